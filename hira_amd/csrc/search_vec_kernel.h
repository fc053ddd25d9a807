// Halfspace range search over the fixed-fan-out ball tree, fused with sparse attention.
//
// One launch covers every tree and every query head.  A wavefront owns a run of
// consecutive level-1 nodes ("leaf parents").  For each of them it re-derives the gates of
// the node's ancestors (levels L-1 .. 2: one row each, shared by whole subtrees and served
// by the caches), then the node's own gate, and then scans the node's child block of keys.
// No global frontier is exchanged between workgroups, so the walk needs no grid-wide
// synchronisation and a pruned subtree costs its waves one or two row reads.
//
// Lane layout: a row of D elements is 16-byte chunks; LPR lanes hold one row (lane % LPR =
// chunk), so a wave reads 64/LPR rows per 128-bit load instruction, fully coalesced.  The
// G query heads that share the tree (GQA group) are scored against every chunk that is
// loaded: one HBM read of a centroid or key row serves the whole group.
//
// Semantics (reference: kernels/cpp/torch_ext_v3.cpp:172-242, with the conservative
// non-unit-query bound of searcher/cpu.py:61-63): keep a node when q.c + ||q||*r >= tau,
// select a key when q.k >= tau.
#pragma once
#include "search.h"

namespace hira {

constexpr int kUnroll = 8;  // row loads in flight per lane while scanning a block

// out[:] = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p over the P partials of one head, by
// all threads of the workgroup (a multiple of 64, at least dvl).  Thread t owns four columns of
// the output (t % dvl) for the partials p = t / dvl (mod ng).  rows: (ng, Dv + 1) floats of
// LDS, red: one float per wave.  The partials are read with device-scope loads: they may have
// been written by workgroups behind another L2.
__device__ __forceinline__ void fold_partials(const float* pm, const float* pl, const float* pa,
                                              int P, int Dv, int dvl, float* out, float* rows,
                                              float* red) {
    auto ld = [](const float* q) {
        return __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    const int t = threadIdx.x, nt = blockDim.x, nw = nt >> 6;
    float mx = -INFINITY;
    for (int i = t; i < P; i += nt) mx = fmaxf(mx, ld(pm + i));
    mx = wave_max(mx);
    if ((t & 63) == 0) red[t >> 6] = mx;
    __syncthreads();
    float M = red[0];
    for (int w = 1; w < nw; ++w) M = fmaxf(M, red[w]);
    if (M == -INFINITY) {  // nothing selected for this head (uniform)
        for (int e = t; e < Dv; e += nt) out[e] = 0.0f;
        return;
    }
    const int ng = nt / dvl;
    const int gi = t / dvl, li = t % dvl;
    float a[4] = {0.f, 0.f, 0.f, 0.f};
    float lsum = 0.0f;
    const bool lane_ok = li * 4 < Dv;
    for (int i = gi; i < P; i += ng) {
        const float mp = ld(pm + i);
        if (mp == -INFINITY) continue;
        const float w = exp2f(mp - M);
        lsum += w * ld(pl + i);
        if (lane_ok) {
#pragma unroll
            for (int c = 0; c < 4; ++c) a[c] += w * ld(pa + (size_t)i * Dv + li * 4 + c);
        }
    }
    float* row = rows + (size_t)gi * (Dv + 1);
    if (lane_ok) {
#pragma unroll
        for (int c = 0; c < 4; ++c) row[li * 4 + c] = a[c];
    }
    if (li == 0) row[Dv] = lsum;
    __syncthreads();
    float ltot = 0.0f;
    for (int g = 0; g < ng; ++g) ltot += rows[(size_t)g * (Dv + 1) + Dv];
    for (int e = t; e < Dv; e += nt) {
        float sum = 0.0f;
        for (int g = 0; g < ng; ++g) sum += rows[(size_t)g * (Dv + 1) + e];
        out[e] = sum / ltot;
    }
}

// NGX: steps of gates (RPW nodes each) a wave batches: 4 where a node holds few keys, else 1.
template <typename T, int LPR, int GMAX, int NGX>
__global__ __launch_bounds__(256) void search_kernel(const SearchParams p) {
    constexpr int EPL = Elem<T>::kPerChunk;
    constexpr int RPW = kWave / LPR;  // rows per wave-wide load
    constexpr int DVP = LPR * EPL;    // widest row a lane group can hold

    extern __shared__ float smem[];

    touch_kernel_arguments();
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int rg = lane / LPR;
    const int ch = lane % LPR;
    const int tree = blockIdx.y;
    const int D = p.dim;
    const int Dv = p.vdim;
    const int L = p.num_levels;
    const bool chunk_ok = ch * EPL < D;
    const bool vchunk_ok = ch * EPL < Dv;
    const bool want_attn = p.part_acc != nullptr;

    // (group_size > 0: head h of the launch belongs to tree h / group_size; the head map is not
    // read, which saves every wave two dependent trips to memory)
    const bool by_group = p.group_size > 0;
    const int hoff = (by_group ? tree * p.group_size : p.tree_q_off[tree]) + blockIdx.z * GMAX;
    const int G = min(GMAX, (by_group ? (tree + 1) * p.group_size : p.tree_q_off[tree + 1]) - hoff);
    if (G <= 0) return;  // uniform for the workgroup
    const unsigned gmask = (1u << G) - 1u;

    // ---- queries of the group: this lane's chunk of each, plus tau, scaling, ||q|| ----
    int qh[GMAX];
    float qf[GMAX][EPL];
    float tau[GMAX], sc[GMAX], qn[GMAX];
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
        qh[g] = (g < G) ? (by_group ? hoff + g : p.tree_q_heads[hoff + g]) : 0;
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (g < G && chunk_ok) raw = load_chunk<T>(p.q, (size_t)qh[g] * D, ch);
        unpack<T>(raw, qf[g]);
        tau[g] = (g < G) ? p.tau[qh[g]] : INFINITY;
        sc[g] = (g < G) ? p.scaling[qh[g]] : 0.0f;
        float ss = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) ss += qf[g][e] * qf[g][e];
        qn[g] = sqrtf(group_sum<LPR>(ss));
    }

    // ---- attention state of this lane group -------------------------------------------
    float acc[GMAX][EPL];
    float mrun[GMAX], lrun[GMAX];
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
        mrun[g] = -INFINITY;
        lrun[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.0f;
    }

    unsigned long long st_nodes[HIRA_MAX_LEVELS];
    unsigned long long st_sel_any = 0, st_sel_pairs = 0;
#pragma unroll
    for (int l = 0; l < HIRA_MAX_LEVELS; ++l) st_nodes[l] = 0;

    const bool is_queue = (int)blockIdx.x >= p.tree_blocks;
    const int blk = is_queue ? (int)blockIdx.x - p.tree_blocks : (int)blockIdx.x;
    const int n_nodes = is_queue ? p.num_queue_blocks : p.num_nodes;
    const bool real_nodes = !is_queue && L >= 2;
    const int node_first = (blk * nwaves + wave) * p.nodes_per_wave;
    const int node_last = min(node_first + p.nodes_per_wave, n_nodes);

    const void* kbase = is_queue ? p.queue_keys : p.keys;
    const void* vbase = is_queue ? p.queue_values : p.values;
    const size_t krow0 = (size_t)tree * (is_queue ? p.queue_cap : p.cap[0]);
    const int n_rows = is_queue ? p.queue_len : p.size[0];
    const int block_rows = real_nodes ? p.bf : kPseudoBlock;
    const int klayout = is_queue ? HIRA_ROW_MAJOR : p.key_layout;

    // The dense output's stretch under this wave's nodes starts out as the fill value; the
    // scores of selected keys follow from the same wave, behind these stores.
    if (p.dense_fill && !is_queue && node_first < node_last) {
        const int r0 = node_first * block_rows, r1 = min(node_last * block_rows, n_rows);
#pragma unroll
        for (int g = 0; g < GMAX; ++g)
            if (g < G)
                for (int i = r0 + lane; i < r1; i += kWave)
                    p.dense[(int64_t)qh[g] * p.dense_stride + i] = p.dense_fill_value;
    }

    if constexpr (NGX == 1) {
        for (int n0 = node_first; n0 < node_last; n0 += RPW) {
            // -------- gates: lane group rg owns node n0 + rg -----------------------------
            const int node = n0 + rg;
            const bool node_ok = node < node_last;
            unsigned alive = node_ok ? gmask : 0u;
            int cnt = 0;
            if (real_nodes) {
                // the node's own row, radius and child count, and its ancestors at levels L-1 .. 2:
                // independent loads, issued together (the node's are wasted when an ancestor
                // prunes it, which costs bandwidth the gates have to spare, not a trip to memory)
                uint4 raw1 = make_uint4(0, 0, 0, 0);
                float rad1 = 0.0f;
                int cnt1 = 0;
                if (node_ok) {
                    const size_t r = (size_t)tree * p.cap[1] + node;
                    if (chunk_ok)
                        raw1 = load_row_chunk<T>(p.centers[1], p.layout, D, (size_t)tree * p.cap[1],
                                                 node, ch);
                    rad1 = p.radii[1][r];
                    cnt1 = p.counts[1][r];
                }
                uint4 araw[HIRA_MAX_LEVELS - 2];
                float arad[HIRA_MAX_LEVELS - 2];
                int aid[HIRA_MAX_LEVELS - 2];
                {
                    int id = node;
    #pragma unroll
                    for (int l = 2; l < HIRA_MAX_LEVELS; ++l) {
                        id /= p.bf;
                        aid[l - 2] = id;
                        araw[l - 2] = make_uint4(0, 0, 0, 0);
                        arad[l - 2] = 0.0f;
                        if (l < L && node_ok) {
                            const size_t r = (size_t)tree * p.cap[l] + id;
                            if (chunk_ok)
                                araw[l - 2] = load_row_chunk<T>(p.centers[l], p.layout, D,
                                                                (size_t)tree * p.cap[l], id, ch);
                            arad[l - 2] = p.radii[l][r];
                        }
                    }
                }
                // top-down so that `alive` before level l says whether level l is evaluated
    #pragma unroll
                for (int l = HIRA_MAX_LEVELS - 1; l >= 2; --l) {
                    if (l < L) {
                        if (p.stats && alive && ch == 0 && arad[l - 2] > -INFINITY) {
                            // count the node once: by its first level-1 descendant
                            int span = 1;
                            for (int t = 1; t < l; ++t) span *= p.bf;
                            if (node % span == 0) st_nodes[l]++;
                        }
                        float kf[EPL];
                        unpack<T>(araw[l - 2], kf);
                        unsigned pass = 0;
    #pragma unroll
                        for (int g = 0; g < GMAX; ++g) {
                            float d = 0.0f;
    #pragma unroll
                            for (int e = 0; e < EPL; ++e) d += kf[e] * qf[g][e];
                            d = group_sum<LPR>(d);
                            if (d + qn[g] * arad[l - 2] >= tau[g]) pass |= 1u << g;
                        }
                        alive &= pass;
                    }
                }
                // the level-1 node itself, only if some head is still alive above it
                if (alive) {
                    const float rad = rad1;
                    cnt = cnt1;
                    if (p.stats && ch == 0 && rad > -INFINITY) st_nodes[1]++;
                    float kf[EPL];
                    unpack<T>(raw1, kf);
                    unsigned pass = 0;
    #pragma unroll
                    for (int g = 0; g < GMAX; ++g) {
                        float d = 0.0f;
    #pragma unroll
                        for (int e = 0; e < EPL; ++e) d += kf[e] * qf[g][e];
                        d = group_sum<LPR>(d);
                        if (d + qn[g] * rad >= tau[g]) pass |= 1u << g;
                    }
                    alive &= pass;
                }
            } else if (node_ok) {
                cnt = min(kPseudoBlock, n_rows - node * kPseudoBlock);
            }
            if (cnt <= 0) alive = 0u;

            // -------- scan the child blocks of the nodes that survived, one at a time -----
    #pragma unroll 1
            for (int b = 0; b < RPW; ++b) {
                const unsigned am = __shfl(alive, b * LPR, 64);  // wave-uniform
                if (am == 0u) continue;
                const int bcnt = __shfl(cnt, b * LPR, 64);
                const int first = (n0 + b) * block_rows;  // first key slot of the block
                if (p.stats && lane == 0) st_nodes[0] += (unsigned long long)bcnt;

    #pragma unroll 1
                for (int i0 = 0; i0 < bcnt; i0 += RPW * kUnroll) {
                    uint4 raw[kUnroll];
    #pragma unroll
                    for (int u = 0; u < kUnroll; ++u) {
                        const int row = i0 + u * RPW + rg;
                        raw[u] = make_uint4(0, 0, 0, 0);
                        if (row < bcnt && chunk_ok)
                            raw[u] = load_row_chunk<T>(kbase, klayout, D, krow0, first + row, ch);
                    }
    #pragma unroll
                    for (int u = 0; u < kUnroll; ++u) {
                        const int row = i0 + u * RPW + rg;
                        float kf[EPL];
                        unpack<T>(raw[u], kf);
                        float s[GMAX];
                        unsigned sel = 0;
    #pragma unroll
                        for (int g = 0; g < GMAX; ++g) {
                            float d = 0.0f;
    #pragma unroll
                            for (int e = 0; e < EPL; ++e) d += kf[e] * qf[g][e];
                            s[g] = group_sum<LPR>(d);
                            if (((am >> g) & 1u) && row < bcnt && (is_queue || s[g] >= tau[g]))
                                sel |= 1u << g;
                        }
                        if (__ballot(sel != 0u) == 0ull) continue;  // wave-uniform

                        const int slot = first + row;
                        const bool owner = (ch == 0) && sel != 0u;
                        if (p.stats && owner) {
                            st_sel_any++;
                            st_sel_pairs += (unsigned long long)__popc(sel);
                        }
                        if (!is_queue && (p.dense != nullptr || p.sel_count != nullptr)) {
                            int idx = slot;
                            if (owner && p.dense_by_position) idx = p.perm[krow0 + slot];
    #pragma unroll
                            for (int g = 0; g < GMAX; ++g) {
                                const bool mine = owner && ((sel >> g) & 1u);
                                if (p.dense != nullptr && mine)
                                    p.dense[(int64_t)qh[g] * p.dense_stride + idx] = s[g] * sc[g];
                                if (p.sel_count != nullptr) {
                                    const unsigned long long bal = __ballot(mine);
                                    if (bal != 0ull) {
                                        int base = 0;
                                        if (lane == 0)
                                            base = atomicAdd(&p.sel_count[qh[g]], __popcll(bal));
                                        base = __shfl(base, 0, 64);
                                        const int pos =
                                            base + __popcll(bal & ((1ull << lane) - 1ull));
                                        if (mine && pos < p.sel_cap) {
                                            p.sel_index[(int64_t)qh[g] * p.sel_cap + pos] = idx;
                                            p.sel_score[(int64_t)qh[g] * p.sel_cap + pos] = s[g];
                                        }
                                    }
                                }
                            }
                        }
                        if (want_attn && sel != 0u) {
                            uint4 vraw = make_uint4(0, 0, 0, 0);
                            if (vchunk_ok) vraw = load_chunk<T>(vbase, (krow0 + slot) * Dv, ch);
                            float vf[EPL];
                            unpack<T>(vraw, vf);
    #pragma unroll
                            for (int g = 0; g < GMAX; ++g) {
                                if ((sel >> g) & 1u) {
                                    const float z = s[g] * sc[g] * kLog2e;
                                    if (z > mrun[g]) {
                                        const float f = exp2f(mrun[g] - z);
                                        lrun[g] = lrun[g] * f + 1.0f;
    #pragma unroll
                                        for (int e = 0; e < EPL; ++e)
                                            acc[g][e] = acc[g][e] * f + vf[e];
                                        mrun[g] = z;
                                    } else {
                                        const float w = exp2f(z - mrun[g]);
                                        lrun[g] += w;
    #pragma unroll
                                        for (int e = 0; e < EPL; ++e) acc[g][e] += w * vf[e];
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
    } else {
        // A wave takes its nodes NGX * RPW at a time.  All their gates first -- the loads of the NGX
        // steps do not depend on each other, so they are in flight together -- then the key slots of
        // the batch, which are consecutive, as ONE block: a row knows from LDS whether its node
        // survived (and for which heads) and whether it holds a key.  With a fan-out of 4 a wave so
        // pays two trips to memory for 32 keys instead of one per node.
        __shared__ uint32_t s_node[4][NGX * RPW];  // heads a node survives for | child count << 16
        constexpr int KU = kUnroll;
        const float inv_rows = 1.0f / (float)block_rows;
        for (int nb0 = node_first; nb0 < node_last; nb0 += NGX * RPW) {
    #pragma unroll
            for (int g = 0; g < NGX; ++g) {
                // -------- gates: lane group rg owns node nb0 + g * RPW + rg -------------------
                const int node = nb0 + g * RPW + rg;
                const bool node_ok = node < node_last;
                unsigned alive = node_ok ? gmask : 0u;
                int cnt = 0;
                if (real_nodes) {
                    // the node's own row, radius and child count, and its ancestors at levels L-1 .. 2:
                    // independent loads, issued together (the node's are wasted when an ancestor
                    // prunes it, which costs bandwidth the gates have to spare, not a trip to memory)
                    uint4 raw1 = make_uint4(0, 0, 0, 0);
                    float rad1 = 0.0f;
                    int cnt1 = 0;
                    if (node_ok) {
                        const size_t r = (size_t)tree * p.cap[1] + node;
                        if (chunk_ok)
                            raw1 = load_row_chunk<T>(p.centers[1], p.layout, D, (size_t)tree * p.cap[1],
                                                     node, ch);
                        rad1 = p.radii[1][r];
                        cnt1 = p.counts[1][r];
                    }
                    uint4 araw[HIRA_MAX_LEVELS - 2];
                    float arad[HIRA_MAX_LEVELS - 2];
                    int aid[HIRA_MAX_LEVELS - 2];
                    {
                        int id = node;
        #pragma unroll
                        for (int l = 2; l < HIRA_MAX_LEVELS; ++l) {
                            id /= p.bf;
                            aid[l - 2] = id;
                            araw[l - 2] = make_uint4(0, 0, 0, 0);
                            arad[l - 2] = 0.0f;
                            if (l < L && node_ok) {
                                const size_t r = (size_t)tree * p.cap[l] + id;
                                if (chunk_ok)
                                    araw[l - 2] = load_row_chunk<T>(p.centers[l], p.layout, D,
                                                                    (size_t)tree * p.cap[l], id, ch);
                                arad[l - 2] = p.radii[l][r];
                            }
                        }
                    }
                    // top-down so that `alive` before level l says whether level l is evaluated
        #pragma unroll
                    for (int l = HIRA_MAX_LEVELS - 1; l >= 2; --l) {
                        if (l < L) {
                            if (p.stats && alive && ch == 0 && arad[l - 2] > -INFINITY) {
                                // count the node once: by its first level-1 descendant
                                int span = 1;
                                for (int t = 1; t < l; ++t) span *= p.bf;
                                if (node % span == 0) st_nodes[l]++;
                            }
                            float kf[EPL];
                            unpack<T>(araw[l - 2], kf);
                            unsigned pass = 0;
        #pragma unroll
                            for (int g = 0; g < GMAX; ++g) {
                                float d = 0.0f;
        #pragma unroll
                                for (int e = 0; e < EPL; ++e) d += kf[e] * qf[g][e];
                                d = group_sum<LPR>(d);
                                if (d + qn[g] * arad[l - 2] >= tau[g]) pass |= 1u << g;
                            }
                            alive &= pass;
                        }
                    }
                    // the level-1 node itself, only if some head is still alive above it
                    if (alive) {
                        const float rad = rad1;
                        cnt = cnt1;
                        if (p.stats && ch == 0 && rad > -INFINITY) st_nodes[1]++;
                        float kf[EPL];
                        unpack<T>(raw1, kf);
                        unsigned pass = 0;
        #pragma unroll
                        for (int g = 0; g < GMAX; ++g) {
                            float d = 0.0f;
        #pragma unroll
                            for (int e = 0; e < EPL; ++e) d += kf[e] * qf[g][e];
                            d = group_sum<LPR>(d);
                            if (d + qn[g] * rad >= tau[g]) pass |= 1u << g;
                        }
                        alive &= pass;
                    }
                } else if (node_ok) {
                    cnt = min(kPseudoBlock, n_rows - node * kPseudoBlock);
                }
                if (cnt <= 0) alive = 0u;
                if (p.stats && ch == 0 && alive) st_nodes[0] += (unsigned long long)cnt;
                if (ch == 0) s_node[wave][g * RPW + rg] = (uint32_t)alive | ((uint32_t)cnt << 16);
            }
            __builtin_amdgcn_wave_barrier();  // the rows below read what other lanes just wrote
            const int batch_nodes = min(NGX * RPW, node_last - nb0);
            const int nrows = batch_nodes * block_rows;
            const int first = nb0 * block_rows;  // first key slot of the batch
            {
    #pragma unroll 1
                for (int i0 = 0; i0 < nrows; i0 += RPW * KU) {
                    uint4 raw[KU];
                    unsigned am_u[KU];
                    bool any = false;
    #pragma unroll
                    for (int u = 0; u < KU; ++u) {
                        const int row = i0 + u * RPW + rg;
                        // (rows of a batch stay far below 2^22: the float quotient is exact enough)
                        const int k = min((int)(((float)row + 0.5f) * inv_rows), NGX * RPW - 1);
                        const uint32_t info = row < nrows ? s_node[wave][k] : 0u;
                        const bool holds = row - k * block_rows < (int)(info >> 16);
                        am_u[u] = holds ? (info & 0xFFFFu) : 0u;
                        any = any || am_u[u] != 0u;
                        raw[u] = make_uint4(0, 0, 0, 0);
                        if (am_u[u] != 0u && chunk_ok)
                            raw[u] = load_row_chunk<T>(kbase, klayout, D, krow0, first + row, ch);
                    }
                    if (__ballot(any) == 0ull) continue;  // wave-uniform: nothing alive in these rows
    #pragma unroll
                    for (int u = 0; u < KU; ++u) {
                        const int row = i0 + u * RPW + rg;
                        const unsigned am = am_u[u];
                        float kf[EPL];
                        unpack<T>(raw[u], kf);
                        float s[GMAX];
                        unsigned sel = 0;
    #pragma unroll
                        for (int g = 0; g < GMAX; ++g) {
                            float d = 0.0f;
    #pragma unroll
                            for (int e = 0; e < EPL; ++e) d += kf[e] * qf[g][e];
                            s[g] = group_sum<LPR>(d);
                            if (((am >> g) & 1u) && (is_queue || s[g] >= tau[g]))
                                sel |= 1u << g;
                        }
                        if (__ballot(sel != 0u) == 0ull) continue;  // wave-uniform

                        const int slot = first + row;
                        const bool owner = (ch == 0) && sel != 0u;
                        if (p.stats && owner) {
                            st_sel_any++;
                            st_sel_pairs += (unsigned long long)__popc(sel);
                        }
                        if (!is_queue && (p.dense != nullptr || p.sel_count != nullptr)) {
                            int idx = slot;
                            if (owner && p.dense_by_position) idx = p.perm[krow0 + slot];
    #pragma unroll
                            for (int g = 0; g < GMAX; ++g) {
                                const bool mine = owner && ((sel >> g) & 1u);
                                if (p.dense != nullptr && mine)
                                    p.dense[(int64_t)qh[g] * p.dense_stride + idx] = s[g] * sc[g];
                                if (p.sel_count != nullptr) {
                                    const unsigned long long bal = __ballot(mine);
                                    if (bal != 0ull) {
                                        int base = 0;
                                        if (lane == 0)
                                            base = atomicAdd(&p.sel_count[qh[g]], __popcll(bal));
                                        base = __shfl(base, 0, 64);
                                        const int pos =
                                            base + __popcll(bal & ((1ull << lane) - 1ull));
                                        if (mine && pos < p.sel_cap) {
                                            p.sel_index[(int64_t)qh[g] * p.sel_cap + pos] = idx;
                                            p.sel_score[(int64_t)qh[g] * p.sel_cap + pos] = s[g];
                                        }
                                    }
                                }
                            }
                        }
                        if (want_attn && sel != 0u) {
                            uint4 vraw = make_uint4(0, 0, 0, 0);
                            if (vchunk_ok) vraw = load_chunk<T>(vbase, (krow0 + slot) * Dv, ch);
                            float vf[EPL];
                            unpack<T>(vraw, vf);
    #pragma unroll
                            for (int g = 0; g < GMAX; ++g) {
                                if ((sel >> g) & 1u) {
                                    const float z = s[g] * sc[g] * kLog2e;
                                    if (z > mrun[g]) {
                                        const float f = exp2f(mrun[g] - z);
                                        lrun[g] = lrun[g] * f + 1.0f;
    #pragma unroll
                                        for (int e = 0; e < EPL; ++e)
                                            acc[g][e] = acc[g][e] * f + vf[e];
                                        mrun[g] = z;
                                    } else {
                                        const float w = exp2f(z - mrun[g]);
                                        lrun[g] += w;
    #pragma unroll
                                        for (int e = 0; e < EPL; ++e) acc[g][e] += w * vf[e];
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
    }

    if (p.stats) {
        unsigned long long* st = p.stats + (size_t)tree * HIRA_STATS_COLS;
#pragma unroll
        for (int l = 0; l < HIRA_MAX_LEVELS; ++l)
            if (st_nodes[l]) atomicAdd(&st[l], st_nodes[l]);
        if (st_sel_any) atomicAdd(&st[HIRA_MAX_LEVELS], st_sel_any);
        if (st_sel_pairs) atomicAdd(&st[HIRA_MAX_LEVELS + 1], st_sel_pairs);
    }

    if (!want_attn) return;  // uniform

    // ---- merge the lane groups of the wave, then the waves of the workgroup -----------
    float* wsm = smem + (size_t)wave * GMAX * (DVP + 2);
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
        const float mall = cross_group_max<LPR>(mrun[g]);
        const float f = (mrun[g] == -INFINITY) ? 0.0f : exp2f(mrun[g] - mall);
        const float lsum = cross_group_sum<LPR>(lrun[g] * f);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const float a = cross_group_sum<LPR>(acc[g][e] * f);
            if (rg == 0) wsm[g * (DVP + 2) + ch * EPL + e] = a;
        }
        if (lane == 0) {
            wsm[g * (DVP + 2) + DVP] = mall;
            wsm[g * (DVP + 2) + DVP + 1] = lsum;
        }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < G * Dv; t += blockDim.x) {
        const int g = t / Dv, e = t % Dv;
        float mall = -INFINITY;
        for (int w = 0; w < nwaves; ++w)
            mall = fmaxf(mall, smem[((size_t)w * GMAX + g) * (DVP + 2) + DVP]);
        float a = 0.0f, lsum = 0.0f;
        for (int w = 0; w < nwaves; ++w) {
            const float* ws = smem + ((size_t)w * GMAX + g) * (DVP + 2);
            const float mw = ws[DVP];
            const float f = (mw == -INFINITY) ? 0.0f : exp2f(mw - mall);
            a += ws[e] * f;
            lsum += ws[DVP + 1] * f;
        }
        const int head = by_group ? hoff + g : p.tree_q_heads[hoff + g];
        const size_t slot = (size_t)head * p.num_parts + blockIdx.x;
        // device-scope stores: written through, so that the workgroup that folds the partials
        // (maybe behind another L2) reads them without cache-wide flushes
        __hip_atomic_store(&p.part_acc[slot * Dv + e], a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (e == 0) {
            __hip_atomic_store(&p.part_m[slot], mall, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&p.part_l[slot], lsum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (p.done == nullptr) return;  // the caller folds the partials in a second launch

    // ---- the last workgroup of this tree (and head pass) to arrive folds its partials ----
    __shared__ int s_last;
    __shared__ float s_fold_red[4];
    hand_off_release();
    __syncthreads();
    if (threadIdx.x == 0) {
        int* ctr = p.done + (size_t)tree * gridDim.z + blockIdx.z;
        const int ticket = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = ticket == (int)gridDim.x - 1;
        if (s_last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    for (int g = 0; g < G; ++g) {  // uniform
        const int head = by_group ? hoff + g : p.tree_q_heads[hoff + g];
        fold_partials(p.part_m + (size_t)head * p.num_parts, p.part_l + (size_t)head * p.num_parts,
                      p.part_acc + (size_t)head * p.num_parts * Dv, p.num_parts, Dv, p.fold_dvl,
                      p.attn_out + (size_t)head * Dv, smem, s_fold_red);
        __syncthreads();
    }
}

template <typename T, int LPR, int NGX>
inline void launch_search_ngx(const SearchPlan& plan, const SearchParams& p, dim3 grid,
                              hipStream_t s) {
    const size_t smem = p.part_acc ? plan.smem : 0;
    switch (plan.gmax) {
        case 1:
            hipLaunchKernelGGL((search_kernel<T, LPR, 1, NGX>), grid, dim3(plan.threads), smem, s, p);
            break;
        case 4:
            hipLaunchKernelGGL((search_kernel<T, LPR, 4, NGX>), grid, dim3(plan.threads), smem, s, p);
            break;
        default:
            hipLaunchKernelGGL((search_kernel<T, LPR, 8, NGX>), grid, dim3(plan.threads), smem, s, p);
            break;
    }
}

template <typename T, int LPR>
inline void launch_search(const SearchPlan& plan, const SearchParams& p, dim3 grid,
                          hipStream_t s) {
    if (plan.gate_steps > 1) launch_search_ngx<T, LPR, 4>(plan, p, grid, s);
    else launch_search_ngx<T, LPR, 1>(plan, p, grid, s);
}

template <typename T>
inline int dispatch_lpr(const SearchPlan& plan, const SearchParams& p, dim3 grid,
                        hipStream_t s) {
    switch (plan.lpr) {
        case 2: launch_search<T, 2>(plan, p, grid, s); break;
        case 4: launch_search<T, 4>(plan, p, grid, s); break;
        case 8: launch_search<T, 8>(plan, p, grid, s); break;
        case 16: launch_search<T, 16>(plan, p, grid, s); break;
        case 32: launch_search<T, 32>(plan, p, grid, s); break;
        case 64: launch_search<T, 64>(plan, p, grid, s); break;
        default: return fail(HIRA_EINVAL, "unsupported row width");
    }
    return HIRA_OK;
}

}  // namespace hira
