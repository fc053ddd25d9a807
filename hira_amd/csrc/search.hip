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

template <typename T, int LPR, int GMAX>
__global__ __launch_bounds__(256) void search_kernel(const SearchParams p) {
    constexpr int EPL = Elem<T>::kPerChunk;
    constexpr int RPW = kWave / LPR;  // rows per wave-wide load
    constexpr int DVP = LPR * EPL;    // widest row a lane group can hold

    extern __shared__ float smem[];

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

// The fold as a launch of its own: one workgroup per head.
__global__ __launch_bounds__(256) void merge_kernel(const float* __restrict__ part_m,
                                                    const float* __restrict__ part_l,
                                                    const float* __restrict__ part_acc, int P,
                                                    int Dv, int dvl, float* __restrict__ out) {
    __shared__ float red[4];
    extern __shared__ float smem[];  // (NG, Dv + 1)
    const int head = blockIdx.x;
    fold_partials(part_m + (size_t)head * P, part_l + (size_t)head * P,
                  part_acc + (size_t)head * P * Dv, P, Dv, dvl, out + (size_t)head * Dv, smem, red);
}

// ---- host side ------------------------------------------------------------------------
static int round_pow2(int v) {
    int r = 1;
    while (r < v) r <<= 1;
    return r;
}

// compute units of the current device (asked once)
static int compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus = n;
    }
    return cus;
}

static int make_plan(const HiraTree* t, const HiraQuery* q, const HiraQueue* queue,
                     const HiraLaunch* launch, SearchPlan* plan) {
    HIRA_CHECK_ARG(t && q, "tree and query must not be NULL");
    HIRA_CHECK_ARG(t->dtype == HIRA_F32 || t->dtype == HIRA_BF16, "dtype %d", t->dtype);
    const int esize = t->dtype == HIRA_F32 ? 4 : 2;
    const int epl = 16 / esize;
    HIRA_CHECK_ARG(t->num_trees >= 1, "num_trees %d", t->num_trees);
    HIRA_CHECK_ARG(t->num_levels >= 1 && t->num_levels <= HIRA_MAX_LEVELS, "num_levels %d",
                   t->num_levels);
    HIRA_CHECK_ARG(t->bf >= 1 && t->bf <= 64, "branching factor %d not in 1..64", t->bf);
    HIRA_CHECK_ARG(t->dim >= epl && t->dim % epl == 0,
                   "dim %d: rows must be a multiple of 16 bytes", t->dim);
    HIRA_CHECK_ARG(t->vdim >= 0 && t->vdim % epl == 0,
                   "vdim %d: rows must be a multiple of 16 bytes", t->vdim);
    const int widest = t->dim > t->vdim ? t->dim : t->vdim;
    int lpr = round_pow2((widest + epl - 1) / epl);
    if (lpr < 2) lpr = 2;
    HIRA_CHECK_ARG(lpr <= 64, "dim %d / vdim %d too wide (max %d)", t->dim, t->vdim, 64 * epl);
    HIRA_CHECK_ARG(t->keys != nullptr, "keys is NULL");
    for (int l = 0; l < t->num_levels; ++l) {
        HIRA_CHECK_ARG(t->size[l] >= 0 && t->size[l] <= t->cap[l], "size[%d]=%d cap=%d", l,
                       t->size[l], t->cap[l]);
        if (l >= 1) {
            HIRA_CHECK_ARG(t->centers[l] && t->radii[l] && t->counts[l],
                           "level %d arrays missing", l);
            HIRA_CHECK_ARG((int64_t)t->size[l] * t->bf >= t->size[l - 1],
                           "size[%d]=%d exceeds size[%d]*bf", l - 1, t->size[l - 1], l);
        }
    }
    HIRA_CHECK_ARG(q->num_q_heads >= 1 && q->q && q->tau && q->scaling && q->tree_q_off &&
                       q->tree_q_heads,
                   "query arrays missing");
    HIRA_CHECK_ARG(q->max_group >= 1, "max_group %d", q->max_group);
    HIRA_CHECK_ARG(t->layout == HIRA_ROW_MAJOR || t->layout == HIRA_TILE16 ||
                       t->layout == HIRA_TILE16_Q8, "layout %d", t->layout);
    if (t->layout == HIRA_TILE16_Q8)
        HIRA_CHECK_ARG(t->dim % 64 == 0 && t->num_levels >= 2 && t->keys8 && t->kscale && t->keps,
                       "the layout with an 8-bit shadow needs rows of a multiple of 64 columns, at "
                       "least two levels, and the keys8 / kscale / keps arrays");
    if (t->layout != HIRA_ROW_MAJOR) {
        HIRA_CHECK_ARG(t->dtype == HIRA_BF16 && t->dim % 32 == 0,
                       "the tiled layout needs bf16 rows of a multiple of 32 columns");
        for (int l = 0; l < t->num_levels; ++l)
            HIRA_CHECK_ARG(t->cap[l] % 16 == 0, "tiled layout: cap[%d]=%d not a multiple of 16",
                           l, t->cap[l]);
    }
    plan->num_queue_blocks = 0;
    if (queue && queue->keys && queue->len > 0) {
        HIRA_CHECK_ARG(queue->len <= queue->cap, "queue len %d > cap %d", queue->len,
                       queue->cap);
        plan->num_queue_blocks = (queue->len + kPseudoBlock - 1) / kPseudoBlock;
    }
    const int want = launch ? launch->kernel : 0;
    HIRA_CHECK_ARG(want >= 0 && want <= 2, "kernel %d", want);
    const bool mfma_ok = mfma_search_supported(t, queue);
    HIRA_CHECK_ARG(want != 2 || mfma_ok,
                   "the MFMA kernel needs bf16, tiled layout, >= 2 levels, fan-out 16/32/48/64, "
                   "dim = vdim in {64,128,256}, under 4 GiB of key slots per tree");
    plan->kernel = (want == 2 || (want == 0 && mfma_ok)) ? 2 : 1;
    plan->lpr = lpr;
    if (plan->kernel == 2) {
        // one workgroup per tile of 16 level-1 nodes; heads in passes of 16
        plan->gmax = q->max_group < 16 ? q->max_group : 16;
        plan->head_chunks = (q->max_group + 15) / 16;
        int threads = launch && launch->block_threads ? launch->block_threads : kMfmaThreads;
        HIRA_CHECK_ARG(threads >= 64 && threads <= kMfmaThreads && threads % 64 == 0,
                       "block_threads %d must be a multiple of 64 up to %d", threads, kMfmaThreads);
        plan->threads = threads;
        // a workgroup walks `tpw` tiles of 16 level-1 nodes (a stride apart): as few as keep
        // one workgroup per CU in the launch (the kernel runs one at a time on a CU) and at
        // most 64 partials per head to fold
        const int tiles = (t->size[1] + 15) / 16;
        int tpw = launch ? launch->nodes_per_wave : 0;
        HIRA_CHECK_ARG(tpw >= 0 && tpw <= kMfmaMaxTilesPerWg,
                       "MFMA kernel: %d tiles per workgroup (at most %d)", tpw, kMfmaMaxTilesPerWg);
        if (tpw == 0) {
            const int64_t all = (int64_t)tiles * t->num_trees * plan->head_chunks;
            const int cus = compute_units();
            tpw = (int)((all + cus - 1) / cus);
            if (tpw * 64 < tiles) tpw = (tiles + 63) / 64;
            if (tpw < 1) tpw = 1;
            // more work than one workgroup per CU can take: several rounds of smaller ones
            if (tpw > kMfmaMaxTilesPerWg) tpw = kMfmaMaxTilesPerWg / 2;
        }
        // groups of `share` workgroups may gate the same share*tpw tiles (at most 16: two a wave)
        // and split the survivors evenly.  Off unless asked for: measured at the benchmark's
        // shapes the spread between workgroups comes from the burst of key reads draining
        // through the memory system, not from uneven node counts, and the longer gate costs
        // more than the even deal gains.
        int share = launch ? launch->share : 0;
        HIRA_CHECK_ARG(share >= 0 && share * tpw <= kMfmaMaxTilesPerWg,
                       "MFMA kernel: share %d x %d tiles per workgroup (at most %d tiles gated)",
                       share, tpw, kMfmaMaxTilesPerWg);
        if (share == 0) share = 1;
        plan->share = share;
        plan->nodes_per_wave = tpw;
        plan->num_nodes = t->size[1];
        plan->tree_blocks = (tiles + tpw * share - 1) / (tpw * share) * share;
        plan->queue_blocks = plan->num_queue_blocks > 0 ? 1 : 0;  // one workgroup takes the whole queue
        plan->smem = 0;
        return HIRA_OK;
    }
    plan->gmax = q->max_group <= 1 ? 1 : (q->max_group <= 4 ? 4 : 8);
    plan->head_chunks = (q->max_group + plan->gmax - 1) / plan->gmax;
    int threads = launch && launch->block_threads ? launch->block_threads : 256;
    HIRA_CHECK_ARG(threads == 64 || threads == 128 || threads == 256,
                   "block_threads %d must be 64, 128 or 256", threads);
    plan->threads = threads;
    const int rpw = 64 / lpr;
    int npw = launch && launch->nodes_per_wave ? launch->nodes_per_wave : rpw;
    HIRA_CHECK_ARG(npw >= 1, "nodes_per_wave %d", npw);
    plan->nodes_per_wave = npw;
    plan->num_nodes = t->num_levels >= 2 ? t->size[1]
                                         : (t->size[0] + kPseudoBlock - 1) / kPseudoBlock;
    const int per_block = (threads / 64) * npw;
    plan->tree_blocks = (plan->num_nodes + per_block - 1) / per_block;
    plan->queue_blocks = (plan->num_queue_blocks + per_block - 1) / per_block;
    plan->smem = (size_t)(threads / 64) * plan->gmax * (lpr * epl + 2) * sizeof(float);
    {   // the fold of the last workgroup reuses the same LDS: (ng, vdim + 1) floats
        const int dvl = round_pow2((t->vdim + 3) / 4);
        if (dvl > 0 && dvl <= threads) {
            const size_t fold = (size_t)(threads / dvl) * (t->vdim + 1) * sizeof(float);
            if (fold > plan->smem) plan->smem = fold;
        }
    }
    return HIRA_OK;
}

template <typename T, int LPR>
static void launch_search(const SearchPlan& plan, const SearchParams& p, dim3 grid,
                          hipStream_t s) {
    const size_t smem = p.part_acc ? plan.smem : 0;
    switch (plan.gmax) {
        case 1:
            hipLaunchKernelGGL((search_kernel<T, LPR, 1>), grid, dim3(plan.threads), smem, s, p);
            break;
        case 4:
            hipLaunchKernelGGL((search_kernel<T, LPR, 4>), grid, dim3(plan.threads), smem, s, p);
            break;
        default:
            hipLaunchKernelGGL((search_kernel<T, LPR, 8>), grid, dim3(plan.threads), smem, s, p);
            break;
    }
}

template <typename T>
static int dispatch_lpr(const SearchPlan& plan, const SearchParams& p, dim3 grid,
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

using namespace hira;

// partials (acc, m, l) followed by the arrival counters of the fused fold
// bytes of the arrival counters, which come first: their place does not depend on the
// number of partials, so a workspace stays usable when the tree grows or a queue comes and goes
static size_t counter_bytes(int trees, int passes) {
    return (((size_t)trees * passes * sizeof(int32_t)) + 255) & ~(size_t)255;
}

static size_t workspace_need(int h_q, size_t P, int vdim, int trees, int passes) {
    return counter_bytes(trees, passes) + (size_t)h_q * P * (size_t)(vdim + 2) * sizeof(float);
}

extern "C" size_t hira_search_workspace_bytes(const HiraTree* tree, const HiraQuery* query,
                                              const HiraQueue* queue,
                                              const HiraLaunch* launch) {
    SearchPlan plan;
    if (make_plan(tree, query, queue, launch, &plan) != HIRA_OK) return 0;
    const size_t P = (size_t)plan.tree_blocks + plan.queue_blocks;
    return workspace_need(query->num_q_heads, P, tree->vdim, tree->num_trees, plan.head_chunks);
}

// The search behind both entry points.  Attention needs arrival counters (one int32 per tree
// and head pass, zero between calls) and room for the partials; `fixed_counters` > 0: the
// counters live in a region of that many entries of their own (the entry point that allocates
// nothing), else at the start of the caller's workspace, the partials right after them.
static int search_impl(const HiraTree* tree, const HiraQuery* query, const HiraQueue* queue,
                       const HiraSearchOut* out, const HiraLaunch* launch, void* workspace,
                       size_t workspace_bytes, size_t fixed_counters, void* stream) {
    SearchPlan plan;
    int rc = make_plan(tree, query, queue, launch, &plan);
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_ARG(out != nullptr, "out is NULL");
    const bool attn = out->attn_out != nullptr;
    if (attn) {
        HIRA_CHECK_ARG(tree->values != nullptr && tree->vdim > 0,
                       "attention needs values in the tree");
        HIRA_CHECK_ARG(tree->vdim % 4 == 0, "vdim %d must be a multiple of 4", tree->vdim);
        HIRA_CHECK_ARG(plan.num_queue_blocks == 0 || queue->values != nullptr,
                       "queue values missing");
    }
    // by position the row length is the number of keys inserted so far, which only the
    // caller knows; by slot it must cover every slot in use
    if (out->dense && !out->dense_by_position)
        HIRA_CHECK_ARG(out->dense_stride >= tree->size[0], "dense_stride %lld < %d slots",
                       (long long)out->dense_stride, tree->size[0]);
    if (out->dense_by_position && (out->dense || out->sel_count))
        HIRA_CHECK_ARG(tree->perm != nullptr, "perm missing");
    if (out->sel_count)
        HIRA_CHECK_ARG(out->sel_index && out->sel_score && out->sel_cap > 0,
                       "selection list arrays missing");

    SearchParams p;
    memset(&p, 0, sizeof(p));
    p.keys = tree->keys;
    p.values = tree->values;
    p.perm = tree->perm;
    for (int l = 0; l < HIRA_MAX_LEVELS; ++l) {
        p.centers[l] = tree->centers[l];
        p.radii[l] = tree->radii[l];
        p.counts[l] = tree->counts[l];
        p.size[l] = tree->size[l];
        p.cap[l] = tree->cap[l];
    }
    p.num_levels = tree->num_levels;
    p.bf = tree->bf;
    p.dim = tree->dim;
    p.vdim = tree->vdim;
    p.layout = center_layout_of(tree->layout);
    p.key_layout = key_layout_of(tree->layout);
    if (tree->layout == HIRA_TILE16_Q8) {
        p.keys8 = tree->keys8;
        p.kscale = tree->kscale;
        p.keps = tree->keps;
    }
    p.q = query->q;
    p.tau = query->tau;
    p.scaling = query->scaling;
    p.tree_q_off = query->tree_q_off;
    p.tree_q_heads = query->tree_q_heads;
    const bool use_queue = attn && plan.num_queue_blocks > 0;
    if (use_queue) {
        p.queue_keys = queue->keys;
        p.queue_values = queue->values;
        p.queue_len = queue->len;
        p.queue_cap = queue->cap;
    }
    p.nodes_per_wave = plan.nodes_per_wave;
    p.tree_blocks = plan.tree_blocks;
    p.share = plan.kernel == 2 ? plan.share : 1;
    p.num_nodes = plan.num_nodes;
    p.num_queue_blocks = use_queue ? plan.num_queue_blocks : 0;
    p.dense = out->dense;
    p.dense_stride = out->dense_stride;
    p.dense_by_position = out->dense_by_position;
    p.sel_index = out->sel_index;
    p.sel_score = out->sel_score;
    p.sel_count = out->sel_count;
    p.sel_cap = out->sel_cap;
    p.stats = out->stats;

    const int P = plan.tree_blocks + (use_queue ? plan.queue_blocks : 0);
    if (P == 0) return HIRA_OK;
    p.num_parts = P;
    if (attn) {
        size_t ctr_bytes = counter_bytes(tree->num_trees, plan.head_chunks);
        if (fixed_counters > 0) {
            if ((size_t)tree->num_trees * plan.head_chunks > fixed_counters)
                return fail(HIRA_EWORKSPACE, "%d trees x %d head passes: more than the %zu arrival "
                            "counters of the built-in scratch buffer", tree->num_trees,
                            plan.head_chunks, fixed_counters);
            ctr_bytes = fixed_counters * sizeof(int32_t);
        }
        const size_t need = ctr_bytes + workspace_need(query->num_q_heads, (size_t)P, tree->vdim, 0, 0);
        if (workspace == nullptr || workspace_bytes < need)
            return fail(HIRA_EWORKSPACE, fixed_counters > 0
                            ? "the built-in scratch buffer holds %zu bytes, this search needs %zu"
                            : "workspace %zu bytes, need %zu", workspace_bytes, need);
        float* w = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + ctr_bytes);
        p.part_acc = w;
        p.part_m = w + (size_t)query->num_q_heads * P * tree->vdim;
        p.part_l = p.part_m + (size_t)query->num_q_heads * P;
        p.attn_out = out->attn_out;
        // the search kernel folds the partials itself (the last workgroup of a tree to arrive
        // does it) unless the caller asks for the second launch
        p.fold_dvl = round_pow2((tree->vdim + 3) / 4);
        // (vector-ALU kernel: its last workgroup folds the heads of its pass one after the
        // other, which only pays for a single head with few partials; the second launch has
        // a workgroup per head)
        const bool can_fold = plan.kernel == 2 ||
                              (p.fold_dvl <= plan.threads && plan.gmax == 1 && P <= 64);
        if (can_fold && !(launch && launch->separate_merge))
            p.done = reinterpret_cast<int32_t*>(workspace);
    }
    p.group_size = query->group_size > 0 ? query->group_size : 0;
    if (p.group_size > 0)
        HIRA_CHECK_ARG((int64_t)p.group_size * tree->num_trees == query->num_q_heads,
                       "group_size %d x %d trees != %d heads", p.group_size, tree->num_trees,
                       query->num_q_heads);

    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    dim3 grid(P, tree->num_trees, plan.head_chunks);
    p.gmax_state = plan.gmax;
    if (plan.kernel == 2)
        rc = launch_search_mfma(plan, p, dim3(tree->num_trees, P, plan.head_chunks), s);
    else
        rc = tree->dtype == HIRA_F32 ? dispatch_lpr<float>(plan, p, grid, s)
                                     : dispatch_lpr<bf16_t>(plan, p, grid, s);
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_LAUNCH("search kernel");

    if (attn && p.done == nullptr) {
        int dvl = round_pow2((tree->vdim + 3) / 4);
        if (dvl > 256) return fail(HIRA_EINVAL, "vdim %d too wide", tree->vdim);
        const int ng = 256 / dvl;
        const size_t smem = (size_t)ng * (tree->vdim + 1) * sizeof(float);
        hipLaunchKernelGGL(merge_kernel, dim3(query->num_q_heads), dim3(256), smem, s, p.part_m,
                           p.part_l, p.part_acc, P, tree->vdim, dvl, out->attn_out);
        HIRA_CHECK_LAUNCH("merge kernel");
    }
    return HIRA_OK;
}

extern "C" int hira_search(const HiraTree* tree, const HiraQuery* query, const HiraQueue* queue,
                           const HiraSearchOut* out, const HiraLaunch* launch, void* workspace,
                           size_t workspace_bytes, void* stream) {
    return search_impl(tree, query, queue, out, launch, workspace, workspace_bytes, 0, stream);
}

// ---- the same search for callers that cannot allocate ----------------------------------------
// Its scratch (arrival counters, then attention partials) is this array in the library's own
// device image: every GPU the library runs on holds a copy until the process ends.  Host code
// never touches `scratch` by name (the name is a host-side stand-in, not a device address): the
// device address is asked for once per device, with that device current, and kept.
namespace hira {
constexpr size_t kScratchBytes = (size_t)8 << 20;
constexpr size_t kScratchCounters = 16384;  // int32 arrival counters at the start (64 KiB)
constexpr int kMaxDevices = 64;
}  // namespace hira
static __device__ __align__(256) unsigned char scratch[hira::kScratchBytes];
static void* g_scratch_ptr[hira::kMaxDevices];  // per device; written once (same value from any thread)

static int scratch_for_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HIRA_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    HIRA_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "device %d: at most %d devices", dev, kMaxDevices);
    void* ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(HIRA_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev,
                        hipGetErrorString(e));
        __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
    }
    *out = ptr;
    return HIRA_OK;
}

extern "C" int hira_search_noalloc(const HiraTree* tree, const HiraQuery* query,
                                   const HiraQueue* queue, const HiraSearchOut* out,
                                   const HiraLaunch* launch, void* stream) {
    void* ptr = nullptr;
    const int rc = scratch_for_current_device(&ptr);
    if (rc != HIRA_OK) return rc;
    return search_impl(tree, query, queue, out, launch, ptr, kScratchBytes, kScratchCounters, stream);
}
