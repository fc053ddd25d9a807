// MFMA search + sparse attention kernel: bf16 keys/centers in the tiled layout
// (HIRA_TILE16), fan-out a multiple of 16, D = Dv in {64, 128, 256}, at least two levels.
//
// One workgroup owns one tile of 16 consecutive level-1 nodes of one tree; workgroup ids
// run fastest over the trees so that, with 8 L2 slices (XCDs) served round-robin, the
// workgroups of one tree share a slice.  Every wave
//   1. issues, before it waits for anything, all the loads the gates need: its heads'
//      queries, the 16 x D tile of level-1 centres, the tiles that hold the ancestors of
//      that tile (one node per level >= 2), radii and child counts;
//   2. gates with v_mfma_f32_16x16x32_bf16: a wave-wide 128-bit load fetches a 16 x 32
//      operand tile from 1 KiB of contiguous memory (that is what the tiled layout is for),
//      the B operand holds the (up to 16) query heads of the GQA group, so the D registers
//      hold score(row, head) with head = lane % 16 and row = 4*(lane/16) + j; a node
//      survives for a head when score + ||q|| r >= tau;
//   3. takes every NW-th surviving node, loads the key tiles of its child block (all at
//      once) and scores them the same way; the leaf filter q.k >= tau is a compare against
//      the lane's own threshold;
//   4. softmax, vectorised over heads: every lane keeps (m, l) of ITS head, raises m by the
//      block's best selected score, turns its selected scores into weights 2^(z - m) and
//      parks them in a wave-private LDS table (row, head); then the value rows of the
//      selected keys are fetched, 8 loads in flight, each row once however many heads
//      selected it, and acc[head][:] += weight(row, head) * v[:] runs branch-free with the
//      accumulators in registers (lane owns Dv/64 columns of every head).
// The waves' states are merged through LDS into one partial per head and workgroup.
//
// Register arrays are only ever indexed by compile-time constants: a run-time index would
// push them to scratch memory.
#pragma once

#include "search.h"

namespace hira {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int kHeadsPerPass = 16;  // MFMA N
constexpr int kMaxTiles = 4;       // key tiles per block: bf <= 64
constexpr int kVBatch = 8;         // value rows in flight per wave

__device__ __forceinline__ bf16x8_t as_bf16x8(const uint4& v) {
    return __builtin_bit_cast(bf16x8_t, v);
}

// chunk pointer of tile `tile` of one tree's tiled matrix (D = 32*KS columns)
template <int KS>
__device__ __forceinline__ const uint4* tile_ptr(const void* base, size_t tree_row0, size_t tile,
                                                 int lane) {
    return reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) +
                                          tree_row0 * (size_t)(32 * KS)) +
           tile * (size_t)(KS * 64) + lane;
}

template <int KS>
__device__ __forceinline__ void load_tile(const uint4* tp, uint4 (&a)[KS]) {
#pragma unroll
    for (int s = 0; s < KS; ++s) a[s] = tp[s * 64];
}

template <int KS>
__device__ __forceinline__ f32x4_t tile_scores(const uint4 (&a)[KS], const bf16x8_t (&bq)[KS]) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[s]), bq[s], acc, 0, 0, 0);
    return acc;
}

__device__ __forceinline__ float pick4(const f32x4_t& v, int j) {
    return j == 0 ? v[0] : (j == 1 ? v[1] : (j == 2 ? v[2] : v[3]));
}

// score of row `i` (0..15) of a scored tile for this lane's head
__device__ __forceinline__ float row_score(const f32x4_t& acc, int i, int col) {
    return __shfl(pick4(acc, i & 3), col + 16 * (i >> 2), 64);
}

__device__ __forceinline__ void stat_add(unsigned long long* st, int slot, unsigned v) {
    if (v) atomicAdd(&st[slot], (unsigned long long)v);
}

// floats of wave-private LDS: the weight table (MT*16 rows x 16 heads) during the scan,
// the wave's state (GS x (D + 2)) afterwards
__host__ __device__ constexpr int mfma_wave_floats(int D, int MT, int GS) {
    return (GS * (D + 2) > MT * 256) ? GS * (D + 2) : MT * 256;
}

template <int KS, int MT, int GS>
__global__ __launch_bounds__(512, (KS <= 4 ? 4 : 2)) void search_mfma_kernel(const SearchParams p) {
    constexpr int D = 32 * KS;
    constexpr int VPL = KS / 2;  // value elements per lane: Dv = D = 64 * VPL
    constexpr int VW = (VPL + 1) / 2;  // dwords of a value row per lane
    constexpr int WAVE_FLOATS = mfma_wave_floats(D, MT, GS);
    extern __shared__ float smem[];

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nw = blockDim.x >> 6;
    const int col = lane & 15;  // head within the pass
    const int kb = lane >> 4;   // column block of 8 inside each 32-column step
    const int tree = blockIdx.x;
    const int t1 = blockIdx.y;  // tile of level-1 nodes
    const int L = p.num_levels, bf = p.bf;
    const bool want_attn = p.part_acc != nullptr;
    unsigned long long* stats = p.stats ? p.stats + (size_t)tree * (HIRA_MAX_LEVELS + 2) : nullptr;

    // ---- heads of this pass ----------------------------------------------------------
    int hoff, G;
    if (p.group_size > 0) {  // head h of the launch belongs to tree h / group_size
        hoff = tree * p.group_size + blockIdx.z * kHeadsPerPass;
        G = min(kHeadsPerPass, p.group_size - (int)blockIdx.z * kHeadsPerPass);
    } else {
        hoff = p.tree_q_off[tree] + blockIdx.z * kHeadsPerPass;
        G = min(kHeadsPerPass, p.tree_q_off[tree + 1] - hoff);
    }
    if (G <= 0) return;  // uniform
    G = min(G, GS);
    const bool head_ok = col < G;
    int qh = 0;
    if (head_ok) qh = p.group_size > 0 ? hoff + col : p.tree_q_heads[hoff + col];

    // ---- every load the gates need, issued before the first wait ------------------------
    uint4 qraw[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qraw[s] = make_uint4(0, 0, 0, 0);
        if (head_ok)
            qraw[s] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.q) +
                                                      (size_t)qh * D + s * 32 + kb * 8);
    }
    const float tau = head_ok ? p.tau[qh] : INFINITY;
    const float sc = head_ok ? p.scaling[qh] : 0.0f;

    const size_t row1 = (size_t)tree * p.cap[1];
    uint4 a1[KS];
    load_tile<KS>(tile_ptr<KS>(p.centers[1], row1, (size_t)t1, lane), a1);
    const float4 r4 = *reinterpret_cast<const float4*>(p.radii[1] + row1 + (size_t)t1 * 16 + 4 * kb);
    const int4 c4 = *reinterpret_cast<const int4*>(p.counts[1] + row1 + (size_t)t1 * 16 + 4 * kb);

    // ancestors: levels L-1 .. 2; the two lowest ones (3 and 2) are fetched right away
    size_t span = 1;  // level-1 nodes under one node of the current level
    for (int l = 2; l < L; ++l) span *= (size_t)bf;
    int lcur = L - 1;
    size_t span_hi = span;
    for (int l = L - 1; l > 3; --l) span_hi /= (size_t)bf;  // span at level min(L-1, 3)
    const int n_par = min(max(L - 2, 0), 2);                // ancestor levels fetched in parallel
    uint4 anc[2][KS];
    float arad[2] = {0.f, 0.f};
    size_t aid[2] = {0, 0};
    {
        size_t sp = span_hi;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (i < n_par) {
                const int l = min(L - 1, 3) - i;
                aid[i] = ((size_t)t1 * 16) / sp;
                load_tile<KS>(tile_ptr<KS>(p.centers[l], (size_t)tree * p.cap[l], aid[i] / 16, lane),
                              anc[i]);
                arad[i] = p.radii[l][(size_t)tree * p.cap[l] + aid[i]];
                sp /= (size_t)bf;
            }
        }
    }

    // ---- B operand and ||q|| -----------------------------------------------------------
    bf16x8_t bq[KS];
    float ss = 0.0f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        bq[s] = as_bf16x8(qraw[s]);
        float f[8];
        unpack<bf16_t>(qraw[s], f);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    const float qn = sqrtf(ss);
    const bool count_nodes = stats != nullptr && wave == 0 && lane == 0;

    // ---- ancestor gates, top-down ---------------------------------------------------------
    bool chain = head_ok;  // this head is still alive above the current level
    for (; lcur > 3; --lcur) {  // trees deeper than four levels: one level at a time
        const size_t a = ((size_t)t1 * 16) / span;
        uint4 t[KS];
        load_tile<KS>(tile_ptr<KS>(p.centers[lcur], (size_t)tree * p.cap[lcur], a / 16, lane), t);
        const float rad = p.radii[lcur][(size_t)tree * p.cap[lcur] + a];
        const bool any_alive = __ballot(chain) != 0ull;
        if (count_nodes && ((size_t)t1 * 16) % span == 0 && any_alive && rad > -INFINITY)
            stat_add(stats, lcur, 1u);
        const float d = row_score(tile_scores<KS>(t, bq), (int)(a % 16), col);
        chain = chain && (d + qn * rad >= tau);
        span /= (size_t)bf;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        if (i < n_par) {
            const bool any_alive = __ballot(chain) != 0ull;
            if (count_nodes && ((size_t)t1 * 16) % span == 0 && any_alive && arad[i] > -INFINITY)
                stat_add(stats, lcur, 1u);
            const float d = row_score(tile_scores<KS>(anc[i], bq), (int)(aid[i] % 16), col);
            chain = chain && (d + qn * arad[i] >= tau);
            span /= (size_t)bf;
            --lcur;
        }
    }
    const bool tile_live = __ballot(chain) != 0ull;  // uniform

    // ---- level-1 gates: 16 nodes at once ----------------------------------------------------
    unsigned alive4 = 0u;
    const int cc[4] = {c4.x, c4.y, c4.z, c4.w};
    if (tile_live) {
        const f32x4_t g1 = tile_scores<KS>(a1, bq);
        const float rr[4] = {r4.x, r4.y, r4.z, r4.w};
        unsigned real = 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (chain && (g1[j] + qn * rr[j] >= tau)) alive4 |= 1u << j;
            if (stats) real += (unsigned)__popcll(__ballot(col == 0 && rr[j] > -INFINITY));
        }
        if (count_nodes) stat_add(stats, 1, real);
    }
    unsigned long long nb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) nb[j] = __ballot((alive4 >> j) & 1u);

    // ---- softmax state: (m, l) of this lane's head; acc[g][e] = column lane*VPL + e of head g
    float* wl = smem + (size_t)wave * WAVE_FLOATS;  // weight table (row, head) during the scan
    const float sc2 = sc * kLog2e;
    const size_t row0 = (size_t)tree * p.cap[0];
    float m_h = -INFINITY, l_h = 0.0f;
    float acc[GS][VPL];
#pragma unroll
    for (int g = 0; g < GS; ++g)
#pragma unroll
        for (int e = 0; e < VPL; ++e) acc[g][e] = 0.0f;

    // ---- my share of the surviving nodes: every nw-th one --------------------------------
    unsigned mine16 = 0u;  // bit n: level-1 node n of the tile survives and is mine
    {
        int k_alive = 0;
#pragma unroll
        for (int n = 0; n < 16; ++n) {
            if (((nb[n & 3] >> (16 * (n >> 2))) & 0xFFFFull) != 0ull) {
                if (k_alive == wave) mine16 |= 1u << n;
                if (++k_alive == nw) k_alive = 0;
            }
        }
    }

    while (mine16 != 0u) {  // uniform
        const int n = __ffs(mine16) - 1;
        mine16 &= mine16 - 1u;
        const int jn = n & 3;
        const unsigned long long nbits = jn == 0 ? nb[0] : (jn == 1 ? nb[1] : (jn == 2 ? nb[2] : nb[3]));
        const unsigned node_mask = (unsigned)((nbits >> (16 * (n >> 2))) & 0xFFFFull);
        const int cnt = __shfl(jn == 0 ? cc[0] : (jn == 1 ? cc[1] : (jn == 2 ? cc[2] : cc[3])),
                               16 * (n >> 2), 64);
        const size_t slot0 = (size_t)(t1 * 16 + n) * bf;
        const bool my_alive = (node_mask >> col) & 1u;
        if (stats && lane == 0) stat_add(stats, 0, (unsigned)cnt);

        // all key tiles of the block in flight at once
        uint4 a[MT][KS];
#pragma unroll
        for (int tt = 0; tt < MT; ++tt)
            if (tt * 16 < cnt) load_tile<KS>(tile_ptr<KS>(p.keys, row0, slot0 / 16 + tt, lane), a[tt]);

        f32x4_t sco[MT];
        unsigned sel4[MT];
        unsigned long long sb[MT][4];
        unsigned long long any = 0ull;
#pragma unroll
        for (int tt = 0; tt < MT; ++tt) {
            sel4[tt] = 0u;
            sco[tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (tt * 16 < cnt) {
                sco[tt] = tile_scores<KS>(a[tt], bq);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (my_alive && (tt * 16 + 4 * kb + j) < cnt && sco[tt][j] >= tau) sel4[tt] |= 1u << j;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sb[tt][j] = __ballot((sel4[tt] >> j) & 1u);
                any |= sb[tt][j];
            }
        }
        if (any == 0ull) continue;  // uniform: nothing selected in this block

        // ---- dense scores / compact lists ----------------------------------------------------
        if (p.dense != nullptr || p.sel_count != nullptr) {
#pragma unroll
            for (int tt = 0; tt < MT; ++tt) {
                if ((sb[tt][0] | sb[tt][1] | sb[tt][2] | sb[tt][3]) == 0ull) continue;
                const unsigned tslot = (unsigned)(slot0 + tt * 16);
                int base = 0;
                if (p.sel_count != nullptr) {  // one atomic per head of the tile (lane g, kb = 0)
                    int mine = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        mine += __popcll(sb[tt][j] & (0x0001000100010001ull << col));
                    int b0 = 0;
                    if (kb == 0 && mine > 0) b0 = atomicAdd(&p.sel_count[qh], mine);
                    base = __shfl(b0, col, 64);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if ((sel4[tt] >> j) & 1u) {
                        const unsigned slot = tslot + 4 * kb + j;
                        int idx = (int)slot;
                        if (p.dense_by_position) idx = p.perm[row0 + slot];
                        if (p.dense != nullptr)
                            p.dense[(int64_t)qh * p.dense_stride + idx] = sco[tt][j] * sc;
                        if (p.sel_count != nullptr) {
                            // hits of my head ordered before (kb, j): rows j' < j of any kb,
                            // then row j of lower kb
                            int before = 0;
#pragma unroll
                            for (int j2 = 0; j2 < 4; ++j2) {
                                unsigned long long bits = sb[tt][j2] & (0x0001000100010001ull << col);
                                if (j2 == j) bits &= (1ull << (16 * kb)) - 1ull;
                                if (j2 <= j) before += __popcll(bits);
                            }
                            const int pos = base + before;
                            if (pos < p.sel_cap) {
                                p.sel_index[(int64_t)qh * p.sel_cap + pos] = idx;
                                p.sel_score[(int64_t)qh * p.sel_cap + pos] = sco[tt][j];
                            }
                        }
                    }
                }
            }
        }
        if (stats && lane == 0) {
            unsigned pairs = 0, rows = 0;
#pragma unroll
            for (int tt = 0; tt < MT; ++tt)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    pairs += (unsigned)__popcll(sb[tt][j]);
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) rows += ((sb[tt][j] >> (16 * q4)) & 0xFFFFull) != 0ull;
                }
            stat_add(stats, HIRA_MAX_LEVELS, rows);
            stat_add(stats, HIRA_MAX_LEVELS + 1, pairs);
        }
        if (!want_attn) continue;

        // ---- softmax bookkeeping, one head per lane -------------------------------------------
        float zmax = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < MT; ++tt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if ((sel4[tt] >> j) & 1u) zmax = fmaxf(zmax, sco[tt][j] * sc2);
        zmax = fmaxf(zmax, __shfl_xor(zmax, 16, 64));
        zmax = fmaxf(zmax, __shfl_xor(zmax, 32, 64));
        const float mnew = fmaxf(m_h, zmax);
        // rescale factor of what this head has accumulated so far (1 if nothing changes)
        const float f = (zmax == -INFINITY || m_h == mnew) ? 1.0f : exp2f(m_h - mnew);
        float lsum = 0.0f;
#pragma unroll
        for (int tt = 0; tt < MT; ++tt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float w = ((sel4[tt] >> j) & 1u) ? exp2f(sco[tt][j] * sc2 - mnew) : 0.0f;
                lsum += w;
                wl[(tt * 16 + 4 * kb + j) * 16 + col] = w;
            }
        lsum += __shfl_xor(lsum, 16, 64);
        lsum += __shfl_xor(lsum, 32, 64);
        l_h = l_h * f + lsum;
        m_h = mnew;
        if (__ballot(f != 1.0f) != 0ull) {  // uniform
#pragma unroll
            for (int g = 0; g < GS; ++g) {
                const float fg = __shfl(f, g, 64);
#pragma unroll
                for (int e = 0; e < VPL; ++e) acc[g][e] *= fg;
            }
        }

        // ---- value rows of the selected keys: each row once, kVBatch loads in flight --------
        unsigned long long rowmask = 0ull;  // bit tt*16 + r
#pragma unroll
        for (int tt = 0; tt < MT; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (((sb[tt][r & 3] >> (16 * (r >> 2))) & 0xFFFFull) != 0ull)
                    rowmask |= 1ull << (tt * 16 + r);
        while (rowmask != 0ull) {  // uniform
            int rows[kVBatch];
            uint32_t vraw[kVBatch][VW];
#pragma unroll
            for (int u = 0; u < kVBatch; ++u) {
                rows[u] = -1;
#pragma unroll
                for (int e = 0; e < VW; ++e) vraw[u][e] = 0u;
                if (rowmask != 0ull) {
                    const int r = __ffsll((long long)rowmask) - 1;
                    rowmask &= rowmask - 1ull;
                    rows[u] = r;
                    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.values) +
                                         (row0 + slot0 + r) * (size_t)D + lane * VPL;
                    if (VPL == 1) {
                        vraw[u][0] = *vp;
                    } else {
#pragma unroll
                        for (int e = 0; e < VPL / 2; ++e)
                            vraw[u][e] = reinterpret_cast<const uint32_t*>(vp)[e];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kVBatch; ++u) {
                if (rows[u] < 0) break;  // uniform
                float vf[VPL];
                if (VPL == 1) {
                    vf[0] = bf16_lo(vraw[u][0]);
                } else {
#pragma unroll
                    for (int e = 0; e < VPL / 2; ++e) {
                        vf[2 * e] = bf16_lo(vraw[u][e]);
                        vf[2 * e + 1] = bf16_hi(vraw[u][e]);
                    }
                }
                const float* wr = wl + rows[u] * 16;  // weights of this row, one per head
#pragma unroll
                for (int g = 0; g < GS; ++g) {
                    const float w = wr[g];  // same address in every lane: a broadcast read
#pragma unroll
                    for (int e = 0; e < VPL; ++e) acc[g][e] += w * vf[e];
                }
            }
        }
    }
    if (!want_attn) return;  // uniform

    // ---- the wave's state goes to LDS: (GS, D + 2) = acc[D], m, l per head ----------------
    float* wsm = smem + (size_t)wave * WAVE_FLOATS;
#pragma unroll
    for (int g = 0; g < GS; ++g)
#pragma unroll
        for (int e = 0; e < VPL; ++e) wsm[g * (D + 2) + lane * VPL + e] = acc[g][e];
    if (kb == 0 && col < GS) {
        wsm[col * (D + 2) + D] = m_h;
        wsm[col * (D + 2) + D + 1] = l_h;
    }
    __syncthreads();

    // ---- merge the waves' states into this workgroup's partial ------------------------------
    const int P = p.num_parts;
    for (int t = threadIdx.x; t < G * D; t += blockDim.x) {
        const int g = t / D, e = t % D;
        float mall = -INFINITY;
        for (int w = 0; w < nw; ++w) mall = fmaxf(mall, smem[(size_t)w * WAVE_FLOATS + g * (D + 2) + D]);
        float a_sum = 0.0f, lsum = 0.0f;
        for (int w = 0; w < nw; ++w) {
            const float* ws = smem + (size_t)w * WAVE_FLOATS + g * (D + 2);
            const float mw = ws[D];
            const float f = (mw == -INFINITY) ? 0.0f : exp2f(mw - mall);
            a_sum += ws[e] * f;
            lsum += ws[D + 1] * f;
        }
        const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
        const size_t slot = (size_t)head * P + t1;
        // device-scope stores: written through, so that the workgroup that folds the
        // partials (maybe on another L2 slice) reads them without cache-wide flushes
        __hip_atomic_store(&p.part_acc[slot * D + e], a_sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (e == 0) {
            __hip_atomic_store(&p.part_m[slot], mall, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&p.part_l[slot], lsum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (p.done == nullptr) return;  // the caller folds the partials in a second launch

    // ---- the last workgroup of this tree (and pass) to arrive folds the tree's partials ----
    __shared__ int s_last;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // my stores have completed
    __syncthreads();
    if (threadIdx.x == 0) {
        int* ctr = p.done + (size_t)tree * gridDim.z + blockIdx.z;
        const int ticket = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = ticket == (int)gridDim.y - 1;
        if (s_last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;

    auto ld = [](const float* q) {
        return __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    float* red = smem;                      // (16, 2): M and L of every head
    float* wts = smem + 2 * kHeadsPerPass;  // (G, P) weights 2^(m_p - M), if they fit
    const bool wts_fit = (size_t)G * P + 2 * kHeadsPerPass <= (size_t)nw * WAVE_FLOATS;
    // phase 1: wave w handles heads w, w + nw, ...: M = max m_p, L = sum 2^(m_p - M) l_p
    for (int g = wave; g < G; g += nw) {
        const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
        const float* pm = p.part_m + (size_t)head * P;
        const float* pl = p.part_l + (size_t)head * P;
        float mx = -INFINITY;
        for (int i = lane; i < P; i += 64) mx = fmaxf(mx, ld(pm + i));
        mx = wave_max(mx);
        float ls = 0.0f;
        for (int i = lane; i < P; i += 64) {
            const float mp = ld(pm + i);
            const float lp = ld(pl + i);
            const float w = (mp > -INFINITY) ? exp2f(mp - mx) : 0.0f;
            ls += w * lp;
            if (wts_fit) wts[g * P + i] = w;
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) ls += __shfl_xor(ls, off, 64);
        if (lane == 0) {
            red[2 * g] = mx;
            red[2 * g + 1] = ls;
        }
    }
    __syncthreads();
    // phase 2: thread t owns output column e of head g; empty partials are skipped
    for (int t = threadIdx.x; t < G * D; t += blockDim.x) {
        const int g = t / D, e = t % D;
        const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
        const float M = red[2 * g], Lg = red[2 * g + 1];
        const float* pm = p.part_m + (size_t)head * P;
        const float* pa = p.part_acc + (size_t)head * P * D + e;
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
        if (Lg > 0.0f) {
            int i = 0;
#pragma unroll 4
            for (; i + 4 <= P; i += 4) {
                float w0, w1, w2, w3;
                if (wts_fit) {
                    w0 = wts[g * P + i], w1 = wts[g * P + i + 1];
                    w2 = wts[g * P + i + 2], w3 = wts[g * P + i + 3];
                } else {
                    const float m0 = ld(pm + i), m1 = ld(pm + i + 1), m2 = ld(pm + i + 2), m3 = ld(pm + i + 3);
                    w0 = m0 > -INFINITY ? exp2f(m0 - M) : 0.0f;
                    w1 = m1 > -INFINITY ? exp2f(m1 - M) : 0.0f;
                    w2 = m2 > -INFINITY ? exp2f(m2 - M) : 0.0f;
                    w3 = m3 > -INFINITY ? exp2f(m3 - M) : 0.0f;
                }
                // weights are uniform over the columns of a head: the skips do not diverge
                if (w0 > 0.0f) s0 += w0 * ld(pa + (size_t)i * D);
                if (w1 > 0.0f) s1 += w1 * ld(pa + (size_t)(i + 1) * D);
                if (w2 > 0.0f) s2 += w2 * ld(pa + (size_t)(i + 2) * D);
                if (w3 > 0.0f) s3 += w3 * ld(pa + (size_t)(i + 3) * D);
            }
            for (; i < P; ++i) {
                const float mi = ld(pm + i);
                const float w = wts_fit ? wts[g * P + i] : (mi > -INFINITY ? exp2f(mi - M) : 0.0f);
                if (w > 0.0f) s0 += w * ld(pa + (size_t)i * D);
            }
        }
        const float inv = Lg > 0.0f ? 1.0f / Lg : 0.0f;
        p.attn_out[(size_t)head * D + e] = (s0 + s1 + s2 + s3) * inv;
    }
}

template <int KS, int MT>
void launch_mfma_gs(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    const dim3 block(plan.threads);
    if (plan.gmax <= 4)
        hipLaunchKernelGGL((search_mfma_kernel<KS, MT, 4>), grid, block, plan.smem, s, p);
    else if (plan.gmax <= 8)
        hipLaunchKernelGGL((search_mfma_kernel<KS, MT, 8>), grid, block, plan.smem, s, p);
    else
        hipLaunchKernelGGL((search_mfma_kernel<KS, MT, 16>), grid, block, plan.smem, s, p);
}

template <int KS>
void launch_mfma_mt(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    const int mt = p.bf / 16;
    if (mt <= 1)
        launch_mfma_gs<KS, 1>(plan, p, grid, s);
    else if (mt == 2)
        launch_mfma_gs<KS, 2>(plan, p, grid, s);
    else
        launch_mfma_gs<KS, 4>(plan, p, grid, s);
}

// one translation unit per key width keeps the build parallel
void launch_mfma_d64(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_d128(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_d256(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);

}  // namespace hira
