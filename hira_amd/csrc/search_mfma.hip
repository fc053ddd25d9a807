// MFMA search + sparse attention kernel: bf16 keys/centers in the tiled layout
// (HIRA_TILE16), fan-out a multiple of 16, D = Dv in {64, 128, 256}, at least two levels.
//
// One workgroup owns one tile of 16 consecutive level-1 nodes of one tree.  Every wave
//   1. gates the tile's ancestors (one node per level >= 2: a 16-byte-chunk dot product on
//      the vector ALU, the row is shared by all lanes that hold the same column block);
//   2. gates the 16 level-1 nodes at once: KS wave-wide 128-bit loads fetch the 16 x D
//      centre tile straight in MFMA A-operand order (1 KiB of contiguous memory per load),
//      v_mfma_f32_16x16x32_bf16 multiplies it with the B operand that holds the (up to 16)
//      query heads of the GQA group;
//   3. takes every NW-th surviving node and scans its child block of keys the same way:
//      bf/16 tiles, KS loads + KS MFMAs each; the D registers hold score(key row, head)
//      with head = lane % 16, key row = 4*(lane/16) + j, so the leaf filter q.k >= tau is a
//      compare against the lane's own threshold and wave ballots give, per key row, the
//      mask of heads that selected it;
//   4. for every selected key row loads the value row once (64 lanes x Dv/64 elements)
//      and folds it into the running softmax state of each selecting head.
// The waves' states are merged through LDS and written as one partial per head and
// workgroup; merge_kernel folds the partials.
#include "search.h"

namespace hira {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int kHeadsPerPass = 16;  // MFMA N
constexpr int kMaxTiles = 4;       // key tiles per block: bf <= 64

__device__ __forceinline__ bf16x8_t as_bf16x8(const uint4& v) {
    return __builtin_bit_cast(bf16x8_t, v);
}

// chunk pointer of tile `tile` of one tree's tiled matrix
template <int KS>
__device__ __forceinline__ const uint4* tile_ptr(const void* base, size_t tree_row0, size_t tile,
                                                 int lane) {
    return reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) +
                                          tree_row0 * (size_t)(32 * KS)) +
           tile * (size_t)(KS * 64) + lane;
}

template <int KS>
__device__ __forceinline__ f32x4_t tile_scores(const uint4 (&a)[KS], const bf16x8_t (&bq)[KS]) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[s]), bq[s], acc, 0, 0, 0);
    return acc;
}

template <int KS, int MT>
__global__ __launch_bounds__(512) void search_mfma_kernel(const SearchParams p) {
    constexpr int D = 32 * KS;
    constexpr int VPL = KS / 2;  // value elements per lane: Dv = D = 64 * VPL
    extern __shared__ float smem[];

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nw = blockDim.x >> 6;
    const int col = lane & 15;  // head within the pass
    const int kb = lane >> 4;   // column block of 8 inside each 32-column step
    const int tree = blockIdx.y;
    const int t1 = blockIdx.x;  // tile of level-1 nodes
    const int L = p.num_levels, bf = p.bf;

    const int hoff = p.tree_q_off[tree] + blockIdx.z * kHeadsPerPass;
    const int G = min(kHeadsPerPass, p.tree_q_off[tree + 1] - hoff);
    if (G <= 0) return;  // uniform
    const bool head_ok = col < G;
    const int qh = head_ok ? p.tree_q_heads[hoff + col] : 0;

    // B operand: this lane's 8 columns of its head's query in each 32-column step
    bf16x8_t bq[KS];
    float qf[KS][8];
    float ss = 0.0f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (head_ok)
            raw = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.q) +
                                                  (size_t)qh * D + s * 32 + kb * 8);
        bq[s] = as_bf16x8(raw);
        unpack<bf16_t>(raw, qf[s]);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += qf[s][e] * qf[s][e];
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    const float qn = sqrtf(ss);
    const float tau = head_ok ? p.tau[qh] : INFINITY;
    const float sc = head_ok ? p.scaling[qh] : 0.0f;

    unsigned long long st_nodes[HIRA_MAX_LEVELS];
    unsigned long long st_any = 0, st_pairs = 0;
#pragma unroll
    for (int l = 0; l < HIRA_MAX_LEVELS; ++l) st_nodes[l] = 0;
    const bool count_nodes = p.stats != nullptr && wave == 0;

    // ---- level-1 tile: loads go out first, the ancestors are checked meanwhile --------
    const size_t row1 = (size_t)tree * p.cap[1];
    uint4 a1[KS];
    {
        const uint4* tp = tile_ptr<KS>(p.centers[1], row1, (size_t)t1, lane);
#pragma unroll
        for (int s = 0; s < KS; ++s) a1[s] = tp[s * 64];
    }
    const float4 r4 = *reinterpret_cast<const float4*>(p.radii[1] + row1 + (size_t)t1 * 16 + 4 * kb);

    bool anc_alive = head_ok;
    {
        size_t span = 1;
        for (int l = 2; l < L; ++l) span *= (size_t)bf;
        for (int l = L - 1; l >= 2; --l) {  // top-down
            const size_t a = ((size_t)t1 * 16) / span;  // the tile's ancestor at level l
            const float rad = p.radii[l][(size_t)tree * p.cap[l] + a];
            if (count_nodes && ((size_t)t1 * 16) % span == 0 && __ballot(anc_alive) != 0ull &&
                rad > -INFINITY)
                st_nodes[l]++;
            const uint4* tp = tile_ptr<KS>(p.centers[l], (size_t)tree * p.cap[l], a / 16,
                                           kb * 16 + (int)(a % 16));
            float d = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const uint4 raw = tp[s * 64];
                float cf[8];
                unpack<bf16_t>(raw, cf);
#pragma unroll
                for (int e = 0; e < 8; ++e) d += cf[e] * qf[s][e];
            }
            d += __shfl_xor(d, 16, 64);
            d += __shfl_xor(d, 32, 64);
            anc_alive = anc_alive && (d + qn * rad >= tau);
            span /= (size_t)bf;
        }
    }
    const bool tile_live = __ballot(anc_alive) != 0ull;  // uniform

    unsigned alive4 = 0u;
    if (tile_live) {
        const f32x4_t g1 = tile_scores<KS>(a1, bq);
        const float rr[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (anc_alive && (g1[j] + qn * rr[j] >= tau)) alive4 |= 1u << j;
            const unsigned long long vb = __ballot(col == 0 && rr[j] > -INFINITY);
            if (count_nodes) st_nodes[1] += (unsigned long long)__popcll(vb);
        }
    }
    unsigned long long nb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) nb[j] = __ballot((alive4 >> j) & 1u);

    // ---- running softmax state of every head: wave-private LDS, (GS, D + 2) floats:
    //      acc[D], then m (in log2 units) and l.  Selections are rare, so the state is
    //      touched seldom; keeping it out of the registers keeps the scan lean.
    const int GS = p.gmax_state;  // heads per pass the LDS rows were sized for
    float* wsm = smem + (size_t)wave * GS * (D + 2);
    const float sc2 = sc * kLog2e;
    const bool want_attn = p.part_acc != nullptr;
    const size_t row0 = (size_t)tree * p.cap[0];
    if (want_attn) {
        for (int i = lane; i < G * (D + 2); i += 64) {
            const int e = i % (D + 2);
            wsm[i] = (e == D) ? -INFINITY : 0.0f;
        }
    }

    // ---- scan the child blocks of the surviving nodes, every nw-th one is mine --------
    int k_alive = 0;
#pragma unroll 1
    for (int n = 0; n < 16; ++n) {
        const unsigned long long b = nb[n & 3];
        const unsigned mask16 = (unsigned)((b >> (16 * (n >> 2))) & 0xFFFFull);
        if (mask16 == 0u) continue;
        if ((k_alive++ % nw) != wave) continue;
        const int node = t1 * 16 + n;
        const int cnt = p.counts[1][row1 + node];
        const bool my_alive = (mask16 >> col) & 1u;
        const size_t slot0 = (size_t)node * bf;
        const int ntiles = (cnt + 15) >> 4;
        if (p.stats && lane == 0) st_nodes[0] += (unsigned long long)cnt;

        uint4 a[MT][KS];
#pragma unroll
        for (int tt = 0; tt < MT; ++tt) {
            if (tt < ntiles) {
                const uint4* tp = tile_ptr<KS>(p.keys, row0, slot0 / 16 + tt, lane);
#pragma unroll
                for (int s = 0; s < KS; ++s) a[tt][s] = tp[s * 64];
            }
        }
#pragma unroll
        for (int tt = 0; tt < MT; ++tt) {
            if (tt >= ntiles) break;
            const f32x4_t sco = tile_scores<KS>(a[tt], bq);
            unsigned sel4 = 0u;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (my_alive && (tt * 16 + 4 * kb + j) < cnt && sco[j] >= tau) sel4 |= 1u << j;
            unsigned long long sb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) sb[j] = __ballot((sel4 >> j) & 1u);
            if ((sb[0] | sb[1] | sb[2] | sb[3]) == 0ull) continue;  // uniform

            // dense scores / compact lists: every lane writes its own (key row, head) hits
            if (sel4 != 0u && (p.dense != nullptr || p.sel_count != nullptr)) {
                int base = 0;
                if (p.sel_count != nullptr) base = atomicAdd(&p.sel_count[qh], __popc(sel4));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if ((sel4 >> j) & 1u) {
                        const size_t slot = slot0 + tt * 16 + 4 * kb + j;
                        int idx = (int)slot;
                        if (p.dense_by_position) idx = p.perm[row0 + slot];
                        if (p.dense != nullptr)
                            p.dense[(int64_t)qh * p.dense_stride + idx] = sco[j] * sc;
                        if (p.sel_count != nullptr) {
                            if (base < p.sel_cap) {
                                p.sel_index[(int64_t)qh * p.sel_cap + base] = idx;
                                p.sel_score[(int64_t)qh * p.sel_cap + base] = sco[j];
                            }
                            ++base;
                        }
                    }
                }
            }
            if (p.stats && lane == 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    st_pairs += (unsigned long long)__popcll(sb[j]);
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) st_any += ((sb[j] >> (16 * q4)) & 0xFFFFull) != 0ull;
                }
            }
            if (!want_attn) continue;

            // value rows of the selected keys, 8 per batch: loads first, then the updates
            unsigned rowmask = 0u;  // bit r: key row r of the tile selected by some head
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (((sb[r & 3] >> (16 * (r >> 2))) & 0xFFFFull) != 0ull) rowmask |= 1u << r;
            while (rowmask != 0u) {  // uniform
                int rows[8];
                uint32_t vraw[8][(VPL + 1) / 2];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    rows[u] = -1;
#pragma unroll
                    for (int e = 0; e < (VPL + 1) / 2; ++e) vraw[u][e] = 0u;
                    if (rowmask != 0u) {
                        const int r = __ffs(rowmask) - 1;
                        rowmask &= rowmask - 1u;
                        rows[u] = r;
                        const size_t vrow = row0 + slot0 + tt * 16 + r;
                        const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.values) +
                                             vrow * (size_t)D + lane * VPL;
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
                for (int u = 0; u < 8; ++u) {
                    if (rows[u] < 0) break;  // uniform
                    const int r = rows[u];
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
                    const int j = r & 3;
                    const float srow = j == 0 ? sco[0] : (j == 1 ? sco[1] : (j == 2 ? sco[2] : sco[3]));
                    // z = score * scaling * log2(e) of (row r, head = my column)
                    const float zrow = srow * sc2;
                    unsigned hm = (unsigned)((sb[j] >> (16 * (r >> 2))) & 0xFFFFull);
                    while (hm != 0u) {  // uniform: heads that selected this key
                        const int g = __ffs(hm) - 1;
                        hm &= hm - 1u;
                        const float z = __shfl(zrow, (r >> 2) * 16 + g, 64);
                        float* st = wsm + g * (D + 2);
                        const float m = st[D];
                        const float mnew = fmaxf(m, z);
                        const float f = exp2f(m - mnew);  // 0 when m = -inf
                        const float w = exp2f(z - mnew);
#pragma unroll
                        for (int e = 0; e < VPL; ++e)
                            st[lane * VPL + e] = st[lane * VPL + e] * f + w * vf[e];
                        if (lane == 0) {
                            st[D] = mnew;
                            st[D + 1] = st[D + 1] * f + w;
                        }
                    }
                }
            }
        }
    }

    if (p.stats && lane == 0) {
        unsigned long long* st = p.stats + (size_t)tree * (HIRA_MAX_LEVELS + 2);
#pragma unroll
        for (int l = 0; l < HIRA_MAX_LEVELS; ++l)
            if (st_nodes[l]) atomicAdd(&st[l], st_nodes[l]);
        if (st_any) atomicAdd(&st[HIRA_MAX_LEVELS], st_any);
        if (st_pairs) atomicAdd(&st[HIRA_MAX_LEVELS + 1], st_pairs);
    }
    if (!want_attn) return;  // uniform

    // ---- merge the waves' states: (nw, GS, D + 2) in LDS -----------------------------------
    __syncthreads();
    for (int t = threadIdx.x; t < G * D; t += blockDim.x) {
        const int g = t / D, e = t % D;
        float mall = -INFINITY;
        for (int w = 0; w < nw; ++w) mall = fmaxf(mall, smem[((size_t)w * GS + g) * (D + 2) + D]);
        float acc = 0.0f, lsum = 0.0f;
        for (int w = 0; w < nw; ++w) {
            const float* ws = smem + ((size_t)w * GS + g) * (D + 2);
            const float mw = ws[D];
            const float f = (mw == -INFINITY) ? 0.0f : exp2f(mw - mall);
            acc += ws[e] * f;
            lsum += ws[D + 1] * f;
        }
        const int head = p.tree_q_heads[hoff + g];
        const size_t slot = (size_t)head * p.num_parts + blockIdx.x;
        p.part_acc[slot * D + e] = acc;
        if (e == 0) {
            p.part_m[slot] = mall;
            p.part_l[slot] = lsum;
        }
    }
}

bool mfma_search_supported(const HiraTree* t, const HiraQueue* queue) {
    if (t->dtype != HIRA_BF16 || t->layout != HIRA_TILE16) return false;
    if (t->num_levels < 2) return false;
    if (t->bf % 16 != 0 || t->bf > 16 * kMaxTiles) return false;
    if (!(t->dim == 64 || t->dim == 128 || t->dim == 256)) return false;
    if (t->vdim != 0 && t->vdim != t->dim) return false;
    if (queue && queue->keys && queue->len > 0) return false;
    return true;
}

template <int KS>
static int launch_gs(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    const size_t smem = p.part_acc ? plan.smem : 0;
    const int mt = p.bf / 16;
    if (mt <= 1)
        hipLaunchKernelGGL((search_mfma_kernel<KS, 1>), grid, dim3(plan.threads), smem, s, p);
    else if (mt == 2)
        hipLaunchKernelGGL((search_mfma_kernel<KS, 2>), grid, dim3(plan.threads), smem, s, p);
    else
        hipLaunchKernelGGL((search_mfma_kernel<KS, 4>), grid, dim3(plan.threads), smem, s, p);
    return HIRA_OK;
}

int launch_search_mfma(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    switch (p.dim) {
        case 64: return launch_gs<2>(plan, p, grid, s);
        case 128: return launch_gs<4>(plan, p, grid, s);
        case 256: return launch_gs<8>(plan, p, grid, s);
        default: return fail(HIRA_EINVAL, "MFMA kernel: dim %d", p.dim);
    }
}

}  // namespace hira
