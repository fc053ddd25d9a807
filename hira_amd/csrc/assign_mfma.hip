// Nearest-centroid assignment of the index build on the matrix cores (bf16 rows).
//
// Replaces the distance step of the reference's k-means (faiss.Kmeans.train / index.search,
// indexer/cpu.py:239-250) and of its capacity packing (indexer/cuda.py:247-334):
//   argmin_k ||x_i - c_k||^2 = argmin_k (||c_k||^2 - 2 x_i.c_k),
// with X.C^T on v_mfma_f32_16x16x32_bf16 and the argmin fused into the epilogue, so the
// n x K distance matrix is never written.  Items are bf16 (exact operands).  Centroids are
// fp32 means: each is split into two bf16 numbers, c = hi + lo (16 bits of mantissa), and
// both halves are multiplied, so the distances are as good as fp32 ones for choosing the
// nearest centroid.
//
// k_cent_prep   centroids (T, K, D) fp32 -> tiles of 16 centroids, hi and lo halves, in the
//               operand layout (chunk (s, kb, i) of 16 bytes at s*64 + kb*16 + i), plus
//               ||hi + lo||^2; a centroid that is full (fill[k] >= bf) or past K gets +inf.
//               (hira_nearest; the build's kernels write the tile of a centroid where they make
//               the centroid, assign.h.)
// k_assign_mfma a workgroup of 4 waves owns 256 items (64 a wave: 4 operand tiles kept in
//               registers) and walks all centroid tiles; four tiles at a time are staged once
//               per workgroup in LDS (double buffered, one barrier a stage).  Lane (n, kb) of a wave sees
//               the products of its centroid column n with rows 4*kb + j, keeps the best
//               (value, index) per row, and the 16 columns are merged at the end
//               (lowest index on ties).  For the build it also counts the items of every
//               centroid and, in a tree's last workgroup, turns the counts into offsets
//               (AssignCounting); over a short list of items it spreads them 64 a workgroup; and
//               it can walk the centroids with room only, put side by side by k_open_scan /
//               k_open_gather (AssignOpen).
#include "assign.h"

namespace hira {

typedef __attribute__((ext_vector_type(8))) __bf16 abf16x8_t;
typedef __attribute__((ext_vector_type(4))) float af32x4_t;

constexpr int kAssignRI = 4;       // operand tiles of 16 items per wave
constexpr int kAssignThreads = 256;
constexpr int kAssignStage = 4;    // centroid tiles staged together: the time they keep the
                                   // matrix cores busy covers the latency of fetching the next
                                   // four (two for D = 256, whose tiles are twice as large)
constexpr int assign_stage(int KS) { return KS <= 4 ? kAssignStage : kAssignStage / 2; }

template <int KS>
__global__ __launch_bounds__(64) void k_cent_prep(const float* cent, int K, const int32_t* fill,
                                                  int bf, uint4* tiles, float* cn2, int Kt) {
    // (Kt counts whole stages of kAssignStage tiles: the tiles past K are zeros with norm +inf)
    constexpr int D = 32 * KS;
    const int lane = threadIdx.x & 63, i = lane & 15, kb = lane >> 4;
    const int tile = blockIdx.x, t = blockIdx.y;
    const int k = tile * 16 + i;
    uint4* out = tiles + ((size_t)t * Kt + tile) * (size_t)(2 * KS * 64);
    float ss = 0.0f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        float c[8], hi[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            c[e] = k < K ? cent[((size_t)t * K + k) * D + s * 32 + kb * 8 + e] : 0.0f;
            hi[e] = bf16_bits_to_f32(f32_to_bf16_bits(c[e]));
            lo[e] = bf16_bits_to_f32(f32_to_bf16_bits(c[e] - hi[e]));
            const float v = hi[e] + lo[e];
            ss += v * v;
        }
        out[s * 64 + kb * 16 + i] = make_uint4(pack_bf16(hi[0], hi[1]), pack_bf16(hi[2], hi[3]),
                                               pack_bf16(hi[4], hi[5]), pack_bf16(hi[6], hi[7]));
        out[KS * 64 + s * 64 + kb * 16 + i] =
            make_uint4(pack_bf16(lo[0], lo[1]), pack_bf16(lo[2], lo[3]), pack_bf16(lo[4], lo[5]),
                       pack_bf16(lo[6], lo[7]));
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (kb == 0) {
        const bool usable = k < K && !(fill != nullptr && fill[(size_t)t * K + k] >= bf);
        cn2[((size_t)t * Kt + tile) * 16 + i] = usable ? ss : INFINITY;
    }
}

// The items of one workgroup: RI operand tiles of 16 items a wave.
template <int KS, int RI>
__device__ __forceinline__ void assign_items(
    const void* x, int n_c, size_t x_tree_stride, const uint4* tiles, const float* cn2, int Kt,
    const int32_t* list, int n_items, size_t list_stride, int32_t* assign, float* dist, int K,
    const AssignCounting& ac, const AssignOpen& open) {
    constexpr int D = 32 * KS;
    constexpr int TILE_CHUNKS = 2 * KS * 64;                 // hi and lo halves of 16 centroids
    constexpr int TPS = assign_stage(KS);
    constexpr int STAGE_CHUNKS = TPS * TILE_CHUNKS;
    constexpr int CPT = STAGE_CHUNKS / kAssignThreads;       // chunks a thread stages per stage
    static_assert(STAGE_CHUNKS % kAssignThreads == 0, "stage does not split over the workgroup");
    extern __shared__ uint4 s_dyn[];                         // two stages of tiles, then their norms
    uint4* s_c0 = s_dyn;
    uint4* s_c1 = s_dyn + STAGE_CHUNKS;
    float* s_n2 = reinterpret_cast<float*>(s_dyn + 2 * STAGE_CHUNKS);  // (2, TPS * 16)

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, kb = lane >> 4;  // operand row / centroid column, column block
    const int t = blockIdx.y;
    const int first = (blockIdx.x * (kAssignThreads / 64) + wave) * (RI * 16);

    // ---- my items: operand tiles in registers, ||x||^2 of row lane % 16 ------------------
    int item[RI];
    uint4 a[RI][KS];
    float x2[RI];
#pragma unroll
    for (int ri = 0; ri < RI; ++ri) {
        const int pos = first + ri * 16 + n;
        item[ri] = -1;
        if (pos < n_items) item[ri] = list ? list[(size_t)t * list_stride + pos] : pos;
        float ss = 0.0f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            a[ri][s] = make_uint4(0, 0, 0, 0);
            if (item[ri] >= 0)
                a[ri][s] = *reinterpret_cast<const uint4*>(
                    reinterpret_cast<const uint16_t*>(x) +
                    ((size_t)t * x_tree_stride + item[ri]) * D + s * 32 + kb * 8);
            float f[8];
            unpack<bf16_t>(a[ri][s], f);
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
        }
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        x2[ri] = ss;
    }
    float best[RI][4];
    int arg[RI][4];
#pragma unroll
    for (int ri = 0; ri < RI; ++ri)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            best[ri][j] = INFINITY;
            arg[ri][j] = -1;
        }

    // ---- all centroid tiles, staged through LDS TPS at a time (the last stage may hold fewer;
    // the arrays are padded to whole stages, their norms with +inf) ---------------------------
    const int Ks_all = (Kt + TPS - 1) / TPS;  // stages a tree's arrays hold
    // (centroids with room side by side: only the stages that hold any)
    const int Ks = open.count ? min(((open.count[t] + 15) / 16 + TPS - 1) / TPS, Ks_all) : Ks_all;
    const uint4* tt = tiles + (size_t)t * Ks_all * STAGE_CHUNKS;
    const float* n2t = cn2 + (size_t)t * Ks_all * (TPS * 16);
    uint4 stage[CPT];
    float stage_n2 = 0.0f;
#pragma unroll
    for (int c = 0; c < CPT; ++c) s_c0[threadIdx.x + c * kAssignThreads] = tt[threadIdx.x + c * kAssignThreads];
    if (threadIdx.x < TPS * 16) s_n2[threadIdx.x] = n2t[threadIdx.x];
    __syncthreads();
    for (int st = 0; st < Ks; ++st) {
        const uint4* cbuf = (st & 1) ? s_c1 : s_c0;
        uint4* nbuf = (st & 1) ? s_c0 : s_c1;
        const float* n2buf = s_n2 + (st & 1) * (TPS * 16);
        // the next stage is on its way while this one is used (after the last stage: the last
        // one again, unused; straight-line code keeps `stage` in registers)
        const int nst = min(st + 1, Ks - 1);  // (Ks >= 1 inside the loop)
#pragma unroll
        for (int c = 0; c < CPT; ++c)
            stage[c] = tt[(size_t)nst * STAGE_CHUNKS + threadIdx.x + c * kAssignThreads];
        stage_n2 = n2t[nst * (TPS * 16) + (threadIdx.x & (TPS * 16 - 1))];
#pragma unroll
        for (int ti = 0; ti < TPS; ++ti) {
            abf16x8_t bh[KS], bl[KS];
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                bh[s] = __builtin_bit_cast(abf16x8_t, cbuf[ti * TILE_CHUNKS + s * 64 + lane]);
                bl[s] = __builtin_bit_cast(abf16x8_t, cbuf[ti * TILE_CHUNKS + KS * 64 + s * 64 + lane]);
            }
            const float n2 = n2buf[ti * 16 + n];
            const int kcol = (st * TPS + ti) * 16 + n;
            // four independent accumulator chains: a product never waits for the one before it
            af32x4_t acc[RI];
#pragma unroll
            for (int ri = 0; ri < RI; ++ri) acc[ri] = af32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s) {
#pragma unroll
                for (int ri = 0; ri < RI; ++ri)
                    acc[ri] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(abf16x8_t, a[ri][s]), bh[s], acc[ri], 0, 0, 0);
#pragma unroll
                for (int ri = 0; ri < RI; ++ri)
                    acc[ri] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(abf16x8_t, a[ri][s]), bl[s], acc[ri], 0, 0, 0);
            }
#pragma unroll
            for (int ri = 0; ri < RI; ++ri)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float v = n2 - 2.0f * acc[ri][j];
                    if (v < best[ri][j]) {  // tiles come in increasing order: ties keep the lower k
                        best[ri][j] = v;
                        arg[ri][j] = kcol;
                    }
                }
        }
#pragma unroll
        for (int c = 0; c < CPT; ++c) nbuf[threadIdx.x + c * kAssignThreads] = stage[c];
        if (threadIdx.x < TPS * 16) s_n2[((st + 1) & 1) * (TPS * 16) + threadIdx.x] = stage_n2;
        __syncthreads();
    }

    // ---- merge the 16 centroid columns of a row group; the wave's 64 results pass through LDS
    // (free behind the loop's last barrier) so that every lane ends up with one item: one store
    // instruction, and one counting instruction, for the whole wave -----------------------------
    static_assert(RI == 1 || RI == 4, "a result per lane, or per lane of the first 16");
    int* s_g = reinterpret_cast<int*>(s_dyn) + wave * 128;
    float* s_b = reinterpret_cast<float*>(s_g + 64);
#pragma unroll
    for (int ri = 0; ri < RI; ++ri)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float b = best[ri][j];
            int g = arg[ri][j];
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) {
                const float ob = __shfl_xor(b, off, 64);
                const int og = __shfl_xor(g, off, 64);
                if (og >= 0 && (g < 0 || ob < b || (ob == b && og < g))) {
                    b = ob;
                    g = og;
                }
            }
            if (n == 0) {  // row 4*kb + j of operand tile ri
                s_g[ri * 16 + 4 * kb + j] = g;
                s_b[ri * 16 + 4 * kb + j] = b;
            }
        }
    __builtin_amdgcn_wave_barrier();
    {
        // lane (kb, n) takes row n of operand tile kb: its item and ||x||^2 are its own
        int g = s_g[lane];  // (meaningless in the lanes that hold no result: kb >= RI)
        const float b = s_b[lane];
        int it = item[0];
        float xx = x2[0];
#pragma unroll
        for (int ri = 1; ri < RI; ++ri)
            if (kb == ri) {
                it = item[ri];
                xx = x2[ri];
            }
        if (kb < RI && it >= 0) {
            if (open.ids != nullptr && g >= 0) g = open.ids[(size_t)t * K + g];  // column -> centroid
            assign[(size_t)t * n_c + it] = g;
            dist[(size_t)t * n_c + it] = fmaxf(b + xx, 0.0f);
            if (ac.counts != nullptr && g >= 0)
                ac.pos[(size_t)t * n_c + it] = atomicAdd(&ac.counts[(size_t)t * K + g], 1);
        }
    }
}

// Few items (the later rounds of the packing walk ever shorter lists) are spread over four times
// as many workgroups, a single operand tile a wave: a workgroup's time is what its walk over all
// centroid tiles takes, and that walk is four times shorter.  The lists' lengths are known on
// the device only, so a launch over a list has workgroups for the narrow shape, and each tree
// picks its shape by the length of its list.
constexpr int kAssignNarrowItems = 256 * 256;  // (all trees together; measured: beyond this many the
                                               // wide shape is faster, its tiles read from LDS once for 64 items)

template <int KS, bool LISTED>
__global__ __launch_bounds__(kAssignThreads, 2) void k_assign_mfma(
    const void* x, int n_c, size_t x_tree_stride, const uint4* tiles, const float* cn2, int Kt,
    const int32_t* list, const int32_t* list_count, size_t list_stride, int32_t* assign,
    float* dist, int K, AssignCounting ac, AssignOpen open) {
    const int t = blockIdx.y;
    const int n_items = LISTED ? list_count[t] : n_c;
    const bool narrow = LISTED && (long long)n_items * gridDim.y <= kAssignNarrowItems;
    const int per_block = (kAssignThreads / 64) * 16 * (narrow ? 1 : kAssignRI);
    // (a launch that counts: the tree's first workgroup draws a ticket also when there is no item)
    const int nblocks = max((n_items + per_block - 1) / per_block, 1);
    if ((int)blockIdx.x >= nblocks) return;  // uniform
    if (ac.zero != nullptr && blockIdx.x == 0 && threadIdx.x == 0) ac.zero[t] = 0;
    if ((int)blockIdx.x * per_block < n_items) {
        if (LISTED && narrow)
            assign_items<KS, 1>(x, n_c, x_tree_stride, tiles, cn2, Kt, list, n_items, list_stride,
                                assign, dist, K, ac, open);
        else
            assign_items<KS, kAssignRI>(x, n_c, x_tree_stride, tiles, cn2, Kt, list, n_items,
                                        list_stride, assign, dist, K, ac, open);
    }
    if (ac.counts != nullptr) finish_counts(ac, t, K, nblocks);
}

// ---- the centroids with room, side by side ---------------------------------------------------
// one workgroup per tree: which centroids are not full, in order
__global__ __launch_bounds__(256) void k_open_scan(const int32_t* fill, int K, int bf, int32_t* ids,
                                                   int32_t* count) {
    const int t = blockIdx.x;
    const int32_t* ft = fill + (size_t)t * K;
    int32_t* it = ids + (size_t)t * K;
    const int total = block_exclusive_scan(
        K, [&](int k) { return ft[k] < bf ? 1 : 0; },
        [&](int k, int v) {
            if (ft[k] < bf) it[v] = k;
        });
    if (threadIdx.x == 0) count[t] = total;
}

// one wave per tile of the side-by-side arrays: column i of tile c is centroid ids[16 c + i]; the
// columns behind the last one, up to the end of the stage, are zeros with norm +inf
template <int KS>
__global__ __launch_bounds__(64) void k_open_gather(const uint4* tiles, const float* cn2,
                                                    const int32_t* ids, const int32_t* count, int K,
                                                    int Kt, uint4* otiles, float* ocn2) {
    constexpr int TILE_CHUNKS = 2 * KS * 64;
    constexpr int TPS = assign_stage(KS);
    const int tile = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    const int no = count[t];
    const int need = min((((no + 15) / 16 + TPS - 1) / TPS) * TPS, Kt);  // tiles the assignment will walk
    if (tile >= need) return;
    const uint4* src = tiles + (size_t)t * Kt * TILE_CHUNKS;
    uint4* dst = otiles + ((size_t)t * Kt + tile) * TILE_CHUNKS;
    const int i = lane & 15;
    const int col = tile * 16 + i;
    const int k = col < no ? ids[(size_t)t * K + col] : -1;
#pragma unroll
    for (int c0 = 0; c0 < TILE_CHUNKS; c0 += 64) {
        const int ci = c0 + lane;  // (ci % 16 == i: a lane always moves chunks of its own column)
        uint4 v = make_uint4(0, 0, 0, 0);
        if (k >= 0) v = src[(size_t)(k >> 4) * TILE_CHUNKS + (ci - i) + (k & 15)];
        dst[ci] = v;
    }
    if (lane < 16) ocn2[((size_t)t * Kt + tile) * 16 + i] = k >= 0 ? cn2[(size_t)t * Kt * 16 + k] : INFINITY;
}

int launch_open_centroids(int dim, const void* tiles, const float* cn2, const int32_t* fill, int bf,
                          int K, int num_trees, int32_t* open_ids, int32_t* open_count,
                          void* open_tiles, float* open_cn2, hipStream_t s) {
    const int Kt = assign_tiles(K);
    hipLaunchKernelGGL(k_open_scan, dim3(num_trees), dim3(256), 0, s, fill, K, bf, open_ids, open_count);
    const dim3 grid(Kt, num_trees);
    const uint4* tl = reinterpret_cast<const uint4*>(tiles);
    uint4* ot = reinterpret_cast<uint4*>(open_tiles);
    switch (dim) {
        case 64: hipLaunchKernelGGL((k_open_gather<2>), grid, dim3(64), 0, s, tl, cn2, open_ids, open_count, K, Kt, ot, open_cn2); break;
        case 128: hipLaunchKernelGGL((k_open_gather<4>), grid, dim3(64), 0, s, tl, cn2, open_ids, open_count, K, Kt, ot, open_cn2); break;
        case 256: hipLaunchKernelGGL((k_open_gather<8>), grid, dim3(64), 0, s, tl, cn2, open_ids, open_count, K, Kt, ot, open_cn2); break;
        default: return fail(HIRA_EINVAL, "MFMA assignment: dim %d", dim);
    }
    return HIRA_OK;
}

// centroid tiles per tree, in whole stages
int assign_tiles(int K) {
    const int kt = (K + 15) / 16;
    return (kt + kAssignStage - 1) / kAssignStage * kAssignStage;
}

// hi/lo tiles and norms of the centroids of every tree
int launch_cent_prep(int dim, const float* cent, int K, int num_trees, const int32_t* fill, int bf,
                     void* tiles, float* cn2, hipStream_t s) {
    const int Kt = assign_tiles(K);
    const dim3 grid(Kt, num_trees);
    uint4* tl = reinterpret_cast<uint4*>(tiles);
    switch (dim) {
        case 64: hipLaunchKernelGGL((k_cent_prep<2>), grid, dim3(64), 0, s, cent, K, fill, bf, tl, cn2, Kt); break;
        case 128: hipLaunchKernelGGL((k_cent_prep<4>), grid, dim3(64), 0, s, cent, K, fill, bf, tl, cn2, Kt); break;
        case 256: hipLaunchKernelGGL((k_cent_prep<8>), grid, dim3(64), 0, s, cent, K, fill, bf, tl, cn2, Kt); break;
        default: return fail(HIRA_EINVAL, "MFMA assignment: dim %d", dim);
    }
    return HIRA_OK;
}

// nearest usable centroid of every item (or of the items list[0 .. *list_count) of each tree)
int launch_assign_mfma(int dim, const void* x, int n_c, size_t x_tree_stride, const void* tiles,
                       const float* cn2, int K, int num_trees, const int32_t* list,
                       const int32_t* list_count, size_t list_stride, int32_t* assign, float* dist,
                       const AssignCounting& counting, const AssignOpen& open, hipStream_t s) {
    const int Kt = assign_tiles(K);
    // (a launch over a list: workgroups for the narrow shape, see kAssignNarrowItems)
    const int per_block = (kAssignThreads / 64) * (list != nullptr ? 1 : kAssignRI) * 16;
    const int tps = assign_stage(dim / 32);
    const size_t smem = 2 * (size_t)tps * (2 * (dim / 32) * 64) * sizeof(uint4) + 2 * (size_t)tps * 16 * sizeof(float);
    const dim3 grid((n_c + per_block - 1) / per_block, num_trees);
    const uint4* tl = reinterpret_cast<const uint4*>(tiles);
    constexpr int kMaxDevices = 64;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(HIRA_ELAUNCH, "MFMA assignment: no current device");
    switch (dim) {
#define HIRA_ASSIGN_MFMA_L(KS, LISTED)                                                              \
    {                                                                                               \
        /* more than 64 KiB of dynamic LDS has to be asked for: once per kernel and device */       \
        static int asked[kMaxDevices];                                                              \
        if (__atomic_load_n(&asked[dev], __ATOMIC_RELAXED) == 0) {                                  \
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_assign_mfma<KS, LISTED>),      \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
                return fail(HIRA_ELAUNCH, "MFMA assignment: %zu bytes of LDS refused", smem);          \
            __atomic_store_n(&asked[dev], 1, __ATOMIC_RELAXED);                                     \
        }                                                                                           \
        hipLaunchKernelGGL((k_assign_mfma<KS, LISTED>), grid, dim3(kAssignThreads), smem, s, x, n_c, \
                           x_tree_stride, tl, cn2, Kt, list, list_count, list_stride, assign, dist, \
                           K, counting, open);                                                      \
    }
#define HIRA_ASSIGN_MFMA(KS)                                                                        \
    if (list != nullptr) HIRA_ASSIGN_MFMA_L(KS, true) else HIRA_ASSIGN_MFMA_L(KS, false)            \
    break;
        case 64: HIRA_ASSIGN_MFMA(2)
        case 128: HIRA_ASSIGN_MFMA(4)
        case 256: HIRA_ASSIGN_MFMA(8)
#undef HIRA_ASSIGN_MFMA
#undef HIRA_ASSIGN_MFMA_L
        default: return fail(HIRA_EINVAL, "MFMA assignment: dim %d", dim);
    }
    return HIRA_OK;
}

}  // namespace hira
