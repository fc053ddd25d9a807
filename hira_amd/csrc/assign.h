// What the nearest-centroid kernels (assign_mfma.hip, and the vector-ALU one of build.hip) share
// with the index build around them: the counting of the items a centroid takes, done by the
// assignment itself, and the operand tiles of the centroids for the matrix cores.
#pragma once

#include "search.h"

namespace hira {

// Counting fused into an assignment launch (all NULL: the launch only assigns).
//   counts  (T, K)    zero when the launch starts; counts[a] += 1 for every item assigned to a
//   pos     (T, n_c)  the value the item's increment returned: its place inside the bucket
//   done    (T)       zero when the launch starts: tickets of the tree's workgroups
//   offsets (T, K+1)  written by the workgroup that draws a tree's last ticket: the exclusive
//                     prefix sums of counts (offsets[K] = number of items assigned)
//   zero    (T)       a counter the launch clears (the list of the round after it), or NULL
struct AssignCounting {
    int32_t* counts;
    int32_t* pos;
    int32_t* done;
    int32_t* offsets;
    int32_t* zero;
};

// The centroids that still take items, put side by side (packing rounds from the second on: most
// blocks are full by then, and a round multiplies every unplaced item with every centroid it is
// given).  ids (T, K): the centroids with room, in increasing order; count (T): how many; the
// assignment then walks tiles and norms holding only those (same arrays' shapes as the full ones)
// and translates the column it finds back through ids.  Both NULL: all centroids, as they lie.
struct AssignOpen {
    const int32_t* count;
    const int32_t* ids;
};

// Exclusive prefix sums of n numbers by a workgroup of 256 threads, 1024 numbers a step; every
// thread returns the total.
template <typename Load, typename Store>
__device__ __forceinline__ int block_exclusive_scan(int n, Load load, Store store) {
    __shared__ int32_t s_w[4];
    __shared__ int32_t s_carry;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    for (int base = 0; base < n; base += 1024) {
        const int k0 = base + (int)threadIdx.x * 4;
        int v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = k0 + j < n ? load(k0 + j) : 0;
        const int mine = v[0] + v[1] + v[2] + v[3];
        int inc = mine;  // inclusive scan in the wave
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        if (lane == 63) s_w[wave] = inc;
        __syncthreads();
        int before = s_carry;
        for (int w = 0; w < wave; ++w) before += s_w[w];
        int run = before + inc - mine;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (k0 + j < n) store(k0 + j, run);
            run += v[j];
        }
        __syncthreads();
        if (threadIdx.x == 255) s_carry = before + inc;
        __syncthreads();
    }
    return s_carry;
}

// a value another workgroup wrote or counted up during this launch, read where it is coherent
__device__ __forceinline__ int32_t load_agent(const int32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// End of an assignment workgroup (256 threads, all of them, also of a workgroup without items):
// a ticket per workgroup; the tree's last one turns the counts into offsets.
__device__ __forceinline__ void finish_counts(const AssignCounting& ac, int t, int K, int nblocks) {
    __shared__ int32_t s_last;
    // (no fence at device scope: it would write the whole L2 back, once per workgroup.  The
    // increments are device-scope atomics; a thread that has waited for what they return knows
    // them done, and the last workgroup reads the counts where they were made.)
    hand_off_release();
    __syncthreads();  // the workgroup's increments have all returned
    if (threadIdx.x == 0) s_last = atomicAdd(&ac.done[t], 1) == nblocks - 1 ? 1 : 0;
    __syncthreads();
    if (!s_last) return;
    const int32_t* cnt = ac.counts + (size_t)t * K;
    int32_t* off = ac.offsets + (size_t)t * (K + 1);
    const int total = block_exclusive_scan(
        K, [&](int k) { return load_agent(cnt + k); }, [&](int k, int v) { off[k] = v; });
    if (threadIdx.x == 0) off[K] = total;
}

// ---- centroids as operands of v_mfma_f32_16x16x32_bf16 --------------------------------------
// A tile holds 16 centroids of D = 32 * KS columns, each split into two bf16 numbers, c = hi + lo:
// 2 * KS * 64 chunks of 16 bytes, chunk (half, s, kb, i) at half*KS*64 + s*64 + kb*16 + i = columns
// [s*32 + kb*8, +8) of centroid i of the tile.  cn2 (T, Kt*16): ||hi + lo||^2, +inf for a centroid
// that takes no items.  A tree has Kt tiles (whole stages of the assignment kernel).
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

// Centroid k of tree t, D fp32 numbers at c (LDS or memory), into its tile; called by the 64
// lanes of one wave.
__device__ __forceinline__ void emit_centroid(const float* c, int D, int Kt, int t, int k,
                                              bool usable, uint4* tiles, float* cn2) {
    const int j = threadIdx.x & 63;
    const int KS = D >> 5;
    float ss = 0.0f;
    if (j < D / 8) {
        const int s = j >> 2, kb = j & 3, i = k & 15;
        uint4* out = tiles + ((size_t)t * Kt + (k >> 4)) * (size_t)(2 * KS * 64);
        float hi[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float v = c[j * 8 + e];
            hi[e] = bf16_bits_to_f32(f32_to_bf16_bits(v));
            lo[e] = bf16_bits_to_f32(f32_to_bf16_bits(v - hi[e]));
            const float w = hi[e] + lo[e];
            ss += w * w;
        }
        out[s * 64 + kb * 16 + i] = make_uint4(pack_bf16(hi[0], hi[1]), pack_bf16(hi[2], hi[3]),
                                               pack_bf16(hi[4], hi[5]), pack_bf16(hi[6], hi[7]));
        out[KS * 64 + s * 64 + kb * 16 + i] =
            make_uint4(pack_bf16(lo[0], lo[1]), pack_bf16(lo[2], lo[3]), pack_bf16(lo[4], lo[5]),
                       pack_bf16(lo[6], lo[7]));
    }
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) ss += __shfl_xor(ss, off, 64);
    if (j == 0) cn2[(size_t)t * Kt * 16 + k] = usable ? ss : INFINITY;
}

// assign_mfma.hip
int assign_tiles(int K);
int launch_cent_prep(int dim, const float* cent, int K, int num_trees, const int32_t* fill, int bf,
                     void* tiles, float* cn2, hipStream_t s);
int launch_assign_mfma(int dim, const void* x, int n_c, size_t x_tree_stride, const void* tiles,
                       const float* cn2, int K, int num_trees, const int32_t* list,
                       const int32_t* list_count, size_t list_stride, int32_t* assign, float* dist,
                       const AssignCounting& counting, const AssignOpen& open, hipStream_t s);
int launch_open_centroids(int dim, const void* tiles, const float* cn2, const int32_t* fill, int bf,
                          int K, int num_trees, int32_t* open_ids, int32_t* open_count,
                          void* open_tiles, float* open_cn2, hipStream_t s);

}  // namespace hira
