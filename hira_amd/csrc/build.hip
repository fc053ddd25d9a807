// Index build: bottom-up k-means-style ball tree in the fixed-fan-out layout.
//
// For each level l = 1 .. L-1 the n_c items of the level below (keys for l = 1, the
// centres of level l-1 above that) are clustered into K = ceil(n_c / bf) groups of at most
// bf items:
//   1. K initial centroids = evenly strided, seeded sample of the items;
//   2. `niter` Lloyd rounds: nearest-centroid assignment, then centroid = mean of members
//      (members are bucketed and summed in a fixed order, so the result is reproducible);
//   3. capacity packing: every item proposes to its nearest centroid that still has room,
//      each centroid takes the closest proposers first (the rule of the reference's GPU
//      build, indexer/cuda.py:247-307), the rest try again against the centroids that are
//      not full yet; what is still unplaced after `pack_rounds` fills free slots in order
//      (the reference drops such items into random free slots, indexer/cuda.py:309-334);
//   4. the centre of a block = mean of the items that ended up in it, rounded to the
//      storage dtype.
// Then the levels are laid out top-down (children of slot p at [p*bf, (p+1)*bf)), keys and
// values are gathered once into slot order, and radii are taken bottom-up from the final
// layout: r_p = max over children (||c_child - c_p|| + r_child), the bound of
// indexer/cpu.py:286-309 / indexer/cuda.py:114-198, against the ROUNDED centres and
// nudged up by a few ulp so that rounding never makes a ball too small.
#include "assign.h"
#include "rows.h"

namespace hira {

// ------------------------------------------------------------------------------------
// small helpers
// ------------------------------------------------------------------------------------
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void k_fill_i32(int32_t* p, size_t n, int32_t v) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ------------------------------------------------------------------------------------
// 0. what a level starts from, in one launch: nothing placed, empty blocks, zero counters; the
//    centroid columns that pad the last stage of operand tiles are zeros that take no items.
//    n_live != NULL: tree t holds n_live[t] <= n_c items, the first ones of its rows; the items
//    it does not hold count as placed from the start (no phase ever touches them), and it uses
//    its first ceil(n_t / bf) centroids only: the others count as full.
// ------------------------------------------------------------------------------------
__global__ void k_level_init(int n_c, int K, int bf, int D, int Kt, const int32_t* n_live,
                             int32_t* placed, int32_t* fill, int32_t* slots, int32_t* counts,
                             int32_t* done, int32_t* list_count /* (2, T) */, uint4* tiles,
                             float* cn2) {
    const int t = blockIdx.y, T = gridDim.y;
    const int n_t = n_live ? min(max(n_live[t], 0), n_c) : n_c;
    const int K_t = n_live ? max((n_t + bf - 1) / bf, 1) : K;
    const int stride = gridDim.x * blockDim.x;
    const int i0 = blockIdx.x * blockDim.x + threadIdx.x;
    if (i0 == 0) {
        done[t] = 0;
        list_count[t] = 0;
        list_count[T + t] = 0;
    }
    for (int i = i0; i < n_c; i += stride) placed[(size_t)t * n_c + i] = i >= n_t ? 1 : 0;
    for (int i = i0; i < K; i += stride) {
        fill[(size_t)t * K + i] = i >= K_t ? bf : 0;
        counts[(size_t)t * K + i] = 0;
    }
    for (size_t i = i0; i < (size_t)K * bf; i += stride) slots[(size_t)t * K * bf + i] = -1;
    if (tiles != nullptr) {
        const int pad = Kt * 16 - K, cpc = D / 4;  // chunks of a column: hi and lo halves
        const int KS = D / 32;
        for (int i = i0; i < pad * cpc; i += stride) {
            const int k = K + i / cpc, c = i % cpc;
            const int half = c / (D / 8), j = c % (D / 8);
            tiles[((size_t)t * Kt + (k >> 4)) * (size_t)(2 * KS * 64) + half * KS * 64 + (j >> 2) * 64 +
                  (j & 3) * 16 + (k & 15)] = make_uint4(0, 0, 0, 0);
        }
        for (int i = i0; i < pad; i += stride) cn2[(size_t)t * Kt * 16 + K + i] = INFINITY;
    }
}

// ------------------------------------------------------------------------------------
// 1. initial centroids: item floor((k + u_k) * n_c / K), u_k in [0,1) from the seed
// ------------------------------------------------------------------------------------
//    (n_live != NULL: tree t holds n_live[t] <= n_c items, the first ones of its rows)
//    tiles != NULL: the centroid also goes into its operand tile (fill: the centroids that
//    count as full from the start take no items)
template <typename T>
__global__ __launch_bounds__(64) void k_init_centroids(const void* x, int n_c, size_t x_tree_stride,
                                                       int K, int D, uint64_t seed, float* cent,
                                                       const int32_t* n_live, int bf, int Kt,
                                                       const int32_t* fill, uint4* tiles,
                                                       float* cn2) {
    __shared__ float s_c[256];
    const int k = blockIdx.x, t = blockIdx.y;
    const uint64_t h = mix64(seed ^ mix64((uint64_t)t * 0x100000001b3ull + (uint64_t)k));
    const double u = (double)(h >> 11) * (1.0 / 9007199254740992.0);
    const int n_t = n_live ? max(min(n_live[t], n_c), 1) : n_c;
    // (a tree with fewer items uses the first K_t = ceil(n_t / bf) centroids only)
    const int K_t = n_live ? min(max((n_t + bf - 1) / bf, 1), K) : K;
    long long idx = (long long)(((double)min(k, K_t - 1) + u) * (double)n_t / (double)K_t);
    if (idx >= n_t) idx = n_t - 1;
    const size_t src = ((size_t)t * x_tree_stride + (size_t)idx) * D;
    float* dst = cent + ((size_t)t * K + k) * D;
    for (int j = threadIdx.x; j < D; j += blockDim.x) {
        const float v = load_elem<T>(x, src + j);
        dst[j] = v;
        if (tiles != nullptr) s_c[j] = v;  // (the matrix-core path has D <= 256)
    }
    if (tiles != nullptr) {
        __syncthreads();
        emit_centroid(s_c, D, Kt, t, k, fill[(size_t)t * K + k] < bf, tiles, cn2);
    }
}

// ------------------------------------------------------------------------------------
// 2. nearest centroid (vector-ALU kernel): argmin_k ||x_i - c_k||^2, lowest k on ties.
//    LPR lanes hold one item row; each lane group keeps PPG items in registers and walks
//    all centroids.  fill != NULL: centroids with fill[k] >= bf are skipped.
//    list != NULL: only the items list[0 .. *list_count) are processed.
//    ac: the items a centroid takes are counted as they are assigned (assign.h).
// ------------------------------------------------------------------------------------
constexpr int kPPG = 4;

template <typename T, int LPR>
__global__ __launch_bounds__(256) void k_assign_simple(
    const void* x, int n_c, size_t x_tree_stride, const float* cent, int K, int D,
    const int32_t* fill, int bf, const int32_t* list, const int32_t* list_count, size_t list_stride,
    int32_t* assign, float* dist, AssignCounting ac) {
    constexpr int EPL = Elem<T>::kPerChunk;
    constexpr int RPW = kWave / LPR;
    const int lane = lane_id();
    const int rg = lane / LPR, ch = lane % LPR;
    const int t = blockIdx.y;
    const int n_items = list ? list_count[t] : n_c;
    const int wave_global = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int first = wave_global * (RPW * kPPG);
    if (ac.counts == nullptr && first >= n_items) return;
    if (ac.zero != nullptr && blockIdx.x == 0 && threadIdx.x == 0) ac.zero[t] = 0;
    const bool chunk_ok = ch * EPL < D;

    if (first < n_items) {  // (wave-uniform; no barrier inside)
        int item[kPPG];
        float xf[kPPG][EPL];
        float best[kPPG];
        int arg[kPPG];
#pragma unroll
        for (int p = 0; p < kPPG; ++p) {
            const int pos = first + p * RPW + rg;
            item[p] = -1;
            if (pos < n_items) item[p] = list ? list[(size_t)t * list_stride + pos] : pos;
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (item[p] >= 0 && chunk_ok)
                raw = load_chunk<T>(x, ((size_t)t * x_tree_stride + item[p]) * D, ch);
            unpack<T>(raw, xf[p]);
            best[p] = INFINITY;
            arg[p] = -1;
        }
        const float* ct = cent + (size_t)t * K * D;
        const int32_t* ft = fill ? fill + (size_t)t * K : nullptr;
        for (int k = 0; k < K; ++k) {
            if (ft && ft[k] >= bf) continue;  // wave-uniform
            float cf[4] = {0.f, 0.f, 0.f, 0.f};
            float cf2[4] = {0.f, 0.f, 0.f, 0.f};
            if (chunk_ok) {
                const float4 a = *reinterpret_cast<const float4*>(ct + (size_t)k * D + ch * EPL);
                cf[0] = a.x, cf[1] = a.y, cf[2] = a.z, cf[3] = a.w;
                if (EPL == 8) {
                    const float4 b =
                        *reinterpret_cast<const float4*>(ct + (size_t)k * D + ch * EPL + 4);
                    cf2[0] = b.x, cf2[1] = b.y, cf2[2] = b.z, cf2[3] = b.w;
                }
            }
#pragma unroll
            for (int p = 0; p < kPPG; ++p) {
                float ss = 0.0f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float df = xf[p][e] - cf[e];
                    ss += df * df;
                }
                if (EPL == 8) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float df = xf[p][4 + e] - cf2[e];
                        ss += df * df;
                    }
                }
                ss = group_sum<LPR>(ss);
                if (ss < best[p]) {
                    best[p] = ss;
                    arg[p] = k;
                }
            }
        }
        if (ch == 0) {
#pragma unroll
            for (int p = 0; p < kPPG; ++p) {
                if (item[p] >= 0) {
                    assign[(size_t)t * n_c + item[p]] = arg[p];
                    dist[(size_t)t * n_c + item[p]] = best[p];
                    if (ac.counts != nullptr && arg[p] >= 0)
                        ac.pos[(size_t)t * n_c + item[p]] =
                            atomicAdd(&ac.counts[(size_t)t * K + arg[p]], 1);
                }
            }
        }
    }
    if (ac.counts != nullptr) finish_counts(ac, t, K, (int)gridDim.x);
}

// ------------------------------------------------------------------------------------
// 3. the items of a round bucketed by the centroid they were assigned to: item i of bucket a
//    goes to members[offsets[a] + pos[i]] (offsets and pos come out of the assignment launch)
// ------------------------------------------------------------------------------------
__global__ void k_bucket_fill(const int32_t* assign, const int32_t* pos, const int32_t* offsets,
                              int n_c, const int32_t* list, const int32_t* list_count,
                              size_t list_stride, int K, int32_t* members) {
    const int t = blockIdx.y;
    const int n_items = list ? list_count[t] : n_c;
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_items) return;
    const int i = list ? list[(size_t)t * list_stride + p] : p;
    const int a = assign[(size_t)t * n_c + i];
    if (a < 0) return;
    members[(size_t)t * n_c + offsets[(size_t)t * (K + 1) + a] + pos[(size_t)t * n_c + i]] = i;
}

// The order in which a bucket's members arrive depends on the run; everything that follows works
// on them in a fixed order, which a workgroup per bucket establishes in LDS:
//   up to 256 members   every thread ranks its member against all others
//   more                a bitonic sorting network over the next power of two
constexpr int kBucketThreads = 256;

template <typename Key>
__device__ __forceinline__ void bitonic_sort(Key* a, int P) {  // (a barrier ahead of the first step)
    for (int k = 2; k <= P; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            __syncthreads();
            for (int i = threadIdx.x; i < P; i += kBucketThreads) {
                const int x = i ^ j;
                if (x > i) {
                    const Key u = a[i], v = a[x];
                    if ((u > v) == ((i & k) == 0)) {
                        a[i] = v;
                        a[x] = u;
                    }
                }
            }
        }
    __syncthreads();
}

__device__ __forceinline__ int pow2_at_least(int n) {
    int p = 1;
    while (p < n) p <<= 1;
    return p;
}

// (what every workgroup of the per-bucket kernels does for the round after it)
__device__ __forceinline__ void reset_counters(int t, int k, int K, int32_t* counts, int32_t* done) {
    if (threadIdx.x == 0) {
        counts[(size_t)t * K + k] = 0;
        if (k == 0) done[t] = 0;
    }
}

// ------------------------------------------------------------------------------------
// 4. Lloyd round: centroid = mean of the member rows.  One workgroup per centroid: the members
//    in the order of their item ids, row e summed by row group e % R, the R sums added in order:
//    the result does not depend on the order of arrival.  An empty centroid keeps its value.
//    tiles != NULL: the new centroid also goes into its operand tile.
// ------------------------------------------------------------------------------------
constexpr int kMeanSort = 4096;      // members ordered in LDS; more: through a bit map of item ids
constexpr int kMeanMapBits = kMeanSort * 32;

template <typename T>
__global__ __launch_bounds__(kBucketThreads) void k_bucket_mean(
    const void* x, size_t x_tree_stride, int n_c, int K, int D, const int32_t* offsets,
    const int32_t* members, int32_t* ordered /* (T, n_c): buckets too large for LDS */,
    const int32_t* fill, int bf, float* cent, int Kt, uint4* tiles, float* cn2, int32_t* counts,
    int32_t* done) {
    constexpr int EPL = Elem<T>::kPerChunk;
    __shared__ uint32_t s_ord[kMeanSort];            // (as a bit map: kMeanMapBits ids)
    __shared__ float s_part[kBucketThreads * EPL];   // (R, D) partial sums, R * D <= 256 * EPL
    __shared__ int32_t s_small[kBucketThreads];
    const int k = blockIdx.x, t = blockIdx.y, tid = threadIdx.x;
    reset_counters(t, k, K, counts, done);
    const int b0 = offsets[(size_t)t * (K + 1) + k];
    const int m = offsets[(size_t)t * (K + 1) + k + 1] - b0;
    if (m <= 0) return;
    const int32_t* mem = members + (size_t)t * n_c + b0;
    const int32_t* ord_g = nullptr;  // the ordered members: in LDS, or here
    if (m <= kBucketThreads) {
        const int mine = tid < m ? mem[tid] : 0x7fffffff;
        s_small[tid] = mine;
        __syncthreads();
        int rank = 0;
        for (int j = 0; j < m; ++j) rank += s_small[j] < mine;
        if (tid < m) s_ord[rank] = (uint32_t)mine;
        __syncthreads();
    } else if (m <= kMeanSort) {
        const int P = pow2_at_least(m);
        for (int e = tid; e < P; e += kBucketThreads) s_ord[e] = e < m ? (uint32_t)mem[e] : 0xffffffffu;
        bitonic_sort(s_ord, P);
    } else {
        // ids in ranges of kMeanMapBits: a bit per member, then the set bits in order
        int32_t* out = ordered + (size_t)t * n_c + b0;
        int written = 0;
        for (int lo = 0; lo < n_c; lo += kMeanMapBits) {
            __syncthreads();
            for (int w = tid; w < kMeanSort; w += kBucketThreads) s_ord[w] = 0;
            __syncthreads();
            for (int e = tid; e < m; e += kBucketThreads) {
                const int d = mem[e] - lo;
                if (d >= 0 && d < kMeanMapBits) atomicOr(&s_ord[d >> 5], 1u << (d & 31));
            }
            __syncthreads();
            // thread `tid` owns the words [tid * W, (tid + 1) * W)
            constexpr int W = kMeanSort / kBucketThreads;
            const int in_range = block_exclusive_scan(
                kBucketThreads, [&](int i) {
                    int c = 0;
                    for (int w = 0; w < W; ++w) c += __popc(s_ord[i * W + w]);
                    return c;
                },
                [&](int i, int v) { s_small[i] = v; });
            __syncthreads();
            int at = written + s_small[tid];
            for (int w = 0; w < W; ++w) {
                uint32_t bits = s_ord[tid * W + w];
                while (bits) {
                    const int b = __ffs(bits) - 1;
                    bits &= bits - 1;
                    out[at++] = lo + (tid * W + w) * 32 + b;
                }
            }
            written += in_range;
        }
        __threadfence_block();
        __syncthreads();
        ord_g = out;
    }
    // ---- sums: CPR threads a row, R rows at a time -------------------------------------------
    const int CPR = D / EPL, R = kBucketThreads / CPR;
    const int r = tid / CPR, c = tid % CPR;
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;
    if (r < R) {
        for (int e = r; e < m; e += R) {
            const int it = ord_g ? ord_g[e] : (int)s_ord[e];
            float f[EPL];
            unpack<T>(load_chunk<T>(x, ((size_t)t * x_tree_stride + it) * D, c), f);
#pragma unroll
            for (int q = 0; q < EPL; ++q) acc[q] += f[q];
        }
#pragma unroll
        for (int q = 0; q < EPL; ++q) s_part[r * D + c * EPL + q] = acc[q];
    }
    __syncthreads();
    float v = 0.0f;
    for (int j = tid; j < D; j += kBucketThreads) {  // (D <= 512: at most two columns a thread)
        float s = 0.0f;
        const int rows = min(R, m);
        for (int q = 0; q < rows; ++q) s += s_part[q * D + j];
        v = s / (float)m;
        cent[((size_t)t * K + k) * D + j] = v;
    }
    if (tiles != nullptr) {  // (D <= 256: column tid)
        __syncthreads();
        if (tid < D) s_part[tid] = v;
        __syncthreads();
        if (tid < 64)
            emit_centroid(s_part, D, Kt, t, k, !(fill != nullptr && fill[(size_t)t * K + k] >= bf),
                          tiles, cn2);
    }
}

// block centre = mean of the items in the bf slots of the block, stored in fp32 and rounded to the
// storage type.  One wave per block: `lpr` lanes (a power of two) hold a row in 16-byte chunks,
// the 64 / lpr lane groups take every (64 / lpr)-th slot, and their sums are added pairwise in a
// fixed order.  An empty block keeps its value.
template <typename T>
__global__ __launch_bounds__(64) void k_block_mean(const void* x, size_t x_tree_stride, int K,
                                                   int D, const int32_t* slots, int bf, int lpr,
                                                   float* cent, void* out_t) {
    constexpr int EPL = Elem<T>::kPerChunk;
    const int k = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x;
    const int rg = lane / lpr, ch = lane % lpr, groups = 64 / lpr;
    const bool chunk_ok = ch * EPL < D;
    const int32_t* lst = slots + ((size_t)t * K + k) * bf;
    float acc[EPL];
#pragma unroll
    for (int q = 0; q < EPL; ++q) acc[q] = 0.0f;
    int cnt = 0;
    for (int e = rg; e < bf; e += groups) {
        const int it = lst[e];
        if (it < 0) continue;
        ++cnt;
        if (!chunk_ok) continue;
        float f[EPL];
        unpack<T>(load_chunk<T>(x, ((size_t)t * x_tree_stride + it) * D, ch), f);
#pragma unroll
        for (int q = 0; q < EPL; ++q) acc[q] += f[q];
    }
    for (int off = lpr; off < 64; off <<= 1) {
        cnt += __shfl_xor(cnt, off, 64);
#pragma unroll
        for (int q = 0; q < EPL; ++q) acc[q] += __shfl_xor(acc[q], off, 64);
    }
    if (rg == 0 && chunk_ok) {
#pragma unroll
        for (int q = 0; q < EPL; ++q) {
            const size_t o = ((size_t)t * K + k) * D + ch * EPL + q;
            float v = cent[o];
            if (cnt > 0) {
                v = acc[q] / (float)cnt;
                cent[o] = v;
            }
            store_elem<T>(out_t, o, v);
        }
    }
}

// ------------------------------------------------------------------------------------
// 5. capacity packing
// ------------------------------------------------------------------------------------
// One workgroup per bucket: the closest proposers (by distance, then item id) take the free
// slots of the block in that order; the others go on the list of the next round.  A block that
// is full now takes no more items: its norm in the operand tiles becomes +inf.
constexpr int kAcceptSort = 2048;  // keys sorted at a time; larger buckets in several goes, the
                                   // best `take` so far carried along

__global__ __launch_bounds__(kBucketThreads) void k_bucket_accept(
    const int32_t* members, const int32_t* offsets, const float* dist, int n_c, int K, int bf,
    int32_t* fill, int32_t* slots, int32_t* placed, int32_t* next_list, int32_t* next_count,
    int Kt, float* cn2, int32_t* counts, int32_t* done) {
    __shared__ uint64_t s_keys[kAcceptSort];
    __shared__ int32_t s_base, s_rej;
    const int k = blockIdx.x, t = blockIdx.y, tid = threadIdx.x;
    reset_counters(t, k, K, counts, done);
    const int b0 = offsets[(size_t)t * (K + 1) + k];
    const int m = offsets[(size_t)t * (K + 1) + k + 1] - b0;
    if (m <= 0) return;
    const int32_t* mem = members + (size_t)t * n_c + b0;
    const float* dt = dist + (size_t)t * n_c;
    const int f = fill[(size_t)t * K + k];
    const int take = max(min(m, bf - f), 0);
    int32_t* my_slots = slots + ((size_t)t * K + k) * bf + f;
    int32_t* pl = placed + (size_t)t * n_c;
    int32_t* nl = next_list + (size_t)t * n_c;
    __syncthreads();  // (every thread has read the block's fill)
    if (tid == 0) {
        s_base = m > take ? atomicAdd(&next_count[t], m - take) : 0;
        s_rej = 0;
        fill[(size_t)t * K + k] = f + take;
        if (cn2 != nullptr && f + take >= bf) cn2[(size_t)t * Kt * 16 + k] = INFINITY;
    }
    auto key_of = [&](int it) { return ((uint64_t)__float_as_uint(dt[it]) << 32) | (uint32_t)it; };
    if (m <= kBucketThreads) {
        int it = -1;
        uint64_t mine = ~0ull;
        if (tid < m) {
            it = mem[tid];
            mine = key_of(it);
        }
        s_keys[tid] = mine;
        __syncthreads();
        int rank = 0;
        for (int j = 0; j < m; ++j) rank += s_keys[j] < mine;
        if (tid < m) {
            if (rank < take) {
                my_slots[rank] = it;
                pl[it] = 1;
            } else {
                nl[s_base + rank - take] = it;
            }
        }
        return;
    }
    int kept = 0;  // s_keys[0 .. kept): the best so far, in order
    for (int e0 = 0; e0 < m;) {
        const int cn = min(kAcceptSort - kept, m - e0);
        const int P = pow2_at_least(kept + cn);
        __syncthreads();
        for (int e = kept + tid; e < P; e += kBucketThreads)
            s_keys[e] = e < kept + cn ? key_of(mem[e0 + e - kept]) : ~0ull;
        bitonic_sort(s_keys, P);
        kept = min(take, kept + cn);
        e0 += cn;
    }
    for (int r = tid; r < take; r += kBucketThreads) {
        const int it = (int)(uint32_t)s_keys[r];
        my_slots[r] = it;
        pl[it] = 1;
    }
    if (m > take) {  // whoever lies behind the last one taken tries again
        const uint64_t last = take > 0 ? s_keys[take - 1] : 0ull;
        for (int e = tid; e < m; e += kBucketThreads) {
            const int it = mem[e];
            if (take == 0 || key_of(it) > last) nl[s_base + atomicAdd(&s_rej, 1)] = it;
        }
    }
}

// (one atomic per workgroup of 256 items, not per wave: the tree's counter is one address)
__global__ __launch_bounds__(256) void k_collect_unplaced(const int32_t* placed, int n_c,
                                                          int32_t* list, int32_t* list_count) {
    __shared__ int32_t s_cnt[4];
    __shared__ int32_t s_base;
    const int t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool mine = i < n_c && placed[(size_t)t * n_c + i] == 0;
    const unsigned long long bal = __ballot(mine);
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    if (lane == 0) s_cnt[wave] = __popcll(bal);
    __syncthreads();
    if (threadIdx.x == 0) {
        const int total = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
        s_base = total > 0 ? atomicAdd(&list_count[t], total) : 0;
    }
    __syncthreads();
    int before = s_base;
    for (int w = 0; w < wave; ++w) before += s_cnt[w];
    if (mine) list[(size_t)t * n_c + before + __popcll(bal & ((1ull << lane) - 1ull))] = i;
}

// Whatever is still unplaced goes to the free slots in order: the u-th unplaced item (by
// item id) takes the u-th free slot (by block, then slot).  Two launches: the unplaced items of
// every 256 are counted, and the tree's last workgroup turns the counts, and the free slots
// of the blocks, into prefix sums; then every item finds its slot by itself.
__global__ __launch_bounds__(256) void k_leftover_count(const int32_t* placed, int n_c, int K,
                                                        int bf, const int32_t* fill,
                                                        int32_t* chunk_pre /* (T, chunks + 1) */,
                                                        int32_t* free_pre /* (T, K + 1) */,
                                                        int32_t* done) {
    __shared__ int32_t s_cnt[4];
    __shared__ int32_t s_last;
    const int t = blockIdx.y, nb = gridDim.x;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool mine = i < n_c && placed[(size_t)t * n_c + i] == 0;
    const unsigned long long bal = __ballot(mine);
    if (lane_id() == 0) s_cnt[threadIdx.x >> 6] = __popcll(bal);
    __syncthreads();
    int32_t* cp = chunk_pre + (size_t)t * (nb + 1);
    if (threadIdx.x == 0) {
        __hip_atomic_store(&cp[blockIdx.x], s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3],
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        hand_off_release();  // (the count is where every workgroup sees it before the ticket)
        s_last = atomicAdd(&done[t], 1) == nb - 1 ? 1 : 0;
    }
    __syncthreads();
    if (!s_last) return;
    const int unplaced = block_exclusive_scan(
        nb, [&](int b) { return load_agent(cp + b); }, [&](int b, int v) { cp[b] = v; });
    int32_t* fp = free_pre + (size_t)t * (K + 1);
    const int32_t* ft = fill + (size_t)t * K;
    const int room = block_exclusive_scan(
        K, [&](int k) { return bf - ft[k]; }, [&](int k, int v) { fp[k] = v; });
    if (threadIdx.x == 0) {
        cp[nb] = unplaced;
        fp[K] = room;
        done[t] = 0;
    }
}

__global__ __launch_bounds__(256) void k_leftover_place(int n_c, int K, int bf, const int32_t* fill,
                                                        const int32_t* chunk_pre,
                                                        const int32_t* free_pre, int32_t* slots,
                                                        int32_t* placed) {
    __shared__ int32_t s_cnt[4];
    const int t = blockIdx.y, nb = gridDim.x;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool mine = i < n_c && placed[(size_t)t * n_c + i] == 0;
    const unsigned long long bal = __ballot(mine);
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    if (lane == 0) s_cnt[wave] = __popcll(bal);
    __syncthreads();
    if (!mine) return;
    int u = chunk_pre[(size_t)t * (nb + 1) + blockIdx.x] + __popcll(bal & ((1ull << lane) - 1ull));
    for (int w = 0; w < wave; ++w) u += s_cnt[w];
    // block k with free_pre[k] <= u < free_pre[k + 1]
    const int32_t* fp = free_pre + (size_t)t * (K + 1);
    int lo = 0, hi = K;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (fp[mid] <= u) lo = mid; else hi = mid;
    }
    const int j = fill[(size_t)t * K + lo] + (u - fp[lo]);
    slots[((size_t)t * K + lo) * bf + j] = i;
    placed[(size_t)t * n_c + i] = 1;
}

// ------------------------------------------------------------------------------------
// 6. final layout
// ------------------------------------------------------------------------------------
// order_child[s*bf + j] = slots[order_parent[s]][j]  (or -1); order_parent == NULL: identity
__global__ void k_compose_order(const int32_t* order_parent, int size_parent, int K_parent,
                                const int32_t* slots, int bf, int32_t* order_child) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= size_parent * bf) return;
    const int s = i / bf, j = i % bf;
    int node = order_parent ? order_parent[(size_t)t * size_parent + s] : (s < K_parent ? s : -1);
    int v = -1;
    if (slots == nullptr)
        v = node;  // bf == 1: plain copy / identity
    else if (node >= 0)
        v = slots[((size_t)t * K_parent + node) * bf + j];
    order_child[(size_t)t * size_parent * bf + i] = v;
}

// dst[t][s] = src[t][order[t][s]] (zero row for -1), a thread per 16-byte chunk of a row (a chunk
// is contiguous in either layout).  perm_out != NULL: also writes perm.
template <typename T>
__global__ void k_gather_rows(const void* src, size_t src_tree_stride, const int32_t* order,
                              int size, int D, void* dst, size_t dst_tree_stride, int dst_layout,
                              int32_t* perm_out, size_t perm_tree_stride) {
    constexpr int EPL = Elem<T>::kPerChunk;
    const int t = blockIdx.y;
    const int chunks = D / EPL;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)size * chunks) return;
    const int s = (int)(i / chunks), c = (int)(i % chunks);
    const int o = order[(size_t)t * size + s];
    uint4 v = make_uint4(0, 0, 0, 0);
    if (o >= 0) v = load_chunk<T>(src, ((size_t)t * src_tree_stride + o) * D, c);
    T* out = reinterpret_cast<T*>(dst) + (size_t)t * dst_tree_stride * D +
             elem_index(dst_layout, D, (size_t)s, c * EPL);
    *reinterpret_cast<uint4*>(out) = v;
    if (perm_out && c == 0) perm_out[(size_t)t * perm_tree_stride + s] = o;
}

// the same, a thread per element: value rows whose length is not a multiple of 16 bytes
template <typename T>
__global__ void k_gather_elems(const void* src, size_t src_tree_stride, const int32_t* order,
                               int size, int D, void* dst, size_t dst_tree_stride) {
    const int t = blockIdx.y;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)size * D) return;
    const int s = (int)(i / D), j = (int)(i % D);
    const int o = order[(size_t)t * size + s];
    float v = 0.0f;
    if (o >= 0) v = load_elem<T>(src, ((size_t)t * src_tree_stride + o) * D + j);
    store_elem<T>(dst, ((size_t)t * dst_tree_stride + s) * D + j, v);
}

// counts[p] = children in use; radii[p] = max over them of (||child - centre|| + r_child),
// -inf when there is none.  One wave per node: `lpr` lanes (a power of two) hold a row in
// 16-byte chunks (a chunk is contiguous in either layout), 64 / lpr children at a time.
template <typename T>
__global__ __launch_bounds__(64) void k_radii(const void* child, size_t child_tree_stride,
                                              const float* child_radii,
                                              size_t child_radii_stride,
                                              const int32_t* child_order, int size_child,
                                              const void* centers, size_t center_tree_stride,
                                              int size, int bf, int D, int lpr, int child_layout,
                                              int layout, float* radii, int32_t* counts,
                                              size_t out_stride) {
    constexpr int EPL = Elem<T>::kPerChunk;
    const int p = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x;
    const int rg = lane / lpr, ch = lane % lpr, groups = 64 / lpr;
    const bool chunk_ok = ch * EPL < D;
    float cf[EPL];
    {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (chunk_ok)
            raw = *reinterpret_cast<const uint4*>(
                reinterpret_cast<const T*>(centers) + (size_t)t * center_tree_stride * D +
                elem_index(layout, D, (size_t)p, ch * EPL));
        unpack<T>(raw, cf);
    }
    float r = -INFINITY;
    int c = 0;
    for (int j0 = 0; j0 < bf; j0 += groups) {  // (uniform trip count: the sums meet in shuffles)
        const int j = j0 + rg;
        const int s = p * bf + j;
        const bool have = j < bf && s < size_child && child_order[(size_t)t * size_child + s] >= 0;
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (have && chunk_ok)
            raw = *reinterpret_cast<const uint4*>(
                reinterpret_cast<const T*>(child) + (size_t)t * child_tree_stride * D +
                elem_index(child_layout, D, (size_t)s, ch * EPL));
        float f[EPL];
        unpack<T>(raw, f);
        float ss = 0.0f;
#pragma unroll
        for (int q = 0; q < EPL; ++q) {
            const float df = f[q] - cf[q];
            ss += df * df;
        }
        for (int off = 1; off < lpr; off <<= 1) ss += __shfl_xor(ss, off, 64);
        if (have) {
            ++c;
            float v = sqrtf(ss);
            if (child_radii) v += child_radii[(size_t)t * child_radii_stride + s];
            r = fmaxf(r, v);
        }
    }
    for (int off = lpr; off < 64; off <<= 1) {
        r = fmaxf(r, __shfl_xor(r, off, 64));
        c += __shfl_xor(c, off, 64);
    }
    if (lane == 0) {
        // a few ulp of head room: the bound must survive fp32 rounding of this sum
        if (r > 0.0f) r = r * (1.0f + 4.0f * 1.1920929e-7f) + 1e-30f;
        radii[(size_t)t * out_stride + p] = r;
        counts[(size_t)t * out_stride + p] = c;
    }
}

// ------------------------------------------------------------------------------------
// host orchestration
// ------------------------------------------------------------------------------------
struct Carver {
    char* base;
    size_t used;
    template <typename U>
    U* take(size_t n) {
        used = (used + 255) & ~(size_t)255;
        U* p = base ? reinterpret_cast<U*>(base + used) : nullptr;
        used += n * sizeof(U);
        return p;
    }
};

struct BuildWs {
    float* cent_f32;
    void* cent_tiles;  // centroids as bf16 operand tiles (matrix-core assignment), or NULL
    float* cent_n2;
    void* open_tiles;  // the same for the centroids with room, side by side (later packing rounds)
    float* open_n2;
    int32_t *open_ids, *open_count;
    int32_t *assign, *pos, *placed, *members, *ordered;
    int32_t* list[2];     // the items of a packing round, and those of the round after it
    int32_t* list_count;  // (2, T)
    float* dist;
    int32_t *counts, *offsets, *done, *fill, *free_pre, *chunk_pre;
    int32_t* slots[HIRA_MAX_LEVELS];
    void* cent_t[HIRA_MAX_LEVELS];
    int32_t* order[HIRA_MAX_LEVELS];
    size_t total;
};

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

// bf16 rows of 64, 128 or 256 columns are assigned on the matrix cores
static bool assign_on_mfma(const HiraTree* t) {
    return t->dtype == HIRA_BF16 && (t->dim == 64 || t->dim == 128 || t->dim == 256);
}

// cluster counts per level: K[0] = n, K[l] = ceil(K[l-1] / bf)
static void cluster_counts(int n, int bf, int L, int* K) {
    K[0] = n;
    for (int l = 1; l < L; ++l) K[l] = K[l - 1] <= 0 ? 0 : (ceil_div(K[l - 1], bf) > 0 ? ceil_div(K[l - 1], bf) : 1);
}

static void carve(const HiraTree* t, int n, void* ws, BuildWs* b) {
    const int L = t->num_levels, T = t->num_trees, D = t->dim, bf = t->bf;
    const size_t esize = t->dtype == HIRA_F32 ? 4 : 2;
    int K[HIRA_MAX_LEVELS];
    cluster_counts(n, bf, L, K);
    Carver c{reinterpret_cast<char*>(ws), 0};
    const size_t k1 = L >= 2 ? (size_t)K[1] : 1;
    b->cent_f32 = c.take<float>((size_t)T * k1 * D);
    b->cent_tiles = nullptr;
    b->cent_n2 = nullptr;
    b->open_tiles = nullptr;
    b->open_n2 = nullptr;
    b->open_ids = b->open_count = nullptr;
    if (assign_on_mfma(t)) {
        const size_t kpad = (size_t)assign_tiles((int)k1) * 16;
        b->cent_tiles = c.take<char>((size_t)T * kpad * D * 4);  // hi and lo halves, 2 bytes each
        b->cent_n2 = c.take<float>((size_t)T * kpad);
        b->open_tiles = c.take<char>((size_t)T * kpad * D * 4);
        b->open_n2 = c.take<float>((size_t)T * kpad);
        b->open_ids = c.take<int32_t>((size_t)T * k1);
        b->open_count = c.take<int32_t>((size_t)T);
    }
    b->assign = c.take<int32_t>((size_t)T * n);
    b->pos = c.take<int32_t>((size_t)T * n);
    b->placed = c.take<int32_t>((size_t)T * n);
    b->members = c.take<int32_t>((size_t)T * n);
    b->ordered = c.take<int32_t>((size_t)T * n);
    b->list[0] = c.take<int32_t>((size_t)T * n);
    b->list[1] = c.take<int32_t>((size_t)T * n);
    b->list_count = c.take<int32_t>((size_t)T * 2);
    b->dist = c.take<float>((size_t)T * n);
    b->counts = c.take<int32_t>((size_t)T * k1);
    b->offsets = c.take<int32_t>((size_t)T * (k1 + 1));
    b->done = c.take<int32_t>((size_t)T);
    b->fill = c.take<int32_t>((size_t)T * k1);
    b->free_pre = c.take<int32_t>((size_t)T * (k1 + 1));
    b->chunk_pre = c.take<int32_t>((size_t)T * ((size_t)ceil_div(n, 256) + 1));
    for (int l = 0; l < HIRA_MAX_LEVELS; ++l) {
        b->slots[l] = nullptr;
        b->cent_t[l] = nullptr;
        b->order[l] = nullptr;
    }
    for (int l = 1; l < L; ++l) {
        b->slots[l] = c.take<int32_t>((size_t)T * K[l] * bf);
        b->cent_t[l] = c.take<char>((size_t)T * K[l] * D * esize);
    }
    for (int l = 0; l < L; ++l) b->order[l] = c.take<int32_t>((size_t)T * t->size[l]);
    b->total = (c.used + 255) & ~(size_t)255;
}

template <typename T>
static int launch_assign(int lpr, dim3 grid, hipStream_t s, const void* x, int n_c,
                         size_t x_stride, const float* cent, int K, int D, const int32_t* fill,
                         int bf, const int32_t* list, const int32_t* list_count,
                         size_t list_stride, int32_t* assign, float* dist,
                         const AssignCounting& counting) {
#define HIRA_ASSIGN_CASE(N)                                                                   \
    case N:                                                                                   \
        hipLaunchKernelGGL((k_assign_simple<T, N>), grid, dim3(256), 0, s, x, n_c, x_stride,   \
                           cent, K, D, fill, bf, list, list_count, list_stride, assign, dist, \
                           counting);                                                          \
        break;
    switch (lpr) {
        HIRA_ASSIGN_CASE(2)
        HIRA_ASSIGN_CASE(4)
        HIRA_ASSIGN_CASE(8)
        HIRA_ASSIGN_CASE(16)
        HIRA_ASSIGN_CASE(32)
        HIRA_ASSIGN_CASE(64)
        default:
            return fail(HIRA_EINVAL, "unsupported row width");
    }
#undef HIRA_ASSIGN_CASE
    return HIRA_OK;
}

static void fill_i32(int32_t* p, size_t n, int32_t v, hipStream_t s) {
    if (n == 0) return;
    hipLaunchKernelGGL(k_fill_i32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n, v);
}

template <typename T>
static int build_impl(const HiraTree* t, const void* keys_in, const void* values_in, int n,
                      const int32_t* n_live, int niter, int pack_rounds, uint64_t seed,
                      const BuildWs& w, hipStream_t s) {
    const int L = t->num_levels, NT = t->num_trees, D = t->dim, bf = t->bf;
    constexpr int EPL = Elem<T>::kPerChunk;
    int lpr = 2;
    while (lpr * EPL < D) lpr <<= 1;
    int K[HIRA_MAX_LEVELS];
    cluster_counts(n, bf, L, K);

    const bool on_mfma = w.cent_tiles != nullptr;
    uint4* tiles = reinterpret_cast<uint4*>(w.cent_tiles);
    for (int l = 1; l < L; ++l) {
        const void* x = l == 1 ? keys_in : w.cent_t[l - 1];
        const int n_c = K[l - 1];
        const size_t xs = (size_t)n_c;  // rows per tree in x
        const int Kl = K[l];
        const int Kt = on_mfma ? assign_tiles(Kl) : 0;
        const int items_per_block = 4 * (64 / lpr) * kPPG;
        const dim3 g_assign(ceil_div(n_c, items_per_block), NT);
        const dim3 g_items(ceil_div(n_c, 256), NT);
        const dim3 g_cent(Kl, NT);

        // Trees with fewer items than rows (n_live): every phase walks the list of the items
        // the tree holds, and the first packing round does too.
        const bool ragged = n_live != nullptr && l == 1;
        hipLaunchKernelGGL(k_level_init, dim3(min(ceil_div(max(n_c, Kl * bf), 256), 2048), NT),
                           dim3(256), 0, s, n_c, Kl, bf, D, Kt, ragged ? n_live : nullptr, w.placed,
                           w.fill, w.slots[l], w.counts, w.done, w.list_count, tiles, w.cent_n2);
        const int32_t* live = nullptr;
        const int32_t* live_cnt = nullptr;
        if (ragged) {
            hipLaunchKernelGGL(k_collect_unplaced, g_items, dim3(256), 0, s, w.placed, n_c,
                               w.list[0], w.list_count);
            live = w.list[0];
            live_cnt = w.list_count;
        }
        hipLaunchKernelGGL((k_init_centroids<T>), g_cent, dim3(64), 0, s, x, n_c, xs, Kl, D,
                           seed + 7919ull * (uint64_t)l, w.cent_f32, ragged ? n_live : nullptr, bf,
                           Kt, w.fill, tiles, w.cent_n2);
        // a round: the assignment (which also counts the items of every centroid and turns the
        // counts into offsets), the buckets, and what the round does with every bucket
        auto assign_round = [&](const int32_t* list, const int32_t* lcnt, const int32_t* fill,
                                int32_t* zero, bool only_open) -> int {
            const AssignCounting ac{w.counts, w.pos, w.done, w.offsets, zero};
            int rc;
            if (on_mfma && only_open) {
                rc = launch_open_centroids(D, w.cent_tiles, w.cent_n2, w.fill, bf, Kl, NT, w.open_ids,
                                           w.open_count, w.open_tiles, w.open_n2, s);
                if (rc == HIRA_OK)
                    rc = launch_assign_mfma(D, x, n_c, xs, w.open_tiles, w.open_n2, Kl, NT, list, lcnt,
                                            (size_t)n_c, w.assign, w.dist, ac,
                                            AssignOpen{w.open_count, w.open_ids}, s);
            } else if (on_mfma)
                rc = launch_assign_mfma(D, x, n_c, xs, w.cent_tiles, w.cent_n2, Kl, NT, list, lcnt,
                                        (size_t)n_c, w.assign, w.dist, ac, AssignOpen{nullptr, nullptr}, s);
            else
                rc = launch_assign<T>(lpr, g_assign, s, x, n_c, xs, w.cent_f32, Kl, D, fill, bf, list,
                                      lcnt, (size_t)n_c, w.assign, w.dist, ac);
            if (rc != HIRA_OK) return rc;
            hipLaunchKernelGGL(k_bucket_fill, g_items, dim3(256), 0, s, w.assign, w.pos, w.offsets,
                               n_c, list, lcnt, (size_t)n_c, Kl, w.members);
            return HIRA_OK;
        };
        for (int it = 0; it < niter; ++it) {
            const int rc = assign_round(live, live_cnt, ragged ? w.fill : nullptr, nullptr, false);
            if (rc != HIRA_OK) return rc;
            hipLaunchKernelGGL((k_bucket_mean<T>), g_cent, dim3(kBucketThreads), 0, s, x, xs, n_c,
                               Kl, D, w.offsets, w.members, w.ordered, ragged ? w.fill : nullptr, bf,
                               w.cent_f32, Kt, tiles, w.cent_n2, w.counts, w.done);
        }
        // capacity packing: round r walks list r % 2 (the first one all items, or the items the
        // trees hold) and leaves those it could not place on the other list
        for (int r = 0; r < pack_rounds; ++r) {
            const int32_t* list = r == 0 ? live : w.list[r & 1];
            const int32_t* lcnt = r == 0 ? live_cnt : w.list_count + (size_t)(r & 1) * NT;
            int32_t* next_cnt = w.list_count + (size_t)((r + 1) & 1) * NT;
            // (from the second round on most blocks are full: the assignment then sees only the
            // centroids with room, side by side; worth its two small launches from 32 tiles on)
            const int rc = assign_round(list, lcnt, w.fill, next_cnt, r >= 1 && Kl >= 512);
            if (rc != HIRA_OK) return rc;
            hipLaunchKernelGGL(k_bucket_accept, g_cent, dim3(kBucketThreads), 0, s, w.members,
                               w.offsets, w.dist, n_c, Kl, bf, w.fill, w.slots[l], w.placed,
                               w.list[(r + 1) & 1], next_cnt, Kt, on_mfma ? w.cent_n2 : nullptr,
                               w.counts, w.done);
        }
        hipLaunchKernelGGL(k_leftover_count, g_items, dim3(256), 0, s, w.placed, n_c, Kl, bf, w.fill,
                           w.chunk_pre, w.free_pre, w.done);
        hipLaunchKernelGGL(k_leftover_place, g_items, dim3(256), 0, s, n_c, Kl, bf, w.fill,
                           w.chunk_pre, w.free_pre, w.slots[l], w.placed);
        // block centre = mean of what is in the block, rounded to the storage type
        hipLaunchKernelGGL((k_block_mean<T>), g_cent, dim3(64), 0, s, x, xs, Kl, D, w.slots[l], bf,
                           lpr, w.cent_f32, w.cent_t[l]);
        HIRA_CHECK_LAUNCH("build level");
    }

    // layout, top-down
    if (L == 1) {
        // keys stay in insertion order
        hipLaunchKernelGGL(k_compose_order, dim3(ceil_div(n, 256), NT), dim3(256), 0, s, nullptr, n,
                           n, nullptr, 1, w.order[0]);
    }
    for (int l = L - 1; l >= 1; --l) {
        const int32_t* po = l == L - 1 ? nullptr : w.order[l];
        hipLaunchKernelGGL(k_compose_order, dim3(ceil_div(t->size[l] * bf, 256), NT), dim3(256), 0,
                           s, po, t->size[l], K[l], w.slots[l], bf, w.order[l - 1]);
        if (l == L - 1)  // identity order of the root, needed by the gathers below
            hipLaunchKernelGGL(k_compose_order, dim3(ceil_div(t->size[l], 256), NT), dim3(256), 0,
                               s, nullptr, t->size[l], K[l], nullptr, 1, w.order[l]);
    }
    // gathers
    {
        const size_t tot = (size_t)t->size[0] * (D / Elem<T>::kPerChunk);
        hipLaunchKernelGGL((k_gather_rows<T>), dim3((unsigned)((tot + 255) / 256), NT), dim3(256),
                           0, s, keys_in, (size_t)n, w.order[0], t->size[0], D, t->keys,
                           (size_t)t->cap[0], key_layout_of(t->layout), t->perm, (size_t)t->cap[0]);
        if (values_in && t->values) {
            if (t->vdim % Elem<T>::kPerChunk == 0) {
                const size_t totv = (size_t)t->size[0] * (t->vdim / Elem<T>::kPerChunk);
                hipLaunchKernelGGL((k_gather_rows<T>), dim3((unsigned)((totv + 255) / 256), NT),
                                   dim3(256), 0, s, values_in, (size_t)n, w.order[0], t->size[0],
                                   t->vdim, t->values, (size_t)t->cap[0], (int)HIRA_ROW_MAJOR, nullptr, (size_t)0);
            } else {
                const size_t totv = (size_t)t->size[0] * t->vdim;
                hipLaunchKernelGGL((k_gather_elems<T>), dim3((unsigned)((totv + 255) / 256), NT),
                                   dim3(256), 0, s, values_in, (size_t)n, w.order[0], t->size[0],
                                   t->vdim, t->values, (size_t)t->cap[0]);
            }
        }
        for (int l = 1; l < L; ++l) {
            const size_t totc = (size_t)t->size[l] * (D / Elem<T>::kPerChunk);
            hipLaunchKernelGGL((k_gather_rows<T>), dim3((unsigned)((totc + 255) / 256), NT),
                               dim3(256), 0, s, w.cent_t[l], (size_t)K[l], w.order[l], t->size[l], D,
                               t->centers[l], (size_t)t->cap[l], center_layout_of(t->layout), nullptr, (size_t)0);
        }
    }
    // radii and counts, bottom-up
    for (int l = 1; l < L; ++l) {
        const void* child = l == 1 ? t->keys : t->centers[l - 1];
        const float* crad = l == 1 ? nullptr : t->radii[l - 1];
        hipLaunchKernelGGL((k_radii<T>), dim3(t->size[l], NT), dim3(64), 0, s, child,
                           (size_t)t->cap[l - 1], crad, (size_t)t->cap[l - 1], w.order[l - 1],
                           t->size[l - 1], t->centers[l], (size_t)t->cap[l], t->size[l], bf, D, lpr,
                           l == 1 ? key_layout_of(t->layout) : center_layout_of(t->layout),
                           center_layout_of(t->layout), t->radii[l], t->counts[l], (size_t)t->cap[l]);
    }
    HIRA_CHECK_LAUNCH("build layout");
    if (t->layout == HIRA_TILE16_Q8)  // steps from all keys, then the 8-bit shadow
        return hira_quantize(t, 0, t->size[0], 1, s);
    return HIRA_OK;
}

static int check_build_args(const HiraTree* t, int n) {
    HIRA_CHECK_ARG(t != nullptr, "tree is NULL");
    HIRA_CHECK_ARG(t->dtype == HIRA_F32 || t->dtype == HIRA_BF16, "dtype %d", t->dtype);
    HIRA_CHECK_ARG(t->num_trees >= 1 && t->num_trees <= 65535, "num_trees %d", t->num_trees);
    HIRA_CHECK_ARG(t->num_levels >= 1 && t->num_levels <= HIRA_MAX_LEVELS, "num_levels %d",
                   t->num_levels);
    HIRA_CHECK_ARG(t->bf >= 1 && t->bf <= 64, "branching factor %d not in 1..64", t->bf);
    const int epl = t->dtype == HIRA_F32 ? 4 : 8;
    HIRA_CHECK_ARG(t->dim >= epl && t->dim % epl == 0 && t->dim <= 64 * epl,
                   "dim %d: rows must be a multiple of 16 bytes", t->dim);
    HIRA_CHECK_ARG(n >= 1, "need at least one key, got %d", n);
    HIRA_CHECK_ARG(t->layout == HIRA_ROW_MAJOR || t->layout == HIRA_TILE16 ||
                       t->layout == HIRA_TILE16_Q8, "layout %d", t->layout);
    if (t->layout == HIRA_TILE16_Q8)
        HIRA_CHECK_ARG((t->dim == 64 || t->dim == 128) && t->num_levels >= 2 && t->keys8 &&
                           t->kscale && t->keps,
                       "the layout with an 8-bit shadow needs rows of 64 or 128 columns, at least "
                       "two levels, and the keys8 / kscale / keps arrays");
    if (t->layout != HIRA_ROW_MAJOR) {
        HIRA_CHECK_ARG(t->dtype == HIRA_BF16 && t->dim % 32 == 0,
                       "the tiled layout needs bf16 rows of a multiple of 32 columns");
        for (int l = 0; l < t->num_levels; ++l)
            HIRA_CHECK_ARG(t->cap[l] % 16 == 0, "tiled layout: cap[%d]=%d not a multiple of 16", l,
                           t->cap[l]);
    }
    int K[HIRA_MAX_LEVELS];
    cluster_counts(n, t->bf, t->num_levels, K);
    // padded sizes the layout needs
    long long want = t->num_levels == 1 ? n : K[t->num_levels - 1];
    for (int l = t->num_levels - 1; l >= 0; --l) {
        HIRA_CHECK_ARG(t->size[l] == want, "size[%d] = %d, the layout of %d keys needs %lld", l,
                       t->size[l], n, want);
        HIRA_CHECK_ARG(t->cap[l] >= t->size[l], "cap[%d] = %d < size %d", l, t->cap[l], t->size[l]);
        want *= t->bf;
    }
    return HIRA_OK;
}

}  // namespace hira

using namespace hira;

extern "C" size_t hira_build_workspace_bytes(const HiraTree* tree, int32_t n) {
    if (check_build_args(tree, n) != HIRA_OK) return 0;
    BuildWs b;
    carve(tree, n, nullptr, &b);
    return b.total;
}

extern "C" int hira_build(const HiraTree* tree, const void* keys_in, const void* values_in,
                          int32_t n, int32_t niter, int32_t pack_rounds, uint64_t seed,
                          void* workspace, size_t workspace_bytes, void* stream) {
    return hira_build_ragged(tree, keys_in, values_in, n, nullptr, niter, pack_rounds, seed,
                             workspace, workspace_bytes, stream);
}

/* see include/hira_hip.h */
extern "C" int hira_build_ragged(const HiraTree* tree, const void* keys_in, const void* values_in,
                                 int32_t n, const int32_t* n_live, int32_t niter,
                                 int32_t pack_rounds, uint64_t seed, void* workspace,
                                 size_t workspace_bytes, void* stream) {
    int rc = check_build_args(tree, n);
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_ARG(n_live == nullptr || tree->num_levels == 2,
                   "per-tree key counts are taken for trees of two levels only (got %d)",
                   tree->num_levels);
    HIRA_CHECK_ARG(keys_in != nullptr && tree->keys != nullptr && tree->perm != nullptr,
                   "keys / perm missing");
    HIRA_CHECK_ARG(niter >= 0 && pack_rounds >= 1, "niter %d, pack_rounds %d", niter, pack_rounds);
    for (int l = 1; l < tree->num_levels; ++l)
        HIRA_CHECK_ARG(tree->centers[l] && tree->radii[l] && tree->counts[l],
                       "level %d arrays missing", l);
    BuildWs b;
    carve(tree, n, workspace, &b);
    if (workspace == nullptr || workspace_bytes < b.total)
        return fail(HIRA_EWORKSPACE, "workspace %zu bytes, need %zu", workspace_bytes, b.total);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    return tree->dtype == HIRA_F32
               ? build_impl<float>(tree, keys_in, values_in, n, n_live, niter, pack_rounds, seed, b, s)
               : build_impl<bf16_t>(tree, keys_in, values_in, n, n_live, niter, pack_rounds, seed, b, s);
}

// ---- nearest centre as a call of its own -------------------------------------------------
namespace hira {

__global__ void k_valid_to_fill(const int32_t* valid, size_t n, int32_t* fill) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) fill[i] = valid[i] != 0 ? 0 : 1;  // "full" (>= 1 of 1 slots) = not usable
}

struct NearestWs {
    void* tiles;
    float* n2;
    int32_t* fill;
    size_t total;
};

static void carve_nearest(int dtype, int T, int m, int D, bool masked, void* ws, NearestWs* b) {
    Carver c{reinterpret_cast<char*>(ws), 0};
    b->tiles = nullptr;
    b->n2 = nullptr;
    if (dtype == HIRA_BF16 && (D == 64 || D == 128 || D == 256)) {
        const size_t kpad = (size_t)assign_tiles(m) * 16;
        b->tiles = c.take<char>((size_t)T * kpad * D * 4);
        b->n2 = c.take<float>((size_t)T * kpad);
    }
    b->fill = masked ? c.take<int32_t>((size_t)T * m) : nullptr;
    b->total = (c.used + 255) & ~(size_t)255;
}

static int check_nearest_args(int dtype, int T, int n, int m, int D) {
    HIRA_CHECK_ARG(dtype == HIRA_F32 || dtype == HIRA_BF16, "dtype %d", dtype);
    const int epl = dtype == HIRA_F32 ? 4 : 8;
    HIRA_CHECK_ARG(T >= 1 && T <= 65535, "num_trees %d", T);
    HIRA_CHECK_ARG(n >= 1 && m >= 1, "n = %d rows, m = %d centres", n, m);
    HIRA_CHECK_ARG(D >= epl && D % epl == 0 && D <= 64 * epl,
                   "dim %d: rows must be a multiple of 16 bytes", D);
    return HIRA_OK;
}

}  // namespace hira

extern "C" size_t hira_nearest_workspace_bytes(int32_t dtype, int32_t num_trees, int32_t m,
                                               int32_t dim) {
    if (check_nearest_args(dtype, num_trees, 1, m, dim) != HIRA_OK) return 0;
    NearestWs b;
    carve_nearest(dtype, num_trees, m, dim, true, nullptr, &b);
    return b.total > 0 ? b.total : 256;
}

extern "C" int hira_nearest(const void* x, int32_t dtype, int32_t num_trees, int32_t n,
                            const float* centers, int32_t m, int32_t dim, const int32_t* valid,
                            int32_t* idx, float* dist2, void* workspace, size_t workspace_bytes,
                            void* stream) {
    int rc = check_nearest_args(dtype, num_trees, n, m, dim);
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_ARG(x && centers && idx && dist2, "x / centers / idx / dist2 missing");
    NearestWs b;
    carve_nearest(dtype, num_trees, m, dim, valid != nullptr, workspace, &b);
    if (b.total > 0 && (workspace == nullptr || workspace_bytes < b.total))
        return fail(HIRA_EWORKSPACE, "workspace %zu bytes, need %zu", workspace_bytes, b.total);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const size_t nm = (size_t)num_trees * m;
    if (valid != nullptr)
        hipLaunchKernelGGL(k_valid_to_fill, dim3((unsigned)((nm + 255) / 256)), dim3(256), 0, s,
                           valid, nm, b.fill);
    // a row without any usable centre keeps idx -1 and an infinite distance
    fill_i32(idx, (size_t)num_trees * n, -1, s);
    fill_i32(reinterpret_cast<int32_t*>(dist2), (size_t)num_trees * n, 0x7f800000, s);
    if (b.tiles != nullptr) {
        rc = launch_cent_prep(dim, centers, m, num_trees, b.fill, 1, b.tiles, b.n2, s);
        if (rc == HIRA_OK)
            rc = launch_assign_mfma(dim, x, n, (size_t)n, b.tiles, b.n2, m, num_trees, nullptr,
                                    nullptr, 0, idx, dist2, AssignCounting{}, AssignOpen{nullptr, nullptr}, s);
    } else {
        const int epl = dtype == HIRA_F32 ? 4 : 8;
        int lpr = 2;
        while (lpr * epl < dim) lpr <<= 1;
        const dim3 grid(ceil_div(n, 4 * (64 / lpr) * kPPG), num_trees);
        rc = dtype == HIRA_F32
                 ? launch_assign<float>(lpr, grid, s, x, n, (size_t)n, centers, m, dim, b.fill, 1,
                                        nullptr, nullptr, 0, idx, dist2, AssignCounting{})
                 : launch_assign<bf16_t>(lpr, grid, s, x, n, (size_t)n, centers, m, dim, b.fill, 1,
                                         nullptr, nullptr, 0, idx, dist2, AssignCounting{});
    }
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_LAUNCH("nearest-centre kernel");
    return HIRA_OK;
}
