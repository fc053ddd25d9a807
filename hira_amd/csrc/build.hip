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
// 1. initial centroids: item floor((k + u_k) * n_c / K), u_k in [0,1) from the seed
// ------------------------------------------------------------------------------------
//    (n_live != NULL: tree t holds n_live[t] <= n_c items, the first ones of its rows)
template <typename T>
__global__ void k_init_centroids(const void* x, int n_c, size_t x_tree_stride, int K, int D,
                                 uint64_t seed, float* cent, const int32_t* n_live, int bf) {
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
    for (int j = threadIdx.x; j < D; j += blockDim.x) dst[j] = load_elem<T>(x, src + j);
}

// ------------------------------------------------------------------------------------
// 2. nearest centroid (vector-ALU kernel): argmin_k ||x_i - c_k||^2, lowest k on ties.
//    LPR lanes hold one item row; each lane group keeps PPG items in registers and walks
//    all centroids.  fill != NULL: centroids with fill[k] >= bf are skipped.
//    list != NULL: only the items list[0 .. *list_count) are processed.
// ------------------------------------------------------------------------------------
constexpr int kPPG = 4;

template <typename T, int LPR>
__global__ __launch_bounds__(256) void k_assign_simple(
    const void* x, int n_c, size_t x_tree_stride, const float* cent, int K, int D,
    const int32_t* fill, int bf, const int32_t* list, const int32_t* list_count, size_t list_stride,
    int32_t* assign, float* dist) {
    constexpr int EPL = Elem<T>::kPerChunk;
    constexpr int RPW = kWave / LPR;
    const int lane = lane_id();
    const int rg = lane / LPR, ch = lane % LPR;
    const int t = blockIdx.y;
    const int n_items = list ? list_count[t] : n_c;
    const int wave_global = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int first = wave_global * (RPW * kPPG);
    if (first >= n_items) return;
    const bool chunk_ok = ch * EPL < D;

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
            }
        }
    }
}

// ------------------------------------------------------------------------------------
// 3. bucket the processed items by assigned centroid, each bucket sorted by (dist, item)
// ------------------------------------------------------------------------------------
__global__ void k_bucket_count(const int32_t* assign, int n_c, const int32_t* list,
                               const int32_t* list_count, size_t list_stride, int K,
                               int32_t* counts) {
    const int t = blockIdx.y;
    const int n_items = list ? list_count[t] : n_c;
    const int pos = blockIdx.x * blockDim.x + threadIdx.x;
    if (pos >= n_items) return;
    const int i = list ? list[(size_t)t * list_stride + pos] : pos;
    const int a = assign[(size_t)t * n_c + i];
    if (a >= 0) atomicAdd(&counts[(size_t)t * K + a], 1);
}

// exclusive scan of counts (K entries) per tree -> offsets (K+1 entries); cursor := offsets
__global__ __launch_bounds__(256) void k_scan(const int32_t* counts, int K, int32_t* offsets,
                                              int32_t* cursor) {
    __shared__ int32_t wsum[4];
    __shared__ int32_t carry;
    const int t = blockIdx.x;
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (int base = 0; base < K; base += 256) {
        const int k = base + threadIdx.x;
        const int v = k < K ? counts[(size_t)t * K + k] : 0;
        int inc = v;  // inclusive scan in the wave
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        int before = carry;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        const int excl = before + inc - v;
        if (k < K) {
            offsets[(size_t)t * (K + 1) + k] = excl;
            cursor[(size_t)t * K + k] = excl;
        }
        __syncthreads();
        if (threadIdx.x == 255) carry = excl + v;
        __syncthreads();
    }
    if (threadIdx.x == 0) offsets[(size_t)t * (K + 1) + K] = carry;
}

__global__ void k_bucket_fill(const int32_t* assign, int n_c, const int32_t* list,
                              const int32_t* list_count, size_t list_stride, int K,
                              int32_t* cursor, int32_t* members) {
    const int t = blockIdx.y;
    const int n_items = list ? list_count[t] : n_c;
    const int pos = blockIdx.x * blockDim.x + threadIdx.x;
    if (pos >= n_items) return;
    const int i = list ? list[(size_t)t * list_stride + pos] : pos;
    const int a = assign[(size_t)t * n_c + i];
    if (a < 0) return;
    const int at = atomicAdd(&cursor[(size_t)t * K + a], 1);
    members[(size_t)t * n_c + at] = i;
}

// one workgroup per bucket: rank every member by (dist, item id) and write it to its rank (four
// waves: nearest-centroid buckets of seeds drawn from the keys are very uneven in 128 dimensions,
// and a bucket of m members costs m * m / threads comparisons)
constexpr int kSortTile = 1024;
constexpr int kSortThreads = 256;
__global__ __launch_bounds__(kSortThreads) void k_bucket_sort(const int32_t* members,
                                                              const int32_t* offsets,
                                                              const float* dist, int n_c, int K,
                                                              int32_t* sorted) {
    __shared__ uint64_t keys[kSortTile];
    const int k = blockIdx.x, t = blockIdx.y;
    const int tid = threadIdx.x;
    const int b0 = offsets[(size_t)t * (K + 1) + k], b1 = offsets[(size_t)t * (K + 1) + k + 1];
    const int m = b1 - b0;
    if (m <= 0) return;
    const int32_t* mem = members + (size_t)t * n_c + b0;
    const float* dt = dist + (size_t)t * n_c;
    for (int e0 = 0; e0 < m; e0 += kSortThreads) {
        const int e = e0 + tid;
        uint64_t mykey = 0;
        int myitem = -1;
        if (e < m) {
            myitem = mem[e];
            mykey = ((uint64_t)__float_as_uint(dt[myitem]) << 32) | (uint32_t)myitem;
        }
        int rank = 0;
        for (int tile = 0; tile < m; tile += kSortTile) {
            const int tn = min(kSortTile, m - tile);
            __syncthreads();
            for (int j = tid; j < tn; j += kSortThreads) {
                const int it = mem[tile + j];
                keys[j] = ((uint64_t)__float_as_uint(dt[it]) << 32) | (uint32_t)it;
            }
            __syncthreads();
            if (e < m)
                for (int j = 0; j < tn; ++j) rank += keys[j] < mykey;
        }
        if (e < m) sorted[(size_t)t * n_c + b0 + rank] = myitem;
    }
}

// ------------------------------------------------------------------------------------
// 4. centroid = mean of the member rows, summed in list order.  One wave per centroid.
//    Lists: CSR (offsets/members) when slots == NULL, else the bf slots of the block.
//    An empty centroid keeps its value.  out_t != NULL: also store rounded to T.
// ------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void k_mean(const void* x, size_t x_tree_stride, int n_c, int K,
                                              int D, const int32_t* offsets,
                                              const int32_t* members, const int32_t* slots, int bf,
                                              float* cent, void* out_t) {
    // launched with one wave (the sums then run in list order) or four (wave w sums members
    // w, w + 4, ..., the four sums are added in wave order: large buckets, still reproducible)
    __shared__ float s_part[3][64];
    __shared__ int s_cnt[3];
    const int k = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int32_t* lst;
    int m;
    if (slots) {
        lst = slots + ((size_t)t * K + k) * bf;
        m = bf;
    } else {
        const int b0 = offsets[(size_t)t * (K + 1) + k];
        m = offsets[(size_t)t * (K + 1) + k + 1] - b0;
        lst = members + (size_t)t * n_c + b0;
    }
    for (int j0 = 0; j0 < D; j0 += 64) {
        const int j = j0 + lane;
        float s = 0.0f;
        int cnt = 0;
        for (int e = wave; e < m; e += nw) {
            const int it = lst[e];
            if (it < 0) continue;
            ++cnt;
            if (j < D) s += load_elem<T>(x, ((size_t)t * x_tree_stride + it) * D + j);
        }
        if (nw > 1) {  // uniform
            __syncthreads();
            if (wave > 0) {
                s_part[wave - 1][lane] = s;
                if (lane == 0) s_cnt[wave - 1] = cnt;
            }
            __syncthreads();
            if (wave == 0)
                for (int w = 1; w < nw; ++w) {
                    s += s_part[w - 1][lane];
                    cnt += s_cnt[w - 1];
                }
        }
        if (wave == 0 && j < D) {
            const size_t o = ((size_t)t * K + k) * D + j;
            float v = cent[o];
            if (cnt > 0) {
                v = s / (float)cnt;
                cent[o] = v;
            }
            if (out_t) store_elem<T>(out_t, o, v);
        }
    }
}

// ------------------------------------------------------------------------------------
// 5. capacity packing
// ------------------------------------------------------------------------------------
// one wave per bucket: the closest proposers take the free slots of the block
__global__ __launch_bounds__(64) void k_accept(const int32_t* sorted, const int32_t* offsets,
                                               int n_c, int K, int bf, int32_t* fill,
                                               int32_t* slots, int32_t* placed) {
    const int k = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x;
    const int b0 = offsets[(size_t)t * (K + 1) + k];
    const int m = offsets[(size_t)t * (K + 1) + k + 1] - b0;
    if (m <= 0) return;
    const int f = fill[(size_t)t * K + k];
    const int take = min(m, bf - f);
    for (int r = lane; r < take; r += 64) {
        const int it = sorted[(size_t)t * n_c + b0 + r];
        slots[((size_t)t * K + k) * bf + f + r] = it;
        placed[(size_t)t * n_c + it] = 1;
    }
    __syncthreads();
    if (lane == 0) fill[(size_t)t * K + k] = f + take;
}

// items a tree does not hold count as placed from the start: no phase ever touches them; and
// a tree with n_t items uses its first ceil(n_t / bf) centroids only: the others count as full
__global__ void k_mark_absent(const int32_t* n_live, int n_c, int K, int bf, int32_t* placed,
                              int32_t* fill) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int n_t = min(max(n_live[t], 0), n_c);
    if (i < n_c) placed[(size_t)t * n_c + i] = i >= n_t ? 1 : 0;
    if (i < K) fill[(size_t)t * K + i] = i >= max((n_t + bf - 1) / bf, 1) ? bf : 0;
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
// item id) takes the u-th free slot (by block, then slot).  One workgroup per tree.
constexpr int kLeftThreads = 1024;  // (the walk over a tree's items is serial in steps of this many)
__global__ __launch_bounds__(kLeftThreads) void k_leftover(int n_c, int K, int bf, int32_t* fill,
                                                  int32_t* slots, int32_t* placed,
                                                  int32_t* scratch /* (T, K+1) */) {
    __shared__ int32_t wsum[kLeftThreads / 64];
    __shared__ int32_t carry;
    const int t = blockIdx.x;
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    int32_t* freepre = scratch + (size_t)t * (K + 1);  // exclusive prefix of free slots
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (int base = 0; base < K; base += kLeftThreads) {
        const int k = base + threadIdx.x;
        const int v = k < K ? bf - fill[(size_t)t * K + k] : 0;
        int inc = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        int before = carry;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        if (k < K) freepre[k] = before + inc - v;
        __syncthreads();
        if (threadIdx.x == kLeftThreads - 1) carry = before + inc;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        freepre[K] = carry;
        carry = 0;
    }
    __syncthreads();
    for (int base = 0; base < n_c; base += kLeftThreads) {
        const int i = base + threadIdx.x;
        const int v = (i < n_c && placed[(size_t)t * n_c + i] == 0) ? 1 : 0;
        int inc = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        int before = carry;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        if (v) {
            const int u = before + inc - 1;  // rank among the unplaced
            // block k with freepre[k] <= u < freepre[k+1]
            int lo = 0, hi = K;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (freepre[mid] <= u) lo = mid; else hi = mid;
            }
            const int j = fill[(size_t)t * K + lo] + (u - freepre[lo]);
            slots[((size_t)t * K + lo) * bf + j] = i;
            placed[(size_t)t * n_c + i] = 1;
        }
        __syncthreads();
        if (threadIdx.x == kLeftThreads - 1) carry = before + inc;
        __syncthreads();
    }
    __syncthreads();
    // the blocks are now as full as the items allow
    for (int k = threadIdx.x; k < K; k += kLeftThreads) {
        int c = 0;
        for (int j = 0; j < bf; ++j) c += slots[((size_t)t * K + k) * bf + j] >= 0;
        fill[(size_t)t * K + k] = c;
    }
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
// -inf when there is none.  One wave per node.
template <typename T>
__global__ __launch_bounds__(64) void k_radii(const void* child, size_t child_tree_stride,
                                              const float* child_radii,
                                              size_t child_radii_stride,
                                              const int32_t* child_order, int size_child,
                                              const void* centers, size_t center_tree_stride,
                                              int size, int bf, int D, int child_layout,
                                              int layout, float* radii, int32_t* counts,
                                              size_t out_stride) {
    const int p = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x;
    float r = -INFINITY;
    int c = 0;
    for (int j = 0; j < bf; ++j) {
        const int s = p * bf + j;
        if (s >= size_child) break;
        if (child_order[(size_t)t * size_child + s] < 0) continue;
        ++c;
        float ss = 0.0f;
        for (int e = lane; e < D; e += 64) {
            const float df =
                load_elem<T>(child, (size_t)t * child_tree_stride * D + elem_index(child_layout, D, (size_t)s, e)) -
                load_elem<T>(centers, (size_t)t * center_tree_stride * D + elem_index(layout, D, (size_t)p, e));
            ss += df * df;
        }
        ss = group_sum<64>(ss);
        float v = sqrtf(ss);
        if (child_radii) v += child_radii[(size_t)t * child_radii_stride + s];
        r = fmaxf(r, v);
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
    int32_t *assign, *placed, *members, *sorted, *list, *list_count;
    float* dist;
    int32_t *counts, *offsets, *cursor, *fill, *scratch;
    int32_t* slots[HIRA_MAX_LEVELS];
    void* cent_t[HIRA_MAX_LEVELS];
    int32_t* order[HIRA_MAX_LEVELS];
    size_t total;
};

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

// assign_mfma.hip
int assign_tiles(int K);
int launch_cent_prep(int dim, const float* cent, int K, int num_trees, const int32_t* fill, int bf,
                     void* tiles, float* cn2, hipStream_t s);
int launch_assign_mfma(int dim, const void* x, int n_c, size_t x_tree_stride, const void* tiles,
                       const float* cn2, int K, int num_trees, const int32_t* list,
                       const int32_t* list_count, size_t list_stride, int32_t* assign, float* dist,
                       hipStream_t s);

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
    if (assign_on_mfma(t)) {
        const size_t kpad = (size_t)assign_tiles((int)k1) * 16;
        b->cent_tiles = c.take<char>((size_t)T * kpad * D * 4);  // hi and lo halves, 2 bytes each
        b->cent_n2 = c.take<float>((size_t)T * kpad);
    }
    b->assign = c.take<int32_t>((size_t)T * n);
    b->placed = c.take<int32_t>((size_t)T * n);
    b->members = c.take<int32_t>((size_t)T * n);
    b->sorted = c.take<int32_t>((size_t)T * n);
    b->list = c.take<int32_t>((size_t)T * n);
    b->list_count = c.take<int32_t>((size_t)T);
    b->dist = c.take<float>((size_t)T * n);
    b->counts = c.take<int32_t>((size_t)T * k1);
    b->offsets = c.take<int32_t>((size_t)T * (k1 + 1));
    b->cursor = c.take<int32_t>((size_t)T * k1);
    b->fill = c.take<int32_t>((size_t)T * k1);
    b->scratch = c.take<int32_t>((size_t)T * (k1 + 1));
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
                         size_t list_stride, int32_t* assign, float* dist) {
#define HIRA_ASSIGN_CASE(N)                                                                   \
    case N:                                                                                   \
        hipLaunchKernelGGL((k_assign_simple<T, N>), grid, dim3(256), 0, s, x, n_c, x_stride,   \
                           cent, K, D, fill, bf, list, list_count, list_stride, assign, dist); \
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

    for (int l = 1; l < L; ++l) {
        const void* x = l == 1 ? keys_in : w.cent_t[l - 1];
        const int n_c = K[l - 1];
        const size_t xs = (size_t)n_c;  // rows per tree in x
        const int Kl = K[l];
        const int items_per_block = 4 * (64 / lpr) * kPPG;
        const dim3 g_assign(ceil_div(n_c, items_per_block), NT);
        const dim3 g_items(ceil_div(n_c, 256), NT);
        const dim3 g_cent(Kl, NT);

        // Trees with fewer items than rows (n_live): the items a tree does not hold are marked
        // placed before anything else, and every phase walks the list of the unplaced ones.
        const bool ragged = n_live != nullptr && l == 1;
        const int32_t* live = nullptr;
        const int32_t* live_cnt = nullptr;
        const size_t live_stride = ragged ? (size_t)n_c : 0;
        if (ragged) {
            hipLaunchKernelGGL(k_mark_absent, dim3(ceil_div(n_c > Kl ? n_c : Kl, 256), NT), dim3(256),
                               0, s, n_live, n_c, Kl, bf, w.placed, w.fill);
            fill_i32(w.list_count, (size_t)NT, 0, s);
            hipLaunchKernelGGL(k_collect_unplaced, g_items, dim3(256), 0, s, w.placed, n_c, w.list,
                               w.list_count);
            live = w.list;
            live_cnt = w.list_count;
        }
        hipLaunchKernelGGL((k_init_centroids<T>), g_cent, dim3(64), 0, s, x, n_c, xs, Kl, D,
                           seed + 7919ull * (uint64_t)l, w.cent_f32, ragged ? n_live : nullptr, bf);
        for (int it = 0; it < niter; ++it) {
            int rc;
            if (w.cent_tiles != nullptr) {
                rc = launch_cent_prep(D, w.cent_f32, Kl, NT, ragged ? w.fill : nullptr, bf,
                                      w.cent_tiles, w.cent_n2, s);
                if (rc == HIRA_OK)
                    rc = launch_assign_mfma(D, x, n_c, xs, w.cent_tiles, w.cent_n2, Kl, NT, live,
                                            live_cnt, live_stride, w.assign, w.dist, s);
            } else {
                rc = launch_assign<T>(lpr, g_assign, s, x, n_c, xs, w.cent_f32, Kl, D,
                                      ragged ? w.fill : nullptr, bf, live, live_cnt, live_stride,
                                      w.assign, w.dist);
            }
            if (rc != HIRA_OK) return rc;
            fill_i32(w.counts, (size_t)NT * Kl, 0, s);
            hipLaunchKernelGGL(k_bucket_count, g_items, dim3(256), 0, s, w.assign, n_c, live,
                               live_cnt, live_stride, Kl, w.counts);
            hipLaunchKernelGGL(k_scan, dim3(NT), dim3(256), 0, s, w.counts, Kl, w.offsets, w.cursor);
            hipLaunchKernelGGL(k_bucket_fill, g_items, dim3(256), 0, s, w.assign, n_c, live,
                               live_cnt, live_stride, Kl, w.cursor, w.members);
            hipLaunchKernelGGL(k_bucket_sort, g_cent, dim3(kSortThreads), 0, s, w.members, w.offsets, w.dist,
                               n_c, Kl, w.sorted);
            hipLaunchKernelGGL((k_mean<T>), g_cent, dim3(256), 0, s, x, xs, n_c, Kl, D, w.offsets,
                               w.sorted, nullptr, bf, w.cent_f32, nullptr);
        }
        // capacity packing
        if (!ragged) {  // (ragged: both were set up ahead of the Lloyd rounds)
            fill_i32(w.fill, (size_t)NT * Kl, 0, s);
            fill_i32(w.placed, (size_t)NT * n_c, 0, s);
        }
        fill_i32(w.slots[l], (size_t)NT * Kl * bf, -1, s);
        for (int r = 0; r < pack_rounds; ++r) {
            // (ragged: the first round walks the list of the items the trees hold, made above)
            const int32_t* list = r == 0 && !ragged ? nullptr : w.list;
            const int32_t* lcnt = r == 0 && !ragged ? nullptr : w.list_count;
            if (r > 0) {
                fill_i32(w.list_count, (size_t)NT, 0, s);
                hipLaunchKernelGGL(k_collect_unplaced, g_items, dim3(256), 0, s, w.placed, n_c,
                                   w.list, w.list_count);
            }
            int rc;
            if (w.cent_tiles != nullptr) {  // full centroids get an infinite norm: never nearest
                rc = launch_cent_prep(D, w.cent_f32, Kl, NT, w.fill, bf, w.cent_tiles, w.cent_n2, s);
                if (rc == HIRA_OK)
                    rc = launch_assign_mfma(D, x, n_c, xs, w.cent_tiles, w.cent_n2, Kl, NT, list,
                                            lcnt, (size_t)n_c, w.assign, w.dist, s);
            } else {
                rc = launch_assign<T>(lpr, g_assign, s, x, n_c, xs, w.cent_f32, Kl, D, w.fill, bf,
                                      list, lcnt, (size_t)n_c, w.assign, w.dist);
            }
            if (rc != HIRA_OK) return rc;
            fill_i32(w.counts, (size_t)NT * Kl, 0, s);
            hipLaunchKernelGGL(k_bucket_count, g_items, dim3(256), 0, s, w.assign, n_c, list, lcnt,
                               (size_t)n_c, Kl, w.counts);
            hipLaunchKernelGGL(k_scan, dim3(NT), dim3(256), 0, s, w.counts, Kl, w.offsets, w.cursor);
            hipLaunchKernelGGL(k_bucket_fill, g_items, dim3(256), 0, s, w.assign, n_c, list, lcnt,
                               (size_t)n_c, Kl, w.cursor, w.members);
            hipLaunchKernelGGL(k_bucket_sort, g_cent, dim3(kSortThreads), 0, s, w.members, w.offsets, w.dist,
                               n_c, Kl, w.sorted);
            hipLaunchKernelGGL(k_accept, g_cent, dim3(64), 0, s, w.sorted, w.offsets, n_c, Kl, bf,
                               w.fill, w.slots[l], w.placed);
        }
        hipLaunchKernelGGL(k_leftover, dim3(NT), dim3(kLeftThreads), 0, s, n_c, Kl, bf, w.fill, w.slots[l],
                           w.placed, w.scratch);
        // block centre = mean of what is in the block, rounded to the storage type
        hipLaunchKernelGGL((k_mean<T>), g_cent, dim3(64), 0, s, x, xs, n_c, Kl, D, nullptr, nullptr,
                           w.slots[l], bf, w.cent_f32, w.cent_t[l]);
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
                           t->size[l - 1], t->centers[l], (size_t)t->cap[l], t->size[l], bf, D,
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
        HIRA_CHECK_ARG(t->dim % 64 == 0 && t->num_levels >= 2 && t->keys8 && t->kscale && t->keps,
                       "the layout with an 8-bit shadow needs rows of a multiple of 64 columns, at "
                       "least two levels, and the keys8 / kscale / keps arrays");
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
                                    nullptr, 0, idx, dist2, s);
    } else {
        const int epl = dtype == HIRA_F32 ? 4 : 8;
        int lpr = 2;
        while (lpr * epl < dim) lpr <<= 1;
        const dim3 grid(ceil_div(n, 4 * (64 / lpr) * kPPG), num_trees);
        rc = dtype == HIRA_F32
                 ? launch_assign<float>(lpr, grid, s, x, n, (size_t)n, centers, m, dim, b.fill, 1,
                                        nullptr, nullptr, 0, idx, dist2)
                 : launch_assign<bf16_t>(lpr, grid, s, x, n, (size_t)n, centers, m, dim, b.fill, 1,
                                         nullptr, nullptr, 0, idx, dist2);
    }
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_LAUNCH("nearest-centre kernel");
    return HIRA_OK;
}
