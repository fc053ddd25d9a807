// Append-on-decode index update: m new keys/values per tree go into the existing tree.
//
// Replaces CUDAIndexer.update and its Triton kernels (indexer/cuda.py:544-701, 707-1231;
// kernels/triton_update_kernels.py:6-123, 126-235, 238-326) with one launch: one workgroup
// per tree walks that tree's new keys in insertion order, so slots, counts and radii need
// no global atomics and the result is reproducible.  For every key:
//   1. nearest level-1 node that still has a free child slot (exact fp32 L2 distance over
//      the nodes in use; full nodes are skipped before their centre is read) -- the
//      reference's nearest_l2 + valid-mask step;
//   2. the key takes the node's next slot (the reference's atomic slot reservation), the
//      node's radius grows to cover it (its atomic-max step) and every ancestor's radius is
//      re-inflated: R_a = max(R_a, ||c_child - c_a|| + r_child) (indexer/cuda.py:1200-1231);
//      centres never move, radii only grow, exactly as in the reference;
//   3. if no node has room the key opens a new level-1 node whose centre is the key itself
//      (the reference draws its new parents from the orphans, indexer/cuda.py:612-635); the
//      new node is attached the same way one level up: nearest level-2 node with a free
//      child slot, else a new level-2 node, ... up to the root level, which simply grows.
// Child counts stay authoritative (the reference over-counts on overflow and repairs the
// counters with an O(N D) rescan after every update, indexer/cuda.py:1233-1298).
//
// state (T, HIRA_MAX_LEVELS + 2) int32: [l] = slots of level l in use (l >= 1; the host keeps
// the maximum over the trees as size[l]), [HIRA_MAX_LEVELS] = keys inserted so far,
// [HIRA_MAX_LEVELS + 1] = error flag (1: a level ran out of capacity; the key was dropped).
// [0] (trees of two or more levels): every level-1 node with a lower index is full -- a lower
// bound that the search for a node with room starts from and raises as it learns more (0 is
// always valid; whoever lowers a count of a level-1 node from outside must lower it too).
#include "rows.h"
#include "threshold_kernel.h"

namespace hira {

constexpr int kUpdThreads = 256;

struct UpdateParams {
    void* keys;
    void* values;
    int32_t* perm;
    void* centers[HIRA_MAX_LEVELS];
    float* radii[HIRA_MAX_LEVELS];
    int32_t* counts[HIRA_MAX_LEVELS];
    int32_t cap[HIRA_MAX_LEVELS];
    int32_t num_levels, bf, dim, vdim, layout;  // layout: of the centers
    int32_t key_layout;
    int8_t* keys8;        // HIRA_TILE16_Q8: the 8-bit shadow of the keys
    const float* kscale;  //   its step per tree and channel
    float* keps;          //   largest error, in steps, among the keys of each level-1 node
    const void* new_keys;    // (T, m, D)
    const void* new_values;  // (T, m, Dv) or NULL
    int32_t m;
    int32_t chunk;  // windows: keys whose rows are in LDS at a time
    int32_t* state;
};

// a bound must survive the fp32 rounding of the sums that produced it
__device__ __forceinline__ float pad_up(float r) { return r > 0.0f ? r * (1.0f + 4.0f * 1.1920929e-7f) + 1e-30f : r; }

// Nearest node of level l (among nodes first .. used - 1; the ones before `first` are known to
// be full) with a free child slot; -1 if none.  Wave w scans nodes w, w+4, ...; a full node
// costs one count read.  Ties go to the lowest id.  *not_full (if given) receives the lowest
// index from `first` on whose node is not full (`used` if there is none).
constexpr int kCountsInFlight = 16;  // reads of child counts a lane has in flight
template <typename T>
__device__ int nearest_with_room(const UpdateParams& p, int tree, int l, int first, int used,
                                 const float* x, float* red_f, int* red_i, int* not_full,
                                 int* count_of = nullptr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int D = p.dim;
    const size_t base = (size_t)tree * p.cap[l];
    const int32_t* cnt = p.counts[l] + base;
    float best = INFINITY;
    int arg = -1, argc = 0;  // the best node so far and its child count
    int low = used;  // lowest index of a node that is not full, among those I have seen
    for (int nb = (first & ~63) + wave * 64; nb < used; nb += kCountsInFlight * 4 * 64) {
        // the reads of the child counts in flight together (a wave's nodes still come in
        // increasing order): one trip to memory for 4096 nodes
        int c4[kCountsInFlight];
#pragma unroll
        for (int u = 0; u < kCountsInFlight; ++u) {
            const int n = nb + u * 4 * 64 + lane;
            c4[u] = n < used ? cnt[n] : p.bf;
        }
#pragma unroll
        for (int u = 0; u < kCountsInFlight; ++u) {
            if (nb + u * 4 * 64 >= used) break;  // uniform
            if (c4[u] < p.bf) low = min(low, nb + u * 4 * 64 + lane);
            // a node in use with a free slot; count 0 marks a pad slot, which is not a node yet
            unsigned long long bal = __ballot(c4[u] > 0 && c4[u] < p.bf);
            while (bal != 0ull) {  // uniform in the wave
                const int src = __ffsll((long long)bal) - 1;
                const int node = nb + u * 4 * 64 + src;
                const int node_c = __shfl(c4[u], src, 64);
                bal &= bal - 1ull;
                float ss = 0.0f;
                for (int j = lane; j < D; j += 64) {
                    const float df = x[j] - load_elem<T>(p.centers[l], base * D + elem_index(p.layout, D, (size_t)node, j));
                    ss += df * df;
                }
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) ss += __shfl_xor(ss, off, 64);
                if (ss < best) {
                    best = ss;
                    arg = node;
                    argc = node_c;
                }
            }
        }
    }
    __syncthreads();
    if (not_full != nullptr) {  // uniform
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) low = min(low, __shfl_xor(low, off, 64));
        if (lane == 0) red_i[wave] = low;
        __syncthreads();
        if (threadIdx.x == 0) *not_full = max(min(min(red_i[0], red_i[1]), min(red_i[2], red_i[3])), first);
        __syncthreads();
    }
    if (lane == 0) {
        red_f[wave] = best;
        red_i[wave] = arg;
    }
    __syncthreads();
    float b = red_f[0];
    int a = red_i[0], aw_of = 0;
#pragma unroll
    for (int w = 1; w < 4; ++w) {
        const float bw = red_f[w];
        const int aw = red_i[w];
        if (aw >= 0 && (a < 0 || bw < b || (bw == b && aw < a))) {
            b = bw;
            a = aw;
            aw_of = w;
        }
    }
    __syncthreads();
    if (count_of != nullptr) {  // uniform: the child count of the chosen node, as the scan read it
        if (lane == 0) red_i[wave] = argc;
        __syncthreads();
        *count_of = red_i[aw_of];
        __syncthreads();
    }
    return a;
}

// One key of the window, placed the general way: key i of the tree's new keys.
//   sm: 2 D floats (the key, the centre of a node being attached upwards).
template <typename T>
__device__ void update_one_key(const UpdateParams& p, const int tree, const int i, float* sm, float* red_f,
                               int* red_i, float* s_dist, float* s_rad) {
    float* x = sm;              // (D) the new key, fp32
    float* cbuf = sm + p.dim;   // (D) centre of the node being attached upwards
    const int t = threadIdx.x;
    const int D = p.dim, Dv = p.vdim, L = p.num_levels, bf = p.bf;
    int32_t* st = p.state + (size_t)tree * (HIRA_MAX_LEVELS + 2);
    const size_t base0 = (size_t)tree * p.cap[0];

    const size_t src = ((size_t)tree * p.m + i) * D;
    for (int j = t; j < D; j += kUpdThreads) x[j] = load_elem<T>(p.new_keys, src + j);
    __syncthreads();
    const int position = st[HIRA_MAX_LEVELS];

    long long slot = -1;  // key slot
    int node1 = -1;       // level-1 node that took the key (L >= 2)
    int count1 = 0;       // keys it held before
    if (L == 1) {
        slot = position < p.cap[0] ? position : -1;
    } else {
        node1 = nearest_with_room<T>(p, tree, 1, min(max(st[0], 0), st[1]), st[1], x, red_f, red_i, &st[0],
                                         &count1);
        if (node1 < 0) {
            // ---- open a new level-1 node; attach it upwards -----------------------
            // child_c = centre of the node being attached (the key itself at level 1)
            for (int j = t; j < D; j += kUpdThreads) cbuf[j] = x[j];
            __syncthreads();
            int lvl = 1;          // level of the node that needs a parent
            int parent = -1;      // node of level lvl+1 that takes it
            int opened_top = 0;   // levels 1..opened_top get a brand-new node
            // find the lowest level that has a parent with room
            while (true) {
                if (lvl == L - 1) {  // the root level grows
                    parent = -1;
                    break;
                }
                parent = nearest_with_room<T>(p, tree, lvl + 1, 0, st[lvl + 1], cbuf, red_f, red_i, nullptr);
                if (parent >= 0) break;
                ++lvl;
            }
            opened_top = lvl;
            // index of the new node at level opened_top
            long long idx;
            if (parent >= 0) {
                idx = (long long)parent * bf + p.counts[opened_top + 1][(size_t)tree * p.cap[opened_top + 1] + parent];
            } else {
                idx = st[opened_top];
            }
            // every new node below it is the first child of the new node above
            bool fits = true;
            long long id = idx;
            for (int l = opened_top; l >= 1; --l) {
                if (id >= p.cap[l]) fits = false;
                id *= bf;
            }
            if (id >= p.cap[0]) fits = false;
            __syncthreads();  // everybody has read the counters the writes below change
            if (!fits) {
                if (t == 0) st[HIRA_MAX_LEVELS + 1] = 1;
                __syncthreads();
                return;  // uniform: the key is dropped, the host sees the flag
            }
            id = idx;
            for (int l = opened_top; l >= 1; --l) {
                const size_t bl = (size_t)tree * p.cap[l];
                for (int j = t; j < D; j += kUpdThreads)
                    store_elem<T>(p.centers[l], bl * D + elem_index(p.layout, D, (size_t)id, j), x[j]);
                if (t == 0) {
                    p.radii[l][bl + id] = 0.0f;
                    p.counts[l][bl + id] = (l == 1) ? 0 : 1;  // level 1 gets its key below
                    if (id + 1 > st[l]) st[l] = (int)(id + 1);
                }
                id *= bf;
            }
            if (t == 0 && parent >= 0)
                p.counts[opened_top + 1][(size_t)tree * p.cap[opened_top + 1] + parent] += 1;
            __syncthreads();
            node1 = (int)(id / bf);  // the new level-1 node (id is now its first key slot)
            count1 = 0;
        }
        // the key takes the next slot of node1
        // (a node found by the scan: the count the scan read; a node just opened: none)
        const size_t b1 = (size_t)tree * p.cap[1];
        const int c = count1;
        slot = (long long)node1 * bf + c;
        __syncthreads();
        if (t == 0) p.counts[1][b1 + node1] = c + 1;
    }
    if (slot < 0 || slot >= p.cap[0]) {
        if (t == 0) st[HIRA_MAX_LEVELS + 1] = 1;
        __syncthreads();
        return;
    }
    // ---- write key, value, perm -------------------------------------------------------
    {
        const T* dummy = nullptr;
        (void)dummy;
        for (int j = t; j < D; j += kUpdThreads)
            store_elem<T>(p.keys, base0 * D + elem_index(p.key_layout, D, (size_t)slot, j), x[j]);
        if (p.keys8 != nullptr) {
            // the key's 8-bit shadow with the tree's steps; a component beyond +-127 steps
            // clips, and the node's error bound then covers it
            float worst = 0.0f;
            for (int j = t; j < D; j += kUpdThreads) {
                const float u = x[j] / p.kscale[(size_t)tree * D + j];
                const float r = fminf(fmaxf(rintf(u), -127.0f), 127.0f);
                worst = fmaxf(worst, fabsf(u - r));
                p.keys8[base0 * D + shadow_index(D, (size_t)slot, j)] = (int8_t)(int)r;
            }
            worst = wave_max(worst);
            if ((t & 63) == 0) red_f[t >> 6] = worst;
            __syncthreads();
            if (t == 0) {
                float* e = p.keps + (size_t)tree * p.cap[1] + node1;
                const float w = fmaxf(fmaxf(red_f[0], red_f[1]), fmaxf(red_f[2], red_f[3]));
                // a node that just opened holds no other key: its bound starts here
                const bool fresh = count1 == 0;
                *e = fresh ? w : fmaxf(*e, w);
            }
            __syncthreads();
        }
        if (p.new_values && p.values) {
            const size_t vs = ((size_t)tree * p.m + i) * Dv;
            for (int j = t; j < Dv; j += kUpdThreads)
                store_elem<T>(p.values, (base0 + slot) * Dv + j, load_elem<T>(p.new_values, vs + j));
        }
        if (t == 0) {
            p.perm[base0 + slot] = position;
            st[HIRA_MAX_LEVELS] = position + 1;
            if (L == 1 && slot + 1 > st[0]) st[0] = (int)(slot + 1);
        }
    }
    // ---- radii: the leaf parent covers the key, every ancestor covers its child.  The
    // distances of all levels are taken at once (a wave per level), then one thread walks
    // the chain R_l = max(R_l, d_l + R_{l-1}). ---------------------------------------------
    if (L >= 2) {
        const int lane = t & 63;
        for (int l = 1 + (t >> 6); l < L; l += kUpdThreads / 64) {  // uniform in the wave
            size_t child = (size_t)node1;  // node of level l - 1 on the key's path (l >= 2)
            for (int i = 2; i < l; ++i) child /= (size_t)bf;
            const size_t node = l == 1 ? (size_t)node1 : child / (size_t)bf;
            const size_t bl = (size_t)tree * p.cap[l], bc = (size_t)tree * p.cap[l - 1];
            const float rad_now = p.radii[l][bl + node];  // (asked for with the centres)
            float ss = 0.0f;
            for (int j = lane; j < D; j += 64) {
                const float a =
                    l == 1 ? x[j]
                           : load_elem<T>(p.centers[l - 1], bc * D + elem_index(p.layout, D, child, j));
                const float b = load_elem<T>(p.centers[l], bl * D + elem_index(p.layout, D, node, j));
                ss += (a - b) * (a - b);
            }
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) ss += __shfl_xor(ss, off, 64);
            if (lane == 0) {
                s_dist[l] = sqrtf(ss);
                s_rad[l] = rad_now;
            }
        }
        __syncthreads();
        if (t == 0) {
            size_t node = (size_t)node1;
            float r_child = 0.0f;
            for (int l = 1; l < L; ++l) {
                const float rn = fmaxf(s_rad[l], pad_up(s_dist[l] + r_child));
                if (rn != s_rad[l]) p.radii[l][(size_t)tree * p.cap[l] + node] = rn;
                r_child = rn;
                node /= (size_t)bf;
            }
        }
    }
    __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(kUpdThreads) void k_update(const UpdateParams p) {
    extern __shared__ float sm[];
    __shared__ float red_f[4];
    __shared__ int red_i[4];
    __shared__ float s_dist[HIRA_MAX_LEVELS], s_rad[HIRA_MAX_LEVELS];
    for (int i = 0; i < p.m; ++i)
        update_one_key<T>(p, (int)blockIdx.x, i, sm, red_f, red_i, s_dist, s_rad);
}

// An append of a few keys per tree and the thresholds of a decode step in one launch: the first
// `trees` workgroups append (their first kUpdThreads threads; the others leave at once, and a
// barrier counts only the waves still there), the ones behind them take a head each.  The two
// halves share nothing: the sample is not touched by the append.
template <typename T, int E>
__global__ __launch_bounds__(kTauThreads) void k_update_threshold(
    const UpdateParams p, const int trees, const T* __restrict__ samples, const int S,
    const T* __restrict__ q, const int32_t* __restrict__ tree_q_off,
    const int32_t* __restrict__ tree_q_heads, const int group_size, const int method, const int k,
    float* __restrict__ tau) {
    extern __shared__ float sm[];
    __shared__ float red_f[4];
    __shared__ int red_i[4];
    __shared__ float s_dist[HIRA_MAX_LEVELS], s_rad[HIRA_MAX_LEVELS];
    if ((int)blockIdx.x < trees) {  // uniform in the workgroup
        if (threadIdx.x >= kUpdThreads) return;
        for (int i = 0; i < p.m; ++i)
            update_one_key<T>(p, (int)blockIdx.x, i, sm, red_f, red_i, s_dist, s_rad);
        return;
    }
    threshold_block<T, E>(samples, S, p.dim, q, tree_q_off, tree_q_heads, group_size, trees, method, k,
                          tau, (int)blockIdx.x - trees);
}

// The general way as a call (the kernel below needs it now and then: its loop stays small, and the
// compiler keeps the loop's values in registers instead of asking for them again every key).
template <typename T>
__device__ __attribute__((noinline)) void update_one_key_called(const UpdateParams& p, const int tree, const int i,
                                                              float* sm, float* red_f, int* red_i, float* s_dist,
                                                              float* s_rad) {
    update_one_key<T>(p, tree, i, sm, red_f, red_i, s_dist, s_rad);
}

// ---- windows of several keys ---------------------------------------------------------------
// Placing a key the general way costs a handful of dependent trips to memory (child counts,
// the centres of the nodes with room, the ancestors' centres and radii): 4-5 us a key, one key
// after the other.  But the nodes with room are few -- the tail nodes opened by earlier appends,
// what a rebuilt subtree left free -- and between two keys of a window only the window itself
// changes them.  So a workgroup that has a window to place reads them ONCE into LDS (ids, child
// counts, centres, radii, and for every ancestor on their paths its radius and the distance
// between consecutive centres, which never changes) and then places key after key from LDS:
// distances to every candidate, the nearest (ties: the lowest id, as the general way), next slot,
// radii along the path; memory only sees stores.  A key that finds no candidate goes the general
// way (it opens a node), after which the candidates are read again.  A tree with more nodes
// with room than the list holds goes the general way altogether.  Same placement, slots and
// radii as key by key (the replaced kernels: kernels/triton_update_kernels.py:85-123 nearest
// centre for a whole window at once, :126-235 slots, :238-326 radii).
constexpr int kCandMax = 48;

struct WindowLds {
    int n;                                  // candidates listed (may exceed kCandMax: then unusable)
    int low;                                // lowest level-1 node from `first` on that is not full
    int id[kCandMax];                       // level-1 node
    int cnt[kCandMax];                      // its child count (bf: full by now)
    float rad[kCandMax];                    // its radius
    float dist[kCandMax];                   // squared distance of the current key
    int anc_id[HIRA_MAX_LEVELS][kCandMax];      // [l][c]: c's ancestor at level l
    int anc_rep[HIRA_MAX_LEVELS][kCandMax];     // [l][c]: the first candidate with the same ancestor at level l
    float anc_rad[HIRA_MAX_LEVELS][kCandMax];   // [l][rep]: that ancestor's radius
    float anc_step[HIRA_MAX_LEVELS][kCandMax];  // [l][c]: distance between c's ancestors at levels l-1 and l
    int best;
};

// level-l ancestor of level-1 node `node1` (l >= 1)
__device__ __forceinline__ size_t ancestor_of(size_t node1, int l, int bf) {
    for (int i = 1; i < l; ++i) node1 /= (size_t)bf;
    return node1;
}

// Reads the tree's level-1 nodes with room into LDS.  cen: (kCandMax, D) floats.  Returns false
// (uniform) when there are more than the list holds.
template <typename T>
__device__ bool window_candidates(const UpdateParams& p, const int tree, WindowLds& w, float* cen) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int D = p.dim, L = p.num_levels, bf = p.bf;
    int32_t* st = p.state + (size_t)tree * (HIRA_MAX_LEVELS + 2);
    const int used = st[1], first = min(max(st[0], 0), used);
    const size_t b1 = (size_t)tree * p.cap[1];
    __syncthreads();  // (everybody has read the state; earlier users of the list are done)
    if (t == 0) {
        w.n = 0;
        w.low = used;
    }
    __syncthreads();
    for (int nb = first & ~63; nb < used; nb += kUpdThreads) {  // uniform
        const int n = nb + t;
        const int c = (n >= first && n < used) ? p.counts[1][b1 + n] : bf;
        if (c < bf) atomicMin(&w.low, n);
        // a node in use with a free slot; count 0 marks a pad slot, which is not a node yet
        const bool room = c > 0 && c < bf;
        const unsigned long long bal = __ballot(room);
        int at = 0;
        if (lane == 0 && bal != 0ull) at = atomicAdd(&w.n, __popcll(bal));
        at = __shfl(at, 0, 64) + __popcll(bal & ((1ull << lane) - 1ull));
        if (room && at < kCandMax) {
            w.id[at] = n;
            w.cnt[at] = c;
        }
    }
    __syncthreads();
    const int nc = w.n;
    if (t == 0) st[0] = max(w.low, first);
    if (nc > kCandMax) return false;
    // (the order in which the waves listed their nodes does not matter: ties between candidates
    // are decided by the node's id)
    for (int c = wave; c < nc; c += kUpdThreads / 64) {  // uniform in the wave
        const size_t node = (size_t)w.id[c];
        for (int j = lane; j < D; j += 64)
            cen[(size_t)c * D + j] = load_elem<T>(p.centers[1], b1 * D + elem_index(p.layout, D, node, j));
        if (lane == 0) w.rad[c] = p.radii[1][b1 + node];
        for (int l = 2; l < L; ++l) {
            const size_t child = ancestor_of(node, l - 1, bf), anc = child / (size_t)bf;
            const size_t bl = (size_t)tree * p.cap[l], bc = (size_t)tree * p.cap[l - 1];
            float ss = 0.0f;
            for (int j = lane; j < D; j += 64) {
                const float a = load_elem<T>(p.centers[l - 1], bc * D + elem_index(p.layout, D, child, j));
                const float b = load_elem<T>(p.centers[l], bl * D + elem_index(p.layout, D, anc, j));
                ss += (a - b) * (a - b);
            }
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) ss += __shfl_xor(ss, off, 64);
            if (lane == 0) {
                w.anc_id[l][c] = (int)anc;
                w.anc_step[l][c] = sqrtf(ss);
                w.anc_rad[l][c] = p.radii[l][bl + anc];  // (read where c is its ancestor's first candidate)
            }
        }
    }
    __syncthreads();
    for (int k = t; k < nc * HIRA_MAX_LEVELS; k += kUpdThreads) {
        const int c = k % nc, l = k / nc;
        if (l < 2 || l >= L) continue;
        const int anc = w.anc_id[l][c];
        int rep = c;
        for (int o = 0; o < c; ++o)
            if (w.anc_id[l][o] == anc) {
                rep = o;
                break;
            }
        w.anc_rep[l][c] = rep;
    }
    __syncthreads();
    return true;
}

// sum over the wave, the same value in every lane (data-path moves inside rows of 16 lanes, then
// the four rows' sums: no trip through LDS, a tenth of the latency of six shuffles)
__device__ __forceinline__ float wave_sum_dpp(float v) {
    auto mv = [](float x, int ctrl_sel) {
        const int xi = __float_as_int(x);
        int r;
        if (ctrl_sel == 0) r = __builtin_amdgcn_update_dpp(0, xi, 0xB1, 0xF, 0xF, false);        // lanes 1 0 3 2
        else if (ctrl_sel == 1) r = __builtin_amdgcn_update_dpp(0, xi, 0x4E, 0xF, 0xF, false);   // lanes 2 3 0 1
        else if (ctrl_sel == 2) r = __builtin_amdgcn_update_dpp(0, xi, 0x141, 0xF, 0xF, false);  // halves of 8 mirrored
        else r = __builtin_amdgcn_update_dpp(0, xi, 0x140, 0xF, 0xF, false);                     // the row mirrored
        return __int_as_float(r);
    };
    v += mv(v, 0);
    v += mv(v, 1);
    v += mv(v, 2);
    v += mv(v, 3);
    const int vi = __float_as_int(v);
    // (added up in the order of the butterfly of shuffles that the general way uses: the two
    // kernels must agree on a distance to the last bit)
    return (__int_as_float(__builtin_amdgcn_readlane(vi, 0)) + __int_as_float(__builtin_amdgcn_readlane(vi, 16))) +
           (__int_as_float(__builtin_amdgcn_readlane(vi, 32)) + __int_as_float(__builtin_amdgcn_readlane(vi, 48)));
}

template <typename T>
__global__ __launch_bounds__(kUpdThreads) void k_update_window(const UpdateParams p) {
    extern __shared__ float sm[];  // 2 D floats of the general way, kCandMax centres, a chunk of rows
    __shared__ float red_f[4];
    __shared__ int red_i[4];
    __shared__ float s_dist[HIRA_MAX_LEVELS], s_rad[HIRA_MAX_LEVELS];
    __shared__ WindowLds w;
    __shared__ int s_slot[16], s_node[16];  // where the chunk's keys went (slot < 0: not placed yet)
    __shared__ int s_done;                   // keys of the chunk dealt with so far
    const int tree = blockIdx.x;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int D = p.dim, Dv = p.vdim, L = p.num_levels, bf = p.bf;
    float* cen = sm + 2 * (size_t)D;
    int32_t* st = p.state + (size_t)tree * (HIRA_MAX_LEVELS + 2);
    const size_t base0 = (size_t)tree * p.cap[0], b1 = (size_t)tree * p.cap[1];
    bool usable = L >= 2 && window_candidates<T>(p, tree, w, cen);  // false: the tree's keys go
                                                                    // the general way, all of them
    // The window's rows come into LDS a chunk of keys at a time.  Wave 0 then places key after key
    // from the list, on its own: no barrier, nothing asked of memory (it carries the number of keys
    // inserted so far; device memory only sees stores) -- until the chunk ends or a key finds no
    // candidate.  Then the workgroup copies the placed keys' rows to their slots, sends the key
    // without a candidate the general way, and wave 0 carries on.
    const bool with_values = p.new_values != nullptr && p.values != nullptr;
    const int chunk = p.chunk;
    float* xs = cen + (size_t)kCandMax * D;  // (chunk, D) keys
    float* vs = xs + (size_t)chunk * D;      // (chunk, Dv) values
    for (int i0 = 0; i0 < p.m; i0 += chunk) {  // uniform
        const int nk = min(chunk, p.m - i0);
        const size_t r0 = (size_t)tree * p.m + i0;
        __syncthreads();  // (the chunk before is done with its rows)
        for (int e = t; e < nk * D; e += kUpdThreads) xs[e] = load_elem<T>(p.new_keys, r0 * D + e);
        if (with_values)
            for (int e = t; e < nk * Dv; e += kUpdThreads) vs[e] = load_elem<T>(p.new_values, r0 * Dv + e);
        if (t == 0) s_done = 0;
        __syncthreads();
        int k = 0;
        while (k < nk) {  // uniform
            if (!usable) {
                for (; k < nk; ++k) update_one_key_called<T>(p, tree, i0 + k, sm, red_f, red_i, s_dist, s_rad);
                break;
            }
            if (wave == 0) {
                int position = st[HIRA_MAX_LEVELS];
                int kk = k;
                for (; kk < nk; ++kk) {
                    const float* x = xs + (size_t)kk * D;
                    const int nc = w.n;
                    float best = INFINITY;
                    int b = -1, best_id = 0x7fffffff;
                    for (int c = 0; c < nc; ++c) {  // uniform
                        if (w.cnt[c] >= bf) continue;
                        float ss = 0.0f;
                        for (int j = lane; j < D; j += 64) {
                            const float df = x[j] - cen[(size_t)c * D + j];
                            ss += df * df;
                        }
                        ss = wave_sum_dpp(ss);
                        const int id = w.id[c];
                        if (ss < best || (ss == best && id < best_id)) {  // ties: the lowest node
                            best = ss;
                            b = c;
                            best_id = id;
                        }
                    }
                    if (b < 0) break;  // no node has room: the workgroup sends this key the general way
                    const int node1 = best_id, count1 = w.cnt[b];
                    const int slot = node1 * bf + count1;
                    if (lane == 0) {
                        s_slot[kk] = slot;
                        s_node[kk] = node1;
                        w.cnt[b] = count1 + 1;
                        p.counts[1][b1 + node1] = count1 + 1;
                        // radii along the key's path: the leaf parent covers the key, every
                        // ancestor its child
                        float r_child = fmaxf(w.rad[b], pad_up(sqrtf(best)));
                        if (r_child != w.rad[b]) {
                            w.rad[b] = r_child;
                            p.radii[1][b1 + node1] = r_child;
                        }
                        for (int l = 2; l < L; ++l) {
                            const int rep = w.anc_rep[l][b];
                            const float have = w.anc_rad[l][rep];
                            const float rn = fmaxf(have, pad_up(w.anc_step[l][b] + r_child));
                            if (rn != have) {
                                w.anc_rad[l][rep] = rn;
                                p.radii[l][(size_t)tree * p.cap[l] + w.anc_id[l][b]] = rn;
                            }
                            r_child = rn;
                        }
                        p.perm[base0 + slot] = position;
                    }
                    ++position;
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");  // (lane 0's list updates
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");  //  before the next key reads)
                }
                if (lane == 0) {
                    st[HIRA_MAX_LEVELS] = position;
                    s_done = kk;
                }
            }
            __syncthreads();
            const int kd = s_done;
            // ---- the rows of the keys placed from the list: keys k .. kd - 1 ---------------------
            for (int q = k; q < kd; ++q) {  // uniform
                const size_t slot = (size_t)s_slot[q];
                const float* x = xs + (size_t)q * D;
                for (int j = t; j < D; j += kUpdThreads)
                    store_elem<T>(p.keys, base0 * D + elem_index(p.key_layout, D, slot, j), x[j]);
                if (p.keys8 != nullptr) {
                    // the key's 8-bit shadow with the tree's steps; a component beyond +-127 steps
                    // clips, and the node's error bound then covers it
                    float worst = 0.0f;
                    for (int j = t; j < D; j += kUpdThreads) {
                        const float u = x[j] / p.kscale[(size_t)tree * D + j];
                        const float r = fminf(fmaxf(rintf(u), -127.0f), 127.0f);
                        worst = fmaxf(worst, fabsf(u - r));
                        p.keys8[base0 * D + shadow_index(D, slot, j)] = (int8_t)(int)r;
                    }
                    worst = wave_max(worst);
                    if (lane == 0) red_f[wave] = worst;
                    __syncthreads();
                    if (t == 0) {
                        float* e = p.keps + b1 + s_node[q];
                        *e = fmaxf(*e, fmaxf(fmaxf(red_f[0], red_f[1]), fmaxf(red_f[2], red_f[3])));
                    }
                    __syncthreads();
                }
                if (with_values)
                    for (int j = t; j < Dv; j += kUpdThreads)
                        store_elem<T>(p.values, (base0 + slot) * Dv + j, vs[(size_t)q * Dv + j]);
            }
            k = kd;
            if (k < nk) {
                // key k found no node with room: it opens one, the general way (which reads device
                // memory that the keys before it wrote: the barrier above was a full one); then
                // the list is read again
                update_one_key_called<T>(p, tree, i0 + k, sm, red_f, red_i, s_dist, s_rad);
                usable = window_candidates<T>(p, tree, w, cen);
                ++k;
            }
        }
    }
}

}  // namespace hira

using namespace hira;

// hira_update's checks and the kernels' arguments; *window: the launch takes the window kernel
static int update_arguments(const HiraTree* tree, const void* new_keys, const void* new_values,
                            int32_t m, int32_t* state, UpdateParams* out, bool* window,
                            size_t* smem, size_t* smem_w) {
    HIRA_CHECK_ARG(tree != nullptr && new_keys != nullptr && state != nullptr,
                   "tree / new_keys / state missing");
    HIRA_CHECK_ARG(tree->dtype == HIRA_F32 || tree->dtype == HIRA_BF16, "dtype %d", tree->dtype);
    HIRA_CHECK_ARG(tree->num_levels >= 1 && tree->num_levels <= HIRA_MAX_LEVELS, "num_levels %d",
                   tree->num_levels);
    HIRA_CHECK_ARG(tree->bf >= 1 && tree->bf <= 64, "branching factor %d", tree->bf);
    HIRA_CHECK_ARG(m >= 0, "m = %d", m);
    HIRA_CHECK_ARG(tree->keys && tree->perm, "keys / perm missing");
    HIRA_CHECK_ARG((new_values == nullptr) || tree->values != nullptr,
                   "values given but the index holds none");
    UpdateParams& p = *out;
    memset(&p, 0, sizeof(p));
    *window = false;
    *smem = *smem_w = 0;
    if (m == 0) return HIRA_OK;  // nothing to append: the callers launch nothing for it
    p.keys = tree->keys;
    p.values = tree->values;
    p.perm = tree->perm;
    for (int l = 0; l < HIRA_MAX_LEVELS; ++l) {
        p.centers[l] = tree->centers[l];
        p.radii[l] = tree->radii[l];
        p.counts[l] = tree->counts[l];
        p.cap[l] = tree->cap[l];
    }
    for (int l = 1; l < tree->num_levels; ++l)
        HIRA_CHECK_ARG(p.centers[l] && p.radii[l] && p.counts[l], "level %d arrays missing", l);
    p.num_levels = tree->num_levels;
    p.bf = tree->bf;
    p.dim = tree->dim;
    p.vdim = tree->vdim;
    p.layout = center_layout_of(tree->layout);
    p.key_layout = key_layout_of(tree->layout);
    if (tree->layout == HIRA_TILE16_Q8) {
        HIRA_CHECK_ARG(tree->keys8 && tree->kscale && tree->keps && tree->num_levels >= 2,
                       "keys8 / kscale / keps missing");
        p.keys8 = tree->keys8;
        p.kscale = tree->kscale;
        p.keps = tree->keps;
    }
    p.new_keys = new_keys;
    p.new_values = new_values;
    p.m = m;
    p.state = state;
    *smem = 2 * (size_t)tree->dim * sizeof(float);
    // windows of a few keys and more: the nodes with room are read into LDS once (where they fit:
    // 48 centres of up to 256 columns beside the rest)
    const size_t cand_bytes = *smem + (size_t)kCandMax * tree->dim * sizeof(float);
    const size_t row_bytes = (size_t)(tree->dim + tree->vdim) * sizeof(float);
    int chunk = cand_bytes + row_bytes <= 60 * 1024 ? (int)((60 * 1024 - cand_bytes) / row_bytes) : 0;
    chunk = chunk > 16 ? 16 : chunk;
    *window = m >= 4 && tree->num_levels >= 2 && chunk >= 1;
    *smem_w = cand_bytes + (size_t)chunk * row_bytes;
    p.chunk = chunk;
    return HIRA_OK;
}

/* see include/hira_hip.h */
extern "C" int hira_update(const HiraTree* tree, const void* new_keys, const void* new_values,
                           int32_t m, int32_t* state, void* stream) {
    UpdateParams p;
    bool window;
    size_t smem, smem_w;
    if (const int rc = update_arguments(tree, new_keys, new_values, m, state, &p, &window, &smem, &smem_w))
        return rc;
    if (m == 0) return HIRA_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (window) {
        if (tree->dtype == HIRA_F32)
            hipLaunchKernelGGL(k_update_window<float>, dim3(tree->num_trees), dim3(kUpdThreads), smem_w, s, p);
        else
            hipLaunchKernelGGL(k_update_window<bf16_t>, dim3(tree->num_trees), dim3(kUpdThreads), smem_w, s, p);
    } else if (tree->dtype == HIRA_F32) {
        hipLaunchKernelGGL(k_update<float>, dim3(tree->num_trees), dim3(kUpdThreads), smem, s, p);
    } else {
        hipLaunchKernelGGL(k_update<bf16_t>, dim3(tree->num_trees), dim3(kUpdThreads), smem, s, p);
    }
    HIRA_CHECK_LAUNCH("update kernel");
    return HIRA_OK;
}

namespace hira {
template <typename T>
static void launch_update_threshold(int e, const UpdateParams& p, const HiraTree* tree, size_t smem,
                                    hipStream_t s, const void* samples, int S, const HiraQuery* qu,
                                    int method, int k, float* tau) {
    const T* x = static_cast<const T*>(samples);
    const T* q = static_cast<const T*>(qu->q);
    const dim3 grid(tree->num_trees + qu->num_q_heads), block(kTauThreads);
#define HIRA_UT_LAUNCH(E)                                                                         \
    hipLaunchKernelGGL((k_update_threshold<T, E>), grid, block, smem, s, p, tree->num_trees, x, S, \
                       q, qu->tree_q_off, qu->tree_q_heads, qu->group_size, method, k, tau)
    if (e == 1) HIRA_UT_LAUNCH(1);
    else if (e == 2) HIRA_UT_LAUNCH(2);
    else HIRA_UT_LAUNCH(4);
#undef HIRA_UT_LAUNCH
}
}  // namespace hira

/* see include/hira_hip.h */
extern "C" int hira_update_threshold(const HiraTree* tree, const void* new_keys,
                                     const void* new_values, int32_t m, int32_t* state,
                                     const void* samples, int32_t num_samples,
                                     const HiraQuery* query, int32_t method, int32_t k,
                                     float* tau_out, void* stream) {
    UpdateParams p;
    bool window;
    size_t smem, smem_w;
    if (const int rc = update_arguments(tree, new_keys, new_values, m, state, &p, &window, &smem, &smem_w))
        return rc;
    if (const int rc = check_threshold_arguments(samples, tree->dtype, tree->num_trees, num_samples,
                                                 tree->dim, query, method, k, tau_out))
        return rc;
    if (m == 0 || window) {
        // nothing to append, or a window that takes the window kernel: the two launches
        if (const int rc = hira_update(tree, new_keys, new_values, m, state, stream)) return rc;
        return hira_threshold(samples, tree->dtype, tree->num_trees, num_samples, tree->dim, query,
                              method, k, tau_out, stream);
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const int e = threshold_sort_registers(num_samples);
    if (tree->dtype == HIRA_F32)
        launch_update_threshold<float>(e, p, tree, smem, s, samples, num_samples, query, method, k, tau_out);
    else
        launch_update_threshold<bf16_t>(e, p, tree, smem, s, samples, num_samples, query, method, k, tau_out);
    HIRA_CHECK_LAUNCH("update + threshold kernel");
    return HIRA_OK;
}
