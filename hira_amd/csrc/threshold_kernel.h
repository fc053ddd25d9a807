// The threshold kernel's device code (see threshold.hip for what it computes), as the work of
// one workgroup: the kernel of hira_threshold runs it in every workgroup, the kernel of
// hira_update_threshold in the workgroups behind those that append.
#pragma once
#include "common.hip.h"

namespace hira {

constexpr int kTauThreads = 1024;
constexpr int kTauWaves = kTauThreads / 64;
constexpr int kTauMaxSamples = 4096;
constexpr int kTauRows = 16;  // sample rows a lane group has in flight

__device__ __forceinline__ float tau_block_reduce(float v, bool is_max, float* s_red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float o = __shfl_xor(v, off, 64);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    if (lane == 0) s_red[wave] = v;
    __syncthreads();
    float r = s_red[0];
#pragma unroll
    for (int w = 1; w < kTauWaves; ++w) r = is_max ? fmaxf(r, s_red[w]) : r + s_red[w];
    return r;
}

constexpr int kTauSorters = 256;  // threads that hold the scores during the sort

// The value that lane ^ J holds: moves inside a row of 16 lanes (J < 16) are data-path moves,
// only J = 16 and 32 go through the LDS crossbar.  rot4_first: which rotation by 4 brings lane ^ 4.
template <int J>
__device__ __forceinline__ float tau_partner(float v, bool rot4_first) {
    if constexpr (J >= 16) {
        return __shfl_xor(v, J, 64);
    } else if constexpr (J == 8) {
        return dpp_move<0x128>(v);  // row rotate by 8
    } else if constexpr (J == 4) {
        const float a = dpp_move<0x124>(v), b = dpp_move<0x12C>(v);  // by 4, by 12
        return rot4_first ? a : b;
    } else if constexpr (J == 2) {
        return dpp_move<0x4E>(v);  // quad [2,3,0,1]
    } else {
        return dpp_move<0xB1>(v);  // quad [1,0,3,2]
    }
}

// One merge stage (stretches of LEN, partners J = LEN/2 .. 1) of a wave's 64 values, one a lane,
// largest first in the end (the last stage sorts the whole wave one way).
template <int LEN, int J>
__device__ __forceinline__ void tau_wave_stage(float& x, int ln, bool rot4_first) {
    const float o = tau_partner<J>(x, rot4_first);
    const bool down = (ln & LEN) == 0 || LEN == 64, lower = (ln & J) == 0;
    x = (down == lower) ? fmaxf(x, o) : fminf(x, o);
    if constexpr (J > 1) tau_wave_stage<LEN, J / 2>(x, ln, rot4_first);
}

// maximum over the wave: inside the rows of 16 by data-path moves, the four rows by reading
// one lane of each
__device__ __forceinline__ float tau_wave_max(float v, bool rot4_first) {
    v = fmaxf(v, tau_partner<1>(v, rot4_first));
    v = fmaxf(v, tau_partner<2>(v, rot4_first));
    v = fmaxf(v, tau_partner<4>(v, rot4_first));
    v = fmaxf(v, tau_partner<8>(v, rot4_first));
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// One step of the bitonic sort (largest first) of 256 * EE entries, entry e*256 + tid in v[e]
// of thread tid < 256: entry i meets entry i ^ J; in a stretch that ends up descending
// ((i & LEN) == 0) the lower index keeps the larger value.  Every thread of the workgroup
// calls it (the steps through LDS hold a barrier); only the sorters hold data.
template <int EE, int LEN, int J>
__device__ __forceinline__ void tau_sort_step(float (&v)[EE], float* s0, float* s1, int& buf,
                                              int tid, bool sorter, bool rot4_first) {
    constexpr int ST = kTauSorters;
    if constexpr (J >= ST) {  // partner in another register of this thread
        constexpr int JE = J / ST;
        if (!sorter) return;
#pragma unroll
        for (int e = 0; e < EE; ++e) {
            if ((e & JE) == 0 && (e | JE) < EE) {
                const bool down = (((e * ST) & LEN) == 0);
                const float lo = v[e], hi = v[e | JE];
                const bool swap = down ? lo < hi : lo > hi;
                v[e] = swap ? hi : lo;
                v[e | JE] = swap ? lo : hi;
            }
        }
    } else {
        auto meet = [&](int e, float o) {
            const int i = e * ST + tid;
            const bool down = (i & LEN) == 0, lower = (i & J) == 0;
            v[e] = (down == lower) ? fmaxf(v[e], o) : fminf(v[e], o);
        };
        if constexpr (J >= 64) {  // partner in another wave
            float* sb = buf ? s1 : s0;
            if (sorter) {
#pragma unroll
                for (int e = 0; e < EE; ++e) sb[e * ST + tid] = v[e];
            }
            __syncthreads();
            if (sorter) {
#pragma unroll
                for (int e = 0; e < EE; ++e) meet(e, sb[e * ST + (tid ^ J)]);
            }
            buf ^= 1;  // the next exchange writes the other half: one barrier per step
        } else if (!sorter) {
            // (whole waves: the steps inside a wave are not theirs to spend issue slots on)
        } else if constexpr (J >= 16) {
#pragma unroll
            for (int e = 0; e < EE; ++e) meet(e, __shfl_xor(v[e], J, 64));
        } else if constexpr (J == 8) {
#pragma unroll
            for (int e = 0; e < EE; ++e) meet(e, dpp_move<0x128>(v[e]));  // row rotate by 8
        } else if constexpr (J == 4) {
#pragma unroll
            for (int e = 0; e < EE; ++e) {
                const float a = dpp_move<0x124>(v[e]), b = dpp_move<0x12C>(v[e]);  // by 4, by 12
                meet(e, rot4_first ? a : b);
            }
        } else if constexpr (J == 2) {
#pragma unroll
            for (int e = 0; e < EE; ++e) meet(e, dpp_move<0x4E>(v[e]));  // quad [2,3,0,1]
        } else {
#pragma unroll
            for (int e = 0; e < EE; ++e) meet(e, dpp_move<0xB1>(v[e]));  // quad [1,0,3,2]
        }
    }
}

// All steps from (LEN = 2^LL, J = 2^JJ) on, in order.
template <int EE, int LOGN, int LL, int JJ>
struct TauSortFrom {
    static __device__ __forceinline__ void run(float (&v)[EE], float* s0, float* s1, int& buf,
                                               int tid, bool sorter, bool rot4_first) {
        tau_sort_step<EE, (1 << LL), (1 << JJ)>(v, s0, s1, buf, tid, sorter, rot4_first);
        if constexpr (JJ > 0)
            TauSortFrom<EE, LOGN, LL, JJ - 1>::run(v, s0, s1, buf, tid, sorter, rot4_first);
        else if constexpr (LL < LOGN)
            TauSortFrom<EE, LOGN, LL + 1, LL>::run(v, s0, s1, buf, tid, sorter, rot4_first);
    }
};

// E = registers per thread of the sort: the padded array has 1024 * E entries
// The work of one workgroup of kTauThreads threads: the threshold of the head that place `pos`
// of the launch stands for.
template <typename T, int E>
__device__ __forceinline__ void threshold_block(
    const T* __restrict__ samples, int S, int D, const T* __restrict__ q,
    const int32_t* __restrict__ tree_q_off, const int32_t* __restrict__ tree_q_heads,
    int group_size, int num_trees, int method, int k, float* __restrict__ tau, const int pos) {
    constexpr int EPL = Elem<T>::kPerChunk;
    constexpr int NPAD = kTauThreads * E;
    __shared__ float s_sc[2][NPAD];  // the scores; the two sides of an exchange through LDS
    __shared__ float s_red[kTauWaves];
    const int tid = threadIdx.x;

    // the head of this workgroup and its tree
    int head, tree;
    if (group_size > 0) {
        // trees in the fast index: workgroup i takes head i / T of tree i % T
        tree = pos % num_trees;
        head = tree * group_size + pos / num_trees;
    } else {
        tree = 0;
        while (tree + 1 < num_trees && tree_q_off[tree + 1] <= pos) ++tree;  // uniform
        head = tree_q_heads[pos];
    }

    // ---- scores: 16 lanes per sample row, 64 rows per pass, kTauRows passes at a time ---------
    // (buffer loads: the tree's sample behind one scalar descriptor, the pass in a scalar offset,
    // one address register for all the rows a lane has in flight -- which is what lets sixteen of
    // them fit.  The range check of a buffer load looks at the vector offset only, so the scalar
    // one must stay inside the sample by itself: the last pass is moved back to end with the
    // sample and scores some rows a second time; with fewer than 64 rows the vector offset alone
    // says which lanes have none.)
    const int sub = tid & 15, grp = tid >> 4;
    const int chunks = D / EPL;
    const T* xs = samples + (size_t)tree * S * D;
    const T* qh = q + (size_t)head * D;
    constexpr int PASS = kTauThreads / 16;
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(xs), 0, (int)((size_t)S * D * sizeof(T)), 0x00020000);
    const int last_pass = max(S - PASS, 0);
    for (int r0 = 0; r0 < S; r0 += PASS * kTauRows) {  // uniform
        float dot[kTauRows];
#pragma unroll
        for (int u = 0; u < kTauRows; ++u) dot[u] = 0.0f;
        for (int c = sub; c < chunks; c += 16) {
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            const unsigned voff = (unsigned)((grp * D + c * EPL) * (int)sizeof(T));
            uint4 raw[kTauRows];
#pragma unroll
            for (int u = 0; u < kTauRows; ++u) {
                raw[u] = make_uint4(0, 0, 0, 0);
                if (r0 + u * PASS < S) {  // uniform
                    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(
                        xrsrc, voff, (unsigned)(min(r0 + u * PASS, last_pass) * D * (int)sizeof(T)), 0);
                    raw[u] = make_uint4(v.x, v.y, v.z, v.w);
                }
            }
            float b[EPL];
            unpack<T>(load_chunk<T>(qh, 0, c), b);
#pragma unroll
            for (int u = 0; u < kTauRows; ++u) {
                float a[EPL];
                unpack<T>(raw[u], a);
#pragma unroll
                for (int e = 0; e < EPL; ++e) dot[u] += a[e] * b[e];
            }
        }
#pragma unroll
        for (int u = 0; u < kTauRows; ++u) {
            const float d = group_sum<16>(dot[u]);
            const int row = min(r0 + u * PASS, last_pass) + grp;
            if (sub == 0 && r0 + u * PASS < S && row < S) s_sc[0][row] = d;
        }
    }
    __syncthreads();
    // ---- from here on only the first four waves hold data; the others keep the barriers company
    constexpr int ST = kTauSorters;
    constexpr int EE = NPAD / ST;     // entries per sorting thread
    constexpr int LOGN = E == 1 ? 10 : (E == 2 ? 11 : 12);
    const bool sorter = tid < ST;
    float v[EE];
#pragma unroll
    for (int e = 0; e < EE; ++e)
        v[e] = (sorter && e * ST + tid < S) ? s_sc[0][e * ST + tid] : -INFINITY;

    if (method == HIRA_TAU_SAMPLE_MAX) {
        float m = v[0];
#pragma unroll
        for (int e = 1; e < EE; ++e) m = fmaxf(m, v[e]);
        m = tau_block_reduce(m, true, s_red);
        if (tid == 0) tau[head] = m;
        return;
    }

    if (E == 1 && k <= 16) {
        // ---- few of up to 1024: every wave sorts its 64 scores, largest first ------------------
        const int ln = tid & 63, wv = tid >> 6;
        const bool rot4 = __builtin_amdgcn_update_dpp(0, ln, 0x124, 0xF, 0xF, true) == (ln ^ 4);
        float x = tid < S ? s_sc[0][tid] : -INFINITY;
        tau_wave_stage<2, 1>(x, ln, rot4);
        tau_wave_stage<4, 2>(x, ln, rot4);
        tau_wave_stage<8, 4>(x, ln, rot4);
        tau_wave_stage<16, 8>(x, ln, rot4);
        tau_wave_stage<32, 16>(x, ln, rot4);
        tau_wave_stage<64, 32>(x, ln, rot4);
        __syncthreads();  // everybody has read its score
        if (ln < 16) s_sc[1][wv * 16 + ln] = x;
        __syncthreads();
        if (wv != 0) return;
        // the k best of the 256 that are left, one at a time: the wave's maximum, taken out of
        // the one place (lowest lane, lowest register) that holds it
        float c[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) c[e] = s_sc[1][e * 64 + ln];
        float sum = 0.0f;
        for (int r = 0; r < k; ++r) {  // uniform
            const float mine = fmaxf(fmaxf(c[0], c[1]), fmaxf(c[2], c[3]));
            const float best = tau_wave_max(mine, rot4);
            sum += best;
            const unsigned long long has = __ballot(mine == best);
            if (ln == __ffsll((long long)has) - 1) {
                if (c[0] == best) c[0] = -INFINITY;
                else if (c[1] == best) c[1] = -INFINITY;
                else if (c[2] == best) c[2] = -INFINITY;
                else c[3] = -INFINITY;
            }
        }
        if (ln == 0) tau[head] = sum / (float)k;
        return;
    }

    // ---- bitonic sort, largest first ---------------------------------------------------------
    // Which of the two rotations by 4 inside a row of 16 lanes brings lane ^ 4: asked of the
    // lane numbers themselves.
    const int lane = tid & 63;
    const bool rot4_first =
        __builtin_amdgcn_update_dpp(0, lane, 0x124, 0xF, 0xF, true) == (lane ^ 4);
    int buf = 1;
    TauSortFrom<EE, LOGN, 1, 0>::run(v, s_sc[0], s_sc[1], buf, tid, sorter, rot4_first);
    float sum = 0.0f;
#pragma unroll
    for (int e = 0; e < EE; ++e)
        if (sorter && e * ST + tid < k) sum += v[e];
    sum = tau_block_reduce(sum, false, s_red);
    if (tid == 0) tau[head] = sum / (float)k;
}

// What hira_threshold checks of its arguments before the launch.
static int check_threshold_arguments(const void* samples, int32_t dtype, int32_t num_trees,
                                     int32_t num_samples, int32_t dim, const HiraQuery* query,
                                     int32_t method, int32_t k, const float* tau_out) {
    HIRA_CHECK_ARG(samples && query && tau_out, "hira_threshold: null argument");
    HIRA_CHECK_ARG(dtype == HIRA_F32 || dtype == HIRA_BF16, "hira_threshold: dtype %d", dtype);
    HIRA_CHECK_ARG(num_trees >= 1 && dim >= 1, "hira_threshold: num_trees %d, dim %d", num_trees, dim);
    const int epl = dtype == HIRA_F32 ? 4 : 8;
    HIRA_CHECK_ARG(dim % epl == 0, "hira_threshold: dim %d must be a multiple of %d (16-byte chunks)", dim, epl);
    HIRA_CHECK_ARG(num_samples >= 1 && num_samples <= kTauMaxSamples,
                   "hira_threshold: %d samples per tree (1..%d)", num_samples, kTauMaxSamples);
    HIRA_CHECK_ARG(method == HIRA_TAU_SAMPLE_MAX || method == HIRA_TAU_SAMPLE_MEAN_TOPK,
                   "hira_threshold: method %d", method);
    HIRA_CHECK_ARG(method == HIRA_TAU_SAMPLE_MAX || (k >= 1 && k <= num_samples),
                   "hira_threshold: k = %d with %d samples", k, num_samples);
    HIRA_CHECK_ARG(query->q && query->num_q_heads >= 1, "hira_threshold: query missing");
    if (query->group_size > 0)
        HIRA_CHECK_ARG(query->num_q_heads == num_trees * query->group_size,
                       "hira_threshold: %d heads != %d trees x group of %d", query->num_q_heads,
                       num_trees, query->group_size);
    else
        HIRA_CHECK_ARG(query->tree_q_off && query->tree_q_heads, "hira_threshold: head map missing");
    return HIRA_OK;
}

// registers per thread of the sort for this many samples: the E of threshold_block
static inline int threshold_sort_registers(int num_samples) {
    return num_samples <= kTauThreads ? 1 : (num_samples <= 2 * kTauThreads ? 2 : 4);
}

}  // namespace hira
