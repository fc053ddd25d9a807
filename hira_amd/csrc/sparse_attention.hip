// hira_sparse_attention: softmax attention over caller-given lists of selected keys (the lists
// hira_search writes, possibly edited in between):
//   out[h] = sum_j softmax_j(scaling[h] * score[h][j]) * values[tree(h)][index[h][j]]
// One workgroup of four waves per query head.  The largest score first (one pass over the
// list), then the waves take the listed rows round-robin, eight value rows in flight each, a
// lane owning every 64th 4-byte word of the row; the waves' sums meet in LDS.
#include "common.hip.h"

namespace hira {

constexpr int kSaThreads = 256;
constexpr int kSaWaves = kSaThreads / 64;
constexpr int kSaRows = 8;      // value rows a wave has in flight
constexpr int kSaMaxWords = 8;  // 4-byte words of a value row per lane: rows of up to 2 KiB

template <typename T>
__device__ __forceinline__ void sa_accumulate(uint32_t word, float w, float& a0, float& a1);
template <>
__device__ __forceinline__ void sa_accumulate<float>(uint32_t word, float w, float& a0, float& a1) {
    a0 += w * __uint_as_float(word);
}
template <>
__device__ __forceinline__ void sa_accumulate<bf16_t>(uint32_t word, float w, float& a0, float& a1) {
    a0 += w * bf16_lo(word);
    a1 += w * bf16_hi(word);
}

// WORDS = 4-byte words of a value row per lane (row bytes <= 256 * WORDS)
template <typename T, int WORDS>
__global__ __launch_bounds__(kSaThreads) void k_sparse_attention(
    const T* __restrict__ values, int64_t cap0, int vdim, const int32_t* __restrict__ sel_index,
    const float* __restrict__ sel_score, const int32_t* __restrict__ sel_count, int sel_cap,
    const float* __restrict__ scaling, const int32_t* __restrict__ tree_q_off,
    const int32_t* __restrict__ tree_q_heads, int group_size, int num_trees, float* __restrict__ out) {
    constexpr int EPW = sizeof(T) == 4 ? 1 : 2;  // elements per word
    __shared__ float s_red[kSaWaves];
    __shared__ float s_l[kSaWaves];
    __shared__ float s_acc[kSaWaves][64 * WORDS * 2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    const int pos = blockIdx.x;
    int head, tree;
    if (group_size > 0) {
        head = pos;
        tree = pos / group_size;
    } else {
        tree = 0;
        while (tree + 1 < num_trees && tree_q_off[tree + 1] <= pos) ++tree;  // uniform
        head = tree_q_heads[pos];
    }
    const int n = min(sel_count[head], sel_cap);
    const int row_words = vdim / EPW;  // 4-byte words of a value row
    float* o = out + (size_t)head * vdim;
    if (n <= 0) {  // uniform: nothing selected
        for (int c = tid; c < vdim; c += kSaThreads) o[c] = 0.0f;
        return;
    }
    const int32_t* idx = sel_index + (size_t)head * sel_cap;
    const float* sco = sel_score + (size_t)head * sel_cap;
    const float sc2 = scaling[head] * kLog2e;

    // the largest logit
    float m = -INFINITY;
    for (int j = tid; j < n; j += kSaThreads) m = fmaxf(m, sco[j] * sc2);
    m = wave_max(m);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = s_red[0];
#pragma unroll
    for (int w = 1; w < kSaWaves; ++w) m = fmaxf(m, s_red[w]);

    // weighted rows
    const uint32_t* vbase = reinterpret_cast<const uint32_t*>(values + (size_t)tree * cap0 * vdim);
    float acc[WORDS][2];
#pragma unroll
    for (int k = 0; k < WORDS; ++k) acc[k][0] = acc[k][1] = 0.0f;
    float l = 0.0f;
    for (int j0 = wave * kSaRows; j0 < n; j0 += kSaWaves * kSaRows) {  // uniform in the wave
        uint32_t raw[kSaRows][WORDS];
        float wgt[kSaRows];
#pragma unroll
        for (int i = 0; i < kSaRows; ++i) {
            const int j = min(j0 + i, n - 1);
            const size_t row = (size_t)min(max(idx[j], 0), (int)cap0 - 1);  // (an index out of range reads a wrong row, never wrong memory)
            wgt[i] = j0 + i < n ? exp2f(sco[j] * sc2 - m) : 0.0f;
#pragma unroll
            for (int k = 0; k < WORDS; ++k) {
                const int wd = lane + 64 * k;
                raw[i][k] = wd < row_words ? vbase[row * row_words + wd] : 0u;
            }
        }
#pragma unroll
        for (int i = 0; i < kSaRows; ++i) {
            l += wgt[i];
#pragma unroll
            for (int k = 0; k < WORDS; ++k) sa_accumulate<T>(raw[i][k], wgt[i], acc[k][0], acc[k][1]);
        }
    }
    // the waves' sums meet
    if (lane == 0) s_l[wave] = l;
#pragma unroll
    for (int k = 0; k < WORDS; ++k) {
        s_acc[wave][(k * 64 + lane) * 2] = acc[k][0];
        s_acc[wave][(k * 64 + lane) * 2 + 1] = acc[k][1];
    }
    __syncthreads();
    float lsum = 0.0f;
#pragma unroll
    for (int w = 0; w < kSaWaves; ++w) lsum += s_l[w];
    for (int c = tid; c < vdim; c += kSaThreads) {
        const int wd = c / EPW, half = c % EPW;  // word (k*64 + lane) and which element of it
        float a = 0.0f;
#pragma unroll
        for (int w = 0; w < kSaWaves; ++w) a += s_acc[w][wd * 2 + half];
        o[c] = a / lsum;
    }
}

template <typename T>
static void launch_sparse_attention(int words, dim3 grid, hipStream_t s, const HiraTree* tree,
                                    const HiraQuery* q, const int32_t* idx, const float* sco,
                                    const int32_t* cnt, int cap, float* out) {
    const T* v = static_cast<const T*>(tree->values);
    const dim3 block(kSaThreads);
#define HIRA_SA_LAUNCH(W)                                                                          \
    hipLaunchKernelGGL((k_sparse_attention<T, W>), grid, block, 0, s, v, (int64_t)tree->cap[0],    \
                       tree->vdim, idx, sco, cnt, cap, q->scaling, q->tree_q_off, q->tree_q_heads, \
                       q->group_size, tree->num_trees, out)
    if (words <= 1) HIRA_SA_LAUNCH(1);
    else if (words <= 2) HIRA_SA_LAUNCH(2);
    else if (words <= 4) HIRA_SA_LAUNCH(4);
    else HIRA_SA_LAUNCH(8);
#undef HIRA_SA_LAUNCH
}

}  // namespace hira

extern "C" int hira_sparse_attention(const HiraTree* tree, const HiraQuery* query,
                                     const int32_t* sel_index, const float* sel_score,
                                     const int32_t* sel_count, int32_t sel_cap, float* attn_out,
                                     void* stream) {
    using namespace hira;
    HIRA_CHECK_ARG(tree && query && sel_index && sel_score && sel_count && attn_out,
                   "hira_sparse_attention: null argument");
    HIRA_CHECK_ARG(tree->dtype == HIRA_F32 || tree->dtype == HIRA_BF16, "dtype %d", tree->dtype);
    HIRA_CHECK_ARG(tree->values != nullptr && tree->vdim > 0, "the index holds no values");
    const int esize = tree->dtype == HIRA_F32 ? 4 : 2;
    HIRA_CHECK_ARG((tree->vdim * esize) % 16 == 0, "vdim %d: rows must be a multiple of 16 bytes", tree->vdim);
    const int words = (tree->vdim * esize / 4 + 63) / 64;
    HIRA_CHECK_ARG(words <= kSaMaxWords, "vdim %d: value rows of at most %d bytes", tree->vdim,
                   kSaMaxWords * 256);
    HIRA_CHECK_ARG(sel_cap > 0, "sel_cap %d", sel_cap);
    HIRA_CHECK_ARG(query->num_q_heads >= 1 && query->scaling, "heads / scaling missing");
    if (query->group_size > 0)
        HIRA_CHECK_ARG(query->num_q_heads == tree->num_trees * query->group_size,
                       "%d heads != %d trees x group of %d", query->num_q_heads, tree->num_trees,
                       query->group_size);
    else
        HIRA_CHECK_ARG(query->tree_q_off && query->tree_q_heads, "head map missing");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const dim3 grid(query->num_q_heads);
    if (tree->dtype == HIRA_F32)
        launch_sparse_attention<float>(words, grid, s, tree, query, sel_index, sel_score, sel_count, sel_cap, attn_out);
    else
        launch_sparse_attention<bf16_t>(words, grid, s, tree, query, sel_index, sel_score, sel_count, sel_cap, attn_out);
    HIRA_CHECK_LAUNCH("hira_sparse_attention");
    return HIRA_OK;
}
