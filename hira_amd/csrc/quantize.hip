// 8-bit shadow of the keys (layout HIRA_TILE16_Q8): one step per tree and channel, the keys
// rounded to whole steps in [-127, 127] and stored in tiles of 16 rows x 64 columns, and per
// level-1 node the largest rounding (or clipping) error, in steps, among its keys.  The search
// scans the shadow first: with k = kscale * (k8 + e), |e| <= keps, a score obeys
//   |q.k - sum_j (q_j kscale_j) k8_j| <= keps * sum_j |q_j kscale_j|,
// so a key whose 8-bit score plus that bound stays below the threshold cannot be selected and
// its bf16 row is never fetched.  The reference keeps fp32 keys only (indexer/cuda.py:365-368);
// this is what halves the bytes of the leaf scan without touching the selected set.
#include "rows.h"

namespace hira {

constexpr int kQuantThreads = 256;
constexpr float kMinStep = 1e-30f;  // a channel that is zero in every key

// largest magnitude per channel: workgroup b of tree t covers rows b*per + r0, stepping by
// gridDim.x*per; its maxima join kscale (zeroed before) through integer atomic maxima -- the
// bits of non-negative floats order like unsigned integers, and a maximum does not depend on
// the order of arrival
__global__ __launch_bounds__(kQuantThreads) void k_absmax(const uint16_t* keys, size_t tree_stride,
                                                          int rows, int D, float* kscale) {
    const int t = blockIdx.y;
    const int per = kQuantThreads / D, c = threadIdx.x % D, r0 = threadIdx.x / D;
    float m = 0.0f;
    if (r0 < per)
        for (int r = blockIdx.x * per + r0; r < rows; r += gridDim.x * per)
            m = fmaxf(m, fabsf(bf16_bits_to_f32(keys[((size_t)t * tree_stride + r) * D + c])));
    __shared__ float sm[kQuantThreads];
    sm[threadIdx.x] = m;
    __syncthreads();
    if (threadIdx.x < D) {
        for (int k = 1; k < per; ++k) m = fmaxf(m, sm[k * D + threadIdx.x]);
        if (m > 0.0f && m < INFINITY)
            atomicMax(reinterpret_cast<unsigned*>(kscale) + (size_t)t * D + threadIdx.x, __float_as_uint(m));
    }
}

__global__ void k_zero_f32(float* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

__global__ void k_step_from_absmax(float* kscale, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) kscale[i] = fmaxf(kscale[i] / 127.0f, kMinStep);
}

// one wave per level-1 node: its bf key slots -> shadow bytes, error bound of the node
__global__ __launch_bounds__(64) void k_quantize(const uint16_t* keys, int8_t* keys8, const float* kscale,
                                                 const int32_t* perm, float* keps, size_t cap0,
                                                 size_t cap1, int node_first, int bf, int D) {
    const int t = blockIdx.y, node = node_first + blockIdx.x, lane = threadIdx.x;
    const size_t base = (size_t)t * cap0;
    float worst = 0.0f;
    for (int i = 0; i < bf; ++i) {
        const size_t slot = (size_t)node * bf + i;
        const bool live = perm[base + slot] >= 0;  // uniform
        for (int j = lane; j < D; j += 64) {
            float r = 0.0f;
            if (live) {
                const float u = bf16_bits_to_f32(keys[(base + slot) * D + j]) / kscale[(size_t)t * D + j];
                r = fminf(fmaxf(rintf(u), -127.0f), 127.0f);
                worst = fmaxf(worst, fabsf(u - r));
            }
            keys8[base * D + shadow_index(D, slot, j)] = (int8_t)(int)r;
        }
    }
    worst = wave_max(worst);
    if (lane == 0) keps[(size_t)t * cap1 + node] = worst;
}

}  // namespace hira

using namespace hira;

/* see include/hira_hip.h */
extern "C" int hira_quantize(const HiraTree* tree, int32_t slot_first, int32_t slot_count,
                             int32_t recompute_scale, void* stream) {
    HIRA_CHECK_ARG(tree != nullptr && tree->layout == HIRA_TILE16_Q8,
                   "hira_quantize needs an index in the layout with an 8-bit shadow");
    HIRA_CHECK_ARG(tree->dtype == HIRA_BF16 && tree->dim % 64 == 0 && tree->dim <= 256 &&
                       tree->num_levels >= 2,
                   "8-bit shadow: bf16 rows of 64, 128, 192 or 256 columns, at least two levels");
    HIRA_CHECK_ARG(tree->keys && tree->perm && tree->keys8 && tree->kscale && tree->keps,
                   "keys / perm / keys8 / kscale / keps missing");
    const int bf = tree->bf;
    HIRA_CHECK_ARG(slot_first >= 0 && slot_count >= 0 && slot_first % bf == 0 && slot_count % bf == 0 &&
                       (int64_t)slot_first + slot_count <= tree->cap[0] &&
                       ((int64_t)slot_first + slot_count) / bf <= tree->cap[1],
                   "slots [%d, +%d): whole level-1 nodes inside the capacity", slot_first, slot_count);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const int D = tree->dim, T = tree->num_trees;
    const uint16_t* keys = reinterpret_cast<const uint16_t*>(tree->keys);
    if (recompute_scale) {
        HIRA_CHECK_ARG(slot_first == 0 && slot_count >= tree->size[0],
                       "new steps need the shadow of every key recomputed");
        const int rows = tree->size[0];
        const size_t n = (size_t)T * D;
        int parts = (rows + 1023) / 1024;
        if (parts > 128) parts = 128;
        if (parts < 1) parts = 1;
        hipLaunchKernelGGL(k_zero_f32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, tree->kscale, n);
        if (rows > 0)
            hipLaunchKernelGGL(k_absmax, dim3(parts, T), dim3(kQuantThreads), 0, s, keys,
                               (size_t)tree->cap[0], rows, D, tree->kscale);
        hipLaunchKernelGGL(k_step_from_absmax, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                           tree->kscale, n);
    }
    if (slot_count == 0) return HIRA_OK;
    hipLaunchKernelGGL(k_quantize, dim3(slot_count / bf, T), dim3(64), 0, s, keys, tree->keys8,
                       tree->kscale, tree->perm, tree->keps, (size_t)tree->cap[0],
                       (size_t)tree->cap[1], slot_first / bf, bf, D);
    HIRA_CHECK_LAUNCH("quantize kernel");
    return HIRA_OK;
}
