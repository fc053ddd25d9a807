// hira_threshold: per-head thresholds from a sample of a tree's keys, one launch.
//   tau[h] = max_s q_h . x_s                      (HIRA_TAU_SAMPLE_MAX)
//   tau[h] = mean of the k largest q_h . x_s      (HIRA_TAU_SAMPLE_MEAN_TOPK)
// One workgroup of sixteen waves per query head; with whole groups of heads per tree the
// workgroups of a tree are a multiple of eight apart in the launch, so that they run behind the
// same L2 (workgroups go to the eight L2s in turn) and the tree's sample is fetched from memory
// once.  Up to 1024 samples and k <= 16: every wave sorts its 64 scores in registers, the
// sixteen best of every wave meet in LDS, and one wave picks the k best of those 256 one by one.  Scores: 16 lanes share a sample row (16 bytes
// each per step), eight rows per lane group in flight.  Then either a maximum, or a bitonic sort
// by the first four waves with the scores in registers (entry e*256 + thread of the padded
// array lives in register e of that thread: partners 256 or more apart are a register swap,
// partners inside a wave a cross-lane move, only the two distances in between go through LDS)
// and a sum over the first k.
#include "threshold_kernel.h"

namespace hira {

template <typename T, int E>
__global__ __launch_bounds__(kTauThreads) void k_threshold(
    const T* __restrict__ samples, int S, int D, const T* __restrict__ q,
    const int32_t* __restrict__ tree_q_off, const int32_t* __restrict__ tree_q_heads,
    int group_size, int num_trees, int method, int k, float* __restrict__ tau) {
    threshold_block<T, E>(samples, S, D, q, tree_q_off, tree_q_heads, group_size, num_trees, method, k,
                          tau, (int)blockIdx.x);
}

template <typename T>
static void launch_threshold(int e, dim3 grid, hipStream_t s, const void* samples, int S, int D,
                             const HiraQuery* qu, int num_trees, int method, int k, float* tau) {
    const T* x = static_cast<const T*>(samples);
    const T* q = static_cast<const T*>(qu->q);
    const dim3 block(kTauThreads);
#define HIRA_TAU_LAUNCH(E)                                                                        \
    hipLaunchKernelGGL((k_threshold<T, E>), grid, block, 0, s, x, S, D, q, qu->tree_q_off,        \
                       qu->tree_q_heads, qu->group_size, num_trees, method, k, tau)
    if (e == 1) HIRA_TAU_LAUNCH(1);
    else if (e == 2) HIRA_TAU_LAUNCH(2);
    else HIRA_TAU_LAUNCH(4);
#undef HIRA_TAU_LAUNCH
}

}  // namespace hira

extern "C" int hira_threshold(const void* samples, int32_t dtype, int32_t num_trees,
                              int32_t num_samples, int32_t dim, const HiraQuery* query,
                              int32_t method, int32_t k, float* tau_out, void* stream) {
    using namespace hira;
    if (const int rc = check_threshold_arguments(samples, dtype, num_trees, num_samples, dim, query,
                                                 method, k, tau_out))
        return rc;
    const int e = threshold_sort_registers(num_samples);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const dim3 grid(query->num_q_heads);
    if (dtype == HIRA_F32)
        launch_threshold<float>(e, grid, s, samples, num_samples, dim, query, num_trees, method, k, tau_out);
    else
        launch_threshold<bf16_t>(e, grid, s, samples, num_samples, dim, query, num_trees, method, k, tau_out);
    HIRA_CHECK_LAUNCH("hira_threshold");
    return HIRA_OK;
}
