// The vector-ALU search kernel for float rows: every row width, head-group width and gate batching.
#include "search_vec_kernel.h"

namespace hira {

int launch_vec_f32(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    return dispatch_lpr<float>(plan, p, grid, s);
}

}  // namespace hira
