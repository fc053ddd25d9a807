// The vector-ALU search kernel for bf16_t rows: every row width, head-group width and gate batching.
#include "search_vec_kernel.h"

namespace hira {

int launch_vec_bf16(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    return dispatch_lpr<bf16_t>(plan, p, grid, s);
}

}  // namespace hira
