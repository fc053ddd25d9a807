// MFMA search kernel instantiations for D = 128.
#include "search_mfma_kernel.h"

namespace hira {
void launch_mfma_d128(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    launch_mfma_mt<4, false, 0>(plan, p, grid, s);
}
}  // namespace hira
