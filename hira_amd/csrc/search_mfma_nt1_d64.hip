// MFMA search kernel instantiations for D = 64, key tiles loaded non-temporal.
#include "search_mfma_kernel.h"

namespace hira {
void launch_mfma_nt1_d64(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    launch_mfma_mt<2, false, 1>(plan, p, grid, s);
}
}  // namespace hira
