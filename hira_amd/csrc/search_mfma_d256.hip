// MFMA search kernel instantiations for D = 256.
#include "search_mfma_kernel.h"

namespace hira {
void launch_mfma_d256(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    launch_mfma_mt<8, false, 0>(plan, p, grid, s);
}
}  // namespace hira
