// Dispatch of the MFMA search kernel (search_mfma_kernel.h).
#include "search_mfma_kernel.h"

namespace hira {

bool mfma_search_supported(const HiraTree* t, const HiraQueue* queue) {
    if (t->dtype != HIRA_BF16 || (t->layout != HIRA_TILE16 && t->layout != HIRA_TILE16_Q8)) return false;
    if (t->num_levels < 2) return false;
    if (t->bf % 16 != 0 || t->bf > 16 * kMaxTiles) return false;
    if (!(t->dim == 64 || t->dim == 128 || t->dim == 256)) return false;
    if (t->vdim != 0 && t->vdim != t->dim) return false;
    (void)queue;  // queued rows get a workgroup of their own
    // the kernel addresses a tree's keys and values with 32-bit offsets
    if ((uint64_t)t->cap[0] * (uint64_t)t->dim * 2ull >= (1ull << 32)) return false;
    return true;
}

// grid: x = tree, y = tile of 16 level-1 nodes, z = pass of 16 heads
int launch_search_mfma(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    const bool q8 = p.keys8 != nullptr;  // the scan reads the keys' 8-bit shadow
    const int pol = q8 ? 0 : p.key_policy;  // cache policy of the bf16 tiles and the value rows
    typedef void (*Launch)(const SearchPlan&, const SearchParams&, dim3, hipStream_t);
    static const Launch table[3][4] = {
        {launch_mfma_d64, launch_mfma_nt1_d64, launch_mfma_nt2_d64, launch_mfma_q8_d64},
        {launch_mfma_d128, launch_mfma_nt1_d128, launch_mfma_nt2_d128, launch_mfma_q8_d128},
        {launch_mfma_d256, launch_mfma_nt1_d256, launch_mfma_nt2_d256, nullptr}};
    const int col = q8 ? 3 : pol;
    // (no shadow scan for rows of 256 columns: its kernels did not fit the register file)
    if (q8 && p.dim == 256) return fail(HIRA_EINVAL, "MFMA kernel: 8-bit shadow with dim 256");
    switch (p.dim) {
        case 64: table[0][col](plan, p, grid, s); return HIRA_OK;
        case 128: table[1][col](plan, p, grid, s); return HIRA_OK;
        case 256: table[2][col](plan, p, grid, s); return HIRA_OK;
        default: return fail(HIRA_EINVAL, "MFMA kernel: dim %d", p.dim);
    }
}

}  // namespace hira
