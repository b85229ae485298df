// Host launcher shared by the four SDDMM translation units.
#pragma once
#include "sddmm_kernel.h"

template <int NR, bool SPLIT>
int psp_sddmm_launch(const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                     const float *A, const float *B, const float *scale, float *out, int nrows, int K,
                     int blkWarpNum, hipStream_t stream, float *row_max)
{
    constexpr bool BCSR = NR > 1;
    const bool balanced = !SPLIT && (blkWarpNum & PSP_BW_BALANCED) != 0;  // plain layouts only; row-split input is balanced
    blkWarpNum &= ~PSP_BW_BALANCED;
    const int stripe_flag = ((blkWarpNum & PSP_BW_STRIPE_MASK) >> PSP_BW_STRIPE_SHIFT) * 256;  // 0: the library option
    blkWarpNum &= ~PSP_BW_STRIPE_MASK;
    PSP_REQUIRE(blkWarpNum == 4 || blkWarpNum == 8, "blkWarpNum must be 4 or 8");
    PSP_REQUIRE(nrows >= 0 && K >= 1, "sddmm: bad size (rows %d, K %d)", nrows, K);
    if (nrows == 0) return PSP_OK;
    // colIdx, out and the block values may be null for a matrix without stored entries: whether there are any is
    // written in rowPtr, which is on the device, and the kernel touches none of the three then
    PSP_REQUIRE(rowPtr && A && B, "sddmm: null pointer");
    PSP_REQUIRE((colIdx != nullptr) == (out != nullptr), "sddmm: colIdx and out must both be given (or both be null for a matrix without entries)");
    PSP_REQUIRE(!SPLIT || target_row, "sddmm: target_row is null");
    PSP_REQUIRE(!BCSR || val || !colIdx, "sddmm: block values are null");
    PSP_REQUIRE(!(BCSR && scale), "sddmm: scale is only supported for csr formats");
    PSP_REQUIRE(!(BCSR && row_max), "sddmm: row maxima are only supported for csr formats");

    const int V = (K % 4 == 0) ? 4 : (K % 2 == 0) ? 2 : 1;
    const int nvec = K / V;
    int C = psp_ceil_div(nvec, 16);
    if (C > 4) C = 4;
    int logL = 0;
    while ((C << logL) < nvec) logL++;
    if (logL > 6) return psp_fail(PSP_ERR_RANGE, "sddmm: K = %d is too wide (max %d for this alignment)", K, 256 * V);
    if (logL < 4 && C > 1) C = 1;

    psp_sddmm_kernel_t k = scale ? psp_sddmm_lookup<NR, SPLIT, !BCSR>(logL, C, V)
                                 : psp_sddmm_lookup<NR, SPLIT, false>(logL, C, V);
    if constexpr (!SPLIT) {
        if (balanced)
            k = scale ? psp_sddmm_lookup<NR, false, !BCSR, true>(logL, C, V) : psp_sddmm_lookup<NR, false, false, true>(logL, C, V);
    }
    if (!k) return psp_fail(PSP_ERR_ARG, "sddmm: no kernel for logL %d coarsen %d vec %d", logL, C, V);
    if (balanced) {
        // A fixed grid that fills the GPU once; its wavefronts divide the stored entries between them in tiles of 256
        // (the entry count is on the device, in rowPtr): each XCD takes one contiguous eighth of the tiles.
        const int wgs = 256 * 32 / blkWarpNum;
        dim3 grid(wgs, 1, 1), block(blkWarpNum * PSP_WAVE, 1, 1);
        hipLaunchKernelGGL(k, grid, block, 0, stream, rowPtr, colIdx, BCSR ? val : scale, target_row, A, B, out, nrows, K,
                           8, wgs, wgs / PSP_XCDS, row_max);
        return psp_check_launch("sddmm kernel (entry-balanced)");
    }

    // segments per wavefront: as for SpMM (one per lane group for plain input, 16 for row-split input, fewer for
    // small matrices)
    const int logR = 6 - logL;
    int logW = SPLIT ? (logR > 4 ? logR : 4) : logR;
    while (logW > 0 && (nrows >> logW) < 4096) logW--;
    if (logW < logR - 1) logW = logR - 1;
    const int segs_per_block = blkWarpNum << logW;
    const psp_grid1d g = psp_xcd_grid(psp_ceil_div(nrows, segs_per_block), (stripe_flag ? stripe_flag : psp_stripe_rows()) / segs_per_block);
    dim3 grid(g.launch, 1, 1), block(blkWarpNum * PSP_WAVE, 1, 1);
    hipLaunchKernelGGL(k, grid, block, 0, stream, rowPtr, colIdx, BCSR ? val : scale, target_row, A, B, out, nrows, K,
                       logW, g.real, g.stripe, row_max);
    return psp_check_launch("sddmm kernel");
}
