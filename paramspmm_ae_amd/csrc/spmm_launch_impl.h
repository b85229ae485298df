// Host launcher shared by the four SpMM translation units (one per format, to compile in parallel).
#pragma once
#include "spmm_kernel.h"

template <int NR, bool SPLIT>
int psp_spmm_launch(const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                    const float *X, float *Y, int nrows, int N, int rows_out, int CF, int blkWarpNum,
                    hipStream_t stream)
{
    psp_spmm_plan plan;
    int rc = psp_spmm_plan_for(N, CF, blkWarpNum, &plan);
    if (rc != PSP_OK) return rc;
    PSP_REQUIRE(nrows >= 0 && rows_out >= 0, "spmm: negative size (rows %d, rows_out %d)", nrows, rows_out);
    PSP_REQUIRE(Y != nullptr || rows_out == 0, "spmm: Y is null");
    if (!SPLIT)
        PSP_REQUIRE((long long)nrows * NR <= rows_out, "spmm: Y has %d rows, the matrix needs %lld", rows_out,
                    (long long)nrows * NR);
    if (nrows > 0) {
        PSP_REQUIRE(rowPtr && X, "spmm: rowPtr / X is null");
        PSP_REQUIRE(!SPLIT || target_row, "spmm: target_row is null");
    }

    // rows the kernel does not store to must read as zero
    if (SPLIT) {
        rc = psp_zero_f32(Y, (size_t)rows_out * N, stream);
    } else {
        const size_t covered = (size_t)nrows * NR;
        rc = psp_zero_f32(Y + covered * N, ((size_t)rows_out - covered) * N, stream);
    }
    if (rc != PSP_OK) return rc;
    if (nrows == 0) return PSP_OK;

    int logL = 0;
    while ((1 << logL) < plan.lanes_per_row) logL++;
    psp_spmm_kernel_t k = psp_spmm_lookup<NR, SPLIT>(plan.coarsen, plan.vec, plan.unroll);
    if (!k) return psp_fail(PSP_ERR_ARG, "spmm: no kernel for coarsen %d vec %d unroll %d", plan.coarsen, plan.vec, plan.unroll);

    // segments per wavefront: 64 when that still leaves thousands of wavefronts, fewer for small matrices,
    // but not so few that most lane groups of a wavefront would find nothing to do
    int logW = 6;
    while (logW > 0 && (nrows >> logW) < 4096) logW--;
    const int logR = 6 - logL;
    if (logW < logR - 1) logW = logR - 1;
    const int segs_per_block = plan.waves_per_block << logW;
    const psp_grid1d g = psp_xcd_grid(psp_ceil_div(nrows, segs_per_block));
    dim3 grid(g.launch, plan.col_tiles, 1), block(plan.waves_per_block * PSP_WAVE, 1, 1);
    hipLaunchKernelGGL(k, grid, block, 0, stream, rowPtr, colIdx, val, target_row, X, Y, nrows, N, logL, logW, g.real, g.chunk);
    return psp_check_launch("spmm kernel");
}
