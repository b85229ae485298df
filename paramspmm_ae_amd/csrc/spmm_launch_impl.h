// Host launcher shared by the four SpMM translation units (one per format, to compile in parallel).
#pragma once
#include <stdlib.h>
#include "spmm_kernel.h"

template <int NR, bool SPLIT>
int psp_spmm_launch(const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                    const float *X, float *Y, int nrows, int N, int rows_out, int CF, int blkWarpNum,
                    hipStream_t stream, const float *row_max, float *row_sum, int relu_x)
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

    int logL = 0;
    while ((1 << logL) < plan.lanes_per_row) logL++;
    // Segments per wavefront.  Plain input gets one row per lane group on average: rows that are neighbours in
    // the matrix are then walked at the same time and share their X rows in the L1 / L2, while the even division
    // of the wavefront's entries still levels moderate differences in row length.  Row-split input means the
    // caller expects skewed rows: 16 segments per wavefront give the lane groups longer, even shares and fold the
    // partial sums of a long row before the single atomic per wavefront (measured on a scale-20 R-MAT graph:
    // 16 beats 8, 32 and 64 at every width).  Small matrices use fewer segments per wavefront so that there are
    // wavefronts for every SIMD.
    const int logR = 6 - logL;
    int logW = SPLIT ? (logR > 4 ? logR : 4) : logR;
    if (plan.log_segs_per_wave >= 0) logW = plan.log_segs_per_wave;  // chosen by a native configuration
    while (logW > 0 && (nrows >> logW) < 4096) logW--;
    if (logW < logR - 1) logW = logR - 1;
    if (logW > 6) logW = 6;
    const psp_options &opt = psp_opts();
    // whole_rows: every lane group is handed whole segments whatever their lengths, so each element of a plain row
    // is one FMA chain over the row's entries in storage order -- the summation order of the reference's
    // one-warp-per-row kernels (SpMM_kernel.cu:1157-1212), bit for bit -- at the price of the balance between the
    // lane groups.  That needs at least one segment per lane group.
    if (opt.whole_rows && logW < logR) logW = logR;

    // rows the kernel does not store to must read as zero
    int tail_rows = 0;
    if (SPLIT) {
        // The kernel stores rows that one wavefront holds alone and adds (atomics) to rows shared by several
        // wavefronts.  Large outputs are therefore not cleared as a whole: a pass over the segments clears only
        // the shared rows and the rows without segments.  Small outputs are cheaper to clear outright.
        if ((long long)rows_out * N >= opt.split_clear_min && nrows > 0)
            rc = psp_split_clear(rowPtr, target_row, Y, nrows, N, NR, rows_out, logW, stream);
        else
            rc = psp_zero_f32(Y, (size_t)rows_out * N, stream);
    } else {
        // rows past the matrix's own: up to PSP_SPMM_TAIL_ROWS_MAX are zeroed by the kernel itself (tail_rows)
        const size_t covered = (size_t)nrows * NR;
        tail_rows = (int)std::min<size_t>((size_t)rows_out - covered, (size_t)PSP_SPMM_TAIL_ROWS_MAX + 1);
        if (tail_rows > PSP_SPMM_TAIL_ROWS_MAX || nrows == 0) {
            tail_rows = 0;
            rc = psp_zero_f32(Y + covered * N, ((size_t)rows_out - covered) * N, stream);
        }
    }
    if (rc != PSP_OK) return rc;
    if (nrows == 0) return PSP_OK;
    const bool softmax = row_max != nullptr;
    PSP_REQUIRE(!(softmax && relu_x), "spmm: the softmax-weighted product takes no activation argument");
    if (softmax && SPLIT) {
        PSP_REQUIRE(row_sum, "spmm softmax: row_sum workspace is null");
        rc = psp_zero_f32(row_sum, (size_t)rows_out, stream);
        if (rc != PSP_OK) return rc;
    }

    const int segs_per_block = plan.waves_per_block << logW;
    psp_spmm_kernel_t k = psp_spmm_lookup<NR, SPLIT>(plan.coarsen, plan.vec, plan.unroll, plan.lanes_per_row, softmax, relu_x != 0);
    if (!k)
        return psp_fail(PSP_ERR_ARG, "spmm%s: no kernel for coarsen %d vec %d unroll %d%s", softmax ? " softmax" : "", plan.coarsen,
                        plan.vec, plan.unroll, softmax ? " (needs N % 4 == 0 and CF <= 4)" : "");

    const int align_pct = opt.whole_rows ? (1 << 30) : (plan.even_split ? 0 : opt.align_pct);
    const psp_grid1d g = psp_xcd_grid(psp_ceil_div(nrows, segs_per_block),
                                      (plan.xcd_stripe_rows ? plan.xcd_stripe_rows : opt.stripe_rows) / segs_per_block);
    dim3 grid(g.launch, plan.col_tiles, 1), block(plan.waves_per_block * PSP_WAVE, 1, 1);
    hipLaunchKernelGGL(k, grid, block, 0, stream, rowPtr, colIdx, val, target_row, X, Y, nrows, N, logL, logW, g.real, g.stripe, align_pct, row_max, row_sum, relu_x, tail_rows);
    rc = psp_check_launch("spmm kernel");
    if (rc != PSP_OK || !(softmax && SPLIT)) return rc;
    return psp_row_scale(Y, row_sum, rows_out, N, stream);  // rows that several wavefronts added to
}
