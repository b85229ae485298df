// Double-precision SpMM and SDDMM for all six layouts (CSR / 2x1 / 3x1 blocks, plain or row-split).  The reference
// dispatches its kernels for double as well as float (AT_DISPATCH_FLOATING_TYPES, SpMM_kernel.cu:149, sddmm_kernel.cu
// :161).  GNN training is single precision, so this path is kept simple rather than tuned: one wavefront per
// segment, lane groups across the columns taking the segment's entries in turn; the float path's balancing, vector
// loads and unrolling are not repeated here.
#include "psp_common.h"

// Y[rows_out, N] has been zeroed.  Plain layouts store, row-split layouts add (several segments may share a row).
// The wavefront is cut into 64 / W groups of W lanes (W = the power of two that covers min(N, 64) columns); the groups
// take the segment's entries in turn and their partial sums are added across the groups at the end, so narrow
// feature matrices still use all lanes.
template <int NR, bool SPLIT>
__global__ void __launch_bounds__(256)
spmm_f64_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const double *__restrict__ val,
                const int *__restrict__ target_row, const double *__restrict__ X, double *__restrict__ Y, int nseg, int N,
                int logW)
{
    const int lane = threadIdx.x & 63;
    const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (s >= nseg) return;  // wave-uniform
    const int lb = rowPtr[s], hb = rowPtr[s + 1];
    if (lb == hb) return;
    const int key = SPLIT ? target_row[s] : s;
    const int W = 1 << logW, G = 64 >> logW;
    const int sub = lane & (W - 1), grp = lane >> logW;
    for (int c0 = blockIdx.y * W; c0 < N; c0 += gridDim.y * W) {  // wave-uniform
        const int c = c0 + sub;
        double acc[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) acc[r] = 0.0;
        if (c < N) {
            for (int p = lb + grp; p < hb; p += G) {
                const double x = X[(size_t)colIdx[p] * N + c];
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    const double v = val[(size_t)p * NR + r];
                    if (NR == 1 || v != 0.0) acc[r] = fma(v, x, acc[r]);  // a zero block entry adds nothing (SpMM_kernel.cu:1399)
                }
            }
        }
        // the groups' partial sums meet in group 0 (all lanes take part in the exchange)
#pragma unroll
        for (int i = 0; i < 6; i++)
#pragma unroll
            for (int r = 0; r < NR; r++) {
                const double other = __shfl_xor(acc[r], 1 << i);
                if ((1 << i) >= W) acc[r] += other;  // wave-uniform
            }
        if (grp == 0 && c < N) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                double *y = Y + (size_t)(key * NR + r) * N + c;
                if (SPLIT) unsafeAtomicAdd(y, acc[r]);
                else *y = acc[r];
            }
        }
    }
}

// out[nblk, NR] (out[nnz] for NR = 1); entries whose block value is zero are written as zero.  Groups of W lanes
// (W covers min(K, 64) columns) take the segment's entries in turn.
template <int NR, bool SPLIT>
__global__ void __launch_bounds__(256)
sddmm_f64_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const double *__restrict__ val_b,
                 const int *__restrict__ target_row, const double *__restrict__ A, const double *__restrict__ B,
                 double *__restrict__ out, int nseg, int K, int logW)
{
    const int lane = threadIdx.x & 63;
    const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (s >= nseg) return;
    const int lb = rowPtr[s], hb = rowPtr[s + 1];
    const int key = SPLIT ? target_row[s] : s;
    const int W = 1 << logW, G = 64 >> logW;
    const int sub = lane & (W - 1), grp = lane >> logW;
    for (int p0 = lb; p0 < hb; p0 += G) {  // wave-uniform trip count: the exchange below needs every lane
        const int p = p0 + grp;
        const bool have = p < hb;
        const double *b = B + (size_t)(have ? colIdx[p] : 0) * K;
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const bool live = have && (NR == 1 || val_b[(size_t)p * NR + r] != 0.0);  // uniform within a group
            double part = 0.0;
            if (live) {
                const double *a = A + (size_t)(key * NR + r) * K;
                for (int k = sub; k < K; k += W) part = fma(a[k], b[k], part);
            }
#pragma unroll
            for (int i = 0; i < 6; i++) {
                const double other = __shfl_xor(part, 1 << i);
                if ((1 << i) < W) part += other;  // wave-uniform
            }
            if (sub == 0 && have) out[(size_t)p * NR + r] = live ? part : 0.0;
        }
    }
}

// lanes per group: the power of two that covers min(width, 64)
static int f64_log_group(int width)
{
    int logW = 0;
    while ((1 << logW) < width && logW < 6) logW++;
    return logW;
}

template <int NR>
static int spmm_f64_launch(const int *rowPtr, const int *colIdx, const double *val, const int *target_row, const double *X,
                           double *Y, int nseg, int N, hipStream_t st)
{
    const int logW = f64_log_group(N);
    int col_tiles = psp_ceil_div(N, 1 << logW);
    if (col_tiles > 64) col_tiles = 64;
    dim3 grid(psp_ceil_div(nseg, 4), col_tiles, 1), block(256, 1, 1);
    if (target_row)
        hipLaunchKernelGGL((spmm_f64_kernel<NR, true>), grid, block, 0, st, rowPtr, colIdx, val, target_row, X, Y, nseg, N, logW);
    else
        hipLaunchKernelGGL((spmm_f64_kernel<NR, false>), grid, block, 0, st, rowPtr, colIdx, val, target_row, X, Y, nseg, N, logW);
    return psp_check_launch("spmm f64 kernel");
}

PSP_EXPORT int psp_spmm_f64(const int *rowPtr, const int *colIdx, const double *val, const int *target_row,
                            const double *X, double *Y, int nseg, int N, int rows_out, int vec_size, psp_stream_t stream)
{
    PSP_REQUIRE(nseg >= 0 && N >= 0 && rows_out >= 0, "spmm_f64: negative size");
    PSP_REQUIRE(vec_size >= 1 && vec_size <= 3, "spmm_f64: vec_size must be 1, 2 or 3 (got %d)", vec_size);
    PSP_REQUIRE(Y || rows_out == 0 || N == 0, "spmm_f64: Y is null");
    if (!target_row) PSP_REQUIRE((long long)nseg * vec_size <= rows_out, "spmm_f64: Y has %d rows, the matrix needs %lld",
                                 rows_out, (long long)nseg * vec_size);
    hipStream_t st = (hipStream_t)stream;
    int rc = psp_zero_f32((float *)Y, (size_t)rows_out * N * 2, st);  // all-zero bits are 0.0 in both precisions
    if (rc != PSP_OK || nseg == 0 || N == 0) return rc;
    PSP_REQUIRE(rowPtr && X, "spmm_f64: rowPtr / X is null");
    if (vec_size == 1) return spmm_f64_launch<1>(rowPtr, colIdx, val, target_row, X, Y, nseg, N, st);
    if (vec_size == 2) return spmm_f64_launch<2>(rowPtr, colIdx, val, target_row, X, Y, nseg, N, st);
    return spmm_f64_launch<3>(rowPtr, colIdx, val, target_row, X, Y, nseg, N, st);
}

template <int NR>
static int sddmm_f64_launch(const int *rowPtr, const int *colIdx, const double *val_b, const int *target_row,
                            const double *A, const double *B, double *out, int nseg, int K, hipStream_t st)
{
    dim3 grid(psp_ceil_div(nseg, 4), 1, 1), block(256, 1, 1);
    const int logW = f64_log_group(K);
    if (target_row)
        hipLaunchKernelGGL((sddmm_f64_kernel<NR, true>), grid, block, 0, st, rowPtr, colIdx, val_b, target_row, A, B, out, nseg, K,
                           logW);
    else
        hipLaunchKernelGGL((sddmm_f64_kernel<NR, false>), grid, block, 0, st, rowPtr, colIdx, val_b, target_row, A, B, out, nseg, K,
                           logW);
    return psp_check_launch("sddmm f64 kernel");
}

PSP_EXPORT int psp_sddmm_f64(const int *rowPtr, const int *colIdx, const double *val_b, const int *target_row,
                             const double *A, const double *B, double *out, int nseg, int K, int vec_size,
                             psp_stream_t stream)
{
    PSP_REQUIRE(nseg >= 0 && K >= 1, "sddmm_f64: bad size (segments %d, K %d)", nseg, K);
    PSP_REQUIRE(vec_size >= 1 && vec_size <= 3, "sddmm_f64: vec_size must be 1, 2 or 3 (got %d)", vec_size);
    if (nseg == 0) return PSP_OK;
    // colIdx, out and the block values may be null for a matrix without stored entries (only rowPtr, on the device, tells)
    PSP_REQUIRE(rowPtr && A && B, "sddmm_f64: null pointer");
    PSP_REQUIRE((colIdx != nullptr) == (out != nullptr), "sddmm_f64: colIdx and out must both be given (or both be null for a matrix without entries)");
    PSP_REQUIRE(vec_size == 1 || val_b || !colIdx, "sddmm_f64: block values are null");
    hipStream_t st = (hipStream_t)stream;
    if (vec_size == 1) return sddmm_f64_launch<1>(rowPtr, colIdx, val_b, target_row, A, B, out, nseg, K, st);
    if (vec_size == 2) return sddmm_f64_launch<2>(rowPtr, colIdx, val_b, target_row, A, B, out, nseg, K, st);
    return sddmm_f64_launch<3>(rowPtr, colIdx, val_b, target_row, A, B, out, nseg, K, st);
}
