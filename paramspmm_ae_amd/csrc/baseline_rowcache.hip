// Row-caching SpMM, the comparison baseline behind ParamSpMM.gespmm_compute / gespmm_profile.
// The reference ships GE-SpMM's "row caching, row balance" kernel for that purpose
// (SpMM/Baseline_kernel.cu:616-742): one warp per sparse row, 32 (column, value) pairs at a time cached in
// shared memory, every lane accumulating CoarsenFactor output columns 32 apart.  This is the same scheme laid
// out for a 64-lane wavefront: 64 pairs per step cached in LDS, lane l owns columns tile*64*CF + l + 64*c, so a
// wavefront reads 256 contiguous bytes of an X row per cached entry and coarsening step.  It is deliberately
// plain (no balancing of long rows, no vector loads): a baseline, not the product kernel.
#include "psp_common.h"

#define RC_THREADS 256

template <int CF>
__global__ void __launch_bounds__(RC_THREADS)
rowcache_spmm_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const float *__restrict__ val,
                     const float *__restrict__ X, float *__restrict__ Y, int M, int N)
{
    __shared__ int s_col[RC_THREADS];
    __shared__ float s_val[RC_THREADS];
    const int lane = threadIdx.x & (PSP_WAVE - 1);
    const int wbase = threadIdx.x - lane;  // this wavefront's slice of the cache
    const int row = blockIdx.x * (RC_THREADS / PSP_WAVE) + (threadIdx.x >> 6);
    if (row >= M) return;  // wave-uniform
    const int col0 = blockIdx.y * (PSP_WAVE * CF) + lane;
    float acc[CF];
#pragma unroll
    for (int c = 0; c < CF; c++) acc[c] = 0.0f;

    const int end = rowPtr[row + 1];
    for (int p0 = rowPtr[row]; p0 < end; p0 += PSP_WAVE) {
        const int p = p0 + lane;
        s_col[wbase + lane] = p < end ? colIdx[p] : 0;
        s_val[wbase + lane] = p < end ? val[p] : 0.0f;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int cnt = min(PSP_WAVE, end - p0);
        for (int j = 0; j < cnt; j++) {
            const float a = s_val[wbase + j];
            const float *xr = X + (size_t)s_col[wbase + j] * (size_t)N;
#pragma unroll
            for (int c = 0; c < CF; c++) {
                const int col = col0 + c * PSP_WAVE;
                if (col < N) acc[c] = __builtin_fmaf(a, xr[col], acc[c]);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();  // the cache is refilled next
    }
#pragma unroll
    for (int c = 0; c < CF; c++) {
        const int col = col0 + c * PSP_WAVE;
        if (col < N) Y[(size_t)row * (size_t)N + col] = acc[c];
    }
}

PSP_EXPORT int psp_baseline_rowcache_spmm_f32(const int *rowPtr, const int *colIdx, const float *val, const float *X,
                                              float *Y, int M, int N, psp_stream_t stream)
{
    PSP_REQUIRE(M >= 0 && N >= 0, "rowcache spmm: negative size");
    if (M == 0 || N == 0) return PSP_OK;
    PSP_REQUIRE(rowPtr && X && Y, "rowcache spmm: null pointer");
    // column coarsening by width, the rule of the reference's launcher (Baseline_kernel.cu:763-765) scaled to 64 lanes
    const int cf = N >= 1024 ? 4 : (N >= 256 ? 2 : 1);
    dim3 grid(psp_ceil_div(M, RC_THREADS / PSP_WAVE), psp_ceil_div(N, PSP_WAVE * cf), 1), block(RC_THREADS, 1, 1);
    hipStream_t st = (hipStream_t)stream;
    if (cf == 4) hipLaunchKernelGGL(rowcache_spmm_kernel<4>, grid, block, 0, st, rowPtr, colIdx, val, X, Y, M, N);
    else if (cf == 2) hipLaunchKernelGGL(rowcache_spmm_kernel<2>, grid, block, 0, st, rowPtr, colIdx, val, X, Y, M, N);
    else hipLaunchKernelGGL(rowcache_spmm_kernel<1>, grid, block, 0, st, rowPtr, colIdx, val, X, Y, M, N);
    return psp_check_launch("rowcache spmm kernel");
}
