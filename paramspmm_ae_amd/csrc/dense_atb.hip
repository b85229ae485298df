// C[K1,K2] = A^T * B for tall-skinny A [n,K1], B [n,K2] (n ~ 10^6, K1,K2 multiples of 16 up to 128): the weight-gradient product
// H^T * (A dY) of the fused GCN layer (SpCONV/SpCONV.h:70 calls torch::mm(H.t(), AG)).  The product is a
// reduction over n with a tiny output; a general GEMM picks tiles for large outputs and runs it 20-40 times
// slower than the memory traffic allows.  Here every workgroup streams a contiguous band of rows through LDS
// (coalesced float4 loads), keeps a K1/16 x K2/16 register tile per lane and adds its partial product to C with
// fp32 atomics.  HBM-bound: 4 n (K1 + K2) bytes.
#include "psp_common.h"
#include "spmm_kernel.h"

template <int K1, int K2>
__global__ void __launch_bounds__(256)
psp_atb_kernel(const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, long long n,
               long long rows_per_block)
{
    constexpr int RM = K1 / 16, RN = K2 / 16;
    constexpr int ATB_ROWS = (K1 + K2 > 128) ? 32 : 64;  // at most 32 KB of LDS per workgroup
    __shared__ float sA[ATB_ROWS][K1];
    __shared__ float sB[ATB_ROWS][K2];
    const int t = threadIdx.x;
    const int ti = t >> 4, tj = t & 15;
    float acc[RM][RN];
#pragma unroll
    for (int a = 0; a < RM; a++)
#pragma unroll
        for (int b = 0; b < RN; b++) acc[a][b] = 0.0f;

    const long long r_begin = (long long)blockIdx.x * rows_per_block;
    const long long r_end = r_begin + rows_per_block < n ? r_begin + rows_per_block : n;
    for (long long base = r_begin; base < r_end; base += ATB_ROWS) {
        // stage ATB_ROWS rows of A and B; rows past the end contribute zeros
        for (int v = t; v < ATB_ROWS * K1 / 4; v += 256) {
            const int r = v / (K1 / 4), c4 = v % (K1 / 4);
            psp_f32x4 x = {0.f, 0.f, 0.f, 0.f};
            if (base + r < r_end) x = *(const psp_f32x4 *)(A + (base + r) * K1 + c4 * 4);
            *(psp_f32x4 *)&sA[r][c4 * 4] = x;
        }
        for (int v = t; v < ATB_ROWS * K2 / 4; v += 256) {
            const int r = v / (K2 / 4), c4 = v % (K2 / 4);
            psp_f32x4 x = {0.f, 0.f, 0.f, 0.f};
            if (base + r < r_end) x = *(const psp_f32x4 *)(B + (base + r) * K2 + c4 * 4);
            *(psp_f32x4 *)&sB[r][c4 * 4] = x;
        }
        __syncthreads();
#pragma unroll 8
        for (int r = 0; r < ATB_ROWS; r++) {
            float av[RM], bv[RN];
#pragma unroll
            for (int a = 0; a < RM; a++) av[a] = sA[r][ti + 16 * a];
#pragma unroll
            for (int b = 0; b < RN; b++) bv[b] = sB[r][tj + 16 * b];
#pragma unroll
            for (int a = 0; a < RM; a++)
#pragma unroll
                for (int b = 0; b < RN; b++) acc[a][b] = __builtin_fmaf(av[a], bv[b], acc[a][b]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < RM; a++)
#pragma unroll
        for (int b = 0; b < RN; b++) unsafeAtomicAdd(&C[(ti + 16 * a) * K2 + tj + 16 * b], acc[a][b]);
}

typedef void (*psp_atb_kernel_t)(const float *, const float *, float *, long long, long long);

static psp_atb_kernel_t atb_lookup(int K1, int K2)
{
#define ATB_CASE(a, b) \
    if (K1 == a && K2 == b) return psp_atb_kernel<a, b>;
#define ATB_ROW(a) ATB_CASE(a, 16) ATB_CASE(a, 32) ATB_CASE(a, 48) ATB_CASE(a, 64) ATB_CASE(a, 80) ATB_CASE(a, 96) ATB_CASE(a, 112) ATB_CASE(a, 128)
    ATB_ROW(16) ATB_ROW(32) ATB_ROW(48) ATB_ROW(64) ATB_ROW(80) ATB_ROW(96) ATB_ROW(112) ATB_ROW(128)
#undef ATB_ROW
#undef ATB_CASE
    return nullptr;
}

PSP_EXPORT int psp_gemm_atb_supported(int K1, int K2) { return atb_lookup(K1, K2) != nullptr; }

PSP_EXPORT int psp_gemm_atb_f32(const float *A, const float *B, float *C, long long n, int K1, int K2,
                                psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && K1 >= 1 && K2 >= 1, "gemm_atb: bad size");
    psp_atb_kernel_t k = atb_lookup(K1, K2);
    PSP_REQUIRE(k != nullptr, "gemm_atb: K1 and K2 must be multiples of 16 up to 128 (got %d, %d)", K1, K2);
    PSP_REQUIRE(C != nullptr && (n == 0 || (A && B)), "gemm_atb: null pointer");
    int rc = psp_zero_f32(C, (size_t)K1 * K2, (hipStream_t)stream);
    if (rc != PSP_OK || n == 0) return rc;
    // about 8 workgroups per CU, each on a contiguous band of whole 64-row tiles
    const int ATB_ROWS = 64;
    long long blocks = (n + ATB_ROWS - 1) / ATB_ROWS;
    if (blocks > 2048) blocks = 2048;
    long long rows_per_block = ((n + blocks - 1) / blocks + ATB_ROWS - 1) / ATB_ROWS * ATB_ROWS;
    blocks = (n + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, A, B, C, n, rows_per_block);
    return psp_check_launch("gemm_atb kernel");
}
