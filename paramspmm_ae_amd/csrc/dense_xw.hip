// Y[n,K2] = X[n,K1] * W  (W [K1,K2] row-major)  or  X * W^T  (W [K2,K1] row-major) for tall-skinny X (n ~ 10^6) and a
// small weight matrix: the dense products around the sparse one in the fused GCN layer, torch::mm(H, W) and
// torch::mm(AG, W.t()) in SpCONV/SpCONV.h:43-71.  The work is reading X and writing Y once; a general GEMM reaches a
// third of the memory rate at these shapes (98 us for 1M x 16 x 16 where the traffic needs 30 us).
//
// One lane per row.  The row of X streams through registers four floats at a time, the K2 sums stay in registers,
// and W is addressed with compile-time indices only, so the compiler fetches it with scalar loads and feeds it to
// the FMAs as a scalar operand: the inner loop is FMAs and nothing else.  The loads of a wavefront touch every
// 128-byte line of its 64 consecutive rows; the lines are fetched once and the remaining accesses hit in L1.
#include "psp_common.h"
#include "spmm_kernel.h"

// RELU_X: X enters the product as max(x, 0) (the activation between two layers, applied as the next layer reads its
// input).  MASK: an output element is kept where the same element of `mask` is positive and zero elsewhere (the
// activation's backward, applied as the gradient with respect to the layer's input is written).
template <int K1, int K2, bool TRANS, bool RELU_X, bool MASK>
__global__ void __launch_bounds__(256)
psp_xw_kernel(const float *__restrict__ X, const float *__restrict__ W, float *__restrict__ Y, long long n,
              const float *__restrict__ mask)
{
    const long long row = (long long)blockIdx.x * 256 + threadIdx.x;
    if (row >= n) return;
    const psp_f32x4 *xr = (const psp_f32x4 *)(X + row * K1);
    float acc[K2];
#pragma unroll
    for (int j = 0; j < K2; j++) acc[j] = 0.0f;
#pragma unroll
    for (int k4 = 0; k4 < K1 / 4; k4++) {
        psp_f32x4 x = xr[k4];
        if constexpr (RELU_X) {
#pragma unroll
            for (int kk = 0; kk < 4; kk++) x[kk] = x[kk] < 0.0f ? 0.0f : x[kk];  // NaN stays NaN, as with torch.relu
        }
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int k = k4 * 4 + kk;
#pragma unroll
            for (int j = 0; j < K2; j++) acc[j] = __builtin_fmaf(x[kk], TRANS ? W[j * K1 + k] : W[k * K2 + j], acc[j]);
        }
    }
    psp_f32x4 *yr = (psp_f32x4 *)(Y + row * K2);
    const psp_f32x4 *mr = (const psp_f32x4 *)(mask + row * K2);
#pragma unroll
    for (int j4 = 0; j4 < K2 / 4; j4++) {
        psp_f32x4 o = {acc[4 * j4], acc[4 * j4 + 1], acc[4 * j4 + 2], acc[4 * j4 + 3]};
        if constexpr (MASK) {
            const psp_f32x4 m = mr[j4];
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = m[e] > 0.0f ? o[e] : 0.0f;
        }
        yr[j4] = o;
    }
}

typedef void (*psp_xw_kernel_t)(const float *, const float *, float *, long long, const float *);

// K2 (the sums a lane holds) is 16 or 32; K1 * K2 FMAs are unrolled, up to 2048.  The forward product exists plain
// and with the activation on its input, the transposed (backward) one plain and with the mask on its output.
static psp_xw_kernel_t xw_lookup(int K1, int K2, bool trans, bool relu_x, bool mask)
{
    if ((trans && relu_x) || (!trans && mask)) return nullptr;
#define XW_CASE(A_, B_)                                                                               \
    if (K1 == A_ && K2 == B_) {                                                                       \
        if (trans) return mask ? psp_xw_kernel<A_, B_, true, false, true> : psp_xw_kernel<A_, B_, true, false, false>; \
        return relu_x ? psp_xw_kernel<A_, B_, false, true, false> : psp_xw_kernel<A_, B_, false, false, false>;      \
    }
    XW_CASE(16, 16) XW_CASE(32, 16) XW_CASE(48, 16) XW_CASE(64, 16) XW_CASE(128, 16)
    XW_CASE(16, 32) XW_CASE(32, 32) XW_CASE(48, 32) XW_CASE(64, 32)
#undef XW_CASE
    return nullptr;
}

// dense_xw_wide.hip: 64 and 128 output columns on the matrix cores
bool psp_xw_wide_supported(int K1, int K2);
int psp_xw_wide_launch(const float *X, const float *W, float *Y, long long n, int K1, int K2, int transW, int relu_x,
                       const float *mask, hipStream_t stream);

PSP_EXPORT int psp_gemm_xw_supported(int K1, int K2)
{
    return xw_lookup(K1, K2, false, false, false) != nullptr || psp_xw_wide_supported(K1, K2);
}

PSP_EXPORT int psp_gemm_xw_act_f32(const float *X, const float *W, float *Y, long long n, int K1, int K2, int transW,
                                   int relu_x, const float *mask, psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && K1 >= 1 && K2 >= 1, "gemm_xw: bad size");
    PSP_REQUIRE(!(transW && relu_x), "gemm_xw: the activation on X exists for the plain product only");
    PSP_REQUIRE(!(!transW && mask), "gemm_xw: the output mask exists for the transposed product only");
    psp_xw_kernel_t k = xw_lookup(K1, K2, transW != 0, relu_x != 0, mask != nullptr);
    const bool wide = k == nullptr && psp_xw_wide_supported(K1, K2);
    PSP_REQUIRE(k != nullptr || wide, "gemm_xw: unsupported widths %d x %d (see psp_gemm_xw_supported)", K1, K2);
    if (n == 0) return PSP_OK;
    PSP_REQUIRE(X && W && Y, "gemm_xw: null pointer");
    PSP_REQUIRE((((size_t)X | (size_t)Y | (size_t)mask) & 15) == 0, "gemm_xw: X, Y and mask must be 16-byte aligned");
    PSP_REQUIRE((n + 255) / 256 <= 0x7fffffffLL, "gemm_xw: too many rows");
    if (wide) return psp_xw_wide_launch(X, W, Y, n, K1, K2, transW, relu_x, mask, (hipStream_t)stream);
    hipLaunchKernelGGL(k, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, X, W, Y, n, mask);
    return psp_check_launch("gemm_xw kernel");
}

PSP_EXPORT int psp_gemm_xw_f32(const float *X, const float *W, float *Y, long long n, int K1, int K2, int transW,
                               psp_stream_t stream)
{
    return psp_gemm_xw_act_f32(X, W, Y, n, K1, K2, transW, 0, nullptr, stream);
}
