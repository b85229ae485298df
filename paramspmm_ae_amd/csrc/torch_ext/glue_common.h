// Shared by the three PyTorch extension modules (ParamSpMM, ParamSDDMM, ParamSpCONV).  The modules own
// argument checking, output allocation and the current-stream lookup; all device work goes through the C ABI
// of libparamsp_hip.so (include/paramsp.h).  No kernels are compiled into the extension modules.
#pragma once
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <hip/hip_runtime_api.h>
#include <vector>
#include "paramsp.h"

namespace pspglue {

// The modules are compiled against include/paramsp.h; a libparamsp_hip.so built from an older header fills smaller
// structs and buffers under the same symbol names.  Called first thing when a module is imported.
inline void check_abi()
{
    TORCH_CHECK(psp_version() >= PSP_ABI_VERSION, "libparamsp_hip.so is version ", psp_version(),
                ", this module was built against ", PSP_ABI_VERSION, ": rebuild the library");
}

// PyTorch-ROCm presents HIP devices under the "cuda" device type; these are its guard / stream types for that.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

// Same contract as the reference's CHECK_INPUT / CHECK_CPU_INPUT (SpMM/SpMM.cpp:5-13): a violation is a
// RuntimeError in Python.  Index tensors must be int32; value / feature tensors float32, or float64 for the
// SpMM / SDDMM operators proper (the reference reaches the same requirement through its int / scalar_t accessors).
inline void need_gpu(const torch::Tensor &t, const char *name)
{
    TORCH_CHECK(t.device().is_cuda(), name, " must be a CUDA tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}
inline void need_cpu(const torch::Tensor &t, const char *name)
{
    TORCH_CHECK(t.device().is_cpu(), name, " must be a CPU tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}
inline void need_i32(const torch::Tensor &t, const char *name)
{
    TORCH_CHECK(t.scalar_type() == torch::kInt32, name, " must be int32");
    TORCH_CHECK(t.dim() == 1, name, " must be 1-D");
}
inline void need_f32(const torch::Tensor &t, const char *name, int dims)
{
    TORCH_CHECK(t.scalar_type() == torch::kFloat32, name, " must be float32 (this build computes in fp32 only)");
    TORCH_CHECK(t.dim() == dims, name, " must be ", dims, "-D");
}
// The six SpMM / six SDDMM operators also take float64, as the reference's dispatch does (SpMM_kernel.cu:149); all
// floating tensors of one call must then agree.
inline void need_fp(const torch::Tensor &t, const char *name, int dims)
{
    TORCH_CHECK(t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kFloat64, name, " must be float32 or float64");
    TORCH_CHECK(t.dim() == dims, name, " must be ", dims, "-D");
}
inline void same_dtype(const torch::Tensor &a, const torch::Tensor &b, const char *what)
{
    TORCH_CHECK(a.scalar_type() == b.scalar_type(), what, ": floating tensors must share one dtype");
}
inline bool is_f64(const torch::Tensor &t) { return t.scalar_type() == torch::kFloat64; }
inline const double *dp(const torch::Tensor &t) { return t.numel() ? t.data_ptr<double>() : nullptr; }
inline double *dpw(torch::Tensor &t) { return t.numel() ? t.data_ptr<double>() : nullptr; }
inline void same_device(const torch::Tensor &a, const torch::Tensor &b, const char *what)
{
    TORCH_CHECK(a.device() == b.device(), what, ": tensors are on different devices");
}

inline void ok(int rc)
{
    TORCH_CHECK(rc >= 0, "libparamsp_hip: ", psp_last_error(), " (status ", rc, ")");
}

inline const int *ip(const torch::Tensor &t) { return t.numel() ? t.data_ptr<int>() : nullptr; }
inline const float *fp(const torch::Tensor &t) { return t.numel() ? t.data_ptr<float>() : nullptr; }
inline float *fpw(torch::Tensor &t) { return t.numel() ? t.data_ptr<float>() : nullptr; }

inline psp_stream_t stream_of(const torch::Tensor &t)
{
    return (psp_stream_t)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// Range checks the device cannot afford: done once per call on the host from tensor sizes only.
inline void check_rowptr_vs(const torch::Tensor &rowPtr, const char *name)
{
    TORCH_CHECK(rowPtr.size(0) >= 1, name, " must have at least one entry");
}

// ---- row split on the host (SpMM/SpMM.cpp:15-75; duplicated in SpCONV/SpCONV.cpp:14-74) -------------
inline std::vector<torch::Tensor> split_csr(torch::Tensor rowPtr, int granularity)
{
    need_cpu(rowPtr, "rowPtr");
    need_i32(rowPtr, "rowPtr");
    check_rowptr_vs(rowPtr, "rowPtr");
    const int n = (int)rowPtr.size(0) - 1;
    const int S = psp_split_csr_count(ip(rowPtr), n, granularity);
    ok(S);
    auto opt = torch::TensorOptions().dtype(torch::kInt32);
    auto rps = torch::empty({(long)S + 1}, opt);
    auto tr = torch::empty({(long)S}, opt);
    ok(psp_split_csr(ip(rowPtr), n, granularity, rps.data_ptr<int>(), S ? tr.data_ptr<int>() : nullptr));
    return {rps, tr};
}

inline std::vector<torch::Tensor> split_csr_par(torch::Tensor rowPtr, torch::Tensor row_split_offset, int granularity)
{
    need_cpu(rowPtr, "rowPtr");
    need_i32(rowPtr, "rowPtr");
    need_cpu(row_split_offset, "row_split_offset");
    need_i32(row_split_offset, "row_split_offset");
    check_rowptr_vs(rowPtr, "rowPtr");
    TORCH_CHECK(row_split_offset.size(0) == rowPtr.size(0), "row_split_offset must have as many entries as rowPtr");
    const int n = (int)rowPtr.size(0) - 1;
    const int S = row_split_offset.data_ptr<int>()[n];
    TORCH_CHECK(S >= 0, "row_split_offset ends negative");
    auto opt = torch::TensorOptions().dtype(torch::kInt32);
    auto rps = torch::empty({(long)S + 1}, opt);
    auto tr = torch::empty({(long)S}, opt);
    ok(psp_split_csr_par(ip(rowPtr), ip(row_split_offset), n, granularity, rps.data_ptr<int>(),
                         S ? tr.data_ptr<int>() : nullptr));
    return {rps, tr};
}

// ---- SpMM into a fresh tensor ------------------------------------------------------------------------
// fmt: 0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split, 4 windowed csr (an addition of this build: rowPtr is the
// [2M + 2] array of psp_window_build, CF selects the kernel variant).  Output rows follow the reference: rows(X) for
// csr formats (zeros_like, SpMM_kernel.cu:136,208), rows(X) rounded up to even for bcsr formats (281-282, 352-353).
inline bool fmt_blocked(int fmt) { return fmt == 2 || fmt == 3; }
inline int fmt_rows(int fmt, const torch::Tensor &rowPtr)
{
    return fmt == 4 ? (int)(rowPtr.size(0) - 2) / 2 : (int)rowPtr.size(0) - 1;
}
inline void check_spmm_args(int fmt, const torch::Tensor &X, const torch::Tensor &rowPtr, const torch::Tensor &colIdx,
                            const torch::Tensor &values, const torch::Tensor *target_row)
{
    need_gpu(X, "input");
    need_gpu(rowPtr, "rowPtr");
    need_gpu(colIdx, "colIdx");
    need_gpu(values, "values");
    need_fp(X, "input", 2);
    need_i32(rowPtr, "rowPtr");
    need_i32(colIdx, "colIdx");
    TORCH_CHECK(fmt >= 0 && fmt <= 4, "format code must be 0..4");
    const bool blocked = fmt_blocked(fmt);
    need_fp(values, "values", blocked ? 2 : 1);
    same_dtype(X, values, "spmm");
    if (blocked) TORCH_CHECK(values.size(1) == 2, "values of a bcsr format must be [nblk, 2]");
    TORCH_CHECK(values.size(0) == colIdx.size(0), "values and colIdx disagree on the number of stored entries");
    check_rowptr_vs(rowPtr, "rowPtr");
    same_device(X, rowPtr, "spmm");
    same_device(X, colIdx, "spmm");
    same_device(X, values, "spmm");
    if (target_row) {
        need_gpu(*target_row, "target_row");
        need_i32(*target_row, "target_row");
        same_device(X, *target_row, "spmm");
        TORCH_CHECK(target_row->size(0) == rowPtr.size(0) - 1, "target_row must have one entry per row segment");
    }
    if (fmt == 4) {
        TORCH_CHECK(rowPtr.size(0) >= 2 && rowPtr.size(0) % 2 == 0, "rowPtr of the windowed format has 2 M + 2 entries");
        TORCH_CHECK(!target_row, "the windowed format has no target_row");
        TORCH_CHECK(X.scalar_type() == torch::kFloat32 && X.size(1) % 4 == 0,
                    "the windowed format takes float32 input whose width is a multiple of 4");
    }
    const long rows = fmt_rows(fmt, rowPtr);
    if (fmt == 0 || fmt == 4) TORCH_CHECK(rows <= X.size(0), "rowPtr describes more rows than input has");
    if (fmt == 2) TORCH_CHECK(2 * rows <= (X.size(0) + 1) / 2 * 2, "rowPtr describes more block-rows than input has");
}

inline void spmm_into(int fmt, torch::Tensor &Y, const torch::Tensor &X, const torch::Tensor &rowPtr,
                      const torch::Tensor &colIdx, const torch::Tensor &values, const torch::Tensor *target_row,
                      int CF, int blkWarpNum)
{
    const int nrows = fmt_rows(fmt, rowPtr), N = (int)X.size(1), rows_out = (int)Y.size(0);
    if (N == 0 || rows_out == 0) return;
    psp_stream_t s = stream_of(X);
    if (fmt == 4) {
        ok(psp_spmm_window_f32(ip(rowPtr), ip(colIdx), fp(values), fp(X), fpw(Y), nrows, (int)colIdx.size(0), N, rows_out, CF, 0,
                               nullptr, s));
        return;
    }
    if (is_f64(X)) {
        ok(psp_spmm_f64(ip(rowPtr), ip(colIdx), dp(values), target_row ? ip(*target_row) : nullptr, dp(X), dpw(Y), nrows, N,
                        rows_out, fmt_blocked(fmt) ? 2 : 1, s));
        return;
    }
    int rc;
    switch (fmt) {
    case 0: rc = psp_spmm_csr_f32(ip(rowPtr), ip(colIdx), fp(values), fp(X), fpw(Y), nrows, N, rows_out, CF, blkWarpNum, s); break;
    case 1: rc = psp_spmm_csr_split_f32(ip(rowPtr), ip(colIdx), fp(values), ip(*target_row), fp(X), fpw(Y), nrows, N, rows_out, CF, blkWarpNum, s); break;
    case 2: rc = psp_spmm_bcsr_f32(ip(rowPtr), ip(colIdx), fp(values), fp(X), fpw(Y), nrows, N, rows_out, CF, blkWarpNum, s); break;
    default: rc = psp_spmm_bcsr_split_f32(ip(rowPtr), ip(colIdx), fp(values), ip(*target_row), fp(X), fpw(Y), nrows, N, rows_out, CF, blkWarpNum, s); break;
    }
    ok(rc);
}

inline torch::Tensor spmm_new(int fmt, const torch::Tensor &X, const torch::Tensor &rowPtr, const torch::Tensor &colIdx,
                              const torch::Tensor &values, const torch::Tensor *target_row, int CF, int blkWarpNum)
{
    check_spmm_args(fmt, X, rowPtr, colIdx, values, target_row);
    pspglue::DeviceGuard guard(X.device());
    const long rows_out = fmt_blocked(fmt) ? (X.size(0) + 1) / 2 * 2 : X.size(0);
    // the library defines every element of Y, so no zero-initialised allocation is needed
    auto Y = torch::empty({rows_out, X.size(1)}, X.options());
    spmm_into(fmt, Y, X, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    return Y;
}

// ---- timing twin: the reference's *_profile loop (SpMM_kernel.cu:576-656) ----------------------------
// `launch` enqueues one complete operation on `stream`.  Returns the mean milliseconds of `iters` launches.
template <class F> inline float time_launches(hipStream_t stream, int warmup, int iters, F launch)
{
    hipEvent_t e0, e1;
    TORCH_CHECK(hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess, "hipEventCreate failed");
    for (int i = 0; i < warmup; i++) launch();
    bool good = hipEventRecord(e0, stream) == hipSuccess;
    for (int i = 0; i < iters; i++) launch();
    good = good && hipEventRecord(e1, stream) == hipSuccess;
    good = good && hipEventSynchronize(e1) == hipSuccess;
    float ms = 0.f;
    good = good && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    TORCH_CHECK(good, "timing the launches failed: ", hipGetErrorString(hipGetLastError()));
    return ms / (float)iters;
}

constexpr int kProfileWarmup = 20;
constexpr int kProfileIters = 200;  // PROFILE in SpMM/SpMM.h:12

inline int gflops(double flops, float ms) { return ms > 0.f ? (int)(flops / 1e6 / (double)ms) : 0; }

}  // namespace pspglue
