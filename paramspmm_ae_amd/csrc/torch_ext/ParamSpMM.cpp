// Python module `ParamSpMM`: the binding surface of the reference's SpMM/SpMM.cpp:891-926, backed by
// libparamsp_hip.so.  Argument order, tensor requirements and return types follow the reference bindings.
#include "glue_common.h"
#include "baseline_rocsparse.h"

using namespace pspglue;
using torch::Tensor;

// ---- the four PCSR SpMM operators (SpMM/SpMM.cpp:77-337) ---------------------------------------------
static Tensor csr_spmm(Tensor input, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return spmm_new(0, input, rowPtr, colIdx, values, nullptr, CF, blkWarpNum);
}
static Tensor csr_split_spmm(Tensor input, Tensor rowPtr_split, Tensor colIdx, Tensor values, Tensor target_row,
                             int CF, int blkWarpNum)
{
    return spmm_new(1, input, rowPtr_split, colIdx, values, &target_row, CF, blkWarpNum);
}
static Tensor bcsr_spmm(Tensor input, Tensor rowPtr_bcsr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return spmm_new(2, input, rowPtr_bcsr, colIdx, values, nullptr, CF, blkWarpNum);
}
static Tensor bcsr_split_spmm(Tensor input, Tensor rowPtr_bcsr_split, Tensor colIdx, Tensor values, Tensor target_row,
                              int CF, int blkWarpNum)
{
    return spmm_new(3, input, rowPtr_bcsr_split, colIdx, values, &target_row, CF, blkWarpNum);
}

// ---- softmax-weighted SpMM (an addition of this build): Y = softmax_rows(e) * X without a separate softmax pass.
// e: scores in CSR order, row_max: an upper bound of every row's scores (ParamSDDMM.*_sddmm_scaled_rowmax delivers
// the maximum).
static Tensor spmm_softmax(int fmt, const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &e,
                           const Tensor &row_max, const Tensor *target_row, int CF, int blkWarpNum)
{
    check_spmm_args(fmt, X, rowPtr, colIdx, e, target_row);
    need_gpu(row_max, "row_max");
    need_f32(row_max, "row_max", 1);
    TORCH_CHECK(row_max.size(0) >= X.size(0) || fmt == 0, "row_max must hold one value per matrix row");
    TORCH_CHECK(X.size(1) % 4 == 0 && ((CF & PSP_CF_NATIVE) ? (CF & 7) < 4 : CF <= 4),
                "softmax-weighted SpMM needs a width that is a multiple of 4 and CF <= 4");
    pspglue::DeviceGuard guard(X.device());
    auto Y = torch::empty_like(X);
    const int nseg = (int)rowPtr.size(0) - 1, N = (int)X.size(1), rows_out = (int)Y.size(0);
    if (N == 0 || rows_out == 0) return Y;
    if (fmt == 0) {
        TORCH_CHECK(row_max.size(0) >= nseg, "row_max must hold one value per matrix row");
        ok(psp_spmm_csr_softmax_f32(ip(rowPtr), ip(colIdx), fp(e), fp(row_max), fp(X), fpw(Y), nseg, N, rows_out, CF,
                                    blkWarpNum, stream_of(X)));
    } else {
        auto row_sum = torch::empty({(long)rows_out}, X.options());
        ok(psp_spmm_csr_split_softmax_f32(ip(rowPtr), ip(colIdx), fp(e), ip(*target_row), fp(row_max), fpw(row_sum), fp(X),
                                          fpw(Y), nseg, N, rows_out, CF, blkWarpNum, stream_of(X)));
    }
    return Y;
}
static Tensor csr_spmm_softmax(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor e, Tensor row_max, int CF, int blkWarpNum)
{
    return spmm_softmax(0, X, rowPtr, colIdx, e, row_max, nullptr, CF, blkWarpNum);
}
static Tensor csr_split_spmm_softmax(Tensor X, Tensor rowPtr_split, Tensor colIdx, Tensor e, Tensor row_max,
                                     Tensor target_row, int CF, int blkWarpNum)
{
    return spmm_softmax(1, X, rowPtr_split, colIdx, e, row_max, &target_row, CF, blkWarpNum);
}

// ---- *_profile twins (SpMM/SpMM.cpp:482-889): mean of 200 launches, int GFLOP/s = 2*nnz*N / t ----------
static int profile_impl(int fmt, const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values,
                        const Tensor *target_row, long nnz, int CF, int blkWarpNum)
{
    check_spmm_args(fmt, X, rowPtr, colIdx, values, target_row);
    pspglue::DeviceGuard guard(X.device());
    const long rows_out = fmt >= 2 ? (X.size(0) + 1) / 2 * 2 : X.size(0);
    auto Y = torch::empty({rows_out, X.size(1)}, X.options());
    hipStream_t s = (hipStream_t)stream_of(X);
    const float ms = time_launches(s, kProfileWarmup, kProfileIters,
                                   [&] { spmm_into(fmt, Y, X, rowPtr, colIdx, values, target_row, CF, blkWarpNum); });
    return gflops(2.0 * (double)nnz * (double)X.size(1), ms);
}
static int csr_spmm_profile(Tensor input, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return profile_impl(0, input, rowPtr, colIdx, values, nullptr, values.size(0), CF, blkWarpNum);
}
static int csr_split_spmm_profile(Tensor input, Tensor rowPtr_split, Tensor colIdx, Tensor values, Tensor target_row,
                                  int CF, int blkWarpNum)
{
    return profile_impl(1, input, rowPtr_split, colIdx, values, &target_row, values.size(0), CF, blkWarpNum);
}
// the blocked twins take the true non-zero count before CF (SpMM/SpMM.cpp:614-621)
static int bcsr_spmm_profile(Tensor input, Tensor rowPtr_bcsr, Tensor colIdx, Tensor values, int nnz, int CF, int blkWarpNum)
{
    return profile_impl(2, input, rowPtr_bcsr, colIdx, values, nullptr, nnz, CF, blkWarpNum);
}
static int bcsr_split_spmm_profile(Tensor input, Tensor rowPtr_bcsr_split, Tensor colIdx, Tensor values,
                                   Tensor target_row, int nnz, int CF, int blkWarpNum)
{
    return profile_impl(3, input, rowPtr_bcsr_split, colIdx, values, &target_row, nnz, CF, blkWarpNum);
}

// ---- explicit timing helper of this build: median-free mean over a caller-chosen iteration count -----
// flush_bytes > 0: every timed launch is preceded by a fill of that many bytes of scratch memory and timed on its
// own (the sum of the launches' own durations is reported), so that the operands come from HBM as they do inside a
// training step; 0 repeats the launch back to back, as the reference's *_profile loop does.
static double spmm_time_ms(int fmt, Tensor input, Tensor rowPtr, Tensor colIdx, Tensor values,
                           c10::optional<Tensor> target_row, int CF, int blkWarpNum, int warmup, int iters,
                           int64_t flush_bytes)
{
    TORCH_CHECK(fmt >= 0 && fmt <= 4, "fmt must be 0 (csr), 1 (csr_split), 2 (bcsr), 3 (bcsr_split) or 4 (windowed csr)");
    TORCH_CHECK((fmt == 1 || fmt == 3) == target_row.has_value(), "target_row must be given exactly for split formats");
    TORCH_CHECK(warmup >= 0 && iters >= 1, "warmup >= 0 and iters >= 1 required");
    const Tensor *tr = target_row.has_value() ? &target_row.value() : nullptr;
    check_spmm_args(fmt, input, rowPtr, colIdx, values, tr);
    pspglue::DeviceGuard guard(input.device());
    const long rows_out = pspglue::fmt_blocked(fmt) ? (input.size(0) + 1) / 2 * 2 : input.size(0);
    auto Y = torch::empty({rows_out, input.size(1)}, input.options());
    hipStream_t s = (hipStream_t)stream_of(input);
    auto launch = [&] { spmm_into(fmt, Y, input, rowPtr, colIdx, values, tr, CF, blkWarpNum); };
    if (flush_bytes <= 0) return (double)time_launches(s, warmup, iters, launch);
    auto scratch = torch::empty({flush_bytes / 4}, input.options().dtype(torch::kFloat32));
    hipEvent_t e0, e1;
    TORCH_CHECK(hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess, "hipEventCreate failed");
    for (int i = 0; i < warmup; i++) launch();
    double total = 0.0;
    bool good = true;
    for (int i = 0; i < iters && good; i++) {
        scratch.fill_((float)i);
        good = good && hipEventRecord(e0, s) == hipSuccess;
        launch();
        good = good && hipEventRecord(e1, s) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
        float ms = 0.f;
        good = good && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
        total += ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    TORCH_CHECK(good, "timing the launches failed: ", hipGetErrorString(hipGetLastError()));
    return total / (double)iters;
}

// ---- generic vec_size x 1 blocks (SpMM/SpMM.cpp:339-480, 757-889) --------------------------------------------------
// The reference instantiates these for vec_size 3 only (SpMM/SpMM.cpp:352,406); values is [nblk, vec_size] and the
// result has the input's rows rounded up to a multiple of vec_size (SpMM_kernel.cu:427-428).  vec_size 2 is accepted
// as well and runs the 2x1 kernels.
static void check_vec_args(const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values,
                           const Tensor *target_row)
{
    need_gpu(X, "input");
    need_gpu(rowPtr, "rowPtr");
    need_gpu(colIdx, "colIdx");
    need_gpu(values, "values");
    need_fp(X, "input", 2);
    need_i32(rowPtr, "rowPtr");
    need_i32(colIdx, "colIdx");
    need_fp(values, "values", 2);
    same_dtype(X, values, "vec_spmm");
    TORCH_CHECK(values.size(1) == 2 || values.size(1) == 3, "vec_spmm: values must be [nblk, 3] (or [nblk, 2]); got vec_size ",
                values.size(1));
    TORCH_CHECK(values.size(0) == colIdx.size(0), "values and colIdx disagree on the number of stored blocks");
    check_rowptr_vs(rowPtr, "rowPtr");
    same_device(X, rowPtr, "vec_spmm");
    same_device(X, colIdx, "vec_spmm");
    same_device(X, values, "vec_spmm");
    const long R = values.size(1), padded = (X.size(0) + R - 1) / R * R;
    if (target_row) {
        need_gpu(*target_row, "target_row");
        need_i32(*target_row, "target_row");
        same_device(X, *target_row, "vec_spmm");
        TORCH_CHECK(target_row->size(0) == rowPtr.size(0) - 1, "target_row must have one entry per row segment");
    } else {
        TORCH_CHECK(R * (rowPtr.size(0) - 1) <= padded, "rowPtr describes more block-rows than input has");
    }
}
static void vec_into(Tensor &Y, const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values,
                     const Tensor *target_row, int CF, int blkWarpNum)
{
    const int nseg = (int)rowPtr.size(0) - 1, N = (int)X.size(1), rows_out = (int)Y.size(0), R = (int)values.size(1);
    if (N == 0 || rows_out == 0) return;
    if (is_f64(X)) {
        ok(psp_spmm_f64(ip(rowPtr), ip(colIdx), dp(values), target_row ? ip(*target_row) : nullptr, dp(X), dpw(Y), nseg, N,
                        rows_out, R, stream_of(X)));
        return;
    }
    if (target_row)
        ok(psp_spmm_vec_split_f32(ip(rowPtr), ip(colIdx), fp(values), ip(*target_row), fp(X), fpw(Y), nseg, N, rows_out, R,
                                  CF, blkWarpNum, stream_of(X)));
    else
        ok(psp_spmm_vec_f32(ip(rowPtr), ip(colIdx), fp(values), fp(X), fpw(Y), nseg, N, rows_out, R, CF, blkWarpNum,
                            stream_of(X)));
}
static Tensor vec_new(const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values,
                      const Tensor *target_row, int CF, int blkWarpNum)
{
    check_vec_args(X, rowPtr, colIdx, values, target_row);
    pspglue::DeviceGuard guard(X.device());
    const long R = values.size(1);
    auto Y = torch::empty({(X.size(0) + R - 1) / R * R, X.size(1)}, X.options());
    vec_into(Y, X, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    return Y;
}
static int vec_profile(const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values,
                       const Tensor *target_row, long nnz, int CF, int blkWarpNum)
{
    check_vec_args(X, rowPtr, colIdx, values, target_row);
    pspglue::DeviceGuard guard(X.device());
    const long R = values.size(1);
    auto Y = torch::empty({(X.size(0) + R - 1) / R * R, X.size(1)}, X.options());
    const float ms = time_launches((hipStream_t)stream_of(X), pspglue::kProfileWarmup, pspglue::kProfileIters,
                                   [&] { vec_into(Y, X, rowPtr, colIdx, values, target_row, CF, blkWarpNum); });
    return gflops(2.0 * (double)nnz * (double)X.size(1), ms);
}
static Tensor vec_spmm(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return vec_new(X, rowPtr, colIdx, values, nullptr, CF, blkWarpNum);
}
static Tensor vec_split_spmm(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor target_row, int CF, int blkWarpNum)
{
    return vec_new(X, rowPtr, colIdx, values, &target_row, CF, blkWarpNum);
}
// the true non-zero count comes before CF, as for the bcsr twins (SpMM/SpMM.cpp:757-765)
static int vec_spmm_profile(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor values, int nnz, int CF, int blkWarpNum)
{
    return vec_profile(X, rowPtr, colIdx, values, nullptr, nnz, CF, blkWarpNum);
}
static int vec_split_spmm_profile(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor target_row, int nnz, int CF,
                                  int blkWarpNum)
{
    return vec_profile(X, rowPtr, colIdx, values, &target_row, nnz, CF, blkWarpNum);
}

// ---- row-caching baseline under the reference's gespmm_* names (SpMM/Baseline_kernel.cu:744-857) ----------------
static void rowcache_into(Tensor &Y, const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values)
{
    ok(psp_baseline_rowcache_spmm_f32(ip(rowPtr), ip(colIdx), fp(values), fp(X), fpw(Y), (int)rowPtr.size(0) - 1,
                                      (int)X.size(1), stream_of(X)));
}
static void check_rowcache_args(const Tensor &X, const Tensor &rowPtr, const Tensor &colIdx, const Tensor &values)
{
    check_spmm_args(0, X, rowPtr, colIdx, values, nullptr);
    TORCH_CHECK(rowPtr.size(0) - 1 <= X.size(0), "gespmm: the matrix has more rows than the dense input");
}
static Tensor gespmm_compute(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor values)
{
    check_rowcache_args(X, rowPtr, colIdx, values);
    pspglue::DeviceGuard guard(X.device());
    auto Y = torch::zeros_like(X);
    rowcache_into(Y, X, rowPtr, colIdx, values);
    return Y;
}
static int gespmm_profile(Tensor X, Tensor rowPtr, Tensor colIdx, Tensor values)
{
    check_rowcache_args(X, rowPtr, colIdx, values);
    pspglue::DeviceGuard guard(X.device());
    auto Y = torch::zeros_like(X);
    const float ms = time_launches((hipStream_t)stream_of(X), pspglue::kProfileWarmup, pspglue::kProfileIters,
                                   [&] { rowcache_into(Y, X, rowPtr, colIdx, values); });
    return (int)(2.0 * (double)values.size(0) * (double)X.size(1) / ((double)ms * 1e-3) / 1e9);
}

// ---- vendor library baselines: the reference's cusparse_* names, served by rocSPARSE (baseline_rocsparse.h) ----
#define PSP_VENDOR(NAME, FMT)                                                                                 \
    static Tensor cusparse_compute##NAME(Tensor X, Tensor ia, Tensor ib, Tensor v) { return vendor_spmm_compute(FMT, X, ia, ib, v); } \
    static int cusparse_profile##NAME(Tensor X, Tensor ia, Tensor ib, Tensor v) { return vendor_spmm_profile(FMT, X, ia, ib, v); }
PSP_VENDOR(, kCsr)
PSP_VENDOR(_csr_alg2, kCsrAlg2)
PSP_VENDOR(_coo_alg4, kCooAlg4)
PSP_VENDOR(_csc, kCsc)

// mean ms per call of the rocSPARSE baseline (format 0 csr, 1 csr load-balanced, 2 coo, 3 csc)
static double vendor_spmm_time_ms(int format, Tensor X, Tensor ia, Tensor ib, Tensor v, int warmup, int iters)
{
    TORCH_CHECK(format >= 0 && format <= 3, "format must be 0..3");
    TORCH_CHECK(warmup >= 0 && iters >= 1, "warmup >= 0 and iters >= 1 required");
    DeviceGuard guard(X.device());
    auto Y = torch::zeros_like(X);
    VendorSpMM op((VendorFormat)format, X, ia, ib, v, Y);
    return (double)time_launches((hipStream_t)stream_of(X), warmup, iters, [&] { op.run(); });
}

// ---- windowed CSR (an addition of this build, include/paramsp.h: psp_window_build / psp_spmm_window_f32) ------------
// [rowPtr_w (2M + 2), colIdx_w, val_w] of a CSR matrix, on the device the arrays live on (CPU tensors: host builder)
static std::vector<Tensor> window_build(Tensor rowPtr, Tensor colIdx, Tensor values)
{
    need_i32(rowPtr, "rowPtr");
    need_i32(colIdx, "colIdx");
    need_f32(values, "values", 1);
    TORCH_CHECK(rowPtr.size(0) >= 1 && values.size(0) == colIdx.size(0), "window_build: array sizes disagree");
    TORCH_CHECK(rowPtr.is_contiguous() && colIdx.is_contiguous() && values.is_contiguous(), "window_build: contiguous arrays");
    pspglue::same_device(rowPtr, colIdx, "window_build");
    pspglue::same_device(rowPtr, values, "window_build");
    const int M = (int)rowPtr.size(0) - 1;
    Tensor rp = torch::empty({2 * (long)M + 2}, rowPtr.options());
    Tensor ci = torch::empty_like(colIdx), v = torch::empty_like(values);
    if (rowPtr.device().is_cpu()) {
        ok(psp_window_build(ip(rowPtr), ip(colIdx), fp(values), M, rp.data_ptr<int>(), colIdx.numel() ? ci.data_ptr<int>() : nullptr,
                            fpw(v)));
    } else {
        DeviceGuard guard(rowPtr.device());
        ok(psp_window_build_dev(ip(rowPtr), ip(colIdx), fp(values), M, rp.data_ptr<int>(),
                                colIdx.numel() ? ci.data_ptr<int>() : nullptr, fpw(v), stream_of(rowPtr)));
    }
    return {rp, ci, v};
}
static Tensor window_spmm(Tensor input, Tensor rowPtr_w, Tensor colIdx_w, Tensor values_w, int variant)
{
    return pspglue::spmm_new(4, input, rowPtr_w, colIdx_w, values_w, nullptr, variant, 4);
}
static py::dict window_plan(int N, int variant)
{
    int tn = 0, rb = 0, lds = 0;
    const int v = psp_spmm_window_plan(N, variant, &tn, &rb, &lds);
    ok(v);
    py::dict d;
    d["variant"] = v;
    d["tile_cols"] = tn;
    d["rows_per_block"] = rb;
    d["lds_bytes"] = lds;
    return d;
}

static py::dict spmm_plan(int N, int CF, int blkWarpNum)
{
    psp_spmm_plan p;
    ok(psp_spmm_plan_for(N, CF, blkWarpNum, &p));
    py::dict d;
    d["vec"] = p.vec;
    d["coarsen"] = p.coarsen;
    d["lanes_per_row"] = p.lanes_per_row;
    d["rows_per_wave"] = p.rows_per_wave;
    d["unroll"] = p.unroll;
    d["col_tiles"] = p.col_tiles;
    d["waves_per_block"] = p.waves_per_block;
    d["log_segs_per_wave"] = p.log_segs_per_wave;
    d["even_split"] = p.even_split;
    d["xcd_stripe_rows"] = p.xcd_stripe_rows;
    d["register_sets"] = psp_spmm_register_sets(p.unroll, p.lanes_per_row);  // which kernel variant the plan launches
    return d;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    pspglue::check_abi();
    m.def("window_build", &window_build, "windowed CSR of a CSR matrix: (rowPtr, colIdx, values) -> [rowPtr_w, colIdx_w, values_w]");
    m.def("window_spmm", &window_spmm, "windowed CSR SpMM (HIP, gfx950): (X, rowPtr_w, colIdx_w, values_w, variant)");
    m.def("window_plan", &window_plan, "(N, variant) -> tile width, rows per workgroup, LDS bytes of the windowed kernel");
    m.def("split_csr", &pspglue::split_csr, "row split on the host (CPU int32 rowPtr, granularity)");
    m.def("split_csr_par", &pspglue::split_csr_par, "row split on the host with a precomputed segment prefix");
    m.def("csr_spmm", &csr_spmm, "CSR SpMM (HIP, gfx950)");
    m.def("csr_split_spmm", &csr_split_spmm, "row-split CSR SpMM (HIP, gfx950)");
    m.def("bcsr_spmm", &bcsr_spmm, "2x1 BCSR SpMM (HIP, gfx950)");
    m.def("bcsr_split_spmm", &bcsr_split_spmm, "row-split 2x1 BCSR SpMM (HIP, gfx950)");
    m.def("vec_spmm", &vec_spmm, "3x1-block SpMM (HIP, gfx950)");
    m.def("vec_split_spmm", &vec_split_spmm, "row-split 3x1-block SpMM (HIP, gfx950)");
    m.def("csr_spmm_profile", &csr_spmm_profile, "GFLOP/s of csr_spmm");
    m.def("csr_split_spmm_profile", &csr_split_spmm_profile, "GFLOP/s of csr_split_spmm");
    m.def("bcsr_spmm_profile", &bcsr_spmm_profile, "GFLOP/s of bcsr_spmm");
    m.def("bcsr_split_spmm_profile", &bcsr_split_spmm_profile, "GFLOP/s of bcsr_split_spmm");
    m.def("vec_spmm_profile", &vec_spmm_profile, "GFLOP/s of vec_spmm");
    m.def("vec_split_spmm_profile", &vec_split_spmm_profile, "GFLOP/s of vec_split_spmm");
    m.def("cusparse_compute", &cusparse_compute, "rocSPARSE SpMM baseline");
    m.def("cusparse_profile", &cusparse_profile, "GFLOP/s of the rocSPARSE SpMM baseline");
    m.def("cusparse_compute_csr_alg2", &cusparse_compute_csr_alg2, "rocSPARSE SpMM baseline");
    m.def("cusparse_profile_csr_alg2", &cusparse_profile_csr_alg2, "GFLOP/s of the rocSPARSE SpMM baseline");
    m.def("cusparse_compute_coo_alg4", &cusparse_compute_coo_alg4, "rocSPARSE SpMM baseline");
    m.def("cusparse_profile_coo_alg4", &cusparse_profile_coo_alg4, "GFLOP/s of the rocSPARSE SpMM baseline");
    m.def("cusparse_compute_csc", &cusparse_compute_csc, "rocSPARSE SpMM baseline");
    m.def("cusparse_profile_csc", &cusparse_profile_csc, "GFLOP/s of the rocSPARSE SpMM baseline");
    m.def("gespmm_compute", &gespmm_compute, "row-caching CSR SpMM baseline (one wavefront per row)");
    m.def("gespmm_profile", &gespmm_profile, "GFLOP/s of the row-caching baseline");
    // additions of this build
    m.def("csr_spmm_softmax", &csr_spmm_softmax, "softmax_rows(e) * X: (X, rowPtr, colIdx, e, row_max, CF, blkWarpNum)");
    m.def("csr_split_spmm_softmax", &csr_split_spmm_softmax,
          "the same on the row-split format: (X, rowPtr_split, colIdx, e, row_max, target_row, CF, blkWarpNum)");
    m.def("spmm_time_ms", &spmm_time_ms, "mean ms per launch: (fmt, X, rowPtr, colIdx, val, target_row|None, CF, bw, warmup, iters, flush_bytes=0)",
          py::arg("fmt"), py::arg("X"), py::arg("rowPtr"), py::arg("colIdx"), py::arg("val"), py::arg("target_row"), py::arg("CF"),
          py::arg("blkWarpNum"), py::arg("warmup"), py::arg("iters"), py::arg("flush_bytes") = 0);
    m.def("vendor_spmm_time_ms", &vendor_spmm_time_ms, "mean ms per rocSPARSE SpMM: (format, X, idx_a, idx_b, val, warmup, iters)");
    m.def("spmm_plan", &spmm_plan, "how (N, CF, blkWarpNum) maps onto the wave64 kernel");
}
