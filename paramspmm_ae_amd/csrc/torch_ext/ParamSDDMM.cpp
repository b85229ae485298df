// Python module `ParamSDDMM`: the binding surface of the reference's SDDMM/sddmm.cpp:675-701, backed by
// libparamsp_hip.so.
#include "glue_common.h"
#include "baseline_rocsparse.h"

using namespace pspglue;
using torch::Tensor;

// fmt: 0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split
static void check_sddmm_args(int fmt, const Tensor &A, const Tensor &B, const Tensor &rowPtr, const Tensor &colIdx,
                             const Tensor &values, const Tensor *target_row, int CF, int blkWarpNum)
{
    need_gpu(A, "A");
    need_gpu(B, "B");
    need_gpu(rowPtr, "rowPtr");
    need_gpu(colIdx, "colIdx");
    need_gpu(values, "values");
    need_fp(A, "A", 2);
    need_fp(B, "B", 2);
    need_i32(rowPtr, "rowPtr");
    need_i32(colIdx, "colIdx");
    const bool blocked = fmt >= 2;
    need_fp(values, "values", blocked ? 2 : 1);
    same_dtype(A, B, "sddmm");
    same_dtype(A, values, "sddmm");
    if (blocked) TORCH_CHECK(values.size(1) == 2, "values of a bcsr format must be [nblk, 2]");
    TORCH_CHECK(values.size(0) == colIdx.size(0), "values and colIdx disagree on the number of stored entries");
    TORCH_CHECK(A.size(1) == B.size(1), "A and B must have the same number of columns");
    TORCH_CHECK(A.size(1) >= 1, "A and B need at least one column");
    check_rowptr_vs(rowPtr, "rowPtr");
    same_device(A, B, "sddmm");
    same_device(A, rowPtr, "sddmm");
    same_device(A, colIdx, "sddmm");
    same_device(A, values, "sddmm");
    // the reference dispatches CF 1..4 only (SDDMM/sddmm.cpp:31-43); wider K is accepted here, CF stays a
    // checked argument so that a caller's mistake still surfaces
    TORCH_CHECK(CF >= 1 && CF <= 8, "CF must be 1..8");
    TORCH_CHECK((blkWarpNum & ~(PSP_BW_BALANCED | PSP_BW_STRIPE_MASK)) == 4 || (blkWarpNum & ~(PSP_BW_BALANCED | PSP_BW_STRIPE_MASK)) == 8, "blkWarpNum must be 4 or 8");
    const long rows = rowPtr.size(0) - 1;
    if (target_row) {
        need_gpu(*target_row, "target_row");
        need_i32(*target_row, "target_row");
        same_device(A, *target_row, "sddmm");
        TORCH_CHECK(target_row->size(0) == rows, "target_row must have one entry per row segment");
    }
    if (fmt == 0) TORCH_CHECK(rows <= A.size(0), "rowPtr describes more rows than A has");
    if (fmt == 2) TORCH_CHECK(2 * rows <= A.size(0), "A needs two rows per block-row (pad it to an even row count)");
    // Row-split block format: the segments do not say how many block-rows there are, but the matrix is square
    // (B has one row per column, as everywhere in the reference), and the kernel reads both rows of a block-row
    // whatever the block values are.  So A must cover B's rows rounded up to whole blocks.
    if (fmt == 3)
        TORCH_CHECK(A.size(0) % 2 == 0 && A.size(0) >= (B.size(0) + 1) / 2 * 2,
                    "A needs two rows per block-row: pad it to an even row count of at least ", (B.size(0) + 1) / 2 * 2);
}

static Tensor sddmm_new(int fmt, const Tensor &A, const Tensor &B, const Tensor &rowPtr, const Tensor &colIdx,
                        const Tensor &values, const Tensor *target_row, const Tensor *scale, int CF, int blkWarpNum)
{
    check_sddmm_args(fmt, A, B, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    pspglue::DeviceGuard guard(A.device());
    auto out = torch::empty_like(values);  // every stored entry is written by the kernel
    const int nrows = (int)rowPtr.size(0) - 1, K = (int)A.size(1);
    if (values.numel() == 0) return out;
    psp_stream_t s = stream_of(A);
    if (is_f64(A)) {
        TORCH_CHECK(!scale, "the scaled SDDMM variants are float32 only");
        ok(psp_sddmm_f64(ip(rowPtr), ip(colIdx), fmt >= 2 ? dp(values) : nullptr, target_row ? ip(*target_row) : nullptr, dp(A),
                         dp(B), dpw(out), nrows, K, fmt >= 2 ? 2 : 1, s));
        return out;
    }
    int rc;
    switch (fmt) {
    case 0: rc = psp_sddmm_csr_f32(ip(rowPtr), ip(colIdx), fp(A), fp(B), scale ? fp(*scale) : nullptr, fpw(out), nrows, K, blkWarpNum, s); break;
    case 1: rc = psp_sddmm_csr_split_f32(ip(rowPtr), ip(colIdx), ip(*target_row), fp(A), fp(B), scale ? fp(*scale) : nullptr, fpw(out), nrows, K, blkWarpNum, s); break;
    case 2: rc = psp_sddmm_bcsr_f32(ip(rowPtr), ip(colIdx), fp(values), fp(A), fp(B), fpw(out), nrows, K, blkWarpNum, s); break;
    default: rc = psp_sddmm_bcsr_split_f32(ip(rowPtr), ip(colIdx), fp(values), ip(*target_row), fp(A), fp(B), fpw(out), nrows, K, blkWarpNum, s); break;
    }
    ok(rc);
    return out;
}

static Tensor csr_sddmm(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return sddmm_new(0, A, B, rowPtr, colIdx, values, nullptr, nullptr, CF, blkWarpNum);
}
static Tensor csr_split_sddmm(Tensor A, Tensor B, Tensor rowPtr_split, Tensor colIdx, Tensor values, Tensor target_row,
                              int CF, int blkWarpNum)
{
    return sddmm_new(1, A, B, rowPtr_split, colIdx, values, &target_row, nullptr, CF, blkWarpNum);
}
static Tensor bcsr_sddmm(Tensor A, Tensor B, Tensor rowPtr_bcsr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return sddmm_new(2, A, B, rowPtr_bcsr, colIdx, values, nullptr, nullptr, CF, blkWarpNum);
}
static Tensor bcsr_split_sddmm(Tensor A, Tensor B, Tensor rowPtr_bcsr_split, Tensor colIdx, Tensor values,
                               Tensor target_row, int CF, int blkWarpNum)
{
    return sddmm_new(3, A, B, rowPtr_bcsr_split, colIdx, values, &target_row, nullptr, CF, blkWarpNum);
}

// SDDMM over the windowed layout (ParamSpMM.window_build): out[p] = alpha <A[row], B[col]> in the layout's entry order.
// alpha: a one-element float32 tensor on the device, or None.  Passing the same tensor for A and B reads it once.
static bool window_sddmm_supported(long K) { return K >= 4 && K % 4 == 0 && K <= PSP_SDDMM_WINDOW_MAX_K; }
static Tensor window_sddmm(Tensor A, Tensor B, Tensor rowPtr_w, Tensor colIdx_w, c10::optional<Tensor> alpha)
{
    need_gpu(A, "A");
    need_gpu(B, "B");
    need_gpu(rowPtr_w, "rowPtr_w");
    need_gpu(colIdx_w, "colIdx_w");
    need_f32(A, "A", 2);
    need_f32(B, "B", 2);
    need_i32(rowPtr_w, "rowPtr_w");
    need_i32(colIdx_w, "colIdx_w");
    same_device(A, B, "window_sddmm");
    same_device(A, rowPtr_w, "window_sddmm");
    same_device(A, colIdx_w, "window_sddmm");
    TORCH_CHECK(rowPtr_w.size(0) >= 2 && rowPtr_w.size(0) % 2 == 0, "rowPtr of the windowed format has 2 M + 2 entries");
    TORCH_CHECK(A.size(1) == B.size(1) && window_sddmm_supported(A.size(1)),
                "window_sddmm: A and B need the same number of columns, a multiple of 4 up to ", PSP_SDDMM_WINDOW_MAX_K);
    const long M = (rowPtr_w.size(0) - 2) / 2;
    TORCH_CHECK(M <= A.size(0), "rowPtr_w describes more rows than A has");
    if (alpha) {
        need_gpu(*alpha, "alpha");
        TORCH_CHECK(alpha->scalar_type() == torch::kFloat32 && alpha->numel() == 1, "alpha is one float32 on the device");
        same_device(A, *alpha, "window_sddmm");
    }
    pspglue::DeviceGuard guard(A.device());
    auto out = torch::empty({colIdx_w.size(0)}, A.options());
    if (colIdx_w.numel() == 0) return out;
    ok(psp_sddmm_window_f32(ip(rowPtr_w), ip(colIdx_w), fp(A), fp(B), alpha ? alpha->data_ptr<float>() : nullptr, fpw(out), (int)M,
                            (int)colIdx_w.size(0), (int)A.size(1), (int)B.size(0), stream_of(A)));
    return out;
}

// out[p] = values[p] * <A[row], B[col]>: the attention-score form (an addition of this build; the reference op
// never multiplies the stored value in)
static Tensor csr_sddmm_scaled(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, int blkWarpNum)
{
    return sddmm_new(0, A, B, rowPtr, colIdx, values, nullptr, &values, 1, blkWarpNum);
}

static Tensor csr_split_sddmm_scaled(Tensor A, Tensor B, Tensor rowPtr_split, Tensor colIdx, Tensor values,
                                     Tensor target_row, int blkWarpNum)
{
    return sddmm_new(1, A, B, rowPtr_split, colIdx, values, &target_row, &values, 1, blkWarpNum);
}

// The scaled scores together with the largest score of every row (fed to ParamSpMM.*_spmm_softmax, which then needs
// no separate softmax pass).  rows: number of matrix rows (the row-split format does not say).
static std::vector<Tensor> sddmm_scaled_rowmax(int fmt, const Tensor &A, const Tensor &B, const Tensor &rowPtr,
                                               const Tensor &colIdx, const Tensor &values, const Tensor *target_row,
                                               long rows, int blkWarpNum)
{
    check_sddmm_args(fmt, A, B, rowPtr, colIdx, values, target_row, 1, blkWarpNum);
    TORCH_CHECK(rows >= 0 && rows <= 0x7fffffffL, "rows out of range");
    pspglue::DeviceGuard guard(A.device());
    auto out = torch::empty_like(values);
    auto row_max = torch::empty({rows}, values.options());
    const int nseg = (int)rowPtr.size(0) - 1, K = (int)A.size(1);
    psp_stream_t s = stream_of(A);
    if (fmt == 0) {
        TORCH_CHECK(rows == nseg, "rows must equal the number of CSR rows");
        ok(psp_sddmm_csr_rowmax_f32(ip(rowPtr), ip(colIdx), fp(A), fp(B), fp(values), fpw(out), fpw(row_max), nseg, K,
                                    blkWarpNum, s));
    } else {
        ok(psp_sddmm_csr_split_rowmax_f32(ip(rowPtr), ip(colIdx), ip(*target_row), fp(A), fp(B), fp(values), fpw(out),
                                          fpw(row_max), nseg, (int)rows, K, blkWarpNum, s));
    }
    return {out, row_max};
}
static std::vector<Tensor> csr_sddmm_scaled_rowmax(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values,
                                                   int blkWarpNum)
{
    return sddmm_scaled_rowmax(0, A, B, rowPtr, colIdx, values, nullptr, rowPtr.size(0) - 1, blkWarpNum);
}
static std::vector<Tensor> csr_split_sddmm_scaled_rowmax(Tensor A, Tensor B, Tensor rowPtr_split, Tensor colIdx,
                                                         Tensor values, Tensor target_row, long rows, int blkWarpNum)
{
    return sddmm_scaled_rowmax(1, A, B, rowPtr_split, colIdx, values, &target_row, rows, blkWarpNum);
}

// ---- *_profile twins (SDDMM/sddmm.cpp:338-661): int GFLOP/s = 2*nnz*K / t -------------------------------
static int profile_impl(int fmt, const Tensor &A, const Tensor &B, const Tensor &rowPtr, const Tensor &colIdx,
                        const Tensor &values, const Tensor *target_row, long nnz, int CF, int blkWarpNum)
{
    check_sddmm_args(fmt, A, B, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    pspglue::DeviceGuard guard(A.device());
    hipStream_t s = (hipStream_t)stream_of(A);
    const float ms = time_launches(s, kProfileWarmup, kProfileIters, [&] {
        (void)sddmm_new(fmt, A, B, rowPtr, colIdx, values, target_row, nullptr, CF, blkWarpNum);
    });
    return gflops(2.0 * (double)nnz * (double)A.size(1), ms);
}
static int csr_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return profile_impl(0, A, B, rowPtr, colIdx, values, nullptr, values.size(0), CF, blkWarpNum);
}
static int csr_split_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor target_row,
                                   int CF, int blkWarpNum)
{
    return profile_impl(1, A, B, rowPtr, colIdx, values, &target_row, values.size(0), CF, blkWarpNum);
}
static int bcsr_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, int nnz, int CF, int blkWarpNum)
{
    return profile_impl(2, A, B, rowPtr, colIdx, values, nullptr, nnz, CF, blkWarpNum);
}
static int bcsr_split_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor target_row,
                                    int nnz, int CF, int blkWarpNum)
{
    return profile_impl(3, A, B, rowPtr, colIdx, values, &target_row, nnz, CF, blkWarpNum);
}

// ---- genmask (SDDMM/sddmm.cpp:663-673) -------------------------------------------------------------------
static Tensor genmask(Tensor rowPtr_bcsr, Tensor rowPtr, Tensor blkval, int nnz)
{
    need_gpu(rowPtr_bcsr, "rowPtr_bcsr");
    need_gpu(rowPtr, "rowPtr");
    need_gpu(blkval, "blkval");
    need_i32(rowPtr_bcsr, "rowPtr_bcsr");
    need_i32(rowPtr, "rowPtr");
    need_f32(blkval, "blkval", 2);
    TORCH_CHECK(blkval.size(1) == 2, "blkval must be [nblk, 2]");
    TORCH_CHECK(nnz >= 0, "nnz must not be negative");
    same_device(rowPtr, rowPtr_bcsr, "genmask");
    same_device(rowPtr, blkval, "genmask");
    check_rowptr_vs(rowPtr_bcsr, "rowPtr_bcsr");
    const int nbr = (int)rowPtr_bcsr.size(0) - 1;
    // block-row t reads rowPtr[2t] and rowPtr[2t+1]
    TORCH_CHECK(rowPtr.size(0) >= 2L * nbr, "rowPtr is too short for the block row pointer");
    pspglue::DeviceGuard guard(rowPtr.device());
    auto mask = torch::empty({(long)nnz}, rowPtr.options());
    ok(psp_genmask(ip(rowPtr_bcsr), ip(rowPtr), fp(blkval), nbr, nnz, nnz ? mask.data_ptr<int>() : nullptr, stream_of(rowPtr)));
    return mask;
}

// ---- row softmax over stored entries (an addition of this build) --------------------------------------
static Tensor segment_softmax(Tensor rowPtr, Tensor e)
{
    need_gpu(rowPtr, "rowPtr");
    need_gpu(e, "e");
    need_i32(rowPtr, "rowPtr");
    need_f32(e, "e", 1);
    same_device(rowPtr, e, "segment_softmax");
    check_rowptr_vs(rowPtr, "rowPtr");
    pspglue::DeviceGuard guard(e.device());
    TORCH_CHECK(e.numel() <= 0x7fffffffLL, "segment_softmax: more than 2^31-1 entries");
    auto out = torch::empty_like(e);
    // the (max, sum) pairs of rows long enough to be spread over several workgroups
    auto ws = torch::empty({2 * (rowPtr.size(0) - 1)}, e.options());
    ok(psp_segment_softmax_ws_f32(ip(rowPtr), fp(e), fpw(out), (int)rowPtr.size(0) - 1, (int)e.numel(), fpw(ws),
                                  stream_of(e)));
    return out;
}

// ---- generic vec_size x 1 blocks (SDDMM/sddmm.cpp:221-336, 547-661): values [nblk, vec_size] -> out [nblk, vec_size].
// The reference instantiates vec_size 3 only, and those kernels are never run (they stride their shared memory by
// CF*2 instead of CF*vec_size); this is their evident intent: the 2x1 rule for each entry of a block.
static void check_vec_sddmm_args(const Tensor &A, const Tensor &B, const Tensor &rowPtr, const Tensor &colIdx,
                                 const Tensor &values, const Tensor *target_row, int CF, int blkWarpNum)
{
    need_gpu(A, "A");
    need_gpu(B, "B");
    need_gpu(rowPtr, "rowPtr");
    need_gpu(colIdx, "colIdx");
    need_gpu(values, "values");
    need_fp(A, "A", 2);
    need_fp(B, "B", 2);
    need_i32(rowPtr, "rowPtr");
    need_i32(colIdx, "colIdx");
    need_fp(values, "values", 2);
    same_dtype(A, B, "vec_sddmm");
    same_dtype(A, values, "vec_sddmm");
    TORCH_CHECK(values.size(1) == 2 || values.size(1) == 3, "vec_sddmm: values must be [nblk, 3] (or [nblk, 2]); got vec_size ",
                values.size(1));
    TORCH_CHECK(values.size(0) == colIdx.size(0), "values and colIdx disagree on the number of stored blocks");
    TORCH_CHECK(A.size(1) == B.size(1) && A.size(1) >= 1, "A and B must have the same, non-zero number of columns");
    check_rowptr_vs(rowPtr, "rowPtr");
    same_device(A, B, "vec_sddmm");
    same_device(A, rowPtr, "vec_sddmm");
    same_device(A, colIdx, "vec_sddmm");
    same_device(A, values, "vec_sddmm");
    TORCH_CHECK(CF >= 1 && CF <= 8, "CF must be 1..8");
    TORCH_CHECK((blkWarpNum & ~(PSP_BW_BALANCED | PSP_BW_STRIPE_MASK)) == 4 || (blkWarpNum & ~(PSP_BW_BALANCED | PSP_BW_STRIPE_MASK)) == 8, "blkWarpNum must be 4 or 8");
    if (target_row) {
        need_gpu(*target_row, "target_row");
        need_i32(*target_row, "target_row");
        same_device(A, *target_row, "vec_sddmm");
        TORCH_CHECK(target_row->size(0) == rowPtr.size(0) - 1, "target_row must have one entry per row segment");
        // square matrix: A must cover B's rows rounded up to whole blocks (the kernel reads every row of a block-row)
        const long R = values.size(1), need = (B.size(0) + R - 1) / R * R;
        TORCH_CHECK(A.size(0) % R == 0 && A.size(0) >= need, "A needs vec_size rows per block-row: pad it to a multiple of ", R,
                    " of at least ", need);
    } else {
        TORCH_CHECK(values.size(1) * (rowPtr.size(0) - 1) <= A.size(0), "A needs vec_size rows per block-row (pad it)");
    }
}
static Tensor vec_sddmm_new(const Tensor &A, const Tensor &B, const Tensor &rowPtr, const Tensor &colIdx,
                            const Tensor &values, const Tensor *target_row, int CF, int blkWarpNum)
{
    check_vec_sddmm_args(A, B, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    pspglue::DeviceGuard guard(A.device());
    auto out = torch::empty_like(values);
    if (values.numel() == 0) return out;
    const int nseg = (int)rowPtr.size(0) - 1, K = (int)A.size(1), R = (int)values.size(1);
    if (is_f64(A)) {
        ok(psp_sddmm_f64(ip(rowPtr), ip(colIdx), dp(values), target_row ? ip(*target_row) : nullptr, dp(A), dp(B), dpw(out),
                         nseg, K, R, stream_of(A)));
        return out;
    }
    if (target_row)
        ok(psp_sddmm_vec_split_f32(ip(rowPtr), ip(colIdx), fp(values), ip(*target_row), fp(A), fp(B), fpw(out), nseg, K, R,
                                   blkWarpNum, stream_of(A)));
    else
        ok(psp_sddmm_vec_f32(ip(rowPtr), ip(colIdx), fp(values), fp(A), fp(B), fpw(out), nseg, K, R, blkWarpNum, stream_of(A)));
    return out;
}
static int vec_sddmm_profile_impl(const Tensor &A, const Tensor &B, const Tensor &rowPtr, const Tensor &colIdx,
                                  const Tensor &values, const Tensor *target_row, long nnz, int CF, int blkWarpNum)
{
    check_vec_sddmm_args(A, B, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    pspglue::DeviceGuard guard(A.device());
    const float ms = time_launches((hipStream_t)stream_of(A), kProfileWarmup, kProfileIters, [&] {
        (void)vec_sddmm_new(A, B, rowPtr, colIdx, values, target_row, CF, blkWarpNum);
    });
    return gflops(2.0 * (double)nnz * (double)A.size(1), ms);
}
static Tensor vec_sddmm(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, int CF, int blkWarpNum)
{
    return vec_sddmm_new(A, B, rowPtr, colIdx, values, nullptr, CF, blkWarpNum);
}
static Tensor vec_split_sddmm(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor target_row, int CF,
                              int blkWarpNum)
{
    return vec_sddmm_new(A, B, rowPtr, colIdx, values, &target_row, CF, blkWarpNum);
}
static int vec_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, int nnz, int CF, int blkWarpNum)
{
    return vec_sddmm_profile_impl(A, B, rowPtr, colIdx, values, nullptr, nnz, CF, blkWarpNum);
}
static int vec_split_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values, Tensor target_row,
                                   int nnz, int CF, int blkWarpNum)
{
    return vec_sddmm_profile_impl(A, B, rowPtr, colIdx, values, &target_row, nnz, CF, blkWarpNum);
}
// vendor baseline under the reference's name (SDDMM/sddmm_baseline_kernel.cu): rocSPARSE SDDMM, written in place
// into `values`, which is also returned
static Tensor cusparse_sddmm_compute(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values)
{
    DeviceGuard guard(A.device());
    VendorSDDMM op(A, B, rowPtr, colIdx, values);
    op.run();
    return values;
}
static int cusparse_sddmm_profile(Tensor A, Tensor B, Tensor rowPtr, Tensor colIdx, Tensor values)
{
    DeviceGuard guard(A.device());
    VendorSDDMM op(A, B, rowPtr, colIdx, values);
    const float ms = time_launches((hipStream_t)stream_of(A), kProfileWarmup, kProfileIters, [&] { op.run(); });
    return gflops(2.0 * (double)values.size(0) * (double)A.size(1), ms);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    pspglue::check_abi();
    m.def("csr_sddmm", &csr_sddmm, "CSR SDDMM (HIP, gfx950)");
    m.def("csr_split_sddmm", &csr_split_sddmm, "row-split CSR SDDMM (HIP, gfx950)");
    m.def("bcsr_sddmm", &bcsr_sddmm, "2x1 BCSR SDDMM (HIP, gfx950)");
    m.def("bcsr_split_sddmm", &bcsr_split_sddmm, "row-split 2x1 BCSR SDDMM (HIP, gfx950)");
    m.def("vec_sddmm", &vec_sddmm, "3x1-block SDDMM (HIP, gfx950)");
    m.def("vec_split_sddmm", &vec_split_sddmm, "row-split 3x1-block SDDMM (HIP, gfx950)");
    m.def("csr_sddmm_profile", &csr_sddmm_profile, "GFLOP/s of csr_sddmm");
    m.def("csr_split_sddmm_profile", &csr_split_sddmm_profile, "GFLOP/s of csr_split_sddmm");
    m.def("bcsr_sddmm_profile", &bcsr_sddmm_profile, "GFLOP/s of bcsr_sddmm");
    m.def("bcsr_split_sddmm_profile", &bcsr_split_sddmm_profile, "GFLOP/s of bcsr_split_sddmm");
    m.def("vec_sddmm_profile", &vec_sddmm_profile, "GFLOP/s of vec_sddmm");
    m.def("vec_split_sddmm_profile", &vec_split_sddmm_profile, "GFLOP/s of vec_split_sddmm");
    m.def("cusparse_sddmm_compute", &cusparse_sddmm_compute, "rocSPARSE SDDMM baseline (in place)");
    m.def("cusparse_sddmm_profile", &cusparse_sddmm_profile, "GFLOP/s of the rocSPARSE SDDMM baseline");
    m.def("genmask", &genmask, "CSR slot -> flat index into the 2x1 block values");
    // additions of this build
    m.def("window_sddmm", &window_sddmm, "windowed CSR SDDMM (HIP, gfx950): (A, B, rowPtr_w, colIdx_w, alpha = None)", py::arg("A"),
          py::arg("B"), py::arg("rowPtr_w"), py::arg("colIdx_w"), py::arg("alpha") = py::none());
    m.def("window_sddmm_supported", &window_sddmm_supported, "is there a windowed SDDMM kernel for K columns?");
    m.def("csr_sddmm_scaled", &csr_sddmm_scaled, "values[p] * <A[row], B[col]>");
    m.def("csr_split_sddmm_scaled", &csr_split_sddmm_scaled, "values[p] * <A[row], B[col]> on the row-split format");
    m.def("csr_sddmm_scaled_rowmax", &csr_sddmm_scaled_rowmax, "[values[p] * <A[row], B[col]>, largest score of every row]");
    m.def("csr_split_sddmm_scaled_rowmax", &csr_split_sddmm_scaled_rowmax,
          "the same on the row-split format: (A, B, rowPtr_split, colIdx, values, target_row, rows, blkWarpNum)");
    m.def("segment_softmax", &segment_softmax, "softmax over the stored entries of each CSR row");
}
