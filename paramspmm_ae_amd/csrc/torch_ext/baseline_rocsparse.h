// Vendor-library comparison baselines, exported under the names of the reference's bindings
// (SpMM/Baseline_kernel.cu:24-613 cuSPARSE SpMM in four flavours, SDDMM/sddmm_baseline_kernel.cu:24-163 cuSPARSE
// SDDMM).  On ROCm the vendor library is rocSPARSE; these are NOT part of the ParamSpMM path and use none of its
// kernels.  As in the reference, the timing twins time 200 calls of the compute stage only (handle, descriptors,
// buffer query and the one-off preprocess stage stay outside the timed loop).
#pragma once
#include <rocsparse/rocsparse.h>
#include "glue_common.h"

namespace pspglue {

#define PSP_ROCSPARSE(call)                                                                     \
    do {                                                                                        \
        rocsparse_status st_ = (call);                                                          \
        TORCH_CHECK(st_ == rocsparse_status_success, "rocSPARSE error ", (int)st_, " in " #call); \
    } while (0)

enum VendorFormat { kCsr = 0, kCsrAlg2 = 1, kCooAlg4 = 2, kCsc = 3 };

// One prepared rocsparse_spmm: C = A * B with B, C row-major [n, N].
class VendorSpMM {
public:
    VendorSpMM(VendorFormat f, const torch::Tensor &X, const torch::Tensor &idx_a, const torch::Tensor &idx_b,
               const torch::Tensor &val, torch::Tensor &Y)
    {
        need_gpu(X, "input");
        need_gpu(idx_a, "first index tensor");
        need_gpu(idx_b, "second index tensor");
        need_gpu(val, "values");
        need_f32(X, "input", 2);
        need_i32(idx_a, "first index tensor");
        need_i32(idx_b, "second index tensor");
        need_f32(val, "values", 1);
        const int64_t n = X.size(0), N = X.size(1), nnz = val.size(0);
        PSP_ROCSPARSE(rocsparse_create_handle(&handle_));
        PSP_ROCSPARSE(rocsparse_set_stream(handle_, (hipStream_t)stream_of(X)));
        void *a = idx_a.data_ptr<int>(), *b = idx_b.data_ptr<int>(), *v = val.data_ptr<float>();
        const auto i32 = rocsparse_indextype_i32;
        switch (f) {
        case kCsr:
            alg_ = rocsparse_spmm_alg_default;
            PSP_ROCSPARSE(rocsparse_create_csr_descr(&A_, n, n, nnz, a, b, v, i32, i32, rocsparse_index_base_zero, rocsparse_datatype_f32_r));
            break;
        case kCsrAlg2:  // cuSPARSE CSR_ALG2 is its load-balanced CSR algorithm; rocSPARSE's is merge path
            alg_ = rocsparse_spmm_alg_csr_merge_path;
            PSP_ROCSPARSE(rocsparse_create_csr_descr(&A_, n, n, nnz, a, b, v, i32, i32, rocsparse_index_base_zero, rocsparse_datatype_f32_r));
            break;
        case kCooAlg4:  // (row, col, val)
            alg_ = rocsparse_spmm_alg_coo_atomic;
            TORCH_CHECK(idx_a.size(0) == nnz && idx_b.size(0) == nnz, "COO index tensors must have nnz entries");
            PSP_ROCSPARSE(rocsparse_create_coo_descr(&A_, n, n, nnz, a, b, v, i32, rocsparse_index_base_zero, rocsparse_datatype_f32_r));
            break;
        default:  // (colPtr, rowIdx, val)
            alg_ = rocsparse_spmm_alg_default;
            PSP_ROCSPARSE(rocsparse_create_csc_descr(&A_, n, n, nnz, a, b, v, i32, i32, rocsparse_index_base_zero, rocsparse_datatype_f32_r));
            break;
        }
        PSP_ROCSPARSE(rocsparse_create_dnmat_descr(&B_, n, N, N, X.data_ptr<float>(), rocsparse_datatype_f32_r, rocsparse_order_row));
        PSP_ROCSPARSE(rocsparse_create_dnmat_descr(&C_, n, N, N, Y.data_ptr<float>(), rocsparse_datatype_f32_r, rocsparse_order_row));
        size_t bytes = 0;
        PSP_ROCSPARSE(call(rocsparse_spmm_stage_buffer_size, &bytes, nullptr));
        buffer_ = torch::empty({(long)std::max<size_t>(bytes, 16)}, X.options().dtype(torch::kUInt8));
        PSP_ROCSPARSE(call(rocsparse_spmm_stage_preprocess, &bytes, buffer_.data_ptr()));
        bytes_ = bytes;
    }
    void run() { PSP_ROCSPARSE(call(rocsparse_spmm_stage_compute, &bytes_, buffer_.data_ptr())); }
    ~VendorSpMM()
    {
        if (A_) (void)rocsparse_destroy_spmat_descr(A_);
        if (B_) (void)rocsparse_destroy_dnmat_descr(B_);
        if (C_) (void)rocsparse_destroy_dnmat_descr(C_);
        if (handle_) (void)rocsparse_destroy_handle(handle_);
    }

private:
    rocsparse_status call(rocsparse_spmm_stage stage, size_t *bytes, void *buf)
    {
        const float alpha = 1.0f, beta = 0.0f;
        return rocsparse_spmm(handle_, rocsparse_operation_none, rocsparse_operation_none, &alpha, A_, B_, &beta, C_,
                              rocsparse_datatype_f32_r, alg_, stage, bytes, buf);
    }
    rocsparse_handle handle_ = nullptr;
    rocsparse_spmat_descr A_ = nullptr;
    rocsparse_dnmat_descr B_ = nullptr, C_ = nullptr;
    rocsparse_spmm_alg alg_ = rocsparse_spmm_alg_default;
    torch::Tensor buffer_;
    size_t bytes_ = 0;
};

inline torch::Tensor vendor_spmm_compute(VendorFormat f, torch::Tensor X, torch::Tensor ia, torch::Tensor ib, torch::Tensor val)
{
    DeviceGuard guard(X.device());
    auto Y = torch::zeros_like(X);
    VendorSpMM op(f, X, ia, ib, val, Y);
    op.run();
    return Y;
}

inline int vendor_spmm_profile(VendorFormat f, torch::Tensor X, torch::Tensor ia, torch::Tensor ib, torch::Tensor val)
{
    DeviceGuard guard(X.device());
    auto Y = torch::zeros_like(X);
    VendorSpMM op(f, X, ia, ib, val, Y);
    const float ms = time_launches((hipStream_t)stream_of(X), kProfileWarmup, kProfileIters, [&] { op.run(); });
    return gflops(2.0 * (double)val.size(0) * (double)X.size(1), ms);
}

// values[p] <- <A[row(p),:], B[col(p),:]> in place (alpha 1, beta 0), SDDMM/sddmm_baseline_kernel.cu:24-80
class VendorSDDMM {
public:
    VendorSDDMM(const torch::Tensor &A, const torch::Tensor &B, const torch::Tensor &rowPtr, const torch::Tensor &colIdx,
                torch::Tensor &values)
    {
        need_gpu(A, "A");
        need_gpu(B, "B");
        need_gpu(rowPtr, "rowPtr");
        need_gpu(colIdx, "colIdx");
        need_gpu(values, "values");
        need_f32(A, "A", 2);
        need_f32(B, "B", 2);
        need_i32(rowPtr, "rowPtr");
        need_i32(colIdx, "colIdx");
        need_f32(values, "values", 1);
        TORCH_CHECK(A.size(1) == B.size(1), "A and B must have the same number of columns");
        const int64_t M = rowPtr.size(0) - 1, Ncols = B.size(0), K = A.size(1), nnz = values.size(0);
        TORCH_CHECK(A.size(0) >= M, "A has fewer rows than the sparse matrix");
        PSP_ROCSPARSE(rocsparse_create_handle(&handle_));
        PSP_ROCSPARSE(rocsparse_set_stream(handle_, (hipStream_t)stream_of(A)));
        PSP_ROCSPARSE(rocsparse_create_csr_descr(&C_, M, Ncols, nnz, rowPtr.data_ptr<int>(), colIdx.data_ptr<int>(),
                                                 values.data_ptr<float>(), rocsparse_indextype_i32, rocsparse_indextype_i32,
                                                 rocsparse_index_base_zero, rocsparse_datatype_f32_r));
        PSP_ROCSPARSE(rocsparse_create_dnmat_descr(&A_, M, K, K, A.data_ptr<float>(), rocsparse_datatype_f32_r, rocsparse_order_row));
        PSP_ROCSPARSE(rocsparse_create_dnmat_descr(&B_, Ncols, K, K, B.data_ptr<float>(), rocsparse_datatype_f32_r, rocsparse_order_row));
        size_t bytes = 0;
        PSP_ROCSPARSE(rocsparse_sddmm_buffer_size(handle_, rocsparse_operation_none, rocsparse_operation_transpose, &alpha_, A_, B_,
                                                  &beta_, C_, rocsparse_datatype_f32_r, rocsparse_sddmm_alg_default, &bytes));
        buffer_ = torch::empty({(long)std::max<size_t>(bytes, 16)}, A.options().dtype(torch::kUInt8));
        PSP_ROCSPARSE(rocsparse_sddmm_preprocess(handle_, rocsparse_operation_none, rocsparse_operation_transpose, &alpha_, A_, B_,
                                                 &beta_, C_, rocsparse_datatype_f32_r, rocsparse_sddmm_alg_default, buffer_.data_ptr()));
    }
    void run()
    {
        PSP_ROCSPARSE(rocsparse_sddmm(handle_, rocsparse_operation_none, rocsparse_operation_transpose, &alpha_, A_, B_, &beta_, C_,
                                      rocsparse_datatype_f32_r, rocsparse_sddmm_alg_default, buffer_.data_ptr()));
    }
    ~VendorSDDMM()
    {
        if (C_) (void)rocsparse_destroy_spmat_descr(C_);
        if (A_) (void)rocsparse_destroy_dnmat_descr(A_);
        if (B_) (void)rocsparse_destroy_dnmat_descr(B_);
        if (handle_) (void)rocsparse_destroy_handle(handle_);
    }

private:
    float alpha_ = 1.0f, beta_ = 0.0f;
    rocsparse_handle handle_ = nullptr;
    rocsparse_spmat_descr C_ = nullptr;
    rocsparse_dnmat_descr A_ = nullptr, B_ = nullptr;
    torch::Tensor buffer_;
};

}  // namespace pspglue
