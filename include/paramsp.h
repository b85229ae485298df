/*
 * libparamsp_hip.so -- C ABI of the MI355X (gfx950, wave64) ParamSpMM / ParamSDDMM hot path.
 *
 * Plain pointers and sizes only: no torch types, no C++ in the signatures.  Every `const float*` /
 * `const int*` marked DEVICE must point to GPU memory valid on the stream's device; HOST pointers are
 * ordinary CPU memory.  `stream` is a hipStream_t passed as void* (NULL = the default stream).  Device
 * entry points only enqueue work; they never synchronise and never allocate.
 *
 * Every function returns 0 on success or a negative psp_status; psp_last_error() gives the text of the
 * last failure on the calling thread.  Nothing here calls exit() (the reference's launchers do on a launch
 * error, SpMM/SpMM_kernel.cu:189-194).
 *
 * Each declaration cites the interface of zzzlxhhh/ParamSpMM_AE it stands in for.  The three PyTorch
 * extension modules ParamSpMM / ParamSDDMM / ParamSpCONV (pybind, same names and argument order as the
 * reference's bindings) are thin glue over this header.
 */
#ifndef PARAMSP_H
#define PARAMSP_H

#ifdef __cplusplus
extern "C" {
#endif

typedef void *psp_stream_t; /* hipStream_t */

enum psp_status {
    PSP_OK = 0,
    PSP_ERR_ARG = -1,    /* bad argument (null pointer, negative size, CF / blkWarpNum out of range) */
    PSP_ERR_LAUNCH = -2, /* hipGetLastError() after the launch was not hipSuccess */
    PSP_ERR_RANGE = -3   /* sizes exceed what the 32-bit index arithmetic of the kernels can address */
};

const char *psp_last_error(void);

/* Version of the ABI this header describes; psp_version() returns the one the loaded library was built from.  A
 * caller compiled against this header must find psp_version() >= PSP_ABI_VERSION before it calls anything else:
 * buffers that the library fills have grown between versions under unchanged symbol names --
 *   200: psp_spmm_plan gained log_segs_per_wave, even_split, xcd_stripe_rows (10 ints; 7 before);
 *        psp_nll_loss_mean_f32 writes 3 + 3*1024 floats of `stats` (2 before);
 *   300: option "whole_rows"; the windowed-CSR entry points;
 *   310: PSP_WINDOW_HALO is 88 (64 before: windowed arrays built by a 300 library do not match these kernels -- build
 *        them again); psp_sddmm_window_f32, psp_attn_window_forward_f32 / _backward_f32, psp_softmax_nll_mean_f32 (+ backward);
 *        option "dense_split";
 *   311: psp_spmm_register_sets (no buffer changed).
 * The extension modules and the ctypes loader of this package check it when they are imported. */
#define PSP_ABI_VERSION 311
int psp_version(void);

/* How a (N, CF, blkWarpNum) request of the Python layer maps onto the wave64 kernels.
 * CF 1..8 keeps its meaning "column coarsening": the number of `vec`-wide column vectors one lane owns;
 * blkWarpNum keeps its meaning "wavefronts per workgroup" (4 or 8, SpMM/SpMM.cpp:77-141).  The reference's callers
 * pass CF through as an opaque int (PCSR.py:224-237), so the same argument also carries the NATIVE parameter space of
 * the wave64 kernel, which the reference's <CF, blkWarpNum> cannot express: a value with PSP_CF_NATIVE set names
 *   coarsen     1..8   column vectors per lane,
 *   log_lanes   0..6   lanes that share one sparse row = 2^log_lanes (rows per wavefront = 64 / lanes),
 *   log_unroll  0..3   stored entries whose feature loads are in flight together per lane = 2^log_unroll
 *                      (coarsen * unroll <= 8, unroll <= lanes),
 *   segs_sel    0..7   0 = segments per wavefront chosen by the library, s >= 1 = 2^(s-1) segments per wavefront
 * (build one with PSP_CF_PACK).  The sweep times such configurations and the decider's forests are trained on them
 * (decider.py:63-80 decodes CF from a list, so the list may hold packed values). */
#define PSP_CF_NATIVE (1 << 16)
#define PSP_CF_EVEN_SPLIT (1 << 11) /* with PSP_CF_NATIVE: always divide a wavefront's entries evenly between the
                                      lane groups, never hand them whole segments (see the option "align_pct") */
#define PSP_CF_PACK(coarsen, log_lanes, log_unroll, segs_sel) \
    (PSP_CF_NATIVE | ((coarsen) - 1) | ((log_lanes) << 3) | ((log_unroll) << 6) | ((segs_sel) << 8))
typedef struct psp_spmm_plan {
    int vec;            /* floats per feature load: 4 (N%4==0), 2 (N%2==0) or 1 */
    int coarsen;        /* column vectors per lane (the request's CF, 1..8) */
    int lanes_per_row;  /* power of two, 1..64: lanes that share one sparse row */
    int rows_per_wave;  /* 64 / lanes_per_row */
    int unroll;         /* non-zeros whose feature loads are in flight together per lane */
    int col_tiles;      /* grid.y: ceil(N / (lanes_per_row*coarsen*vec)) */
    int waves_per_block;
    int log_segs_per_wave; /* -1: chosen at launch from the format and the matrix size */
    int even_split;        /* 1: the wavefront's entries are always divided evenly between the lane groups */
    int xcd_stripe_rows;   /* rows (segments) dealt to one XCD at a time; 0: the library option "xcd_stripe_rows" */
} psp_spmm_plan;
int psp_spmm_plan_for(int N, int CF, int blkWarpNum, psp_spmm_plan *plan);
/* Register sets of the SpMM kernel a plan runs (the last argument of the kernel's symbol as a profiler prints it: true
 * for 1).  2: the feature loads of a batch of `unroll` entries are issued while the batch before is added.  1: a batch
 * is gathered, added, and the next one gathered -- fewer registers, more wavefronts per SIMD; faster wherever at least
 * four entries are in flight, or two with 8 or more lanes per row.  No counterpart in the reference. */
int psp_spmm_register_sets(int unroll, int lanes_per_row);

/* SpMM and SDDMM entry points (row-wise walks), blkWarpNum | PSP_BW_STRIPE(rows): this launch deals `rows`
 * consecutive rows (segments, block-rows) to one XCD at a time instead of the library option "xcd_stripe_rows".
 * rows = a multiple of 256 up to 65280 (the field
 * holds rows / 256 in bits 12..19; 0 = the option).  The reference has no counterpart (one L2 on its GPUs): a caller
 * that knows the matrix picks the longest stripe that still gives the eight XCDs equal shares of the stored entries
 * (graph_input does: csr_data.xcd_stripe), long stripes keeping neighbouring rows -- and the X rows they share -- in
 * one L2, short ones levelling a matrix whose long rows cluster in an index range. */
#define PSP_BW_STRIPE_SHIFT 12
#define PSP_BW_STRIPE_MASK (0xff << PSP_BW_STRIPE_SHIFT)
#define PSP_BW_STRIPE(rows) ((((rows) / 256) << PSP_BW_STRIPE_SHIFT) & PSP_BW_STRIPE_MASK)

/* Library-wide tuning options (no counterpart in the reference, whose launch shapes are compile-time constants):
 *   "xcd_stripe_rows"  rows (segments) dealt to one XCD at a time by the SpMM kernels (default 8192),
 *   "align_pct"        lane groups take whole segments when that costs at most this many percent more steps than
 *                      the even division of a wavefront's entries (default 50),
 *   "split_clear_min"  row-split outputs of at least this many floats are cleared selectively (default 4 Mi),
 *   "whole_rows"       1: a lane group is always handed whole rows (segments), however uneven that is.  Every element
 *                      of a plain CSR / BCSR product is then one FMA chain over the row's stored entries in storage
 *                      order, which is the summation order of the reference's one-warp-per-row kernels
 *                      (SpMM/SpMM_kernel.cu:1157-1212, 1362-1440): results repeat the sequential chain bit for bit.
 *                      Default 0: rows may be cut between lane groups and summed piecewise (faster on skewed rows).
 *   "dense_split"      1 (default): the dense layer products (the gemm_xw and gemm_atb entry points) at 128 x 128 form
 *                      every fp32 product from the three bf16 terms of each operand (six bf16 matrix-core products,
 *                      fp32 accumulation: error 2^-23 of |x||w| per product, the rounding level of fp32) and are
 *                      bound by their memory traffic; an infinite input (or one within a bf16 rounding step of
 *                      FLT_MAX) turns its row into NaN.  0: the fp32 matrix-core instruction, 25-40 % slower at that shape.
 * The environment (PSP_XCD_STRIPE_ROWS, PSP_ALIGN_PCT, PSP_SPLIT_CLEAR_MIN, PSP_WHOLE_ROWS, PSP_DENSE_SPLIT) sets the
 * initial values, once.
 * psp_get_option returns the value, or a negative psp_status for an unknown name.  Not synchronised with running
 * launches: set options before the calls they should affect. */
int psp_set_option(const char *name, long long value);
long long psp_get_option(const char *name);

/* ---------------------------------------------------------------------------------------------
 * HOST: PCSR index construction
 * ------------------------------------------------------------------------------------------- */

/* Row splitting, SpMM/SpMM.cpp:15-40 (`split_csr`).  Row i with [lb,hb) becomes ceil((hb-lb)/g) segments
 * of at most g non-zeros.  psp_split_csr_count returns S; psp_split_csr fills rowPtr_split[S+1] and
 * target_row[S] and returns S. */
int psp_split_csr_count(const int *rowPtr, int nrows, int g);
int psp_split_csr(const int *rowPtr, int nrows, int g, int *rowPtr_split, int *target_row);

/* SpMM/SpMM.cpp:42-75 (`split_csr_par`): same output; the caller supplies the exclusive prefix sum of the
 * per-row segment counts (graph_input.py:135-136); rows are processed by several host threads.
 * Returns S = row_split_offset[nrows]. */
int psp_split_csr_par(const int *rowPtr, const int *row_split_offset, int nrows, int g,
                      int *rowPtr_split, int *target_row);

/* BCSR with 2x1 blocks in SciPy `tobsr` order (graph_input.py:243-266 calls csr.tobsr(blocksize=(2,1))):
 * inside block-row t the blocks appear in first-encounter order, row 2t's columns first, then the columns
 * only row 2t+1 has.  nrows may be odd (the missing row is empty, graph_input.py:248-255).
 * psp_bcsr_count returns nblk; psp_bcsr_build fills rowPtr_b[(nrows+1)/2+1], colIdx_b[nblk],
 * val_b[nblk*2] and returns nblk. */
int psp_bcsr_count(const int *rowPtr, const int *colIdx, int nrows, int ncols);
int psp_bcsr_build(const int *rowPtr, const int *colIdx, const float *val, int nrows, int ncols,
                   int *rowPtr_b, int *colIdx_b, float *val_b);

/* Blocks of R x 1 for any R in 1..8 (graph_input.py:243-266 with blk_size = R; the reference has kernels for R = 3
 * besides 2): same block order as above, val_b is [nblk, R], rowPtr_b has ceil(nrows/R)+1 entries. */
int psp_vbsr_count(const int *rowPtr, const int *colIdx, int nrows, int ncols, int R);
int psp_vbsr_build(const int *rowPtr, const int *colIdx, const float *val, int nrows, int ncols, int R,
                   int *rowPtr_b, int *colIdx_b, float *val_b);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: PCSR index construction on the GPU, the twins of the host builders above (same outputs, bit for
 * bit).  The reference builds on the host only (SpMM/SpMM.cpp:15-75, graph_input.py:243-274).  Each builder is
 * two calls with one read-back of a size in between: offsets (count + exclusive scan), then fill.
 *   workspace: psp_scan_workspace_ints(n) ints of device memory, n = number of scanned items (nrows for the
 *              split, (nrows+1)/2 for BCSR);
 *   status:    one device int the caller has set to 0; the kernels OR psp_build_flag bits into it.  With a
 *              non-zero status the outputs are not valid (the host builders accept such input).
 * ------------------------------------------------------------------------------------------- */
enum psp_build_flag {
    PSP_BUILD_OVERFLOW = 1,  /* a prefix sum left the int32 range */
    PSP_BUILD_UNSORTED = 2,  /* a row's column indices are not strictly ascending (BCSR builder only) */
    PSP_BUILD_BAD_ROWPTR = 4, /* rowPtr decreases, does not start at 0 or does not end at nnz */
    PSP_BUILD_BAD_COLUMN = 8, /* a column index lies outside [0, ncols)        (psp_check_index_dev only) */
    PSP_BUILD_BAD_TARGET = 16 /* target_row decreases or leaves [0, target_rows) (psp_check_index_dev only) */
};
int psp_scan_workspace_ints(int n);

/* row_split_offset[nrows+1] = exclusive prefix sum of ceil(nnz_i / g): the array graph_input.py:135 computes
 * with torch.cumsum; row_split_offset[nrows] is S. */
int psp_split_csr_offsets_dev(const int *rowPtr, int nrows, int g, int *row_split_offset, int *workspace,
                              int workspace_ints, int *status, psp_stream_t stream);
/* fills rowPtr_split[S+1] and target_row[S] like psp_split_csr_par. */
int psp_split_csr_fill_dev(const int *rowPtr, const int *row_split_offset, int nrows, int g, int S,
                           int *rowPtr_split, int *target_row, psp_stream_t stream);

/* rowPtr_b[(nrows+1)/2+1]; rowPtr_b[(nrows+1)/2] is nblk.  Input rows must hold strictly ascending columns. */
int psp_bcsr_offsets_dev(const int *rowPtr, const int *colIdx, int nrows, int *rowPtr_b, int *workspace,
                         int workspace_ints, int *status, psp_stream_t stream);
/* fills colIdx_b[nblk] and val_b[nblk*2] in the block order of psp_bcsr_build. */
int psp_bcsr_fill_dev(const int *rowPtr, const int *colIdx, const float *val, int nrows, const int *rowPtr_b,
                      int *colIdx_b, float *val_b, psp_stream_t stream);

/* Validation of index arrays of unknown origin, any of the four formats: rowPtr[M+1] (or rowPtr_split[S+1]) starts at
 * 0, does not decrease and ends at nnz; every colIdx is inside [0, ncols); target_row (NULL for the plain formats)
 * does not decrease and stays inside [0, target_rows).  The SpMM / SDDMM kernels trust their inputs, as the
 * reference's do (no check anywhere in SpMM/SpMM.cpp): an index outside X makes them read outside the buffer.  ORs
 * psp_build_flag bits into *status (set to 0 by the caller). */
int psp_check_index_dev(const int *rowPtr, const int *colIdx, const int *target_row, int M, int nnz, int ncols,
                        int target_rows, int *status, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: genmask, SDDMM/sddmm.cpp:663-673 -> sddmm_kernel.cu:78-141.
 * mask[nnz] (int32) is fully written: CSR slot -> flat index into val_b of the same non-zero.
 * rowPtr must hold at least 2*nblkrows entries (+1 when the row count is even).
 * ------------------------------------------------------------------------------------------- */
int psp_genmask(const int *rowPtr_b, const int *rowPtr, const float *val_b, int nblkrows, int nnz,
                int *mask, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: SpMM  Y = A * X, fp32.  X is [*, N] row-major with leading dimension N; Y is
 * [rows_out, N] and is completely defined on return (rows the matrix does not cover are zero), so the
 * caller passes uninitialised memory -- the reference allocates zeros and then launches
 * (SpMM/SpMM_kernel.cu:136, 281-282).
 * ------------------------------------------------------------------------------------------- */

/* ParamSpMM.csr_spmm, SpMM/SpMM.cpp:77-141 -> SpMM_kernel.cu:129-197, 1157-1243.  M = rows of A. */
int psp_spmm_csr_f32(const int *rowPtr, const int *colIdx, const float *val, const float *X, float *Y,
                     int M, int N, int rows_out, int CF, int blkWarpNum, psp_stream_t stream);

/* ParamSpMM.csr_split_spmm, SpMM/SpMM.cpp:143-207 -> SpMM_kernel.cu:199-268, 1245-1360.
 * S = number of segments.  Rows made of one segment are stored, rows made of several are accumulated
 * with fp32 atomics (order not fixed, as in the reference). */
int psp_spmm_csr_split_f32(const int *rowPtr_split, const int *colIdx, const float *val,
                           const int *target_row, const float *X, float *Y, int S, int N, int rows_out,
                           int CF, int blkWarpNum, psp_stream_t stream);

/* Softmax-weighted SpMM on the CSR layouts (no counterpart in the reference: the attention pipeline SDDMM ->
 * softmax -> SpMM in two kernels instead of three passes):
 *   Y[i] = sum_j w_ij X[j] / sum_j w_ij,  w_ij = exp(e_ij - row_max[i]),
 * e in CSR entry order, row_max[i] >= every e_ij of row i (psp_sddmm_*_rowmax_f32 delivers the maximum).  Rows without
 * entries give zeros.  N % 4 == 0 and CF <= 4.  The split variant needs row_sum: rows_out floats of device
 * workspace (contents irrelevant on entry); rows shared by several wavefronts are accumulated with fp32 atomics and
 * normalised by a second launch. */
int psp_spmm_csr_softmax_f32(const int *rowPtr, const int *colIdx, const float *e, const float *row_max,
                             const float *X, float *Y, int M, int N, int rows_out, int CF, int blkWarpNum,
                             psp_stream_t stream);
int psp_spmm_csr_split_softmax_f32(const int *rowPtr_split, const int *colIdx, const float *e, const int *target_row,
                                   const float *row_max, float *row_sum, const float *X, float *Y, int S, int N,
                                   int rows_out, int CF, int blkWarpNum, psp_stream_t stream);

/* ParamSpMM.bcsr_spmm, SpMM/SpMM.cpp:209-271 -> SpMM_kernel.cu:273-343, 1362-1493.
 * Mb block-rows; val_b is [nblk,2]; rows_out >= 2*Mb.  A zero block entry contributes nothing. */
int psp_spmm_bcsr_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *X,
                      float *Y, int Mb, int N, int rows_out, int CF, int blkWarpNum, psp_stream_t stream);

/* ParamSpMM.bcsr_split_spmm, SpMM/SpMM.cpp:273-337 -> SpMM_kernel.cu:345-420, 1495-1651.
 * target_row holds block-row indices. */
int psp_spmm_bcsr_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                            const int *target_row, const float *X, float *Y, int Sb, int N, int rows_out,
                            int CF, int blkWarpNum, psp_stream_t stream);

/* ParamSpMM.vec_spmm / vec_split_spmm, SpMM/SpMM.cpp:339-480 -> SpMM_kernel.cu:420-562, 1653-1972: blocks of
 * vec_size x 1 (val_b is [nblk, vec_size]); the reference instantiates vec_size 3 only, this library 3 and, through the
 * 2x1 kernels, 2.  rows_out >= vec_size * Mb.  CF 7 and 8 with vec_size 3 exceed the register file and run slowly. */
int psp_spmm_vec_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *X, float *Y, int Mb,
                     int N, int rows_out, int vec_size, int CF, int blkWarpNum, psp_stream_t stream);
int psp_spmm_vec_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b, const int *target_row,
                           const float *X, float *Y, int Sb, int N, int rows_out, int vec_size, int CF,
                           int blkWarpNum, psp_stream_t stream);

/* The four SpMM formats with the ReLU between two layers folded in (no counterpart among the reference's kernels:
 * its driver applies F.relu as a pass of its own, GNN.py:43-61, 63-78).  fmt: 0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split,
 * arrays and sizes as for the plain entry point of that format (target_row NULL for the plain ones).
 *   relu_x != 0: Y = A * max(X, 0) -- the product reads the previous layer's output through the ReLU, applied to the
 *   rows as they are gathered (no activated copy of X is written);
 *   mask != NULL ([rows_out, N], 16-byte aligned like Y): Y = (A * X) where mask > 0, else 0 -- the gradient with respect
 *   to the pre-activation values a layer was given; a pass over Y that follows the product on the same stream. */
int psp_spmm_act_f32(int fmt, const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                     const float *X, float *Y, int nseg, int N, int rows_out, int CF, int blkWarpNum, int relu_x,
                     const float *mask, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: SDDMM  out[p] = <A[row(p),:], B[col(p),:]>, fp32, NOT scaled by the stored values (the reference
 * kernels never multiply them in, SDDMM/sddmm_kernel.cu:917-983).  A and B are [*, K] row-major.
 * `scale` may be NULL; when given (an extension of this library used by the attention benchmark) the result
 * is multiplied by scale[p] (csr) -- pass NULL for the reference semantics.
 * blkWarpNum | PSP_BW_BALANCED (plain layouts; ignored by the row-split ones): the stored entries, not the rows, are
 * divided between the wavefronts of a fixed grid, so a plain matrix with hub rows runs as evenly as its row-split form
 * (every entry's result is independent, a row can be cut anywhere).  The reference balances through the row-split
 * format only (SDDMM/sddmm_kernel.cu:986-1057).
 * colIdx, out and the block values may all be NULL for a matrix without stored entries (an empty device
 * allocation has no address, and only rowPtr -- on the device -- says whether there are any).
 * ------------------------------------------------------------------------------------------- */

#define PSP_BW_BALANCED 0x100

/* ParamSDDMM.csr_sddmm, SDDMM/sddmm.cpp:15-65 -> sddmm_kernel.cu:143-192, 917-983.  out[nnz]. */
int psp_sddmm_csr_f32(const int *rowPtr, const int *colIdx, const float *A, const float *B,
                      const float *scale, float *out, int M, int K, int blkWarpNum, psp_stream_t stream);

/* ParamSDDMM.csr_split_sddmm, SDDMM/sddmm.cpp:67-120 -> sddmm_kernel.cu:194-246, 986-1057. */
int psp_sddmm_csr_split_f32(const int *rowPtr_split, const int *colIdx, const int *target_row,
                            const float *A, const float *B, const float *scale, float *out, int S, int K,
                            int blkWarpNum, psp_stream_t stream);

/* The two CSR variants with the largest result of every row delivered as well: row_max[rows] (overwritten; rows
 * without entries keep the lowest float).  No counterpart in the reference; feeds psp_spmm_*_softmax_f32. */
int psp_sddmm_csr_rowmax_f32(const int *rowPtr, const int *colIdx, const float *A, const float *B,
                             const float *scale, float *out, float *row_max, int M, int K, int blkWarpNum,
                             psp_stream_t stream);
int psp_sddmm_csr_split_rowmax_f32(const int *rowPtr_split, const int *colIdx, const int *target_row,
                                   const float *A, const float *B, const float *scale, float *out, float *row_max,
                                   int S, int rows, int K, int blkWarpNum, psp_stream_t stream);

/* ParamSDDMM.bcsr_sddmm, SDDMM/sddmm.cpp:122-172 -> sddmm_kernel.cu:248-300, 1059-1176.
 * out is [nblk,2]; entries whose block value is zero are written as zero.  A needs 2*Mb rows. */
int psp_sddmm_bcsr_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *A,
                       const float *B, float *out, int Mb, int K, int blkWarpNum, psp_stream_t stream);

/* ParamSDDMM.bcsr_split_sddmm, SDDMM/sddmm.cpp:174-228 -> sddmm_kernel.cu:302-352, 1178-1287. */
int psp_sddmm_bcsr_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                             const int *target_row, const float *A, const float *B, float *out, int Sb,
                             int K, int blkWarpNum, psp_stream_t stream);

/* ParamSDDMM.vec_sddmm / vec_split_sddmm, SDDMM/sddmm.cpp:230-336 -> sddmm_kernel.cu:1289-1468: blocks of vec_size x 1,
 * out is [nblk, vec_size].  The reference's kernels for this are never run and address their shared memory with a
 * stride of CF*2 instead of CF*vec_size; this is their evident intent (the 2x1 rule for every entry of a block), for
 * vec_size 3 and, through the 2x1 kernels, 2.  A needs vec_size*Mb rows. */
int psp_sddmm_vec_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *A, const float *B,
                      float *out, int Mb, int K, int vec_size, int blkWarpNum, psp_stream_t stream);
int psp_sddmm_vec_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b, const int *target_row,
                            const float *A, const float *B, float *out, int Sb, int K, int vec_size,
                            int blkWarpNum, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Windowed CSR: a fifth representation, for matrices whose entries cluster around the diagonal (community-ordered
 * graphs, meshes, banded matrices).  No counterpart in the reference.  Rows are cut into blocks of PSP_WINDOW_BLOCK;
 * an entry is local when its column lies in [block start - PSP_WINDOW_HALO, block end + PSP_WINDOW_HALO) and below M.  The format
 * keeps every row's entries, local ones first (each part in its original order), columns absolute:
 *   rowPtr_w[2M + 2]: 2i = start of row i, 2i + 1 = start of its remote part; 2M and 2M + 1 = nnz;
 *   colIdx_w[nnz], val_w[nnz]: the permuted entries.
 * psp_window_build fills them on the host, psp_window_build_dev on the device (same result).
 * psp_spmm_window_f32: Y[0..M) = A X (A with M rows and nnz = rowPtr_w[2M] stored entries, X with a row for every
 * column and at least M of them),
 * Y[M..rows_out) = 0.  The X rows of a workgroup's window are staged in LDS and the local entries read them there;
 * only remote entries gather from global memory.  N must be a multiple of 4.  variant: 0 automatic, 1 / 2 / 3 = column tiles of 16 / 32 / 64 floats
 * (psp_spmm_window_plan reports tile width, rows per workgroup and LDS bytes, and returns the variant chosen).
 * relu_x != 0: the rows of X enter as max(x, 0); mask (may be null): an output element is kept only where
 * mask > 0, else it is an exact zero (mask has Y's shape).  Results lie within the fp32 tolerance of the CSR product
 * (local entries are summed before remote ones), they are not bit-identical to it.
 * ------------------------------------------------------------------------------------------- */
#define PSP_WINDOW_BLOCK 64
#define PSP_WINDOW_HALO 88
int psp_window_build(const int *rowPtr, const int *colIdx, const float *val, int M, int *rowPtr_w, int *colIdx_w,
                     float *val_w);
int psp_window_build_dev(const int *rowPtr, const int *colIdx, const float *val, int M, int *rowPtr_w, int *colIdx_w,
                         float *val_w, psp_stream_t stream);
int psp_spmm_window_plan(int N, int variant, int *tile_cols, int *rows_per_block, int *lds_bytes);
int psp_spmm_window_f32(const int *rowPtr_w, const int *colIdx_w, const float *val_w, const float *X, float *Y, int M,
                        int nnz, int N, int rows_out, int variant, int relu_x, const float *mask, psp_stream_t stream);
/* The same product with a small dense one folded into its epilogue (the dense product of a square GCN layer,
 * SpCONV/SpCONV.h:43-71: torch::mm(H, W) around the sparse product): Y = mask (.) ((A f(X)) W) for transW == 0 or
 * ((A f(X)) W^T) for transW != 0, with W[N, N] row-major, N = 16 or 32, f = max(., 0) when relu_x.  Y_raw (may be null)
 * receives A f(X) itself.  Since A (H W) = (A H) W the forward pass of a layer is one launch, and its backward pass one
 * launch that delivers A dY (for the weight gradient) and (A dY) W^T masked (the input gradient). */
int psp_spmm_window_xw_f32(const int *rowPtr_w, const int *colIdx_w, const float *val_w, const float *X, const float *W,
                           int transW, float *Y, float *Y_raw, int M, int nnz, int N, int rows_out, int relu_x,
                           const float *mask, psp_stream_t stream);

/* SDDMM over the same layout: out[p] = alpha <A[row(p), :], B[col(p), :]> for every stored entry, in the layout's entry
 * order (out is parallel to colIdx_w).  The B rows of a block's window sit in LDS; only remote entries gather.
 * A[>= M, K], B[rows_b, K] row-major and 16-byte aligned, rows_b above every column index, K a multiple of 4 up to
 * PSP_SDDMM_WINDOW_MAX_K.  alpha: one float in device memory, or NULL for 1.  A == B (the attention scores of a graph
 * layer) reads the matrix once.  No counterpart in the reference (its kernels, SDDMM/sddmm_kernel.cu:917-1057, gather
 * B[col] per entry); results agree with psp_sddmm_csr_f32 on (rowPtr_w[0::2], colIdx_w) within the fp32 tolerance. */
#define PSP_SDDMM_WINDOW_MAX_K 128
int psp_sddmm_window_f32(const int *rowPtr_w, const int *colIdx_w, const float *A, const float *B, const float *alpha,
                         float *out, int M, int nnz, int K, int rows_b, psp_stream_t stream);

/* One attention layer's sparse work over the same layout, the SDDMM and the SpMM of a direction in one pass over the
 * window (the layer of gnn_conv.py:128-180 runs them as separate operators; no counterpart in the reference).
 * X, dY: [>= M, K] row-major, 16-byte aligned; the matrix is square (every column index below M); K a multiple of 4 up
 * to PSP_ATTN_WINDOW_MAX_K; Y, G: [rows_out, K], rows past M are cleared.
 *   forward:  att[p] = alpha <X[row(p)], X[col(p)]> (alpha: one float on the device, or NULL for 1) in the layout's
 *             entry order, Y[i] = sum_p att[p] X[col(p)].
 *   backward: G[i] = sum_p att[p] dY[col(p)] and *wsum = sum_p <dY[row(p)], dY[col(p)]> (float)col(p), the reference's
 *             literal formula for the gradient of the attention weight (gnn_conv.py:166-172: the SDDMM of the gradient
 *             with itself times colIdx as floats); *wsum (device memory) is overwritten, the per-entry products are
 *             never stored.  Workgroups add their shares to *wsum atomically, in no fixed order. */
#define PSP_ATTN_WINDOW_MAX_K 64
int psp_attn_window_forward_f32(const int *rowPtr_w, const int *colIdx_w, const float *X, const float *alpha, float *att,
                                float *Y, int M, int nnz, int K, int rows_out, psp_stream_t stream);
int psp_attn_window_backward_f32(const int *rowPtr_w, const int *colIdx_w, const float *att, const float *dY, float *G,
                                 float *wsum, int M, int nnz, int K, int rows_out, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: softmax over the stored entries of every CSR row (out[p] = exp(e[p]-max_r) / sum_r).
 * No counterpart in the reference (its AGNN layer applies no softmax, gnn_conv.py:136-142); it exists for
 * the SDDMM -> softmax -> SpMM attention pipeline.  in and out may alias.
 * ------------------------------------------------------------------------------------------- */
int psp_segment_softmax_f32(const int *rowPtr, const float *in, float *out, int M, psp_stream_t stream);
/* Same result with the work of rows longer than 128 entries spread over the whole GPU (four launches instead of
 * one; a hub row otherwise runs on a single workgroup).  nnz = rowPtr[M]; workspace: 2*M floats of device memory,
 * contents irrelevant on entry.  The sum of a long row is accumulated with fp32 atomics. */
int psp_segment_softmax_ws_f32(const int *rowPtr, const float *in, float *out, int M, int nnz, float *workspace,
                               psp_stream_t stream);

/* The same softmax for callers that cannot allocate device memory.  It has no counterpart in the reference: it is
 * for code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same result as
 * psp_segment_softmax_ws_f32, whose kernels it runs, but the 2*M floats of workspace are a fixed array inside the
 * library (16 MiB of device memory on every GPU the library is used on, held until the process ends); the call
 * allocates and frees nothing.  M may not exceed PSP_SEGMENT_SOFTMAX_STATIC_MAX_ROWS (PSP_ERR_ARG beyond it: use the
 * _ws_ form).  The stream's device must be the current device.  All calls on one GPU share the array: two calls
 * that overlap on one GPU (different streams, or graphs replayed concurrently) race on it; calls on one stream, or
 * otherwise ordered, do not.  The first call on a device looks the array's address up (hipGetDevice, a lock,
 * hipGetSymbolAddress: host work, no allocation); every later call on that device is kernel launches only.  Make one
 * call per device outside any stream capture before capturing one -- an empty call (M = 0) does the lookup and
 * launches nothing. */
#define PSP_SEGMENT_SOFTMAX_STATIC_MAX_ROWS (1 << 21)
int psp_segment_softmax_static_f32(const int *rowPtr, const float *in, float *out, int M, int nnz,
                                   psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: C[K1,K2] = A^T * B for tall-skinny row-major A [n,K1] and B [n,K2]; C is overwritten.
 * Stands in for the weight-gradient product torch::mm(H.t(), AG) of the fused GCN backward
 * (SpCONV/SpCONV.h:70) when both widths are multiples of 16 up to 128 (psp_gemm_atb_supported tells); partial products of
 * row bands are added with fp32 atomics, so the summation order is not fixed.
 * ------------------------------------------------------------------------------------------- */
int psp_gemm_atb_supported(int K1, int K2);
int psp_gemm_atb_f32(const float *A, const float *B, float *C, long long n, int K1, int K2, psp_stream_t stream);
/* Same product without atomics: every workgroup stores its partial product in the caller's workspace and a second
 * kernel adds them in a fixed order (so results repeat bit for bit, and the 20-60 us the contended atomics take are
 * saved).  workspace: psp_gemm_atb_workspace_floats(n, K1, K2) floats of device memory, contents irrelevant on
 * entry; 0 means the shape runs the atomic kernel and needs none. */
long long psp_gemm_atb_workspace_floats(long long n, int K1, int K2);
int psp_gemm_atb_ws_f32(const float *A, const float *B, float *C, long long n, int K1, int K2, float *workspace,
                        long long workspace_floats, psp_stream_t stream);
/* relu_a != 0: A enters the product as max(a, 0): the weight gradient of a layer that reads the previous layer's
 * output through a ReLU (GNN.py:43-61 applies F.relu between the layers) without that activation being stored. */
int psp_gemm_atb_ws_act_f32(const float *A, const float *B, float *C, long long n, int K1, int K2, int relu_a,
                            float *workspace, long long workspace_floats, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: Y[n,K2] = X[n,K1] * W (transW = 0, W is [K1,K2] row-major) or X * W^T (transW != 0, W is [K2,K1]) for
 * tall-skinny X and a small weight matrix: torch::mm(H, W) and torch::mm(AG, W.t()) of the fused GCN layer
 * (SpCONV/SpCONV.h:43-71).  Supported widths: K2 in {16, 32} with K1 in {16, 32, 48, 64} (and 128 with K2 = 16): one
 * lane per row, FMAs; K2 in {64, 128} with K1 in {16, 32, 64, 128}: fp32 matrix cores (v_mfma_f32_16x16x4_f32), W in
 * LDS.  psp_gemm_xw_supported tells.  Y is overwritten; X and Y 16-byte aligned.  Deterministic (no atomics, one
 * fixed summation order per output element).
 * ------------------------------------------------------------------------------------------- */
int psp_gemm_xw_supported(int K1, int K2);
int psp_gemm_xw_f32(const float *X, const float *W, float *Y, long long n, int K1, int K2, int transW,
                    psp_stream_t stream);
/* The same products with the ReLU between two GCN layers (F.relu in GNN.py:43-61) folded in, so that neither the
 * activation nor its backward is a pass of its own:
 *   relu_x != 0 (transW == 0 only): Y = max(X, 0) * W -- the layer reads the previous layer's output through the ReLU;
 *   mask != NULL (transW != 0 only): Y = (X * W^T) where mask > 0, else 0; mask is [n, K2] -- the gradient with respect
 *   to the pre-activation values the layer was given. */
int psp_gemm_xw_act_f32(const float *X, const float *W, float *Y, long long n, int K1, int K2, int transW, int relu_x,
                        const float *mask, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: mean negative log-likelihood, the loss of the reference's training step (F.nll_loss(model(), labels),
 * GNN.py:131-146), forward and backward.  logp is [n, C] row-major log-probabilities, labels are int64; rows whose
 * label is outside [0, C) do not count.  loss: one float.  stats: psp_nll_loss_stats_floats() floats of device memory
 * (contents irrelevant on entry) that the forward call fills -- [0] the sum, [1] the number of rows that count, [2] the
 * number of labels outside [0, C) other than PyTorch's ignore_index -100 (PyTorch raises for those; check it where
 * that matters), the rest workspace -- and the backward call reads.  grad_loss: one float on the device (the incoming
 * gradient); grad_logp [n, C] is overwritten.  The partial sums of the workgroups are added in a fixed order: the
 * loss repeats bit for bit.
 * ------------------------------------------------------------------------------------------- */
int psp_nll_loss_stats_floats(void);
int psp_nll_loss_mean_f32(const float *logp, const long long *labels, long long n, int C, float *loss, float *stats,
                          psp_stream_t stream);
int psp_nll_loss_mean_backward_f32(const long long *labels, const float *grad_loss, const float *stats, long long n,
                                   int C, float *grad_logp, psp_stream_t stream);

/* The same loss from the logits: F.nll_loss(F.log_softmax(x, 1), labels) (GNN.py:61,78,101 with 131-146) in one pass
 * over x instead of five over the [n, C] matrix.  C a multiple of 4 up to 64 (psp_softmax_nll_supported), x 16-byte
 * aligned; loss and stats as above (stats[0] is the sum of the log-probabilities of the labels).  The backward call
 * writes d loss / d x = (softmax(x) - onehot(label)) * grad_loss / count for rows that count, 0 for the others. */
int psp_softmax_nll_supported(int C);
int psp_softmax_nll_mean_f32(const float *logits, const long long *labels, long long n, int C, float *loss, float *stats,
                             psp_stream_t stream);
int psp_softmax_nll_mean_backward_f32(const float *logits, const long long *labels, const float *grad_loss,
                                      const float *stats, long long n, int C, float *grad_logits, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: double precision.  The reference dispatches its SpMM / SDDMM kernels for double as well
 * (AT_DISPATCH_FLOATING_TYPES, SpMM_kernel.cu:149, sddmm_kernel.cu:161); these two entry points serve all six layouts:
 * vec_size 1 (CSR), 2 or 3 (blocks of vec_size x 1, val [nblk, vec_size]); target_row NULL = plain layout, else
 * row-split.  Same semantics as the float entry points (Y completely defined; SDDMM unscaled, zero where a block value
 * is zero).  One wavefront per segment, not tuned: GNN training is single precision.  CF / blkWarpNum do not apply.
 * ------------------------------------------------------------------------------------------- */
int psp_spmm_f64(const int *rowPtr, const int *colIdx, const double *val, const int *target_row, const double *X,
                 double *Y, int nseg, int N, int rows_out, int vec_size, psp_stream_t stream);
int psp_sddmm_f64(const int *rowPtr, const int *colIdx, const double *val_b, const int *target_row, const double *A,
                  const double *B, double *out, int nseg, int K, int vec_size, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: comparison baseline, ParamSpMM.gespmm_compute (SpMM/Baseline_kernel.cu:616-788): CSR SpMM with one
 * wavefront per row and the row's (column, value) pairs cached in LDS.  Y [M,N] is fully written.
 * ------------------------------------------------------------------------------------------- */
int psp_baseline_rowcache_spmm_f32(const int *rowPtr, const int *colIdx, const float *val, const float *X,
                                   float *Y, int M, int N, psp_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * DEVICE: measurement aid, no counterpart in the reference.  The gathers of an SpMM without the SpMM: for every
 * stored entry and every column tile (lanes_per_row lanes x float4) the X row tile is loaded and added up per
 * lane; there is no row structure, no multiplication and one 16-byte store per lane and wavefront.  Its duration
 * is the floor the memory system sets for any SpMM on the pattern (bench.py reports the kernel's time against it).
 * entries_per_wave: stored entries one wavefront walks (a multiple of 64); unroll: loads in flight per lane
 * (1, 2, 4, 8).  out: psp_probe_gather_out_floats(...) floats of device memory, overwritten.
 * ------------------------------------------------------------------------------------------- */
long long psp_probe_gather_out_floats(long long nnz, int N, int lanes_per_row, int entries_per_wave);
int psp_probe_gather_f32(const int *colIdx, long long nnz, const float *X, int N, int lanes_per_row, int unroll,
                         int entries_per_wave, float *out, long long out_floats, psp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PARAMSP_H */
