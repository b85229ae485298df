/*
 * CPU oracle for the ParamSpMM / ParamSDDMM hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package links, loads or
 * calls this file; only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py may use it, and only as the checker.
 *
 * Every function restates, in plain scalar C, the algorithm of one piece of
 * the reference (zzzlxhhh/ParamSpMM_AE); the cited file:line is the code it
 * follows.  Floating point follows the reference kernels' evaluation order:
 * one fp32 fused multiply-add per non-zero, in storage order (nvcc contracts
 * `res += val * x` into an FMA by default), and for SDDMM the 32-lane strided
 * partial sums followed by the xor butterfly 16,8,4,2,1.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   orc_split_csr(_par)   brute-force Python loop, numpy closed form, the
 *                         pubmed segment counts (20005 / 10293 / 10240)
 *   orc_bcsr_build        scipy.sparse csr.tobsr((2,1)) (the routine the
 *                         reference itself calls), the hand case
 *                         rows {0:[1,5],1:[0,5,7]}, pubmed block counts
 *   orc_vbsr_build        scipy.sparse csr.tobsr((R,1)) for R = 3, 4; equals
 *                         orc_bcsr_build for R = 2
 *   orc_genmask           brute force + permutation-within-row invariant
 *   orc_spmm_*            torch.sparse.mm on CPU (the reference's own
 *                         checker), fp64 dense product, X = ones -> row sums
 *   orc_spmm_vec          equals orc_spmm_bcsr(_split) for R = 2; for R = 3 the
 *                         CSR product of the same matrix (entry by entry the
 *                         same FMA chain), fp64 dense product
 *   orc_sddmm_vec         equals orc_sddmm_bcsr(_split) for R = 2; fp64 dots
 *   orc_sddmm_*           fp64 gathered dot products, A = B = ones -> K
 *   orc_segment_softmax   closed form in fp64 (no reference counterpart)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------------- */
/* Row splitting: SpMM/SpMM.cpp:15-40 (serial) and 42-75 (parallel twin). */
/* Returns the number of segments S.  Outputs may be NULL to count only.  */
ORC_API int orc_split_csr(const int *rowPtr, int nrows, int g,
                          int *rowPtr_split, int *target_row)
{
    int s = 0;
    if (rowPtr_split) rowPtr_split[0] = 0;
    for (int i = 0; i < nrows; i++) {
        int lb = rowPtr[i], hb = rowPtr[i + 1];
        for (; lb < hb; lb += g) {
            if (target_row) target_row[s] = i;
            if (rowPtr_split) rowPtr_split[s + 1] = (lb + g > hb) ? hb : lb + g;
            s++;
        }
    }
    return s;
}

/* SpMM/SpMM.cpp:42-75: same result, but every row starts at a caller-supplied
 * exclusive prefix of the per-row segment counts (graph_input.py:135-136). */
ORC_API int orc_split_csr_par(const int *rowPtr, const int *row_split_offset,
                              int nrows, int g, int *rowPtr_split, int *target_row)
{
    int S = row_split_offset[nrows];
    rowPtr_split[0] = 0;
    for (int i = 0; i < nrows; i++) {
        int lb = rowPtr[i], hb = rowPtr[i + 1];
        int off = row_split_offset[i];
        for (; lb < hb; lb += g) {
            target_row[off] = i;
            rowPtr_split[off + 1] = (lb + g > hb) ? hb : lb + g;
            off++;
        }
    }
    return S;
}

/* ---------------------------------------------------------------------- */
/* BCSR with 2x1 blocks: graph_input.py:243-266 calls SciPy's tobsr, whose
 * csr_tobsr walks the two rows of a block-row in order and opens a new block
 * the first time a column is met (no re-sorting).  nrows may be odd: the
 * missing last row is empty (graph_input.py:248-255 pads rowPtr).
 * Call with colIdx_b == NULL to obtain the block count first.            */
ORC_API int orc_bcsr_build(const int *rowPtr, const int *colIdx, const float *val,
                           int nrows, int ncols,
                           int *rowPtr_b, int *colIdx_b, float *val_b)
{
    int nbr = (nrows + 1) / 2;
    int *slot = (int *)malloc(sizeof(int) * (size_t)(ncols > 0 ? ncols : 1));
    for (int c = 0; c < ncols; c++) slot[c] = -1;
    int nblk = 0;
    if (rowPtr_b) rowPtr_b[0] = 0;
    for (int t = 0; t < nbr; t++) {
        int first = nblk;
        for (int k = 0; k < 2; k++) {
            int r = 2 * t + k;
            if (r >= nrows) break;
            for (int p = rowPtr[r]; p < rowPtr[r + 1]; p++) {
                int c = colIdx[p];
                if (slot[c] < first) { /* not yet opened in this block-row */
                    slot[c] = nblk;
                    if (colIdx_b) {
                        colIdx_b[nblk] = c;
                        val_b[2 * (size_t)nblk] = 0.0f;
                        val_b[2 * (size_t)nblk + 1] = 0.0f;
                    }
                    nblk++;
                }
                if (colIdx_b) val_b[2 * (size_t)slot[c] + k] += val[p];
            }
        }
        if (rowPtr_b) rowPtr_b[t + 1] = nblk;
    }
    free(slot);
    return nblk;
}

/* Blocks of R x 1 for any R (graph_input.py:243-266 with blk_size = R; the reference instantiates its kernels for
 * R = 3 besides the 2 x 1 case above).  Same first-encounter block order: SciPy's csr_tobsr walks the R rows of a
 * block-row in turn and opens a block at the first entry of a column.  val_b is [nblk, R].                        */
ORC_API int orc_vbsr_build(const int *rowPtr, const int *colIdx, const float *val,
                           int nrows, int ncols, int R,
                           int *rowPtr_b, int *colIdx_b, float *val_b)
{
    int nbr = (nrows + R - 1) / R;
    int *slot = (int *)malloc(sizeof(int) * (size_t)(ncols > 0 ? ncols : 1));
    for (int c = 0; c < ncols; c++) slot[c] = -1;
    int nblk = 0;
    if (rowPtr_b) rowPtr_b[0] = 0;
    for (int t = 0; t < nbr; t++) {
        int first = nblk;
        for (int k = 0; k < R; k++) {
            int r = R * t + k;
            if (r >= nrows) break;
            for (int p = rowPtr[r]; p < rowPtr[r + 1]; p++) {
                int c = colIdx[p];
                if (slot[c] < first) {
                    slot[c] = nblk;
                    if (colIdx_b) {
                        colIdx_b[nblk] = c;
                        for (int q = 0; q < R; q++) val_b[(size_t)R * nblk + q] = 0.0f;
                    }
                    nblk++;
                }
                if (colIdx_b) val_b[(size_t)R * slot[c] + k] += val[p];
            }
        }
        if (rowPtr_b) rowPtr_b[t + 1] = nblk;
    }
    free(slot);
    return nblk;
}

/* genmask: SDDMM/sddmm_kernel.cu:78-107.  mask has nnz entries and is
 * pre-zeroed by the caller (sddmm_kernel.cu:126).                        */
ORC_API void orc_genmask(const int *rowPtr_b, const int *rowPtr, const float *val_b,
                         int nblkrows, int *mask)
{
    for (int t = 0; t < nblkrows; t++) {
        int lb = rowPtr_b[t], hb = rowPtr_b[t + 1];
        if (lb == hb) continue;
        int cnt0 = rowPtr[2 * t], cnt1 = rowPtr[2 * t + 1];
        for (int i = lb; i < hb; i++) {
            if (val_b[2 * (size_t)i] != 0.0f) mask[cnt0++] = i * 2;
            if (val_b[2 * (size_t)i + 1] != 0.0f) mask[cnt1++] = i * 2 + 1;
        }
    }
}

/* ---------------------------------------------------------------------- */
/* SpMM.  Y is [rows_out, N] row-major and is zeroed here first
 * (SpMM/SpMM_kernel.cu:136 zeros_like; 281-282 padded zeros for bcsr).   */

/* SpMM/SpMM_kernel.cu:1157-1243 */
ORC_API void orc_spmm_csr(const int *rowPtr, const int *colIdx, const float *val,
                          const float *X, float *Y, int M, int N, int rows_out)
{
    memset(Y, 0, sizeof(float) * (size_t)rows_out * N);
    for (int r = 0; r < M; r++)
        for (int c = 0; c < N; c++) {
            float res = 0.0f;
            for (int p = rowPtr[r]; p < rowPtr[r + 1]; p++)
                res = fmaf(val[p], X[(size_t)colIdx[p] * N + c], res);
            Y[(size_t)r * N + c] = res;
        }
}

/* SpMM/SpMM_kernel.cu:1245-1360: per-segment FMA chain, then an add into the
 * target row.  The reference adds with atomics in arbitrary order; the oracle
 * fixes segment order.                                                    */
ORC_API void orc_spmm_csr_split(const int *rowPtr_split, const int *colIdx, const float *val,
                                const int *target_row, const float *X, float *Y,
                                int S, int N, int rows_out)
{
    memset(Y, 0, sizeof(float) * (size_t)rows_out * N);
    for (int s = 0; s < S; s++) {
        int r = target_row[s];
        for (int c = 0; c < N; c++) {
            float res = 0.0f;
            for (int p = rowPtr_split[s]; p < rowPtr_split[s + 1]; p++)
                res = fmaf(X[(size_t)colIdx[p] * N + c], val[p], res);
            Y[(size_t)r * N + c] += res;
        }
    }
}

/* SpMM/SpMM_kernel.cu:1362-1493: 2x1 blocks, a lane's FMA is skipped when the
 * block entry is zero (1399,1405). rows_out must be >= 2*Mb.              */
ORC_API void orc_spmm_bcsr(const int *rowPtr_b, const int *colIdx_b, const float *val_b,
                           const float *X, float *Y, int Mb, int N, int rows_out)
{
    memset(Y, 0, sizeof(float) * (size_t)rows_out * N);
    for (int t = 0; t < Mb; t++)
        for (int c = 0; c < N; c++) {
            float r0 = 0.0f, r1 = 0.0f;
            for (int p = rowPtr_b[t]; p < rowPtr_b[t + 1]; p++) {
                float b = X[(size_t)colIdx_b[p] * N + c];
                float v0 = val_b[2 * (size_t)p], v1 = val_b[2 * (size_t)p + 1];
                if (v0 != 0.0f) r0 = fmaf(v0, b, r0);
                if (v1 != 0.0f) r1 = fmaf(v1, b, r1);
            }
            Y[(size_t)(2 * t) * N + c] = r0;
            Y[(size_t)(2 * t + 1) * N + c] = r1;
        }
}

/* SpMM/SpMM_kernel.cu:1495-1651 */
ORC_API void orc_spmm_bcsr_split(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                                 const int *target_row, const float *X, float *Y,
                                 int Sb, int N, int rows_out)
{
    memset(Y, 0, sizeof(float) * (size_t)rows_out * N);
    for (int s = 0; s < Sb; s++) {
        int t = target_row[s];
        for (int c = 0; c < N; c++) {
            float r0 = 0.0f, r1 = 0.0f;
            for (int p = rowPtr_bs[s]; p < rowPtr_bs[s + 1]; p++) {
                float b = X[(size_t)colIdx_b[p] * N + c];
                float v0 = val_b[2 * (size_t)p], v1 = val_b[2 * (size_t)p + 1];
                if (v0 != 0.0f) r0 = fmaf(v0, b, r0);
                if (v1 != 0.0f) r1 = fmaf(v1, b, r1);
            }
            Y[(size_t)(2 * t) * N + c] += r0;
            Y[(size_t)(2 * t + 1) * N + c] += r1;
        }
    }
}

/* SpMM/SpMM_kernel.cu:1653-1770 (vec_spmm) and 1772-1972 (vec_split_spmm): R x 1 blocks, the 2 x 1 rule for
 * every one of the R entries of a block (a zero entry adds nothing, 1693-1699).  target_row = NULL: plain format
 * (segment s is block-row s).  rows_out >= R * (number of block-rows).                                             */
ORC_API void orc_spmm_vec(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const int *target_row,
                          const float *X, float *Y, int S, int N, int rows_out, int R)
{
    memset(Y, 0, sizeof(float) * (size_t)rows_out * N);
    for (int s = 0; s < S; s++) {
        int t = target_row ? target_row[s] : s;
        for (int c = 0; c < N; c++)
            for (int q = 0; q < R; q++) {
                float r = 0.0f;
                for (int p = rowPtr_b[s]; p < rowPtr_b[s + 1]; p++) {
                    float v = val_b[(size_t)R * p + q];
                    if (v != 0.0f) r = fmaf(v, X[(size_t)colIdx_b[p] * N + c], r);
                }
                Y[(size_t)(R * t + q) * N + c] += r;
            }
    }
}

/* ---------------------------------------------------------------------- */
/* SDDMM.  One 32-lane warp per row: lane l accumulates k = l, l+32, ... by
 * FMA from zero, then res += shfl_xor(res, s) for s = 16,8,4,2,1
 * (SDDMM/sddmm_kernel.cu:944-981).  `values` never scales the result.     */
static float warp_dot(const float *a, const float *b, int K)
{
    float lane[32];
    for (int l = 0; l < 32; l++) {
        float res = 0.0f;
        for (int k = l; k < K; k += 32) res = fmaf(a[k], b[k], res);
        lane[l] = res;
    }
    for (int stride = 16; stride > 0; stride >>= 1) {
        float nxt[32];
        for (int l = 0; l < 32; l++) nxt[l] = lane[l] + lane[l ^ stride];
        memcpy(lane, nxt, sizeof(lane));
    }
    return lane[0];
}

/* SDDMM/sddmm_kernel.cu:917-983; out has nnz entries, zeroed first (149). */
ORC_API void orc_sddmm_csr(const int *rowPtr, const int *colIdx,
                           const float *A, const float *B, float *out,
                           int M, int K, int nnz)
{
    memset(out, 0, sizeof(float) * (size_t)nnz);
    for (int r = 0; r < M; r++)
        for (int p = rowPtr[r]; p < rowPtr[r + 1]; p++)
            out[p] = warp_dot(A + (size_t)r * K, B + (size_t)colIdx[p] * K, K);
}

/* SDDMM/sddmm_kernel.cu:986-1057: the A row is target_row[segment]. */
ORC_API void orc_sddmm_csr_split(const int *rowPtr_split, const int *colIdx, const int *target_row,
                                 const float *A, const float *B, float *out,
                                 int S, int K, int nnz)
{
    memset(out, 0, sizeof(float) * (size_t)nnz);
    for (int s = 0; s < S; s++) {
        int r = target_row[s];
        for (int p = rowPtr_split[s]; p < rowPtr_split[s + 1]; p++)
            out[p] = warp_dot(A + (size_t)r * K, B + (size_t)colIdx[p] * K, K);
    }
}

/* SDDMM/sddmm_kernel.cu:1059-1176: out is [nblk,2]; an entry is computed only
 * where the block value is non-zero (1103,1115), else it stays zero.      */
ORC_API void orc_sddmm_bcsr(const int *rowPtr_b, const int *colIdx_b, const float *val_b,
                            const float *A, const float *B, float *out,
                            int Mb, int K, int nblk)
{
    memset(out, 0, sizeof(float) * 2 * (size_t)nblk);
    for (int t = 0; t < Mb; t++)
        for (int p = rowPtr_b[t]; p < rowPtr_b[t + 1]; p++) {
            const float *b = B + (size_t)colIdx_b[p] * K;
            if (val_b[2 * (size_t)p] != 0.0f)
                out[2 * (size_t)p] = warp_dot(A + (size_t)(2 * t) * K, b, K);
            if (val_b[2 * (size_t)p + 1] != 0.0f)
                out[2 * (size_t)p + 1] = warp_dot(A + (size_t)(2 * t + 1) * K, b, K);
        }
}

/* SDDMM/sddmm_kernel.cu:1178-1287 */
ORC_API void orc_sddmm_bcsr_split(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                                  const int *target_row, const float *A, const float *B, float *out,
                                  int Sb, int K, int nblk)
{
    memset(out, 0, sizeof(float) * 2 * (size_t)nblk);
    for (int s = 0; s < Sb; s++) {
        int t = target_row[s];
        for (int p = rowPtr_bs[s]; p < rowPtr_bs[s + 1]; p++) {
            const float *b = B + (size_t)colIdx_b[p] * K;
            if (val_b[2 * (size_t)p] != 0.0f)
                out[2 * (size_t)p] = warp_dot(A + (size_t)(2 * t) * K, b, K);
            if (val_b[2 * (size_t)p + 1] != 0.0f)
                out[2 * (size_t)p + 1] = warp_dot(A + (size_t)(2 * t + 1) * K, b, K);
        }
    }
}

/* R x 1 blocks, the intended generalisation of the 2 x 1 functions above (the reference's vec_sddmm kernels,
 * sddmm_kernel.cu:1289-1468, index their shared memory with CF*2 instead of CF*vec_size and are never run; their
 * evident intent is restated here, not their bug).  out is [nblk, R]; target_row = NULL: plain format.           */
ORC_API void orc_sddmm_vec(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const int *target_row,
                           const float *A, const float *B, float *out, int S, int K, int nblk, int R)
{
    memset(out, 0, sizeof(float) * (size_t)R * nblk);
    for (int s = 0; s < S; s++) {
        int t = target_row ? target_row[s] : s;
        for (int p = rowPtr_b[s]; p < rowPtr_b[s + 1]; p++) {
            const float *b = B + (size_t)colIdx_b[p] * K;
            for (int q = 0; q < R; q++)
                if (val_b[(size_t)R * p + q] != 0.0f)
                    out[(size_t)R * p + q] = warp_dot(A + (size_t)(R * t + q) * K, b, K);
        }
    }
}

/* ---------------------------------------------------------------------- */
/* Row softmax over the stored entries of each CSR row.  The reference has no
 * such op (gnn_conv.py:136-142 applies no softmax); it exists for the AGNN
 * attention benchmark.  Computed in double, rounded once to fp32.         */
ORC_API void orc_segment_softmax(const int *rowPtr, const float *in, float *out, int M)
{
    for (int r = 0; r < M; r++) {
        int lb = rowPtr[r], hb = rowPtr[r + 1];
        if (lb == hb) continue;
        double mx = in[lb];
        for (int p = lb + 1; p < hb; p++) if (in[p] > mx) mx = in[p];
        double sum = 0.0;
        for (int p = lb; p < hb; p++) sum += exp((double)in[p] - mx);
        for (int p = lb; p < hb; p++) out[p] = (float)(exp((double)in[p] - mx) / sum);
    }
}
