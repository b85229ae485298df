// PCSR index construction on the device: row splitting and 2x1 BCSR, the device twins of the host builders in
// capi.hip.  Same outputs, bit for bit, for CSR input whose rows hold strictly ascending column indices (what
// SciPy's coo -> csr conversion in graph_input.py:52-60 produces); other input is reported through a status word
// and left to the host builder.  The reference builds both on the host (SpMM/SpMM.cpp:15-75,
// graph_input.py:243-274); at millions of rows that is seconds of single-thread work per graph.
//
// Everything is count -> exclusive scan -> fill, so every output slot is written by exactly one lane and the
// result does not depend on scheduling.  Nothing allocates: the scan's workspace comes from the caller.
#include "psp_common.h"

#define SCAN_THREADS 256
#define SCAN_ITEMS 8
#define SCAN_TILE (SCAN_THREADS * SCAN_ITEMS)

// ---- exclusive scan of int32 ----------------------------------------------------------------------------------
// pass 1: tile-local exclusive scan, tile totals to ws; pass 2: one workgroup scans the totals (64-bit running
// sum, overflow past int32 raises PSP_BUILD_OVERFLOW in *status); pass 3: add the tile offsets, write out[n].
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane)
{
#pragma unroll
    for (int d = 1; d < PSP_WAVE; d <<= 1) {
        const int t = __shfl_up(v, d);
        if (lane >= d) v += t;
    }
    return v;
}

// block-wide exclusive scan of one value per thread; returns the exclusive prefix, *total = block sum
__device__ __forceinline__ int block_exclusive_scan(int v, int *total)
{
    __shared__ int s_wave[SCAN_THREADS / PSP_WAVE];
    const int lane = threadIdx.x & (PSP_WAVE - 1), wave = threadIdx.x >> 6;
    const int inc = wave_inclusive_scan(v, lane);
    __syncthreads();  // s_wave may still be read by the previous call
    if (lane == PSP_WAVE - 1) s_wave[wave] = inc;
    __syncthreads();
    int base = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < SCAN_THREADS / PSP_WAVE; w++) {
        const int t = s_wave[w];
        if (w < wave) base += t;
        sum += t;
    }
    *total = sum;
    return base + inc - v;
}

__global__ void __launch_bounds__(SCAN_THREADS) scan_tiles_kernel(const int *__restrict__ in, int *__restrict__ out,
                                                                  int *__restrict__ ws, int n)
{
    const long long t0 = (long long)blockIdx.x * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
    int v[SCAN_ITEMS], sum = 0;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; i++) {
        v[i] = (t0 + i < n) ? in[t0 + i] : 0;
        sum += v[i];
    }
    int total;
    int run = block_exclusive_scan(sum, &total);
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; i++) {
        if (t0 + i < n) out[t0 + i] = run;
        run += v[i];
    }
    if (threadIdx.x == 0) ws[blockIdx.x] = total;
}

__global__ void __launch_bounds__(SCAN_THREADS) scan_totals_kernel(int *__restrict__ ws, int ntiles, int *__restrict__ status)
{
    __shared__ long long s_carry;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    for (int b0 = 0; b0 < ntiles; b0 += SCAN_THREADS) {
        const int i = b0 + threadIdx.x;
        const int v = i < ntiles ? ws[i] : 0;
        int total;
        const int ex = block_exclusive_scan(v, &total);
        const long long carry = s_carry;
        if (carry + ex + v > 0x7fffffffLL && i < ntiles) atomicOr(status, PSP_BUILD_OVERFLOW);
        if (i < ntiles) ws[i] = (int)(carry + ex);
        __syncthreads();
        if (threadIdx.x == 0) s_carry = carry + total;
        __syncthreads();
    }
    if (threadIdx.x == 0) ws[ntiles] = (int)s_carry;  // grand total
}

__global__ void __launch_bounds__(SCAN_THREADS) scan_add_kernel(int *__restrict__ out, const int *__restrict__ ws, int n, int ntiles)
{
    const int add = ws[blockIdx.x];
    const long long t0 = (long long)blockIdx.x * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; i++)
        if (t0 + i < n) out[t0 + i] += add;
    if (blockIdx.x == 0 && threadIdx.x == 0) out[n] = ws[ntiles];
}

static int scan_tiles_of(int n) { return n <= 0 ? 0 : (int)(((long long)n + SCAN_TILE - 1) / SCAN_TILE); }

PSP_EXPORT int psp_scan_workspace_ints(int n) { return n < 0 ? 0 : scan_tiles_of(n) + 1; }

// out[0..n] = exclusive prefix sums of in[0..n) (out[n] = total); in and out may be the same array
static int exclusive_scan(const int *in, int *out, int n, int *ws, int ws_ints, int *status, hipStream_t stream)
{
    const int ntiles = scan_tiles_of(n);
    PSP_REQUIRE(ws && ws_ints >= ntiles + 1, "scan: workspace of %d ints, need %d", ws_ints, ntiles + 1);
    if (ntiles > 0) hipLaunchKernelGGL(scan_tiles_kernel, dim3(ntiles), dim3(SCAN_THREADS), 0, stream, in, out, ws, n);
    hipLaunchKernelGGL(scan_totals_kernel, dim3(1), dim3(SCAN_THREADS), 0, stream, ws, ntiles, status);
    hipLaunchKernelGGL(scan_add_kernel, dim3(ntiles > 0 ? ntiles : 1), dim3(SCAN_THREADS), 0, stream, out, ws, n, ntiles);
    return psp_check_launch("scan kernels");
}

// ---- row splitting ----------------------------------------------------------------------------------------------
__global__ void split_count_kernel(const int *__restrict__ rowPtr, int nrows, int g, int *__restrict__ counts,
                                   int *__restrict__ status)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nrows) return;
    const int k = rowPtr[i + 1] - rowPtr[i];
    if (k < 0) atomicOr(status, PSP_BUILD_BAD_ROWPTR);
    counts[i] = k > 0 ? (k + g - 1) / g : 0;
}

// one lane per segment: its row is the last one whose offset is <= s among rows that own segments
__global__ void split_fill_kernel(const int *__restrict__ rowPtr, const int *__restrict__ seg_off, int nrows, int g,
                                  int S, int *__restrict__ rowPtr_split, int *__restrict__ target_row)
{
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s == 0) rowPtr_split[0] = 0;
    if (s >= S) return;
    int lo = 0, hi = nrows;  // first row with seg_off[row + 1] > s
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (seg_off[mid + 1] > s) hi = mid; else lo = mid + 1;
    }
    const int j = s - seg_off[lo];
    const int lb = rowPtr[lo] + j * g;
    target_row[s] = lo;
    rowPtr_split[s + 1] = min(lb + g, rowPtr[lo + 1]);
}

PSP_EXPORT int psp_split_csr_offsets_dev(const int *rowPtr, int nrows, int g, int *row_split_offset, int *workspace,
                                         int workspace_ints, int *status, psp_stream_t stream)
{
    PSP_REQUIRE(rowPtr && row_split_offset && status && nrows >= 0, "split_csr_offsets_dev: bad input");
    PSP_REQUIRE(g >= 1, "split_csr_offsets_dev: granularity must be positive (got %d)", g);
    hipStream_t st = (hipStream_t)stream;
    if (nrows > 0)
        hipLaunchKernelGGL(split_count_kernel, dim3(psp_ceil_div(nrows, 256)), dim3(256), 0, st, rowPtr, nrows, g,
                           row_split_offset, status);
    return exclusive_scan(row_split_offset, row_split_offset, nrows, workspace, workspace_ints, status, st);
}

PSP_EXPORT int psp_split_csr_fill_dev(const int *rowPtr, const int *row_split_offset, int nrows, int g, int S,
                                      int *rowPtr_split, int *target_row, psp_stream_t stream)
{
    PSP_REQUIRE(rowPtr && row_split_offset && rowPtr_split && nrows >= 0 && S >= 0, "split_csr_fill_dev: bad input");
    PSP_REQUIRE(target_row || S == 0, "split_csr_fill_dev: target_row is null");
    PSP_REQUIRE(g >= 1, "split_csr_fill_dev: granularity must be positive (got %d)", g);
    hipLaunchKernelGGL(split_fill_kernel, dim3(psp_ceil_div(S > 0 ? S : 1, 256)), dim3(256), 0, (hipStream_t)stream, rowPtr,
                       row_split_offset, nrows, g, S, rowPtr_split, target_row);
    return psp_check_launch("split fill kernel");
}

// ---- BCSR 2x1 -----------------------------------------------------------------------------------------------------
// position of column c in the ascending range col[lo, hi), or -1
__device__ __forceinline__ int find_col(const int *__restrict__ col, int lo, int hi, int c)
{
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        const int v = col[mid];
        if (v == c) return mid;
        if (v < c) lo = mid + 1; else hi = mid;
    }
    return -1;
}

// first position in the ascending range col[lo, hi) whose column is not below c[k], for ILP columns at once: the
// searches have the same depth (`top` = largest power of two not above hi - lo, at least 1), so their loads overlap
template <int ILP>
__device__ __forceinline__ void lower_bound_batch(const int *__restrict__ col, int lo, int hi, int top, const int (&c)[ILP],
                                                  int (&pos)[ILP])
{
#pragma unroll
    for (int k = 0; k < ILP; k++) pos[k] = lo;
    if (hi <= lo) return;
    for (int step = top; step >= 1; step >>= 1) {
#pragma unroll
        for (int k = 0; k < ILP; k++)
            if (pos[k] + step <= hi && col[pos[k] + step - 1] < c[k]) pos[k] += step;
    }
}
__device__ __forceinline__ int top_power_of_two(int len)
{
    int top = 1;
    while (top * 2 <= len) top *= 2;
    return top;
}

// Block-rows with more stored entries than this are built by a whole workgroup (bcsr_long_kernel): walked by a single
// wavefront, the hub rows of a skewed graph were the tail of the launch (4.5 of 4.8 ms on an R-MAT graph).
#define BCSR_LONG 2048

// One wavefront per block-row t (rows 2t and 2t+1).  Blocks: the entries of row 2t in order, then the entries of
// row 2t+1 whose column row 2t does not hold, in order -- the first-encounter order of the host builder.
template <bool FILL>
__global__ void __launch_bounds__(256) bcsr_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx,
                                                   const float *__restrict__ val, int nrows, int nbr,
                                                   int *__restrict__ counts, const int *__restrict__ rowPtr_b,
                                                   int *__restrict__ colIdx_b, float *__restrict__ val_b,
                                                   int *__restrict__ status)
{
    const int lane = threadIdx.x & (PSP_WAVE - 1);
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= nbr) return;  // wave-uniform
    const int a0 = rowPtr[2 * t], a1 = rowPtr[2 * t + 1];
    const int b1 = (2 * t + 1 < nrows) ? rowPtr[2 * t + 2] : a1;  // odd row count: the last block-row has one row
    const int len0 = a1 - a0;
    if (a1 >= a0 && b1 >= a1 && b1 - a0 > BCSR_LONG) return;  // wave-uniform: bcsr_long_kernel takes this block-row

    if (!FILL) {
        // strictly ascending columns inside both rows?
        bool bad = a1 < a0 || b1 < a1;
        for (int p = a0 + lane; p < b1; p += PSP_WAVE)
            if (p != a0 && p != a1 && colIdx[p] <= colIdx[p - 1]) bad = true;
        if (bad) atomicOr(status, a1 < a0 || b1 < a1 ? PSP_BUILD_BAD_ROWPTR : PSP_BUILD_UNSORTED);
        if (a1 < a0 || b1 < a1) {
            if (lane == 0) counts[t] = 0;
            return;
        }
    } else {
        const int base = rowPtr_b[t];
        for (int i = lane; i < len0; i += PSP_WAVE) {
            const int c = colIdx[a0 + i];
            const int q = find_col(colIdx, a1, b1, c);
            colIdx_b[base + i] = c;
            val_b[2 * (size_t)(base + i)] = val[a0 + i];
            val_b[2 * (size_t)(base + i) + 1] = q >= 0 ? val[q] : 0.0f;
        }
    }

    // entries of row 2t+1 that open a block of their own, ranked in order
    int fresh = 0;
    for (int p0 = a1; p0 < b1; p0 += PSP_WAVE) {
        const int p = p0 + lane;
        bool mine = false;
        int c = 0;
        if (p < b1) {
            c = colIdx[p];
            mine = find_col(colIdx, a0, a1, c) < 0;
        }
        const unsigned long long m = __ballot(mine);
        if (FILL && mine) {
            const int slot = rowPtr_b[t] + len0 + fresh + __popcll(m & ((1ull << lane) - 1ull));
            colIdx_b[slot] = c;
            val_b[2 * (size_t)slot] = 0.0f;
            val_b[2 * (size_t)slot + 1] = val[p];
        }
        fresh += __popcll(m);
    }
    if (!FILL && lane == 0) counts[t] = len0 + fresh;
}

// The long block-rows, one workgroup of 1024 lanes at a time.  Workgroup w looks at the block-rows w, w + G, w + 2G, ...
// (hub rows often sit next to each other; this spreads them over the workgroups), 1024 of them per round: the lanes
// list the long ones in LDS, then build each together.  Every lane looks up four entries at once, the ranks of the
// entries that open their own block come from ballots, a prefix over the 16 wavefronts and the running total.
template <bool FILL>
__global__ void __launch_bounds__(1024) bcsr_long_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx,
                                                         const float *__restrict__ val, int nrows, int nbr,
                                                         int *__restrict__ counts, const int *__restrict__ rowPtr_b,
                                                         int *__restrict__ colIdx_b, float *__restrict__ val_b,
                                                         int *__restrict__ status)
{
    constexpr int ILP = 4, WAVES = 16;
    __shared__ int s_list[1024];
    __shared__ int s_nlist;
    __shared__ int s_wave[ILP][WAVES];
    const int tid = threadIdx.x, lane = tid & (PSP_WAVE - 1), wave = tid >> 6;
    const long long G = gridDim.x;
    for (long long i0 = 0; i0 * G < nbr; i0 += 1024) {
        if (tid == 0) s_nlist = 0;
        __syncthreads();
        const long long tt = (i0 + tid) * G + blockIdx.x;
        const int mine_t = (int)tt;
        if (tt < nbr) {
            const int a0 = rowPtr[2 * mine_t], a1 = rowPtr[2 * mine_t + 1];
            const int b1 = (2 * mine_t + 1 < nrows) ? rowPtr[2 * mine_t + 2] : a1;
            if (a1 >= a0 && b1 >= a1 && b1 - a0 > BCSR_LONG) s_list[atomicAdd(&s_nlist, 1)] = mine_t;
        }
        __syncthreads();
        const int nlist = s_nlist;
        for (int li = 0; li < nlist; li++) {
            const int t = s_list[li];  // the order of the list does not matter: every block-row has its own output range
            const int a0 = rowPtr[2 * t], a1 = rowPtr[2 * t + 1];
            const int b1 = (2 * t + 1 < nrows) ? rowPtr[2 * t + 2] : a1;
            const int len0 = a1 - a0;
            if (!FILL) {
                bool bad = false;  // strictly ascending columns inside both rows?
                for (int p = a0 + tid; p < b1; p += 1024)
                    if (p != a0 && p != a1 && colIdx[p] <= colIdx[p - 1]) bad = true;
                if (bad) atomicOr(status, PSP_BUILD_UNSORTED);
            } else {
                const int base = rowPtr_b[t];
                const int top1 = top_power_of_two(b1 - a1);
                for (int i0e = 0; i0e < len0; i0e += ILP * 1024) {
                    int c[ILP], q[ILP];
#pragma unroll
                    for (int k = 0; k < ILP; k++) {
                        const int i = i0e + k * 1024 + tid;
                        c[k] = i < len0 ? colIdx[a0 + i] : 0;
                    }
                    lower_bound_batch<ILP>(colIdx, a1, b1, top1, c, q);
#pragma unroll
                    for (int k = 0; k < ILP; k++) {
                        const int i = i0e + k * 1024 + tid;
                        if (i < len0) {
                            const bool hit = q[k] < b1 && colIdx[q[k]] == c[k];
                            colIdx_b[base + i] = c[k];
                            val_b[2 * (size_t)(base + i)] = val[a0 + i];
                            val_b[2 * (size_t)(base + i) + 1] = hit ? val[q[k]] : 0.0f;
                        }
                    }
                }
            }
            // entries of row 2t+1 that open a block of their own, ranked in order
            const int top = top_power_of_two(len0);
            int fresh = 0;
            for (int p0 = a1; p0 < b1; p0 += ILP * 1024) {
                int c[ILP], lo[ILP];
                bool in[ILP], mine[ILP];
#pragma unroll
                for (int k = 0; k < ILP; k++) {
                    const int p = p0 + k * 1024 + tid;
                    in[k] = p < b1;
                    c[k] = in[k] ? colIdx[p] : 0;
                }
                lower_bound_batch<ILP>(colIdx, a0, a1, top, c, lo);
#pragma unroll
                for (int k = 0; k < ILP; k++) {
                    mine[k] = in[k] && !(lo[k] < a1 && colIdx[lo[k]] == c[k]);
                    const unsigned long long m = __ballot(mine[k]);
                    if (lane == 0) s_wave[k][wave] = __popcll(m);
                    lo[k] = __popcll(m & ((1ull << lane) - 1ull));  // rank inside the wavefront
                }
                __syncthreads();
                int before = fresh;  // blocks opened by earlier chunks, earlier wavefronts of this chunk
#pragma unroll
                for (int k = 0; k < ILP; k++) {
                    int chunk_total = 0, ahead = 0;
#pragma unroll
                    for (int w = 0; w < WAVES; w++) {
                        const int n_w = s_wave[k][w];
                        if (w < wave) ahead += n_w;
                        chunk_total += n_w;
                    }
                    if (FILL && mine[k]) {
                        const int slot = rowPtr_b[t] + len0 + before + ahead + lo[k];
                        const int p = p0 + k * 1024 + tid;
                        colIdx_b[slot] = c[k];
                        val_b[2 * (size_t)slot] = 0.0f;
                        val_b[2 * (size_t)slot + 1] = val[p];
                    }
                    before += chunk_total;
                }
                fresh = before;
                __syncthreads();  // s_wave is rewritten by the next round
            }
            if (!FILL && tid == 0) counts[t] = len0 + fresh;
        }
        __syncthreads();  // s_list / s_nlist are rewritten by the next slab
    }
}

static void launch_bcsr(bool fill, const int *rowPtr, const int *colIdx, const float *val, int nrows, int nbr, int *counts,
                        const int *rowPtr_b, int *colIdx_b, float *val_b, int *status, hipStream_t st)
{
    // about two workgroups of 1024 lanes per CU; a prime (odd) count, because the workgroups take block-rows by index
    // modulo the count and hub rows of generated graphs share their low index bits
    int long_wgs = psp_ceil_div(nbr, 64);
    long_wgs = long_wgs >= 509 ? 509 : (long_wgs | 1);
    if (fill) {
        hipLaunchKernelGGL(bcsr_kernel<true>, dim3(psp_ceil_div(nbr, 4)), dim3(256), 0, st, rowPtr, colIdx, val, nrows, nbr,
                           counts, rowPtr_b, colIdx_b, val_b, status);
        hipLaunchKernelGGL(bcsr_long_kernel<true>, dim3(long_wgs), dim3(1024), 0, st, rowPtr, colIdx, val, nrows, nbr, counts,
                           rowPtr_b, colIdx_b, val_b, status);
    } else {
        hipLaunchKernelGGL(bcsr_kernel<false>, dim3(psp_ceil_div(nbr, 4)), dim3(256), 0, st, rowPtr, colIdx, val, nrows, nbr,
                           counts, rowPtr_b, colIdx_b, val_b, status);
        hipLaunchKernelGGL(bcsr_long_kernel<false>, dim3(long_wgs), dim3(1024), 0, st, rowPtr, colIdx, val, nrows, nbr, counts,
                           rowPtr_b, colIdx_b, val_b, status);
    }
}

PSP_EXPORT int psp_bcsr_offsets_dev(const int *rowPtr, const int *colIdx, int nrows, int *rowPtr_b, int *workspace,
                                    int workspace_ints, int *status, psp_stream_t stream)
{
    PSP_REQUIRE(rowPtr && rowPtr_b && status && nrows >= 0, "bcsr_offsets_dev: bad input");
    const int nbr = (nrows + 1) / 2;
    hipStream_t st = (hipStream_t)stream;
    if (nbr > 0) {  // colIdx may be null for a matrix without entries (the host cannot tell, rowPtr is on the device)
        launch_bcsr(false, rowPtr, colIdx, nullptr, nrows, nbr, rowPtr_b, nullptr, nullptr, nullptr, status, st);
    }
    return exclusive_scan(rowPtr_b, rowPtr_b, nbr, workspace, workspace_ints, status, st);
}

PSP_EXPORT int psp_bcsr_fill_dev(const int *rowPtr, const int *colIdx, const float *val, int nrows, const int *rowPtr_b,
                                 int *colIdx_b, float *val_b, psp_stream_t stream)
{
    PSP_REQUIRE(rowPtr && rowPtr_b && nrows >= 0, "bcsr_fill_dev: bad input");
    const int nbr = (nrows + 1) / 2;
    if (nbr == 0) return PSP_OK;  // the entry arrays may be null when rowPtr_b says there are no blocks
    launch_bcsr(true, rowPtr, colIdx, val, nrows, nbr, nullptr, rowPtr_b, colIdx_b, val_b, nullptr, (hipStream_t)stream);
    return psp_check_launch("bcsr fill kernel");
}

// ---- index validation ---------------------------------------------------------------------------------------------
// The SpMM / SDDMM kernels trust their index arrays, as the reference's kernels do: a column index outside X makes
// them read outside the buffer.  This pass lets a caller check arrays of unknown origin once, on the device.
__global__ void check_index_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx,
                                   const int *__restrict__ target_row, int M, int nnz, int ncols, int target_rows,
                                   int *__restrict__ status)
{
    const long long stride = (long long)gridDim.x * blockDim.x;
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    int bad = 0;
    if (t == 0 && (rowPtr[0] != 0 || rowPtr[M] != nnz)) bad |= PSP_BUILD_BAD_ROWPTR;
    for (long long i = t; i < M; i += stride) {
        const int a = rowPtr[i], b = rowPtr[i + 1];
        if (a > b || a < 0 || b > nnz) bad |= PSP_BUILD_BAD_ROWPTR;
        if (target_row) {
            const int r = target_row[i];
            if (r < 0 || r >= target_rows || (i > 0 && target_row[i - 1] > r)) bad |= PSP_BUILD_BAD_TARGET;
        }
    }
    for (long long p = t; p < nnz; p += stride) {
        const int c = colIdx[p];
        if (c < 0 || c >= ncols) bad |= PSP_BUILD_BAD_COLUMN;
    }
    if (bad) atomicOr(status, bad);
}

PSP_EXPORT int psp_check_index_dev(const int *rowPtr, const int *colIdx, const int *target_row, int M, int nnz, int ncols,
                                   int target_rows, int *status, psp_stream_t stream)
{
    PSP_REQUIRE(rowPtr && status && M >= 0 && nnz >= 0 && ncols >= 0, "check_index_dev: bad input");
    PSP_REQUIRE(colIdx || nnz == 0, "check_index_dev: colIdx is null");
    const long long work = (long long)M > nnz ? M : nnz;
    int blocks = psp_ceil_div(work > 0 ? work : 1, 256);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(check_index_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, rowPtr, colIdx, target_row, M, nnz,
                       ncols, target_rows, status);
    return psp_check_launch("index check kernel");
}
