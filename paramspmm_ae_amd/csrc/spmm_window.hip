// Windowed CSR SpMM for gfx950: Y = A X for matrices whose entries cluster around the diagonal (community-ordered
// graphs, meshes, banded matrices).  No counterpart in the reference; it is a fifth representation beside the four
// PCSR ones, for the case the counters show the row-wise kernel bound by the gather path (texture addresser and L1)
// instead of by HBM: on a community-ordered block model nine out of ten gathered X rows are rows the neighbouring
// sparse rows gather as well.
//
// Format (psp_window_build / psp_window_build_dev).  The rows are cut into blocks of PSP_WINDOW_BLOCK = 64; the
// window of a block is the row range [64 b - 88, 64 b + 152), i.e. the block and PSP_WINDOW_HALO = 88 rows either
// side (the widest halo with which two workgroups of the 64-column variant still share a CU's 160 KB of LDS: every
// remote entry costs a gather of its own and, past the few whose rows are prefetched, a wait).  An entry is *local* when its column lies inside its row's window.  Every row keeps its entries, local ones
// first (each part in the original order), and rowPtr_w[2M + 2] holds for row i the start of the row at 2i and the
// start of its remote part at 2i + 1; entries 2M and 2M + 1 hold nnz.  Columns stay absolute, so any CSR kernel can
// read (rowPtr_w[0::2], colIdx_w, val_w) as an ordinary matrix with unsorted rows.
//
// Kernel.  A workgroup of 256 lanes walks a run of consecutive 64-row blocks for one column tile of TN = 16 / 32 / 64
// floats.  The X rows of the current block's window sit in LDS in a ring of 64 + 2 * 88 + 64 = 304 rows (row g in slot
// g mod 304): the windows of neighbouring blocks differ by 64 rows, so a step to the next block loads only the 64 rows
// that enter -- and they land in the slots of the 64 rows that the block after next no longer needs, so the ring never
// overwrites a row that is still being read and one barrier per block is enough.  A lane group of L = 4 or 8 lanes
// owns one row of a block (workgroups of 512 lanes for L = 8).  The walk is software-pipelined, so that after the first block of a run no lane waits for
// a load it has just issued: while block j is summed from LDS, the loads in flight are
//   * the X row tiles of block j's remote entries (up to UR = 4 per row, gathered from global memory into registers,
//     issued when block j - 1 was finished),
//   * the 64 new window rows, the (column, value) pairs and the row bounds of the blocks that follow.
// Local entries are read with ds_read_b128 -- no global gather instruction in that loop; the (column, value) pairs
// travel round the lane group with DPP moves, not through the LDS crossbar.  A lane group of 8 keeps the pairs of a
// row's first eight remote entries (entry e in lane e) and gathers the rows of entries 4 .. 7 together, in a second
// round, when some row of the wavefront has that many; prefetch slots past a row's remote part read one shared address.
// Rows with more than 32 local or 8 (groups of 4 lanes: 4) remote entries finish in plain loops (correct for any
// matrix, slow for matrices the format is not meant for).  Per
// element the sum runs over the local entries in storage order, then the remote ones: within the stated fp32
// tolerance of the reference's chain, not bit-identical to it.
// EPI (square layers of 16 or 32 columns, one column tile): the finished row is multiplied by a small dense matrix
// before it is stored, Y = (A f(X)) W or (A f(X)) W^T -- the dense product of a GCN layer folded into the sparse one.
// W sits in LDS (transposed on the way in for W^T); a lane group gathers its row of A f(X) with DPP moves and each lane
// forms its four output columns (N multiply-adds per column).  The row of A f(X) itself can be stored as well (Y_raw:
// the backward pass needs A dY for the weight gradient and (A dY) W^T for the input gradient).  Measured and dropped:
// the same product on the matrix cores (the block's 64 rows parked in LDS, one 16 x 16 tile per wavefront):
// the extra barrier per block and the 4-byte stores of the tile layout cost more than the multiply-adds they replace
// (GCN epoch, hidden 16 / 32: 1.71 / 2.60 ms against 1.61 / 2.49).
// relu_x applies max(x, 0) to X as it enters (once per window element rather than once per gather); mask keeps an
// output element only where mask > 0, read where the row is stored -- the two halves of a ReLU folded into the
// product, as psp_spmm_act_f32 offers for the other formats.
#include "psp_common.h"

#include "window_common.h"

template <int C, int LOGL, int PSPW_THREADS, bool EPI = false>
__global__ void __launch_bounds__(PSPW_THREADS)
psp_spmm_window_kernel(const int *__restrict__ rowPtr_w, const int *__restrict__ colIdx, const float *__restrict__ val,
                       const float *__restrict__ X, float *__restrict__ Y, const float *__restrict__ mask, int M, int N,
                       int nnz, int nruns, int stripe, int run, int relu_x, const float *__restrict__ W, int transW,
                       float *__restrict__ Y_raw)
{
    constexpr int L = 1 << LOGL;
    static_assert(!EPI || C == 1, "the dense epilogue exists for one vector per lane (one column tile of 16 or 32)");
    constexpr int TN = L * C * 4;                  // columns per tile
    constexpr int RB = PSPW_BLOCK;                 // rows per step
    constexpr int RPG = RB * L / PSPW_THREADS;     // rows per lane group
    constexpr int RING = RB + 2 * PSPW_HALO + RB;  // window + the rows that enter with the next block
    constexpr int T = PSPW_LOCAL / L;
    constexpr int UR = PSPW_UR;
    constexpr int REM = L == 8 ? 2 * UR : UR;      // remote entries per row whose pairs sit in registers (entry e in lane e)
    constexpr int V4 = TN / 4;                     // 16-byte pieces per window row
    constexpr int FPT = RB * V4 / PSPW_THREADS;    // pieces per lane when 64 rows enter
    static_assert(RPG >= 1 && RB * V4 % PSPW_THREADS == 0, "shape");
    static_assert(UR <= L, "one lane per prefetched remote entry");
    // [RING + 1][TN]: the ring and one row of zeros, which the padding of a row's entry registers points at (value 0
    // times a zero, so the summing loop needs no predicate and a padding slot can never bring an Inf or NaN in)
    extern __shared__ __align__(16) float s_x[];
    constexpr int ZERO_OFF = RING * TN * 4;  // byte offset of the zero row

    const int run_id = psp_xcd_tile(stripe);
    if (run_id >= nruns) return;
    const int nblocks = (M + RB - 1) / RB;
    const int j0 = run_id * run, j1 = min(j0 + run, nblocks);
    const int tid = threadIdx.x;
    const int sub = tid & (L - 1);
    const int grp = tid >> LOGL;
    const int tile_col0 = blockIdx.y * TN;
    const int2 *rp2 = (const int2 *)rowPtr_w;
    if (tid < V4) *(psp_f32x4 *)(s_x + RING * TN + tid * 4) = (psp_f32x4){0.f, 0.f, 0.f, 0.f};
    float *s_w = s_x + (RING + 1) * TN;  // EPI: [TN][TN], s_w[k][j] = factor of input column k in output column j
    if constexpr (EPI) {
        for (int idx = tid; idx < TN * TN; idx += PSPW_THREADS) {
            const int k_ = idx / TN, j_ = idx - k_ * TN;
            s_w[idx] = transW ? W[j_ * TN + k_] : W[idx];
        }
    }

    bool live[C];
    int off[C];
#pragma unroll
    for (int i = 0; i < C; i++) {
        off[i] = (i * L + sub) * 4;  // column inside the tile
        live[i] = tile_col0 + off[i] < N;
    }

    // row bounds of this lane group's rows in block j (the same addresses for the lanes of a group); entry M of the
    // pair array holds (nnz, nnz), so rows past the matrix are empty
    auto load_bounds = [&](int j, int(&a)[RPG], int(&m)[RPG], int(&b)[RPG]) {
        const int r0 = j * RB + grp * RPG;
#pragma unroll
        for (int k = 0; k < RPG; k++) {
            const int2 am = rp2[min(r0 + k, M)];
            a[k] = am.x;
            m[k] = am.y;
        }
        const int end = rp2[min(r0 + RPG, M)].x;
#pragma unroll
        for (int k = 0; k < RPG; k++) b[k] = k + 1 < RPG ? a[k + 1] : end;
    };
    // Every load below is unconditional and reads a clamped, valid address; what a lane must not use is masked where
    // it is used.  A load under a condition would meet its "not loaded" value in a register copy right behind the
    // load, and the copy would wait for the load: the pipeline of this kernel lives on loads that stay in flight.
    //
    // lane s takes the rows' local entries a + tL + s (t < T) and remote entry m + s
    auto load_pairs = [&](const int(&a)[RPG], const int(&m)[RPG], int(&cl)[RPG][T], float(&vl)[RPG][T], int(&cr)[RPG],
                          float(&vr)[RPG]) {
#pragma unroll
        for (int k = 0; k < RPG; k++) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                const int p = min(a[k] + t * L + sub, nnz - 1);
                cl[k][t] = colIdx[p];
                vl[k][t] = val[p];
            }
            const int p = min(m[k] + sub, nnz - 1);  // remote entry e in lane e
            cr[k] = colIdx[p];
            vr[k] = val[p];
        }
    };
    // X rows first .. first + 64 of this tile: global -> registers, registers -> ring.  Rows outside the matrix and
    // columns past N are read from the nearest valid place; no local entry refers to them.
    auto fill_load = [&](int first, psp_f32x4(&w)[FPT]) {
#pragma unroll
        for (int i = 0; i < FPT; i++) {
            const int q = i * PSPW_THREADS + tid;
            const int wr = q / V4, c4 = q - wr * V4;
            const int gr = min(max(first + wr, 0), M - 1), gc = min(tile_col0 + c4 * 4, N - 4);
            w[i] = *(const psp_f32x4 *)(X + (size_t)gr * (size_t)N + gc);
        }
    };
    auto fill_store = [&](int first, psp_f32x4(&w)[FPT]) {
#pragma unroll
        for (int i = 0; i < FPT; i++) {
            const int q = i * PSPW_THREADS + tid;
            const int wr = q / V4, c4 = q - wr * V4;
            if (relu_x) {
#pragma unroll
                for (int e = 0; e < 4; e++) w[i][e] = w[i][e] < 0.0f ? 0.0f : w[i][e];
            }
            *(psp_f32x4 *)(s_x + (pspw_slot<RING>(first + wr) * TN + c4 * 4)) = w[i];
        }
    };
    // (a slot past the row's remote part reads row 0: the same address for every such lane of the wavefront, which the
    // memory pipeline serves as one request, where the clamped column would cost a request of its own)
    auto gather_remote = [&](const int(&cr)[RPG], const int(&m)[RPG], const int(&b)[RPG], psp_f32x4(&xr)[RPG][UR][C]) {
#pragma unroll
        for (int k = 0; k < RPG; k++) {
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const int c = m[k] + u < b[k] ? pspw_remote<L>(cr[k], u, sub) : 0;
#pragma unroll
                for (int i = 0; i < C; i++)
                    xr[k][u][i] = *(const psp_f32x4 *)(X + (size_t)c * (size_t)N + min(tile_col0 + off[i], N - 4));
            }
        }
    };

    // A lane turns the local entries it fetched into what the summing loop reads: the byte offset of the entry's X
    // row in the ring (the zero row for a slot past the row's local part) and the value (0 there).
    auto to_ring = [&](const int(&a)[RPG], const int(&m)[RPG], int(&cl)[RPG][T], float(&vl)[RPG][T]) {
#pragma unroll
        for (int k = 0; k < RPG; k++)
#pragma unroll
            for (int t = 0; t < T; t++) {
                const bool ok = a[k] + t * L + sub < m[k];
                cl[k][t] = ok ? pspw_slot<RING>(cl[k][t]) * (TN * 4) : ZERO_OFF;
                vl[k][t] = ok ? vl[k][t] : 0.0f;
            }
    };

    int a[RPG], m[RPG], b[RPG], an[RPG], mn[RPG], bn[RPG];
    int cl[RPG][T], cr[RPG], cln[RPG][T], crn[RPG];
    float vl[RPG][T], vr[RPG], vln[RPG][T], vrn[RPG];
    psp_f32x4 xr[RPG][UR][C], w[FPT];

    // ---- first block of the run: its whole window, its pairs, its remote tiles ------------------------------------
    load_bounds(j0, a, m, b);
    load_bounds(j0 + 1, an, mn, bn);
#pragma unroll 1
    for (int piece = 0; piece < PSPW_FIRST_PIECES; piece++) {
        fill_load(j0 * RB - PSPW_HALO + piece * RB, w);
        fill_store(j0 * RB - PSPW_HALO + piece * RB, w);
    }
    load_pairs(a, m, cl, vl, cr, vr);
    gather_remote(cr, m, b, xr);
    to_ring(a, m, cl, vl);
    __syncthreads();

#pragma unroll 1
    for (int j = j0; j < j1; j++) {
        // loads for the blocks that follow (past the end of the run they read clamped addresses and are not used)
        int a2[RPG], m2[RPG], b2[RPG];
        load_pairs(an, mn, cln, vln, crn, vrn);
        load_bounds(j + 2, a2, m2, b2);
        fill_load((j + 1) * RB + PSPW_HALO, w);  // the rows that enter with block j + 1

        // ---- local entries from the ring ------------------------------------------------------------------------
        psp_f32x4 acc[RPG][C];
#pragma unroll
        for (int k = 0; k < RPG; k++)
#pragma unroll
            for (int i = 0; i < C; i++) acc[k][i] = (psp_f32x4){0.f, 0.f, 0.f, 0.f};

        // one entry of every lane group: ring offset and value from the lane that holds them, C reads of 16 bytes from
        // the ring, 4 C multiply-adds; straight-line code, so the reads of the following entries overlap the adds
#define PSPW_STEP(K_, T_, J_)                                                                   \
    {                                                                                           \
        const int o_ = pspw_bcast<L, J_>(cl[K_][T_], sub) + sub * 16;                           \
        const float v_ = pspw_bcast_f<L, J_>(vl[K_][T_], sub);                                  \
        _Pragma("unroll") for (int i = 0; i < C; i++)                                           \
        {                                                                                       \
            const psp_f32x4 x_ = *(const psp_f32x4 *)((const char *)s_x + (o_ + i * (L * 16))); \
            _Pragma("unroll") for (int e = 0; e < 4; e++)                                       \
                acc[K_][i][e] = __builtin_fmaf(v_, x_[e], acc[K_][i][e]);                       \
        }                                                                                       \
    }
#pragma unroll
        for (int k = 0; k < RPG; k++) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                // a chunk no lane group of the wavefront reaches is skipped as a whole
                if (__builtin_amdgcn_ballot_w64(a[k] + t * L < m[k]) == 0ull) continue;
                PSPW_STEP(k, t, 0)
                PSPW_STEP(k, t, 1)
                PSPW_STEP(k, t, 2)
                PSPW_STEP(k, t, 3)
                if constexpr (L == 8) {
                    PSPW_STEP(k, t, 4)
                    PSPW_STEP(k, t, 5)
                    PSPW_STEP(k, t, 6)
                    PSPW_STEP(k, t, 7)
                }
            }
            // local entries beyond the ones fetched up front
            for (int p = a[k] + T * L; p < m[k]; p++) {
                const int c_ = pspw_slot<RING>(colIdx[p]);
                const float v_ = val[p];
#pragma unroll
                for (int i = 0; i < C; i++) {
                    const psp_f32x4 x_ = *(const psp_f32x4 *)(s_x + (c_ * TN + off[i]));
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[k][i][e] = __builtin_fmaf(v_, x_[e], acc[k][i][e]);
                }
            }
        }
#undef PSPW_STEP

        // ---- remote entries, then the rows go out -------------------------------------------------------------------
#pragma unroll
        for (int k = 0; k < RPG; k++) {
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const float v = pspw_remote_f<L>(vr[k], u, sub);
                if (m[k] + u < b[k]) {
#pragma unroll
                    for (int i = 0; i < C; i++) {
                        psp_f32x4 x_ = xr[k][u][i];
                        if (relu_x) {
#pragma unroll
                            for (int e = 0; e < 4; e++) x_[e] = x_[e] < 0.0f ? 0.0f : x_[e];
                        }
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[k][i][e] = __builtin_fmaf(v, x_[e], acc[k][i][e]);
                    }
                }
            }
            // Second round (lane groups of 8): remote entries 4 .. 7, whose columns and values lanes 4 .. 7 already hold.
            // Their X rows are gathered together, into the registers the first round has just left, only when some row of
            // the wavefront has that many -- one wait instead of two dependent ones per entry in the loop below.
            if constexpr (REM > UR) {
                if (__builtin_amdgcn_ballot_w64(m[k] + UR < b[k]) != 0ull) {
                    psp_f32x4 x2[UR][C];
#pragma unroll
                    for (int u = 0; u < UR; u++) {
                        const int c = pspw_remote<L>(cr[k], UR + u, sub);
#pragma unroll
                        for (int i = 0; i < C; i++)
                            x2[u][i] = *(const psp_f32x4 *)(X + (size_t)c * (size_t)N + min(tile_col0 + off[i], N - 4));
                    }
#pragma unroll
                    for (int u = 0; u < UR; u++) {
                        const float v = pspw_remote_f<L>(vr[k], UR + u, sub);
                        if (m[k] + UR + u < b[k]) {
#pragma unroll
                            for (int i = 0; i < C; i++) {
                                psp_f32x4 x_ = x2[u][i];
                                if (relu_x) {
#pragma unroll
                                    for (int e = 0; e < 4; e++) x_[e] = x_[e] < 0.0f ? 0.0f : x_[e];
                                }
#pragma unroll
                                for (int e = 0; e < 4; e++) acc[k][i][e] = __builtin_fmaf(v, x_[e], acc[k][i][e]);
                            }
                        }
                    }
                }
            }
            for (int p = m[k] + REM; p < b[k]; p++) {
                const int c_ = colIdx[p];
                const float v_ = val[p];
#pragma unroll
                for (int i = 0; i < C; i++) {
                    if (!live[i]) continue;
                    psp_f32x4 x_ = *(const psp_f32x4 *)(X + (size_t)c_ * (size_t)N + tile_col0 + off[i]);
                    if (relu_x) {
#pragma unroll
                        for (int e = 0; e < 4; e++) x_[e] = x_[e] < 0.0f ? 0.0f : x_[e];
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[k][i][e] = __builtin_fmaf(v_, x_[e], acc[k][i][e]);
                }
            }
            const int r = j * RB + grp * RPG + k;
            if constexpr (EPI) {
                // the row of A f(X) is complete: store it if asked, then multiply it by the staged matrix (every lane
                // of the wavefront takes part in the DPP moves; N == TN here, so every lane has columns)
                const psp_f32x4 raw = acc[k][0];
                if (Y_raw != nullptr && r < M)
                    __builtin_nontemporal_store(raw, (psp_f32x4 *)(Y_raw + (size_t)r * (size_t)N + off[0]));
                psp_f32x4 o = (psp_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j2 = 0; j2 < L; j2++) {
#pragma unroll
                    for (int e2 = 0; e2 < 4; e2++) {
                        const float a_ = pspw_bcast_any_f<L>(raw[e2], j2, sub);
                        const psp_f32x4 wv = *(const psp_f32x4 *)(s_w + ((j2 * 4 + e2) * TN + off[0]));
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = __builtin_fmaf(a_, wv[e], o[e]);
                    }
                }
                acc[k][0] = o;
            }
            if (r < M) {
#pragma unroll
                for (int i = 0; i < C; i++) {
                    if (!live[i]) continue;
                    const size_t at = (size_t)r * (size_t)N + tile_col0 + off[i];
                    psp_f32x4 y = acc[k][i];
                    if (mask) {
                        const psp_f32x4 mk = *(const psp_f32x4 *)(mask + at);
#pragma unroll
                        for (int e = 0; e < 4; e++) y[e] = mk[e] > 0.0f ? y[e] : 0.0f;
                    }
                    __builtin_nontemporal_store(y, (psp_f32x4 *)(Y + at));
                }
            }
        }

        // ---- hand over to block j + 1 ---------------------------------------------------------------------------------
        gather_remote(crn, mn, bn, xr);                     // in flight while block j + 1 is summed from the ring
        fill_store((j + 1) * RB + PSPW_HALO, w);    // slots no row of block j's or j + 1's window occupies
#pragma unroll
        for (int k = 0; k < RPG; k++) {
            a[k] = an[k], m[k] = mn[k], b[k] = bn[k];
            an[k] = a2[k], mn[k] = m2[k], bn[k] = b2[k];
            cr[k] = crn[k], vr[k] = vrn[k];
#pragma unroll
            for (int t = 0; t < T; t++) cl[k][t] = cln[k][t], vl[k][t] = vln[k][t];
        }
        to_ring(a, m, cl, vl);
        __syncthreads();
    }
}

// ---- format construction ----------------------------------------------------------------------------------------
// (a column past the last row is never local: the kernels stage rows 0 .. M - 1 of the dense operand, and a matrix with
// more columns than rows reaches the rest through the gathers)
__device__ __host__ static inline bool pspw_is_local(int row, int col, int M)
{
    const int lo = row / PSPW_BLOCK * PSPW_BLOCK - PSPW_HALO;
    return col >= lo && col < lo + PSPW_BLOCK + 2 * PSPW_HALO && col < M;
}

// one lane per row: local entries first, remote ones after, each part in the original order
__global__ void __launch_bounds__(256)
psp_window_build_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const float *__restrict__ val,
                        int M, int *__restrict__ rowPtr_w, int *__restrict__ colIdx_w, float *__restrict__ val_w)
{
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r > M) return;
    if (r == M) {
        rowPtr_w[2 * M] = rowPtr_w[2 * M + 1] = rowPtr[M];
        return;
    }
    const int lb = rowPtr[r], hb = rowPtr[r + 1];
    int w = lb;
    for (int p = lb; p < hb; p++) {
        const int c = colIdx[p];
        if (pspw_is_local(r, c, M)) {
            colIdx_w[w] = c;
            val_w[w] = val[p];
            w++;
        }
    }
    rowPtr_w[2 * r] = lb;
    rowPtr_w[2 * r + 1] = w;
    for (int p = lb; p < hb; p++) {
        const int c = colIdx[p];
        if (!pspw_is_local(r, c, M)) {
            colIdx_w[w] = c;
            val_w[w] = val[p];
            w++;
        }
    }
}

PSP_EXPORT int psp_window_build(const int *rowPtr, const int *colIdx, const float *val, int M, int *rowPtr_w,
                                int *colIdx_w, float *val_w)
{
    PSP_REQUIRE(M >= 0 && rowPtr && rowPtr_w, "window_build: null pointer or negative size");
    const int nnz = rowPtr[M];
    PSP_REQUIRE(nnz >= 0 && (nnz == 0 || (colIdx && val && colIdx_w && val_w)), "window_build: null entry arrays");
    for (int r = 0; r < M; r++) {
        const int lb = rowPtr[r], hb = rowPtr[r + 1];
        PSP_REQUIRE(lb >= 0 && hb >= lb && hb <= nnz, "window_build: rowPtr is not a monotone prefix at row %d", r);
        int w = lb;
        for (int p = lb; p < hb; p++)
            if (pspw_is_local(r, colIdx[p], M)) {
                colIdx_w[w] = colIdx[p];
                val_w[w++] = val[p];
            }
        rowPtr_w[2 * r] = lb;
        rowPtr_w[2 * r + 1] = w;
        for (int p = lb; p < hb; p++)
            if (!pspw_is_local(r, colIdx[p], M)) {
                colIdx_w[w] = colIdx[p];
                val_w[w++] = val[p];
            }
    }
    rowPtr_w[2 * M] = rowPtr_w[2 * M + 1] = nnz;
    return PSP_OK;
}

PSP_EXPORT int psp_window_build_dev(const int *rowPtr, const int *colIdx, const float *val, int M, int *rowPtr_w,
                                    int *colIdx_w, float *val_w, psp_stream_t stream)
{
    PSP_REQUIRE(M >= 0 && rowPtr && rowPtr_w, "window_build_dev: null pointer or negative size");
    hipLaunchKernelGGL(psp_window_build_kernel, dim3(psp_ceil_div((long long)M + 1, 256)), dim3(256), 0,
                       (hipStream_t)stream, rowPtr, colIdx, val, M, rowPtr_w, colIdx_w, val_w);
    return psp_check_launch("window build kernel");
}

// ---- launch -----------------------------------------------------------------------------------------------------------
typedef void (*pspw_kernel_t)(const int *, const int *, const float *, const float *, float *, const float *, int, int,
                              int, int, int, int, int, const float *, int, float *);

struct pspw_variant {
    pspw_kernel_t fn;
    int tn, threads;
};

// one row of a block per lane group: 64 groups of 4 lanes, or 64 groups of 8 lanes in a workgroup of 512
static pspw_variant pspw_lookup(int variant, bool epilogue = false)
{
    if (epilogue) {
        switch (variant) {
        case 1: return {psp_spmm_window_kernel<1, 2, 256, true>, 16, 256};
        case 2: return {psp_spmm_window_kernel<1, 3, 512, true>, 32, 512};
        default: return {nullptr, 0, 0};
        }
    }
    switch (variant) {
    case 1: return {psp_spmm_window_kernel<1, 2, 256>, 16, 256};  // 4 lanes x 1 vector
    case 2: return {psp_spmm_window_kernel<1, 3, 512>, 32, 512};  // 8 lanes x 1 vector
    case 3: return {psp_spmm_window_kernel<2, 3, 512>, 64, 512};  // 8 lanes x 2 vectors
    default: return {nullptr, 0, 0};
    }
}

PSP_EXPORT int psp_spmm_window_plan(int N, int variant, int *tile_cols, int *rows_per_block, int *lds_bytes)
{
    PSP_REQUIRE(N >= 4 && N % 4 == 0, "spmm_window: N must be a positive multiple of 4 (got %d)", N);
    PSP_REQUIRE(variant >= 0 && variant <= 3, "spmm_window: variant %d (0 automatic, 1: 16, 2: 32, 3: 64 columns per tile)", variant);
    if (variant == 0) variant = N <= 16 ? 1 : (N <= 32 ? 2 : 3);
    const pspw_variant v = pspw_lookup(variant);
    if (tile_cols) *tile_cols = v.tn;
    if (rows_per_block) *rows_per_block = PSPW_BLOCK;
    if (lds_bytes) *lds_bytes = (2 * PSPW_BLOCK + 2 * PSPW_HALO + 1) * v.tn * 4;  // the ring and a row of zeros
    return variant;
}

static int pspw_launch(const int *rowPtr_w, const int *colIdx_w, const float *val_w, const float *X, float *Y, int M, int nnz,
                       int N, int rows_out, int variant, int relu_x, const float *mask, const float *W, int transW,
                       float *Y_raw, hipStream_t st)
{
    const bool epi = W != nullptr;
    int tn = 0, rb = 0, lds = 0;
    const int v = psp_spmm_window_plan(N, variant, &tn, &rb, &lds);
    if (v < 0) return v;
    PSP_REQUIRE(M >= 0 && nnz >= 0 && rows_out >= M, "spmm_window: Y has %d rows, the matrix %d (%d entries)", rows_out, M, nnz);
    PSP_REQUIRE((((size_t)X | (size_t)Y | (size_t)mask | (size_t)Y_raw) & 15) == 0, "spmm_window: X, Y and mask must be 16-byte aligned");
    if (epi) {
        PSP_REQUIRE(N == tn && (N == 16 || N == 32), "spmm_window: the dense epilogue exists for N = 16 and 32 (got %d)", N);
        lds += tn * tn * 4;
    }
    if (nnz == 0) {  // (the kernel clamps its loads to entry nnz - 1)
        const int rc = psp_zero_f32(Y, (size_t)rows_out * N, st);
        return rc != PSP_OK || !Y_raw ? rc : psp_zero_f32(Y_raw, (size_t)rows_out * N, st);
    }
    int rc = psp_zero_f32(Y + (size_t)M * N, ((size_t)rows_out - (size_t)M) * N, st);  // rows past the matrix
    if (rc == PSP_OK && Y_raw) rc = psp_zero_f32(Y_raw + (size_t)M * N, ((size_t)rows_out - (size_t)M) * N, st);
    if (rc != PSP_OK || M == 0) return rc;
    PSP_REQUIRE(rowPtr_w && colIdx_w && val_w && X && Y, "spmm_window: null pointer");
    const pspw_variant k = pspw_lookup(v, epi);
    const int key = v + (epi ? 4 : 0);
    static bool lds_raised[8];
    if (lds > 48 * 1024 && !lds_raised[key]) {
        const hipError_t e = hipFuncSetAttribute((const void *)k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return psp_fail(PSP_ERR_LAUNCH, "spmm_window: %d bytes of LDS refused: %s", lds, hipGetErrorString(e));
        lds_raised[key] = true;
    }
    const int nblocks = psp_ceil_div(M, rb), tiles = psp_ceil_div(N, tn);
    const int run = pspw_run_length(nblocks, tiles, key, (const void *)k.fn, k.threads, lds);
    const int nruns = psp_ceil_div(nblocks, run);
    const psp_grid1d g = psp_xcd_grid(nruns, 1);  // long runs: neighbouring runs share two halo windows, nothing to keep in one L2
    dim3 grid(g.launch, tiles, 1), block(k.threads, 1, 1);
    hipLaunchKernelGGL(k.fn, grid, block, lds, st, rowPtr_w, colIdx_w, val_w, X, Y, mask, M, N, nnz, nruns, g.stripe, run,
                       relu_x != 0, W, transW != 0, Y_raw);
    return psp_check_launch("spmm window kernel");
}

PSP_EXPORT int psp_spmm_window_f32(const int *rowPtr_w, const int *colIdx_w, const float *val_w, const float *X, float *Y,
                                   int M, int nnz, int N, int rows_out, int variant, int relu_x, const float *mask,
                                   psp_stream_t stream)
{
    return pspw_launch(rowPtr_w, colIdx_w, val_w, X, Y, M, nnz, N, rows_out, variant, relu_x, mask, nullptr, 0, nullptr,
                       (hipStream_t)stream);
}

PSP_EXPORT int psp_spmm_window_xw_f32(const int *rowPtr_w, const int *colIdx_w, const float *val_w, const float *X,
                                      const float *W, int transW, float *Y, float *Y_raw, int M, int nnz, int N, int rows_out,
                                      int relu_x, const float *mask, psp_stream_t stream)
{
    PSP_REQUIRE(W != nullptr, "spmm_window_xw: W is null");
    return pspw_launch(rowPtr_w, colIdx_w, val_w, X, Y, M, nnz, N, rows_out, 0, relu_x, mask, W, transW, Y_raw,
                       (hipStream_t)stream);
}
