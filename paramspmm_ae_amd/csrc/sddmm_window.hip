// Windowed CSR SDDMM for gfx950: out[p] = alpha <A[row(p), :], B[col(p), :]> over the stored entries of a matrix in
// the windowed layout (psp_window_build; see spmm_window.hip for the layout and for the walk this kernel shares with
// the SpMM kernel).  No counterpart in the reference: its SDDMM kernels (SDDMM/sddmm_kernel.cu:917-1057) gather
// B[col] per entry from global memory; here the B rows of a 64-row block's window sit in an LDS ring, so the local
// entries -- nine out of ten on a community-ordered graph -- are dot products of two LDS / register operands, and
// only the remote ones gather.
//
// A workgroup walks a run of consecutive 64-row blocks; a lane group of L = 4 or 8 lanes owns one row of the block and
// holds that row of A in registers, 4 C floats per lane (the whole of K is covered by one lane group: 4 C L >= K).
// Per chunk of L local entries the group forms L partial dot products (one ds_read_b128 of
// the B row and 4 C multiply-adds per lane and entry) and sums them across the lanes with L - 1 DPP additions, after
// which lane s holds entry s of the chunk and the group stores L consecutive floats.  The B rows of a row's first four
// remote entries were gathered into registers while the previous block was processed; lane groups of 8 gather those
// of entries 4 .. 7 together in a second round when some row of the wavefront has them; longer rows finish in plain
// loops.  SAME: A and B are the same matrix (the attention scores of a graph layer, <X_i, X_j>), so the row of A is
// read from the ring as well and X is read from HBM once.
// Per entry the products are summed in the order k = s, s + L, ... inside a lane, then across the lanes: within the
// stated fp32 tolerance of the reference's 32-lane strided sum and butterfly, not bit-identical to it.
#include "window_common.h"

template <int C, int LOGL, int THREADS, bool SAME>
__global__ void __launch_bounds__(THREADS)
psp_sddmm_window_kernel(const int *__restrict__ rowPtr_w, const int *__restrict__ colIdx, const float *__restrict__ A,
                        const float *__restrict__ B, const float *__restrict__ alpha_ptr, float *__restrict__ out, int M,
                        int K, int rows_b, int nnz, int nruns, int stripe, int run)
{
    constexpr int L = 1 << LOGL;
    constexpr int TN = L * C * 4;                  // columns a lane group covers
    constexpr int RB = PSPW_BLOCK;                 // rows per step
    constexpr int RING = RB + 2 * PSPW_HALO + RB;  // window + the rows that enter with the next block
    constexpr int T = PSPW_LOCAL / L;
    constexpr int UR = PSPW_UR;
    constexpr int REM = L == 8 ? 2 * UR : UR;      // remote entries per row whose pairs sit in registers (entry e in lane e)
    constexpr int V4 = TN / 4;                     // 16-byte pieces per window row
    constexpr int FPT = RB * V4 / THREADS;         // pieces per lane when 64 rows enter
    static_assert(RB * L == THREADS, "one row of the block per lane group");
    static_assert(RB * V4 % THREADS == 0 && UR <= L && UR == 4, "shape");
    // [RING + 1][TN]: the ring and a row of zeros for the padding of a row's entry registers
    extern __shared__ __align__(16) float s_x[];
    constexpr int ZERO_OFF = RING * TN * 4;

    const int run_id = psp_xcd_tile(stripe);
    if (run_id >= nruns) return;
    const int nblocks = (M + RB - 1) / RB;
    const int j0 = run_id * run, j1 = min(j0 + run, nblocks);
    const int tid = threadIdx.x;
    const int sub = tid & (L - 1);
    const int grp = tid >> LOGL;
    const int2 *rp2 = (const int2 *)rowPtr_w;
    if (tid < V4) *(psp_f32x4 *)(s_x + RING * TN + tid * 4) = (psp_f32x4){0.f, 0.f, 0.f, 0.f};
    const float alpha = alpha_ptr ? alpha_ptr[0] : 1.0f;

    bool live[C];
    int off[C];
#pragma unroll
    for (int i = 0; i < C; i++) {
        off[i] = (i * L + sub) * 4;
        live[i] = off[i] < K;
    }

    // Every load below is unconditional and reads a clamped, valid address (a load under a condition would be waited
    // for right behind its issue); what a lane must not use is masked where it is used.
    auto load_bounds = [&](int j, int &a, int &m, int &b) {
        const int r = j * RB + grp;
        const int2 am = rp2[min(r, M)];
        a = am.x;
        m = am.y;
        b = rp2[min(r + 1, M)].x;
    };
    // lane s takes the row's local entries a + tL + s (t < T) and remote entry m + s
    auto load_cols = [&](int a, int m, int(&cl)[T], int &cr) {
#pragma unroll
        for (int t = 0; t < T; t++) cl[t] = colIdx[min(a + t * L + sub, nnz - 1)];
        cr = colIdx[min(m + sub, nnz - 1)];  // remote entry e in lane e
    };
    auto fill_load = [&](int first, psp_f32x4(&w)[FPT]) {
#pragma unroll
        for (int i = 0; i < FPT; i++) {
            const int q = i * THREADS + tid;
            const int wr = q / V4, c4 = q - wr * V4;
            const int gr = min(max(first + wr, 0), rows_b - 1), gc = min(c4 * 4, K - 4);
            w[i] = *(const psp_f32x4 *)(B + (size_t)gr * (size_t)K + gc);
        }
    };
    auto fill_store = [&](int first, const psp_f32x4(&w)[FPT]) {
#pragma unroll
        for (int i = 0; i < FPT; i++) {
            const int q = i * THREADS + tid;
            const int wr = q / V4, c4 = q - wr * V4;
            *(psp_f32x4 *)(s_x + (pspw_slot<RING>(first + wr) * TN + c4 * 4)) = w[i];
        }
    };
    // (a slot past the row's remote part reads row 0: the same address for every such lane of the wavefront, which the
    // memory pipeline serves as one request, where the clamped column would cost a request of its own)
    auto gather_remote = [&](int cr, int m, int b, int first, psp_f32x4(&xr)[UR][C]) {
#pragma unroll
        for (int u = 0; u < UR; u++) {
            const int c = m + first + u < b ? pspw_remote<L>(cr, first + u, sub) : 0;
#pragma unroll
            for (int i = 0; i < C; i++) xr[u][i] = *(const psp_f32x4 *)(B + (size_t)c * (size_t)K + min(off[i], K - 4));
        }
    };
    auto load_row = [&](int j, psp_f32x4(&ar)[C]) {  // the group's row of A (not SAME)
        const int r = min(j * RB + grp, M - 1);
#pragma unroll
        for (int i = 0; i < C; i++) ar[i] = *(const psp_f32x4 *)(A + (size_t)r * (size_t)K + min(off[i], K - 4));
    };
    // local columns -> byte offsets of the B rows in the ring (the zero row for a slot past the row's local part)
    auto to_ring = [&](int a, int m, int(&cl)[T]) {
#pragma unroll
        for (int t = 0; t < T; t++) cl[t] = a + t * L + sub < m ? pspw_slot<RING>(cl[t]) * (TN * 4) : ZERO_OFF;
    };
    auto dot = [&](const psp_f32x4(&x)[C], const psp_f32x4(&ar)[C]) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < C; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) s = __builtin_fmaf(x[i][e], ar[i][e], s);
        return s;
    };

    int a, m, b, an, mn, bn;
    int cl[T], cr, cln[T], crn;
    psp_f32x4 xr[UR][C], w[FPT], ar[C], arn[C];

    // ---- first block of the run: its whole window, its columns, its remote rows ------------------------------------------
    load_bounds(j0, a, m, b);
    load_bounds(j0 + 1, an, mn, bn);
#pragma unroll 1
    for (int piece = 0; piece < PSPW_FIRST_PIECES; piece++) {
        fill_load(j0 * RB - PSPW_HALO + piece * RB, w);
        fill_store(j0 * RB - PSPW_HALO + piece * RB, w);
    }
    load_cols(a, m, cl, cr);
    gather_remote(cr, m, b, 0, xr);
    if constexpr (!SAME) load_row(j0, arn);
    to_ring(a, m, cl);
    __syncthreads();

#pragma unroll 1
    for (int j = j0; j < j1; j++) {
        int a2, m2, b2;
        load_cols(an, mn, cln, crn);
        load_bounds(j + 2, a2, m2, b2);
        fill_load((j + 1) * RB + PSPW_HALO, w);  // the rows that enter with block j + 1
        if constexpr (SAME) {
            // (a row past the matrix has no entries; its slot holds the nearest valid row)
            const int slot = pspw_slot<RING>(j * RB + grp) * TN;
#pragma unroll
            for (int i = 0; i < C; i++) ar[i] = *(const psp_f32x4 *)(s_x + slot + off[i]);
        } else {
#pragma unroll
            for (int i = 0; i < C; i++) ar[i] = arn[i];
            load_row(j + 1, arn);
        }
        // columns past K hold copies of the last four (the clamped loads): they must not count
#pragma unroll
        for (int i = 0; i < C; i++)
            if (!live[i]) ar[i] = (psp_f32x4){0.f, 0.f, 0.f, 0.f};

        // ---- local entries: both operands on chip -------------------------------------------------------------------------
#define PSPW_DOT(T_, J_)                                                                           \
    {                                                                                              \
        const int o_ = pspw_bcast<L, J_>(cl[T_], sub) + sub * 16;                                  \
        psp_f32x4 x_[C];                                                                           \
        _Pragma("unroll") for (int i = 0; i < C; i++)                                              \
            x_[i] = *(const psp_f32x4 *)((const char *)s_x + (o_ + i * (L * 16)));                 \
        part[J_] = dot(x_, ar);                                                                    \
    }
#pragma unroll
        for (int t = 0; t < T; t++) {
            // a chunk no lane group of the wavefront reaches is skipped as a whole
            if (__builtin_amdgcn_ballot_w64(a + t * L < m) == 0ull) continue;
            float part[L];
            PSPW_DOT(t, 0)
            PSPW_DOT(t, 1)
            PSPW_DOT(t, 2)
            PSPW_DOT(t, 3)
            if constexpr (L == 8) {
                PSPW_DOT(t, 4)
                PSPW_DOT(t, 5)
                PSPW_DOT(t, 6)
                PSPW_DOT(t, 7)
            }
            const float r = pspw_reduce_transposed<L>(part, sub);
            const int p = a + t * L + sub;
            if (p < m) out[p] = alpha * r;
        }
#undef PSPW_DOT
        // local entries beyond the ones fetched up front
        for (int p = a + T * L; p < m; p++) {
            const int c_ = pspw_slot<RING>(colIdx[p]);
            psp_f32x4 x_[C];
#pragma unroll
            for (int i = 0; i < C; i++) x_[i] = *(const psp_f32x4 *)(s_x + (c_ * TN + off[i]));
            const float r = pspw_reduce_all<L>(dot(x_, ar));
            if (sub == 0) out[p] = alpha * r;
        }

        // ---- remote entries ----------------------------------------------------------------------------------------------
        {
            float part[UR];
#pragma unroll
            for (int u = 0; u < UR; u++) part[u] = dot(xr[u], ar);
            const float r = pspw_reduce_transposed4<L>(part, sub);
            const int p = m + sub;
            if (sub < UR && p < b) out[p] = alpha * r;
        }
        // second round (lane groups of 8): remote entries 4 .. 7 (columns already in lanes 4 .. 7), gathered together
        // when some row of the wavefront has that many
        if (REM > UR && __builtin_amdgcn_ballot_w64(m + UR < b) != 0ull) {
            psp_f32x4 x2[UR][C];
            gather_remote(cr, m, b, UR, x2);
            float part[UR];
#pragma unroll
            for (int u = 0; u < UR; u++) part[u] = dot(x2[u], ar);
            const float r = pspw_reduce_transposed4<L>(part, sub);
            const int p = m + UR + sub;
            if (sub < UR && p < b) out[p] = alpha * r;
        }
        for (int p = m + REM; p < b; p++) {
            const int c_ = colIdx[p];
            psp_f32x4 x_[C];
#pragma unroll
            for (int i = 0; i < C; i++) x_[i] = *(const psp_f32x4 *)(B + (size_t)c_ * (size_t)K + min(off[i], K - 4));
            const float r = pspw_reduce_all<L>(dot(x_, ar));
            if (sub == 0) out[p] = alpha * r;
        }

        // ---- hand over to block j + 1 ---------------------------------------------------------------------------------
        gather_remote(crn, mn, bn, 0, xr);                     // in flight while block j + 1 is processed
        fill_store((j + 1) * RB + PSPW_HALO, w);    // slots no row of block j's or j + 1's window occupies
        a = an, m = mn, b = bn;
        an = a2, mn = m2, bn = b2;
        cr = crn;
#pragma unroll
        for (int t = 0; t < T; t++) cl[t] = cln[t];
        to_ring(a, m, cl);
        __syncthreads();
    }
}

// ---- launch -----------------------------------------------------------------------------------------------------------
typedef void (*pspdw_kernel_t)(const int *, const int *, const float *, const float *, const float *, float *, int, int, int,
                               int, int, int, int);
struct pspdw_variant {
    pspdw_kernel_t fn;
    int tn, threads;
};
static pspdw_variant pspdw_lookup(int K, bool same)
{
    if (K <= 16) return {same ? psp_sddmm_window_kernel<1, 2, 256, true> : psp_sddmm_window_kernel<1, 2, 256, false>, 16, 256};
    if (K <= 32) return {same ? psp_sddmm_window_kernel<1, 3, 512, true> : psp_sddmm_window_kernel<1, 3, 512, false>, 32, 512};
    if (K <= 64) return {same ? psp_sddmm_window_kernel<2, 3, 512, true> : psp_sddmm_window_kernel<2, 3, 512, false>, 64, 512};
    return {same ? psp_sddmm_window_kernel<4, 3, 512, true> : psp_sddmm_window_kernel<4, 3, 512, false>, 128, 512};
}

PSP_EXPORT int psp_sddmm_window_f32(const int *rowPtr_w, const int *colIdx_w, const float *A, const float *B,
                                    const float *alpha, float *out, int M, int nnz, int K, int rows_b, psp_stream_t stream)
{
    PSP_REQUIRE(K >= 4 && K % 4 == 0 && K <= PSP_SDDMM_WINDOW_MAX_K,
                "sddmm_window: K must be a multiple of 4 between 4 and %d (got %d)", PSP_SDDMM_WINDOW_MAX_K, K);
    PSP_REQUIRE(M >= 0 && nnz >= 0 && rows_b >= 0, "sddmm_window: negative size");
    if (M == 0 || nnz == 0) return PSP_OK;
    PSP_REQUIRE(rowPtr_w && colIdx_w && A && B && out && rows_b > 0, "sddmm_window: null pointer or no rows of B");
    PSP_REQUIRE((((size_t)A | (size_t)B) & 15) == 0, "sddmm_window: A and B must be 16-byte aligned");
    const bool same = A == B;
    PSP_REQUIRE(!same || rows_b >= M, "sddmm_window: A == B with fewer rows (%d) than the matrix (%d)", rows_b, M);
    const pspdw_variant k = pspdw_lookup(K, same);
    const int lds = (2 * PSPW_BLOCK + 2 * PSPW_HALO + 1) * k.tn * 4;
    const int key = (k.tn == 16 ? 0 : k.tn == 32 ? 1 : k.tn == 64 ? 2 : 3) + (same ? 4 : 0);
    static bool lds_raised[8];
    if (lds > 48 * 1024 && !lds_raised[key]) {
        const hipError_t e = hipFuncSetAttribute((const void *)k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return psp_fail(PSP_ERR_LAUNCH, "sddmm_window: %d bytes of LDS refused: %s", lds, hipGetErrorString(e));
        lds_raised[key] = true;
    }
    const int nblocks = psp_ceil_div(M, PSPW_BLOCK);
    const int run = pspw_run_length(nblocks, 1, key, (const void *)k.fn, k.threads, lds);
    const int nruns = psp_ceil_div(nblocks, run);
    const psp_grid1d g = psp_xcd_grid(nruns, 1);
    hipLaunchKernelGGL(k.fn, dim3(g.launch), dim3(k.threads), lds, (hipStream_t)stream, rowPtr_w, colIdx_w, A, B, alpha, out, M,
                       K, rows_b, nnz, nruns, g.stripe, run);
    return psp_check_launch("sddmm window kernel");
}
