// One attention layer's sparse work on the windowed CSR layout, for gfx950 (no counterpart in the reference, whose layer,
// gnn_conv.py:128-180, runs an SDDMM and an SpMM per direction -- and a 1 x nnz x 1 matrix product for the gradient of
// the head's weight -- as separate operators).  With the feature rows of a block's window in an LDS ring (see
// spmm_window.hip for the layout and the walk) every stored entry's B row is on chip once and serves both:
//
//   forward   att[p] = alpha <X[row(p)], X[col(p)]>,  Y[i] = sum_p att[p] X[col(p)]            (SDDMM, then SpMM)
//   backward  G[i] = sum_p att[p] dY[col(p)],  *wsum += sum_p <dY[row(p)], dY[col(p)]> float(col(p))
//             (the SpMM of the incoming gradient with the saved scores; the SDDMM of the gradient with itself
//             contracted with the column indices as floats -- the reference's literal formula for the gradient of the
//             attention weight, gnn_conv.py:166-172 -- without the scores of that SDDMM ever being stored)
//
// A lane group of L = 4 or 8 lanes owns one row and covers the whole width (K <= 4 C L).  Per local entry: one
// ds_read_b128 per lane and vector, 4 C multiply-adds for the partial dot product, log2(L) DPP additions to complete
// it in every lane, 4 C multiply-adds into the row's sum.  Remote entries go the same way from global memory: the
// first four of a row from registers filled a block ahead, entries 4 .. 7 of lane groups of 8 in a second round when
// some row of the wavefront has them, the rest in a plain loop.
// Summation order: a score is summed inside a lane over k = s, s + L, ..., then across the lanes; a row of Y over its
// local entries in storage order, then the remote ones.  Within the stated fp32 tolerance of the two reference
// operators, not bit-identical to them.  *wsum is accumulated with one atomic addition per workgroup.
#include "window_common.h"

template <int C, int LOGL, int THREADS, bool BWD>
__global__ void __launch_bounds__(THREADS)
psp_attn_window_kernel(const int *__restrict__ rowPtr_w, const int *__restrict__ colIdx, const float *__restrict__ att_in,
                       const float *__restrict__ X, const float *__restrict__ alpha_ptr, float *__restrict__ att_out,
                       float *__restrict__ Y, float *__restrict__ wsum_out, int M, int K, int nnz, int nruns, int stripe,
                       int run)
{
    constexpr int L = 1 << LOGL;
    constexpr int TN = L * C * 4;
    constexpr int RB = PSPW_BLOCK;
    constexpr int RING = RB + 2 * PSPW_HALO + RB;
    constexpr int T = PSPW_LOCAL / L;
    constexpr int UR = PSPW_UR;
    constexpr int REM = L == 8 ? 2 * UR : UR;      // remote entries per row whose pairs sit in registers (entry e in lane e)
    constexpr int V4 = TN / 4;
    constexpr int FPT = RB * V4 / THREADS;
    static_assert(RB * L == THREADS, "one row of the block per lane group");
    static_assert(RB * V4 % THREADS == 0 && UR <= L && UR == 4, "shape");
    extern __shared__ __align__(16) float s_x[];  // [RING + 1][TN]: the ring and a row of zeros
    constexpr int ZERO_OFF = RING * TN * 4;
    __shared__ float s_part[THREADS / 64];

    const int run_id = psp_xcd_tile(stripe);
    if (run_id >= nruns) return;
    const int nblocks = (M + RB - 1) / RB;
    const int j0 = run_id * run, j1 = min(j0 + run, nblocks);
    const int tid = threadIdx.x;
    const int sub = tid & (L - 1);
    const int grp = tid >> LOGL;
    const int2 *rp2 = (const int2 *)rowPtr_w;
    if (tid < V4) *(psp_f32x4 *)(s_x + RING * TN + tid * 4) = (psp_f32x4){0.f, 0.f, 0.f, 0.f};
    float alpha = 1.0f;
    if constexpr (!BWD) alpha = alpha_ptr ? alpha_ptr[0] : 1.0f;
    float wsum = 0.0f;

    bool live[C];
    int off[C];
#pragma unroll
    for (int i = 0; i < C; i++) {
        off[i] = (i * L + sub) * 4;
        live[i] = off[i] < K;
    }

    // Every load below is unconditional and reads a clamped, valid address; what a lane must not use is masked where it
    // is used (a load under a condition would be waited for right behind its issue).
    auto load_bounds = [&](int j, int &a, int &m, int &b) {
        const int r = j * RB + grp;
        const int2 am = rp2[min(r, M)];
        a = am.x;
        m = am.y;
        b = rp2[min(r + 1, M)].x;
    };
    // lane s takes the row's local entries a + tL + s (t < T) and remote entry m + s
    auto load_entries = [&](int a, int m, int(&cl)[T], float(&vl)[T], int &cr, float &vr) {
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int p = min(a + t * L + sub, nnz - 1);
            cl[t] = colIdx[p];
            if constexpr (BWD) vl[t] = att_in[p];
        }
        const int p = min(m + sub, nnz - 1);  // remote entry e in lane e
        cr = colIdx[p];
        if constexpr (BWD) vr = att_in[p];
    };
    auto fill_load = [&](int first, psp_f32x4(&w)[FPT]) {
#pragma unroll
        for (int i = 0; i < FPT; i++) {
            const int q = i * THREADS + tid;
            const int wr = q / V4, c4 = q - wr * V4;
            const int gr = min(max(first + wr, 0), M - 1), gc = min(c4 * 4, K - 4);
            w[i] = *(const psp_f32x4 *)(X + (size_t)gr * (size_t)K + gc);
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
            for (int i = 0; i < C; i++) xr[u][i] = *(const psp_f32x4 *)(X + (size_t)c * (size_t)K + min(off[i], K - 4));
        }
    };
    // local columns -> byte offsets of their rows in the ring (the zero row for a slot past the row's local part);
    // BWD keeps the columns as floats beside them (the factor of the weight gradient) and clears the padding's values
    auto to_ring = [&](int a, int m, int(&cl)[T], float(&vl)[T], float(&cf)[T]) {
#pragma unroll
        for (int t = 0; t < T; t++) {
            const bool ok = a + t * L + sub < m;
            if constexpr (BWD) {
                cf[t] = ok ? (float)cl[t] : 0.0f;
                vl[t] = ok ? vl[t] : 0.0f;
            }
            cl[t] = ok ? pspw_slot<RING>(cl[t]) * (TN * 4) : ZERO_OFF;
        }
    };
    auto dot = [&](const psp_f32x4(&x)[C], const psp_f32x4(&ar)[C]) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < C; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) s = __builtin_fmaf(x[i][e], ar[i][e], s);
        return s;
    };
    auto axpy = [&](float s, const psp_f32x4(&x)[C], psp_f32x4(&acc)[C]) {
#pragma unroll
        for (int i = 0; i < C; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][e] = __builtin_fmaf(s, x[i][e], acc[i][e]);
    };

    int a, m, b, an, mn, bn;
    int cl[T], cr, cln[T], crn;
    float vl[T], vr = 0.0f, vln[T], vrn = 0.0f, cf[T];
    psp_f32x4 xr[UR][C], w[FPT], ar[C];

    // ---- first block of the run: its whole window, its entries, its remote rows -------------------------------------------
    load_bounds(j0, a, m, b);
    load_bounds(j0 + 1, an, mn, bn);
#pragma unroll 1
    for (int piece = 0; piece < PSPW_FIRST_PIECES; piece++) {
        fill_load(j0 * RB - PSPW_HALO + piece * RB, w);
        fill_store(j0 * RB - PSPW_HALO + piece * RB, w);
    }
    load_entries(a, m, cl, vl, cr, vr);
    gather_remote(cr, m, b, 0, xr);
    to_ring(a, m, cl, vl, cf);
    __syncthreads();

#pragma unroll 1
    for (int j = j0; j < j1; j++) {
        int a2, m2, b2;
        load_entries(an, mn, cln, vln, crn, vrn);
        load_bounds(j + 2, a2, m2, b2);
        fill_load((j + 1) * RB + PSPW_HALO, w);  // the rows that enter with block j + 1
        const int r = j * RB + grp;
        {
            // the group's own row (a row past the matrix has no entries; its slot holds the nearest valid row)
            const int slot = pspw_slot<RING>(r) * TN;
#pragma unroll
            for (int i = 0; i < C; i++) {
                ar[i] = *(const psp_f32x4 *)(s_x + slot + off[i]);
                if (!live[i]) ar[i] = (psp_f32x4){0.f, 0.f, 0.f, 0.f};  // columns past K hold copies of the last four
            }
        }
        psp_f32x4 acc[C];
#pragma unroll
        for (int i = 0; i < C; i++) acc[i] = (psp_f32x4){0.f, 0.f, 0.f, 0.f};

        // ---- local entries: both rows on chip ---------------------------------------------------------------------------
        // (a padding slot reads the zero row; its score is cleared as well, so that a non-finite row of X cannot turn
        // it into a NaN)
#define PSPA_STEP(T_, J_)                                                                          \
    {                                                                                              \
        const int o_ = pspw_bcast<L, J_>(cl[T_], sub) + sub * 16;                                  \
        psp_f32x4 x_[C];                                                                           \
        _Pragma("unroll") for (int i = 0; i < C; i++)                                              \
            x_[i] = *(const psp_f32x4 *)((const char *)s_x + (o_ + i * (L * 16)));                 \
        float s_ = pspw_reduce_all<L>(dot(x_, ar));                                                \
        s_ = a + T_ * L + J_ < m ? s_ : 0.0f;                                                      \
        if constexpr (BWD) {                                                                       \
            if (sub == J_) wsum = __builtin_fmaf(s_, cf[T_], wsum);                                \
            axpy(pspw_bcast_f<L, J_>(vl[T_], sub), x_, acc);                                       \
        } else {                                                                                   \
            s_ *= alpha;                                                                           \
            if (sub == J_) mine = s_;                                                              \
            axpy(s_, x_, acc);                                                                     \
        }                                                                                          \
    }
#pragma unroll
        for (int t = 0; t < T; t++) {
            // a chunk no lane group of the wavefront reaches is skipped as a whole
            if (__builtin_amdgcn_ballot_w64(a + t * L < m) == 0ull) continue;
            float mine = 0.0f;
            PSPA_STEP(t, 0)
            PSPA_STEP(t, 1)
            PSPA_STEP(t, 2)
            PSPA_STEP(t, 3)
            if constexpr (L == 8) {
                PSPA_STEP(t, 4)
                PSPA_STEP(t, 5)
                PSPA_STEP(t, 6)
                PSPA_STEP(t, 7)
            }
            if constexpr (!BWD) {
                const int p = a + t * L + sub;
                if (p < m) att_out[p] = mine;
            }
        }
#undef PSPA_STEP
        // local entries beyond the ones fetched up front
        for (int p = a + T * L; p < m; p++) {
            const int c_ = colIdx[p];
            const int slot = pspw_slot<RING>(c_) * TN;
            psp_f32x4 x_[C];
#pragma unroll
            for (int i = 0; i < C; i++) x_[i] = *(const psp_f32x4 *)(s_x + (slot + off[i]));
            float s_ = pspw_reduce_all<L>(dot(x_, ar));
            if constexpr (BWD) {
                if (sub == 0) wsum = __builtin_fmaf(s_, (float)c_, wsum);
                axpy(att_in[p], x_, acc);
            } else {
                s_ *= alpha;
                if (sub == 0) att_out[p] = s_;
                axpy(s_, x_, acc);
            }
        }

        // ---- remote entries ----------------------------------------------------------------------------------------------
        // first round: entries 0 .. 3, whose rows were gathered while the previous block was processed; second round:
        // entries 4 .. 7 of lane groups of 8 (columns already in lanes 4 .. 7), gathered together when some row of the
        // wavefront has that many
        auto remote_round = [&](int first, const psp_f32x4(&x)[UR][C]) {
#pragma unroll
            for (int u = 0; u < UR; u++) {
                // (the moves between lanes stay outside the branch: every lane of the group takes part in them)
                const int e = first + u;
                const float vu = BWD ? pspw_remote_f<L>(vr, e, sub) : 0.0f;
                float s_ = pspw_reduce_all<L>(dot(x[u], ar));
                if (m + e < b) {
                    if constexpr (BWD) {
                        if (sub == e) wsum = __builtin_fmaf(s_, (float)cr, wsum);
                        axpy(vu, x[u], acc);
                    } else {
                        s_ *= alpha;
                        if (sub == e) att_out[m + e] = s_;
                        axpy(s_, x[u], acc);
                    }
                }
            }
        };
        remote_round(0, xr);
        if (REM > UR && __builtin_amdgcn_ballot_w64(m + UR < b) != 0ull) {
            psp_f32x4 x2[UR][C];
            gather_remote(cr, m, b, UR, x2);
            remote_round(UR, x2);
        }
        for (int p = m + REM; p < b; p++) {
            const int c_ = colIdx[p];
            psp_f32x4 x_[C];
#pragma unroll
            for (int i = 0; i < C; i++) x_[i] = *(const psp_f32x4 *)(X + (size_t)c_ * (size_t)K + min(off[i], K - 4));
            float s_ = pspw_reduce_all<L>(dot(x_, ar));
            if constexpr (BWD) {
                if (sub == 0) wsum = __builtin_fmaf(s_, (float)c_, wsum);
                axpy(att_in[p], x_, acc);
            } else {
                s_ *= alpha;
                if (sub == 0) att_out[p] = s_;
                axpy(s_, x_, acc);
            }
        }
        if (r < M) {
#pragma unroll
            for (int i = 0; i < C; i++)
                if (live[i]) __builtin_nontemporal_store(acc[i], (psp_f32x4 *)(Y + (size_t)r * (size_t)K + off[i]));
        }

        // ---- hand over to block j + 1 ---------------------------------------------------------------------------------
        gather_remote(crn, mn, bn, 0, xr);                     // in flight while block j + 1 is processed
        fill_store((j + 1) * RB + PSPW_HALO, w);    // slots no row of block j's or j + 1's window occupies
        a = an, m = mn, b = bn;
        an = a2, mn = m2, bn = b2;
        cr = crn, vr = vrn;
#pragma unroll
        for (int t = 0; t < T; t++) cl[t] = cln[t], vl[t] = vln[t];
        to_ring(a, m, cl, vl, cf);
        __syncthreads();
    }

    if constexpr (BWD) {
        // the workgroup's share of the weight gradient: lanes -> wavefront -> workgroup -> one atomic addition
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) wsum += __shfl_xor(wsum, o, 64);
        if ((tid & 63) == 0) s_part[tid >> 6] = wsum;
        __syncthreads();
        if (tid == 0) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < THREADS / 64; i++) s += s_part[i];
            atomicAdd(wsum_out, s);
        }
    }
}

// ---- launch -----------------------------------------------------------------------------------------------------------
typedef void (*pspa_kernel_t)(const int *, const int *, const float *, const float *, const float *, float *, float *, float *,
                              int, int, int, int, int, int);
struct pspa_variant {
    pspa_kernel_t fn;
    int tn, threads;
};
static pspa_variant pspa_lookup(int K, bool bwd)
{
    if (K <= 16) return {bwd ? psp_attn_window_kernel<1, 2, 256, true> : psp_attn_window_kernel<1, 2, 256, false>, 16, 256};
    if (K <= 32) return {bwd ? psp_attn_window_kernel<1, 3, 512, true> : psp_attn_window_kernel<1, 3, 512, false>, 32, 512};
    // (a lane group covering 128 columns would spill registers: wider layers run the SDDMM and the SpMM separately)
    return {bwd ? psp_attn_window_kernel<2, 3, 512, true> : psp_attn_window_kernel<2, 3, 512, false>, 64, 512};
}

static int pspa_launch(bool bwd, const int *rowPtr_w, const int *colIdx_w, const float *att_in, const float *X, const float *alpha,
                       float *att_out, float *Y, float *wsum, int M, int nnz, int K, int rows_out, hipStream_t st)
{
    PSP_REQUIRE(K >= 4 && K % 4 == 0 && K <= PSP_ATTN_WINDOW_MAX_K,
                "attn_window: K must be a multiple of 4 between 4 and %d (got %d)", PSP_ATTN_WINDOW_MAX_K, K);
    PSP_REQUIRE(M >= 0 && nnz >= 0 && rows_out >= M, "attn_window: the output has %d rows, the matrix %d (%d entries)", rows_out, M, nnz);
    PSP_REQUIRE((((size_t)X | (size_t)Y) & 15) == 0, "attn_window: the dense operands must be 16-byte aligned");
    int rc = PSP_OK;
    if (bwd) {
        PSP_REQUIRE(wsum != nullptr, "attn_window: null pointer for the weight gradient");
        rc = psp_zero_f32(wsum, 1, st);
    }
    if (rc != PSP_OK) return rc;
    if (nnz == 0 || M == 0) return psp_zero_f32(Y, (size_t)rows_out * K, st);
    rc = psp_zero_f32(Y + (size_t)M * K, ((size_t)rows_out - (size_t)M) * K, st);  // rows past the matrix
    if (rc != PSP_OK) return rc;
    PSP_REQUIRE(rowPtr_w && colIdx_w && X && Y && (bwd ? att_in != nullptr : att_out != nullptr), "attn_window: null pointer");
    const pspa_variant k = pspa_lookup(K, bwd);
    const int lds = (2 * PSPW_BLOCK + 2 * PSPW_HALO + 1) * k.tn * 4;
    const int key = (k.tn == 16 ? 0 : k.tn == 32 ? 1 : 2) + (bwd ? 4 : 0);
    static bool lds_raised[8];
    if (lds > 48 * 1024 && !lds_raised[key]) {
        const hipError_t e = hipFuncSetAttribute((const void *)k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return psp_fail(PSP_ERR_LAUNCH, "attn_window: %d bytes of LDS refused: %s", lds, hipGetErrorString(e));
        lds_raised[key] = true;
    }
    const int nblocks = psp_ceil_div(M, PSPW_BLOCK);
    const int run = pspw_run_length(nblocks, 1, key, (const void *)k.fn, k.threads, lds);
    const int nruns = psp_ceil_div(nblocks, run);
    const psp_grid1d g = psp_xcd_grid(nruns, 1);
    hipLaunchKernelGGL(k.fn, dim3(g.launch), dim3(k.threads), lds, st, rowPtr_w, colIdx_w, att_in, X, alpha, att_out, Y, wsum, M, K,
                       nnz, nruns, g.stripe, run);
    return psp_check_launch("attention window kernel");
}

PSP_EXPORT int psp_attn_window_forward_f32(const int *rowPtr_w, const int *colIdx_w, const float *X, const float *alpha, float *att,
                                           float *Y, int M, int nnz, int K, int rows_out, psp_stream_t stream)
{
    return pspa_launch(false, rowPtr_w, colIdx_w, nullptr, X, alpha, att, Y, nullptr, M, nnz, K, rows_out, (hipStream_t)stream);
}

PSP_EXPORT int psp_attn_window_backward_f32(const int *rowPtr_w, const int *colIdx_w, const float *att, const float *dY, float *G,
                                            float *wsum, int M, int nnz, int K, int rows_out, psp_stream_t stream)
{
    return pspa_launch(true, rowPtr_w, colIdx_w, att, dY, nullptr, nullptr, G, wsum, M, nnz, K, rows_out, (hipStream_t)stream);
}
