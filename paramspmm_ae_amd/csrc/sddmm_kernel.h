// Parameterised SDDMM kernel for gfx950 (wave64): out[p] = <A[row(p),:], B[col(p),:]> for every stored
// entry p.  Semantics follow SDDMM/sddmm_kernel.cu:917-1287 (the stored values never scale the result; for
// 2x1 blocks they only decide which of the two entries is computed).
//
// A lane group of L = 2^LOGL lanes works on one sparse row at a time; each lane keeps C vectors of V floats of
// the A row in registers and loads the matching part of the B row, so a group reads L*V*4 contiguous bytes per load.
// The per-lane partial dot products are summed across the group with DPP / ds_swizzle butterflies.  The L
// results of one chunk of L non-zeros are parked one per lane and written with a single coalesced store
// (the reference stores one float per warp per non-zero).
#pragma once
#include "psp_common.h"
#include "spmm_kernel.h"  // psp_vec

// Sum over aligned groups of 2^LOGL lanes; every lane of the group receives the total.
template <int LOGL> __device__ __forceinline__ float psp_group_sum(float v)
{
    if constexpr (LOGL >= 1)  // lane ^ 1
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
    if constexpr (LOGL >= 2)  // lane ^ 2
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
    if constexpr (LOGL >= 3)  // mirror inside 8 lanes: the partner sits in the other quad
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
    if constexpr (LOGL >= 4)  // mirror inside 16 lanes
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
    if constexpr (LOGL >= 5)  // lane ^ 16 inside 32 lanes
        v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
    if constexpr (LOGL >= 6)  // lane ^ 32
        v += __int_as_float(__builtin_amdgcn_ds_bpermute((int)((threadIdx.x ^ 32) & 63) << 2, __float_as_int(v)));
    return v;
}

// Maximum over aligned groups of 2^LOGL lanes (all lanes of the group active); every lane receives it.
template <int LOGL> __device__ __forceinline__ float psp_group_max(float v)
{
#define PSP_DPP_MAX(CTRL) v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, false)))
    if constexpr (LOGL >= 1) PSP_DPP_MAX(0xB1);
    if constexpr (LOGL >= 2) PSP_DPP_MAX(0x4E);
    if constexpr (LOGL >= 3) PSP_DPP_MAX(0x141);
    if constexpr (LOGL >= 4) PSP_DPP_MAX(0x140);
#undef PSP_DPP_MAX
    if constexpr (LOGL >= 5) v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F)));
    if constexpr (LOGL >= 6) v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_bpermute((int)((threadIdx.x ^ 32) & 63) << 2, __float_as_int(v))));
    return v;
}

// val: bcsr -> [nblk,2] block values (gate); csr -> optional per-entry scale (may be null when !SCALE)
//
// The walk is the one of the SpMM kernel: a wavefront owns W = 2^logW consecutive segments, their stored entries
// are divided evenly between the 64/L lane groups, and a group reloads its A row (prefetched one segment ahead)
// whenever it crosses into another row.  Every stored entry is written exactly once, so `out` needs no clearing.
//
// row_max (CSR layouts, may be null): the largest result of every row is also raised into row_max[row] (atomic
// max, once per lane group and row; the caller has filled the array with the lowest float).  The attention
// pipeline's softmax-weighted SpMM takes its reference maxima from there instead of sweeping the entries again.
//
// BAL (plain layouts): the launch is a fixed grid of wavefronts that divide the *stored entries* between them -- each
// takes consecutive tiles of 2^logW entries, finds the rows that hold them with a 64-ary search in rowPtr and walks
// them window by window (up to 64 rows at a time, cut at the tile's ends).  Every entry's result is independent, so a
// row may be cut anywhere, and a hub row of 10^5 entries spreads over a hundred wavefronts instead of pinning one.
template <int LOGL, int C, int V, int U, int NR, bool SPLIT, bool SCALE, bool BAL = false>
__global__ void __launch_bounds__(512)
psp_sddmm_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const float *__restrict__ val,
                 const int *__restrict__ target_row, const float *__restrict__ A, const float *__restrict__ B,
                 float *__restrict__ out, int nseg, int K, int logW, int tiles, int stripe, float *__restrict__ row_max)
{
    typedef typename psp_vec<V>::type vec_t;
    constexpr bool BCSR = NR > 1;  // NR rows per stored entry: 1 = CSR, 2 = 2x1 blocks, 3 = 3x1 blocks
    constexpr int L = 1 << LOGL;
    constexpr int R = PSP_WAVE >> LOGL;
    static_assert(U <= L, "unroll must not exceed the group width");
    static_assert(!BAL || !SPLIT, "the entry-balanced walk is for the plain layouts (row-split input is balanced already)");
    __shared__ int2 s_seg[PSP_MAX_WAVES][PSP_WAVE];  // (end offset, A row) of the wavefront's filled segments
    // CSR results of narrow groups wait here until the group has 32 of them (a 128-byte line of `out`) and then leave
    // in one burst of stores: a group stores only L floats at a time, and lines written piecemeal are evicted from the
    // L2 half-written by the gather stream (measured: 3x the result's bytes in HBM writes at L = 4).
    // 2x1 blocks hold pairs (16 blocks to a line); 3x1 blocks are stored directly.
    constexpr int HOLD = (NR <= 2 && LOGL >= 2 && LOGL + NR <= 5) ? ((32 / NR) >> LOGL) : 1;  // chunks held back per group
    __shared__ __align__(8) float s_hold[HOLD > 1 ? PSP_MAX_WAVES : 1][HOLD > 1 ? HOLD * PSP_WAVE * NR : 1];

    const int lane = threadIdx.x & (PSP_WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int sub = lane & (L - 1);
    const int grp = lane >> LOGL;
    const int grp_base = lane - sub;

    int off[C];
    bool live[C];
#pragma unroll
    for (int i = 0; i < C; i++) {
        const int col = ((i << LOGL) + sub) * V;
        live[i] = col < K;
        off[i] = live[i] ? col : K - V;
    }

    // One window: the segments s0 .. s0+nvalid-1 (at most 64), of which only the entries inside [pbeg, pend) count
    // (the plain walk passes the whole range of the segments).  tabW: power of two >= nvalid.
    auto run_window = [&](const int s0, const int nvalid, const int pbeg, const int pend, const int tabW) {
    const int W = tabW;
    const int P0 = pbeg;
    const int P1 = min(rowPtr[s0 + nvalid], pend);
    {
        const bool in = lane < nvalid;
        const int e = in ? min(rowPtr[s0 + lane + 1], pend) : P1;
        const int e_up = __shfl_up(e, 1);  // cross-lane reads stay outside any lane-dependent branch
        const int b_ = (lane == 0) ? P0 : e_up;
        const bool filled = in && e > b_;
        const unsigned long long fmask = __ballot(filled);
        const int slot = __popcll(fmask & ((1ull << lane) - 1ull));
        s_seg[wave][lane] = make_int2(P1, -1);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (filled) s_seg[wave][slot] = make_int2(e, SPLIT ? target_row[s0 + lane] : s0 + lane);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int2 *w_seg = s_seg[wave];
    if (P0 >= P1) return;

    const int q = (P1 - P0 + R - 1) >> (6 - LOGL);
    int a0 = P0 + grp * q;
    if (a0 > P1) a0 = P1;
    const int b0 = min(P1, a0 + q);
    if (a0 >= b0) return;  // the whole group leaves together; nothing below reads other groups' lanes

    // A row(s) of a segment; dead tail vectors are zero so they add nothing to the dot product
    auto load_a = [&](int key, float (&dst)[NR][C][V]) {
#pragma unroll
        for (int r = 0; r < NR; r++)
#pragma unroll
            for (int i = 0; i < C; i++) {
                vec_t t;
                if constexpr (V == 1) t = 0.0f;
                else {
#pragma unroll
                    for (int e = 0; e < V; e++) t[e] = 0.0f;
                }
                if (live[i]) t = *(const vec_t *)(A + (size_t)(key * NR + r) * (size_t)K + off[i]);
#pragma unroll
                for (int e = 0; e < V; e++) dst[r][i][e] = psp_elem<V>(t, e);
            }
    };

    int cur = 0;
    for (int step = W >> 1; step >= 1; step >>= 1)
        if (w_seg[cur + step - 1].x <= a0) cur += step;
    int row_end = w_seg[cur].x;
    int mykey = w_seg[cur].y;
    float a[NR][C][V], a_nxt[NR][C][V];
    load_a(mykey, a);
    {
        const int nk = cur + 1 < PSP_WAVE ? w_seg[cur + 1].y : -1;
        load_a(nk >= 0 ? nk : mykey, a_nxt);
    }

    float lmax = PSP_F32_LOWEST;  // largest result among this lane's entries of the current row
    auto emit_row_max = [&](int key) {
        const float m = psp_group_max<LOGL>(lmax);
        if (sub == 0 && m > PSP_F32_LOWEST) psp_atomic_max_f32(row_max + key, m);
        lmax = PSP_F32_LOWEST;
    };
    const bool want_max = !BCSR && row_max != nullptr;  // uniform

    // lane `sub` of the group picks up entry base+sub (column index and, where the format has one, its value); the
    // next chunk's are requested before the current chunk is worked on
    auto fetch = [&](int base, int &c_out, float (&g_out)[NR]) {
        const int q = base + sub;
        const int qq = q < b0 ? q : b0 - 1;
        c_out = colIdx[qq];
        if constexpr (NR == 2) {
            const psp_f32x2 t = ((const psp_f32x2 *)val)[qq];
            g_out[0] = t[0];
            g_out[1] = t[1];
        } else if constexpr (NR > 2) {
#pragma unroll
            for (int r = 0; r < NR; r++) g_out[r] = val[(size_t)qq * NR + r];
        } else {
            g_out[0] = SCALE ? val[qq] : 1.0f;
        }
    };
    int c_cur;
    float gate[NR];
    fetch(a0, c_cur, gate);
    int held = 0;         // chunks waiting in s_hold (group-uniform)
    int hold_base = a0;   // entry of the first of them
    // every lane reads back what it wrote itself, so the wavefront's program order is all the ordering needed
    auto release = [&]() {
#pragma unroll
        for (int j = 0; j < HOLD; j++) {
            const int pp = hold_base + (j << LOGL) + sub;
            if (j < held && pp < b0) {
                if constexpr (NR == 2) ((psp_f32x2 *)out)[pp] = ((const psp_f32x2 *)s_hold[wave])[j * PSP_WAVE + lane];
                else out[pp] = s_hold[wave][j * PSP_WAVE + lane];
            }
        }
        hold_base += held << LOGL;
        held = 0;
    };

    for (int base = a0; base < b0; base += L) {
        const int p = base + sub;
        const bool ok = p < b0;
        int c_nxt = 0;
        float gate_nxt[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) gate_nxt[r] = 0.0f;
        if (base + L < b0) fetch(base + L, c_nxt, gate_nxt);
        float res[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) res[r] = 0.0f;

        const int cnt = min(L, b0 - base);
        int k = 0;
        while (k < cnt) {
            // the current row's entries inside this chunk: positions [k, run_end)
            const int run_end = min(cnt, row_end - base);
            for (; k < run_end; k += U) {
                int ck[U];
#pragma unroll
                for (int u = 0; u < U; u++) ck[u] = psp_bperm_i(grp_base + min(k + u, L - 1), c_cur);
                vec_t bv[U][C];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const float *br = B + (size_t)ck[u] * (size_t)K;
#pragma unroll
                    for (int i = 0; i < C; i++) bv[u][i] = *(const vec_t *)(br + off[i]);
                }
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int r = 0; r < NR; r++) {
                        float part = 0.0f;
#pragma unroll
                        for (int i = 0; i < C; i++)
#pragma unroll
                            for (int e = 0; e < V; e++) part = __builtin_fmaf(a[r][i][e], psp_elem<V>(bv[u][i], e), part);
                        part = psp_group_sum<LOGL>(part);
                        // positions past run_end belong to the next row: their dot product with this A row is dropped
                        if (sub == k + u && k + u < run_end) {
                            res[r] = part;
                            if (!BCSR && want_max) lmax = fmaxf(lmax, SCALE ? part * gate[0] : part);
                        }
                    }
            }
            k = run_end;
            if (base + k == row_end && base + k < b0) {
                const int2 nx = w_seg[++cur];
                row_end = nx.x;
                if (nx.y != mykey) {
                    if (want_max) emit_row_max(mykey);  // the group is converged here: the condition is group-uniform
                    mykey = nx.y;
#pragma unroll
                    for (int r = 0; r < NR; r++)
#pragma unroll
                        for (int i = 0; i < C; i++)
#pragma unroll
                            for (int e = 0; e < V; e++) a[r][i][e] = a_nxt[r][i][e];
                }
                const int nk = cur + 1 < PSP_WAVE ? w_seg[cur + 1].y : -1;
                if (nk >= 0 && nk != mykey) load_a(nk, a_nxt);
            }
        }
        if (ok) {
            if constexpr (NR == 2 && HOLD == 1) {
                // entries of a block whose value is zero are padding: written as zero (sddmm_kernel.cu:1103,1115)
                psp_f32x2 o;
                o[0] = gate[0] != 0.0f ? res[0] : 0.0f;
                o[1] = gate[1] != 0.0f ? res[1] : 0.0f;
                ((psp_f32x2 *)out)[p] = o;
            } else if constexpr (NR > 2) {
#pragma unroll
                for (int r = 0; r < NR; r++) out[(size_t)p * NR + r] = gate[r] != 0.0f ? res[r] : 0.0f;
            } else if constexpr (HOLD == 1) {
                out[p] = SCALE ? res[0] * gate[0] : res[0];
            }
        }
        if constexpr (HOLD > 1) {
            if constexpr (NR == 2) {
                psp_f32x2 o;  // padding entries of a block (value zero) are written as zero (sddmm_kernel.cu:1103,1115)
                o[0] = gate[0] != 0.0f ? res[0] : 0.0f;
                o[1] = gate[1] != 0.0f ? res[1] : 0.0f;
                ((psp_f32x2 *)s_hold[wave])[held * PSP_WAVE + lane] = o;
            } else {
                s_hold[wave][held * PSP_WAVE + lane] = SCALE ? res[0] * gate[0] : res[0];
            }
            if (++held == HOLD) release();
        }
        c_cur = c_nxt;
#pragma unroll
        for (int r = 0; r < NR; r++) gate[r] = gate_nxt[r];
    }
    if constexpr (HOLD > 1) release();
    if (want_max) emit_row_max(mykey);
    };  // run_window

    if constexpr (!BAL) {
        const int tile = psp_xcd_tile(stripe);
        if (tile >= tiles) return;
        const int s0 = (tile * (int)(blockDim.x >> 6) + wave) << logW;
        if (s0 >= nseg) return;  // wave-uniform
        run_window(s0, min(1 << logW, nseg - s0), rowPtr[s0], 0x7fffffff, 1 << logW);
    } else {
        // Tiles of 2^logW stored entries.  Each XCD (workgroups are dealt to them round-robin) owns one contiguous
        // eighth of the tiles and its wavefronts take them in turn, so at any time an XCD works on a run of
        // neighbouring tiles -- neighbouring rows, whose B rows share its L2 -- and all XCDs carry the same load.
        const int nnz = rowPtr[nseg];
        const int ntiles = (int)(((long long)nnz + (1 << logW) - 1) >> logW);
        const int wpb = blockDim.x >> 6;
        const int xcd = blockIdx.x % PSP_XCDS;
        const int waves_per_xcd = (gridDim.x / PSP_XCDS) * wpb;
        const int tiles_per_xcd = (ntiles + PSP_XCDS - 1) / PSP_XCDS;
        const int band_end = min(ntiles, (xcd + 1) * tiles_per_xcd);
        for (int t = xcd * tiles_per_xcd + (blockIdx.x / PSP_XCDS) * wpb + wave; t < band_end; t += waves_per_xcd) {
        const int e0 = t << logW;
        const int e1 = min(nnz, e0 + (1 << logW));
        // first row whose end lies past e0: 64-ary search, one independent load per lane and round
        int lo = 0, hi = nseg;  // rowPtr[i + 1] <= e0 for i < lo, > e0 for i >= hi
        while (lo < hi) {
            const int step = (hi - lo + 63) >> 6;
            const int i = lo + lane * step;
            const bool gt = i >= hi || rowPtr[i + 1] > e0;  // ascending probes: false up to some lane, true from there on
            const unsigned long long m = __ballot(gt);
            const int f = m ? __ffsll((long long)m) - 1 : 64;
            int nlo = f == 0 ? lo : lo + (f - 1) * step + 1;
            int nhi = f == 64 ? hi : lo + f * step;
            lo = nlo < hi ? nlo : hi;
            hi = nhi < hi ? nhi : hi;
        }
        int s0 = lo, pbeg = e0;
        while (pbeg < e1 && s0 < nseg) {  // wave-uniform
            const int nvalid = min(PSP_WAVE, nseg - s0);
            run_window(s0, nvalid, pbeg, e1, PSP_WAVE);
            // the next window's table overwrites this one's: every group has finished reading it here
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            pbeg = min(rowPtr[s0 + nvalid], e1);
            s0 += nvalid;
        }
        }  // tiles of this wavefront
    }
}

typedef void (*psp_sddmm_kernel_t)(const int *, const int *, const float *, const int *, const float *,
                                   const float *, float *, int, int, int, int, int, float *);

// (LOGL, C, U) triples that exist.  C grows only once the group is 16 lanes wide (DPP-only reduction);
// beyond 64 vectors the group widens to 32 and 64 lanes.
#define PSP_SDDMM_FOR_EACH_LCU(M_) \
    M_(0, 1, 1) M_(1, 1, 2) M_(2, 1, 4) M_(3, 1, 4) M_(4, 1, 4) \
    M_(4, 2, 4) M_(4, 3, 2) M_(4, 4, 2) M_(5, 4, 2) M_(6, 4, 2)

template <int NR, bool SPLIT, bool SCALE, bool BAL = false>
static psp_sddmm_kernel_t psp_sddmm_lookup(int logL, int C, int V)
{
#define PSP_CASE(L_, C_, U_)                                                               \
    if (logL == L_ && C == C_) {                                                           \
        if (V == 4) return psp_sddmm_kernel<L_, C_, 4, U_, NR, SPLIT, SCALE, BAL>;       \
        if (V == 2) return psp_sddmm_kernel<L_, C_, 2, U_, NR, SPLIT, SCALE, BAL>;       \
        return psp_sddmm_kernel<L_, C_, 1, U_, NR, SPLIT, SCALE, BAL>;                   \
    }
    PSP_SDDMM_FOR_EACH_LCU(PSP_CASE)
#undef PSP_CASE
    return nullptr;
}

template <int NR, bool SPLIT>
int psp_sddmm_launch(const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                     const float *A, const float *B, const float *scale, float *out, int nrows, int K,
                     int blkWarpNum, hipStream_t stream, float *row_max);
