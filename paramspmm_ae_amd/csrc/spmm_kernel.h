// Parameterised SpMM kernel for gfx950 (wave64).  One template serves the four PCSR formats
// (CSR / 2x1 BCSR, each plain or row-split).  Semantics follow the reference kernels
// SpMM/SpMM_kernel.cu:1157-1651: per output element one fp32 FMA per stored non-zero, in storage order.
//
// Work decomposition (what replaces "one 32-lane warp per row, CF columns per lane"):
//   * a sparse row (or block-row, or row segment) is owned by a group of L = 2^logL lanes of a wavefront,
//     so one wavefront carries 64/L rows;
//   * every lane owns C column vectors of V floats (V = 4 -> global_load_dwordx4); vector i of lane s
//     covers columns tile*L*C*V + (i*L + s)*V .. +V, so the L lanes of a group read L*V*4 contiguous bytes
//     of an X row per load;
//   * colIdx / values are read once per L non-zeros, coalesced (lane s takes non-zero base+s), and handed
//     round the group with ds_bpermute; the next L are prefetched while the current ones are consumed;
//   * U non-zeros are unrolled so U*C feature loads are in flight per lane before the first FMA.
// Tail columns (N not a multiple of L*C*V): loads are redirected to the last valid vector, stores are
// predicated.  Lanes past the end of a row hold (last valid column, value 0).
#pragma once
#include "psp_common.h"

typedef float psp_f32x2 __attribute__((ext_vector_type(2)));
typedef float psp_f32x4 __attribute__((ext_vector_type(4)));

template <int V> struct psp_vec;
template <> struct psp_vec<1> { typedef float type; };
template <> struct psp_vec<2> { typedef psp_f32x2 type; };
template <> struct psp_vec<4> { typedef psp_f32x4 type; };

template <int V> __device__ __forceinline__ float psp_elem(const typename psp_vec<V>::type &v, int e) { return v[e]; }
template <> __device__ __forceinline__ float psp_elem<1>(const float &v, int) { return v; }

template <int V> __device__ __forceinline__ void psp_store_vec(float *p, const float (&a)[V])
{
    typename psp_vec<V>::type t;
    if constexpr (V == 1) t = a[0];
    else {
#pragma unroll
        for (int e = 0; e < V; e++) t[e] = a[e];
    }
    *(typename psp_vec<V>::type *)p = t;
}

template <int C, int V, int U, bool BCSR, bool SPLIT>
__global__ void __launch_bounds__(512)
psp_spmm_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const float *__restrict__ val,
                const int *__restrict__ target_row, const float *__restrict__ X, float *__restrict__ Y,
                int nrows, int N, int logL, int tiles, int chunk)
{
    typedef typename psp_vec<V>::type vec_t;
    constexpr int NR = BCSR ? 2 : 1;

    const int tile = psp_xcd_tile(chunk);
    if (tile >= tiles) return;

    const int L = 1 << logL;
    const int lane = threadIdx.x & (PSP_WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int sub = lane & (L - 1);
    const int grp_base = lane - sub;
    const int row = ((tile * (int)(blockDim.x >> 6) + wave) << (6 - logL)) + (lane >> logL);

    int off[C];
    bool live[C];
    {
        const int tile_col0 = blockIdx.y * ((C * V) << logL);
#pragma unroll
        for (int i = 0; i < C; i++) {
            const int col = tile_col0 + ((i << logL) + sub) * V;
            live[i] = col < N;
            off[i] = live[i] ? col : N - V;
        }
    }

    int lb = 0, hb = 0;
    if (row < nrows) {
        lb = rowPtr[row];
        hb = rowPtr[row + 1];
    }

    float acc[NR][C][V];
#pragma unroll
    for (int r = 0; r < NR; r++)
#pragma unroll
        for (int i = 0; i < C; i++)
#pragma unroll
            for (int e = 0; e < V; e++) acc[r][i][e] = 0.0f;

    int c_cur = 0;
    float v_cur[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) v_cur[r] = 0.0f;

    // lane `sub` of the group picks up non-zero base+sub; past the end: (last column of the row, 0)
#define PSP_FETCH(base, c_out, v_out)                                      \
    {                                                                      \
        const int p_ = (base) + sub;                                       \
        const bool ok_ = p_ < hb;                                          \
        const int pp_ = ok_ ? p_ : hb - 1;                                 \
        c_out = colIdx[pp_];                                               \
        if constexpr (BCSR) {                                              \
            const psp_f32x2 t_ = ((const psp_f32x2 *)val)[pp_];            \
            v_out[0] = ok_ ? t_[0] : 0.0f;                                 \
            v_out[1] = ok_ ? t_[1] : 0.0f;                                 \
        } else {                                                           \
            const float t_ = val[pp_];                                     \
            v_out[0] = ok_ ? t_ : 0.0f;                                    \
        }                                                                  \
    }

    if (lb < hb) PSP_FETCH(lb, c_cur, v_cur);

    for (int base = lb; base < hb; base += L) {
        int c_nxt = 0;
        float v_nxt[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) v_nxt[r] = 0.0f;
        if (base + L < hb) PSP_FETCH(base + L, c_nxt, v_nxt);

        const int cnt = min(L, hb - base);
        for (int k = 0; k < cnt; k += U) {
            int ck[U];
            float vk[U][NR];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int src = (grp_base + k + u) << 2;
                ck[u] = __builtin_amdgcn_ds_bpermute(src, c_cur);
#pragma unroll
                for (int r = 0; r < NR; r++)
                    vk[u][r] = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(v_cur[r])));
            }
            vec_t x[U][C];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float *xr = X + (size_t)ck[u] * (size_t)N;
#pragma unroll
                for (int i = 0; i < C; i++) x[u][i] = *(const vec_t *)(xr + off[i]);
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    // 2x1 blocks: a zero entry is skipped (SpMM_kernel.cu:1399,1405)
                    if (!BCSR || vk[u][r] != 0.0f) {
#pragma unroll
                        for (int i = 0; i < C; i++)
#pragma unroll
                            for (int e = 0; e < V; e++)
                                acc[r][i][e] = __builtin_fmaf(vk[u][r], psp_elem<V>(x[u][i], e), acc[r][i][e]);
                    }
                }
        }
        c_cur = c_nxt;
#pragma unroll
        for (int r = 0; r < NR; r++) v_cur[r] = v_nxt[r];
    }
#undef PSP_FETCH

    if (row >= nrows) return;

    if constexpr (!SPLIT) {
        // every covered row is written, empty ones as zeros: the caller need not clear Y first
#pragma unroll
        for (int r = 0; r < NR; r++) {
            float *yr = Y + (size_t)(row * NR + r) * (size_t)N;
#pragma unroll
            for (int i = 0; i < C; i++)
                if (live[i]) psp_store_vec<V>(yr + off[i], acc[r][i]);
        }
    } else {
        if (lb == hb) return;
        const int t = target_row[row];
        const bool shared = (row > 0 && target_row[row - 1] == t) || (row + 1 < nrows && target_row[row + 1] == t);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            float *yr = Y + (size_t)(t * NR + r) * (size_t)N;
#pragma unroll
            for (int i = 0; i < C; i++) {
                if (!live[i]) continue;
                if (!shared) {
                    // the only segment of its row: Y was cleared, a plain store equals 0 + partial
                    psp_store_vec<V>(yr + off[i], acc[r][i]);
                } else {
#pragma unroll
                    for (int e = 0; e < V; e++) unsafeAtomicAdd(yr + off[i] + e, acc[r][i][e]);
                }
            }
        }
    }
}

// (C, U) pairs that exist: U = non-zeros in flight, bounded by the register budget U*C*V
#define PSP_SPMM_FOR_EACH_CU(M_) \
    M_(1, 8) M_(1, 4) M_(1, 2) M_(1, 1) \
    M_(2, 4) M_(2, 2) M_(2, 1) \
    M_(3, 2) M_(3, 1) M_(4, 2) M_(4, 1) \
    M_(5, 1) M_(6, 1) M_(7, 1) M_(8, 1)

typedef void (*psp_spmm_kernel_t)(const int *, const int *, const float *, const int *, const float *, float *,
                                  int, int, int, int, int);

template <bool BCSR, bool SPLIT>
static psp_spmm_kernel_t psp_spmm_lookup(int C, int V, int U)
{
#define PSP_CASE(C_, U_)                                                          \
    if (C == C_ && U == U_) {                                                     \
        if (V == 4) return psp_spmm_kernel<C_, 4, U_, BCSR, SPLIT>;               \
        if (V == 2) return psp_spmm_kernel<C_, 2, U_, BCSR, SPLIT>;               \
        return psp_spmm_kernel<C_, 1, U_, BCSR, SPLIT>;                           \
    }
    PSP_SPMM_FOR_EACH_CU(PSP_CASE)
#undef PSP_CASE
    return nullptr;
}

// nrows: rows / block-rows / segments.  Y rows covered: nrows*NR (plain) or all of rows_out (split, cleared first).
template <bool BCSR, bool SPLIT>
int psp_spmm_launch(const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                    const float *X, float *Y, int nrows, int N, int rows_out, int CF, int blkWarpNum,
                    hipStream_t stream);
