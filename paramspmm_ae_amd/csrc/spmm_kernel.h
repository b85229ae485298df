// Parameterised SpMM kernel for gfx950 (wave64).  One template serves the four PCSR formats
// (CSR / 2x1 BCSR, each plain or row-split).  Semantics follow the reference kernels
// SpMM/SpMM_kernel.cu:1157-1651: per output element one fp32 FMA per stored non-zero, in storage order
// (rows that are cut between lane groups or wavefronts are summed piecewise, see below).
//
// Work decomposition (what replaces "one 32-lane warp per row, CF columns per lane"):
//   * a wavefront owns W = 2^logW consecutive segments (rows, block-rows or row-split segments), i.e. one
//     contiguous range [P0,P1) of stored entries; their bounds and output rows sit in LDS;
//   * the wavefront is cut into R = 64/L groups of L = 2^logL lanes; the range [P0,P1) is divided evenly
//     between the groups, whatever the row lengths are, so a group walks ceil((P1-P0)/R) entries and
//     writes a row out whenever it crosses a row end.  Skewed rows therefore cost no idle lanes;
//   * every lane owns C column vectors of V floats (V = 4 -> global_load_dwordx4); vector i of lane s
//     covers columns tile*L*C*V + (i*L + s)*V .. +V, so the L lanes of a group read L*V*4 contiguous bytes
//     of an X row per load;
//   * colIdx / values are read once per L*U entries: lane s of a group takes the U consecutive entries
//     base + s*U .. in one 4U-byte load per array (a group reads whole 128-byte lines), the pairs are handed
//     round the group with ds_bpermute, and the next L*U are prefetched while the current ones are consumed;
//   * the walk goes over batches of U entries, whatever rows they belong to, so every lane group issues the
//     same U*C feature loads at the same time and only the closing of a row -- a store where a row ends --
//     diverges between groups.  With two register sets (SINGLE = false) the loads of batch t+1 are issued
//     before batch t is added; with one set (SINGLE = true) a batch is gathered, added, and the next one
//     gathered, which frees registers for more wavefronts per SIMD (psp_spmm_single_set picks);
//   * a row cut by a group boundary is summed across the groups in registers (ds_bpermute), in group order,
//     so plain CSR needs neither atomics nor a cleared Y.  Only a row whose segments lie in several
//     wavefronts (row-split formats) is accumulated with fp32 atomics, once per wavefront.
// Tail columns (N not a multiple of L*C*V): loads are redirected to the last valid vector, stores are
// predicated.  Lanes past the end of a group's range hold (last valid column, value 0).
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

// max(x, 0) per element; a NaN stays a NaN, as with torch.relu
template <int V> __device__ __forceinline__ void psp_relu_vec(typename psp_vec<V>::type &v)
{
    if constexpr (V == 1) v = v < 0.0f ? 0.0f : v;
    else {
#pragma unroll
        for (int e = 0; e < V; e++) v[e] = v[e] < 0.0f ? 0.0f : v[e];
    }
}

template <int V> __device__ __forceinline__ void psp_store_vec(float *p, const float (&a)[V])
{
    typename psp_vec<V>::type t;
    if constexpr (V == 1) t = a[0];
    else {
#pragma unroll
        for (int e = 0; e < V; e++) t[e] = a[e];
    }
    // Y is written once and not read again by this kernel: the streaming hint keeps it from displacing rows of X
    // in the L2 (measured 1-5 % faster; the same hint on colIdx / val loads is slower, other column tiles re-read them)
    __builtin_nontemporal_store(t, (typename psp_vec<V>::type *)p);
}

// COUNT consecutive 4-byte words starting at a 4-byte aligned address, fetched in the widest pieces (16, 8, 4 bytes)
typedef int psp_i32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef int psp_i32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));
template <int COUNT> __device__ __forceinline__ void psp_load_words(const int *p, int (&out)[COUNT])
{
    int done = 0;
#pragma unroll
    for (; done + 4 <= COUNT; done += 4) {
        const psp_i32x4_a4 t = *(const psp_i32x4_a4 *)(p + done);
#pragma unroll
        for (int e = 0; e < 4; e++) out[done + e] = t[e];
    }
    if constexpr ((COUNT & 2) != 0) {
        const psp_i32x2_a4 t = *(const psp_i32x2_a4 *)(p + done);
        out[done] = t[0];
        out[done + 1] = t[1];
        done += 2;
    }
    if constexpr ((COUNT & 1) != 0) out[done] = p[done];
}

__device__ __forceinline__ int psp_bperm_i(int src_lane, int v) { return __builtin_amdgcn_ds_bpermute(src_lane << 2, v); }
__device__ __forceinline__ float psp_bperm_f(int src_lane, float v)
{
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}

#define PSP_MAX_WAVES 8  // blkWarpNum is 4 or 8

// NR: rows per stored entry (1 = CSR, 2 = 2x1 BCSR, 3 = 3x1 blocks: the reference's vec_spmm, SpMM_kernel.cu:1653-1972).  SPLIT: segments carry an explicit output row.
// SM (CSR layouts): the stored values are attention scores e; the product is taken with softmax weights,
//   Y[i] = sum_j exp(e_ij - m_i) X[j] / sum_j exp(e_ij - m_i),   m_i = row_max[i] (any upper bound of the row works,
// the SDDMM kernel delivers the exact maximum).  The weights are formed on the fly, their sum travels with the
// partial sums like one more column, and a row is divided by it when it is written.  A row that several wavefronts
// share is accumulated unnormalised (atomics) together with its weight sum in row_sum; psp_row_scale_kernel divides
// such rows afterwards.  This replaces the separate softmax pass over the entries.
// ACT (a variant of its own, so that the plain kernel keeps its loop): relu_x != 0 makes the rows of X enter as
// max(x, 0) -- the ReLU between two layers applied to the gathered values (NaN stays NaN) instead of in a pass that
// writes the activated copy.  It costs no registers.  The matching backward, keeping an output element only where a
// mask is positive, is NOT done in this kernel: fetched where a row closes -- the point where the walk holds the
// most registers and where every lane group of the wavefront waits for the slowest -- the mask took the most used
// configuration from five to four wavefronts per SIMD and made the product 25-45 % slower on the community-ordered
// graph (341 against 243 us at N = 32, 1018 against 703 at N = 128; the separate pass costs 66 and 256 us).
// SINGLE: one register set instead of two (the walk below).
template <int C, int V, int U, int NR, bool SPLIT, bool SM, bool ACT = false, bool SINGLE = false>
__global__ void __launch_bounds__(512)
psp_spmm_kernel(const int *__restrict__ rowPtr, const int *__restrict__ colIdx, const float *__restrict__ val,
                const int *__restrict__ target_row, const float *__restrict__ X, float *__restrict__ Y,
                int nseg, int N, int logL, int logW, int tiles, int stripe, int align_pct,
                const float *__restrict__ row_max, float *__restrict__ row_sum, int relu_x, int tail_rows)
{
    static_assert(!SM || NR == 1, "softmax weights exist for the CSR layouts only");
    static_assert(!(SM && ACT), "the softmax-weighted product takes no activation argument");
    typedef typename psp_vec<V>::type vec_t;
    __shared__ int2 s_seg[PSP_MAX_WAVES][PSP_WAVE];  // (end offset, output row) of the wavefront's segments
    __shared__ float s_m[SM ? PSP_MAX_WAVES : 1][SM ? PSP_WAVE : 1];  // SM: reference maximum of each segment's row

    // tail_rows: the few rows Y has past the matrix's own (a feature matrix padded to an even row count): the first
    // wavefront of the launch writes their zeros, one column tile per blockIdx.y, instead of a launch of its own -- on
    // a matrix of 10^5 entries that launch and the gap behind it took as long as the product
    if (!SPLIT && tail_rows > 0 && blockIdx.x == 0 && threadIdx.x < PSP_WAVE) {
        const int tile_w = (C * V) << logL;
        const int col0 = blockIdx.y * tile_w;
        const int w = min(tile_w, N - col0);
        float *yt = Y + (size_t)nseg * NR * (size_t)N + col0;
        for (int i = threadIdx.x; i < tail_rows * w; i += PSP_WAVE) yt[(size_t)(i / w) * (size_t)N + i % w] = 0.0f;
    }

    const int tile = psp_xcd_tile(stripe);
    if (tile >= tiles) return;

    const int L = 1 << logL, W = 1 << logW;
    const int lane = threadIdx.x & (PSP_WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int sub = lane & (L - 1);
    const int grp = lane >> logL;
    const int grp_base = lane - sub;
    const int s0 = (tile * (int)(blockDim.x >> 6) + wave) << logW;  // first segment of this wavefront
    if (s0 >= nseg) return;                                         // wave-uniform
    const int nvalid = min(W, nseg - s0);

    // ---- segment table of this wavefront: only segments that hold entries, packed to the front ----------
    const int P0 = rowPtr[s0];
    const int P1 = rowPtr[s0 + nvalid];
    int e_lane;  // end offset of segment `lane` of this wavefront
    {
        const bool in = lane < nvalid;
        const int e = in ? rowPtr[s0 + lane + 1] : P1;
        e_lane = e;
        const int e_up = __shfl_up(e, 1);  // cross-lane reads stay outside any lane-dependent branch
        const int b_ = (lane == 0) ? P0 : e_up;
        const bool filled = in && e != b_;
        const unsigned long long fmask = __ballot(filled);
        const int slot = __popcll(fmask & ((1ull << lane) - 1ull));
        s_seg[wave][lane] = make_int2(P1, -1);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (filled) {
            const int key = SPLIT ? target_row[s0 + lane] : s0 + lane;
            s_seg[wave][slot] = make_int2(e, key);
            if constexpr (SM) s_m[wave][slot] = row_max[key];
        }
        if constexpr (!SPLIT) {
            // rows without entries are never visited below: write their zeros here, one row per lane group
            unsigned long long empties = __ballot(in && e == b_);
            int turn = 0;
            while (empties) {
                const int i = __ffsll((long long)empties) - 1;
                empties &= empties - 1;
                if ((turn++ & ((PSP_WAVE >> logL) - 1)) == grp) {
                    const int tile_col0 = blockIdx.y * ((C * V) << logL);
#pragma unroll
                    for (int r = 0; r < NR; r++) {
                        float *yr = Y + (size_t)((s0 + i) * NR + r) * (size_t)N;
#pragma unroll
                        for (int c = 0; c < C; c++) {
                            const int col = tile_col0 + ((c << logL) + sub) * V;
                            const float z[V] = {};
                            if (col < N) psp_store_vec<V>(yr + col, z);
                        }
                    }
                }
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int2 *w_seg = s_seg[wave];  // .x = end offset, .y = output row (block-row for NR = 2)
    if (P0 == P1) return;

    bool ext_head = false, ext_tail = false;  // the first / last row of this wavefront also has entries elsewhere
    int tr_prev = -1, tr_next = -1;
    if constexpr (SPLIT) {
        if (s0 > 0) tr_prev = target_row[s0 - 1];
        if (s0 + nvalid < nseg) tr_next = target_row[s0 + nvalid];
    }

    // ---- this group's share of [P0,P1) ---------------------------------------------------------------
    // Even division by default.  When giving every group whole segments (W/R each) costs at most align_pct
    // percent more steps than that, the segments are not cut: neighbouring rows then advance together and no
    // partial sums have to be merged.
    const int R = PSP_WAVE >> logL;
    const int q = (P1 - P0 + R - 1) >> (6 - logL);
    int a = P0 + grp * q;
    if (a > P1) a = P1;
    int b = min(P1, a + q);
    if (logW + logL >= 6) {
        const int m = 1 << (logW + logL - 6);  // segments per group
        const int first = grp * m;
        const int a_up = psp_bperm_i((first + PSP_WAVE - 1) & (PSP_WAVE - 1), e_lane);
        const int a_al = first == 0 ? P0 : a_up;
        const int b_al = psp_bperm_i(first + m - 1, e_lane);
        int longest = b_al - a_al;
#pragma unroll
        for (int d = 1; d < PSP_WAVE; d <<= 1) longest = max(longest, psp_bperm_i(lane ^ d, longest));
        if ((long long)longest * 100 <= (long long)q * (100 + align_pct)) {
            a = a_al;
            b = b_al;
        }
    }
    const bool busy = a < b;

    // segment that holds entry x: the first whose end exceeds x (unused table slots end at P1)
    auto seg_of = [&](int x) {
        int lo = 0;
        for (int step = W >> 1; step >= 1; step >>= 1)
            if (w_seg[lo + step - 1].x <= x) lo += step;
        return lo;
    };

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

    float acc[NR][C][V], head[NR][C][V];
#pragma unroll
    for (int r = 0; r < NR; r++)
#pragma unroll
        for (int i = 0; i < C; i++)
#pragma unroll
            for (int e = 0; e < V; e++) acc[r][i][e] = head[r][i][e] = 0.0f;
    float acc_l = 0.0f, head_l = 0.0f, m_cur = 0.0f;  // SM: weight sum of the running row / stashed head, row maximum

    // out: a finished row goes to Y; `shared` = other wavefronts add to the same row (row-split formats)
    auto write_out = [&](int key, bool shared) {
        if constexpr (SM) {
            if (!SPLIT || !shared) {
                const float inv = 1.0f / acc_l;  // the row's largest entry alone contributes exp(0) = 1
#pragma unroll
                for (int i = 0; i < C; i++)
#pragma unroll
                    for (int e = 0; e < V; e++) acc[0][i][e] *= inv;
            } else if (sub == 0 && blockIdx.y == 0) {
                unsafeAtomicAdd(row_sum + key, acc_l);  // one column tile reports the weight sum
            }
        }
#pragma unroll
        for (int r = 0; r < NR; r++) {
            float *yr = Y + (size_t)(key * NR + r) * (size_t)N;
#pragma unroll
            for (int i = 0; i < C; i++) {
                if (!live[i]) continue;
                if (!SPLIT || !shared) {
                    psp_store_vec<V>(yr + off[i], acc[r][i]);
                } else {
#pragma unroll
                    for (int e = 0; e < V; e++) unsafeAtomicAdd(yr + off[i] + e, acc[r][i][e]);
                }
            }
        }
    };

    enum { F_HEAD = 1, F_CLOSED = 2, F_SHARED = 4 };
    // what `head` holds, for the groups before this one; a group without entries passes a row on unchanged
    int flags = busy ? 0 : F_HEAD;
    bool has_tail = false;  // acc holds the start of a row that goes on in the next group
    bool tail_shared = false;
    int cur = 0, row_end = 0, mykey = -1;
    bool first_run = true, head_valid = false;

    if (busy) {
        cur = seg_of(a);
        const int2 sg = w_seg[cur];
        row_end = sg.x;
        mykey = sg.y;
        if constexpr (SM) m_cur = s_m[wave][cur];
        const int seg_begin = cur == 0 ? P0 : w_seg[cur - 1].x;
        head_valid = a > seg_begin;
        if constexpr (SPLIT) {
            if (!head_valid && cur > 0) head_valid = w_seg[cur - 1].y == mykey;
            if (a == P0) ext_head = tr_prev == mykey;
        }
    }

    // Lane `sub` of the group picks up the U consecutive entries base + sub*U ..: one 4U-byte load of column
    // indices and one of 4U*NR bytes of values, so a group reads L*U*4 contiguous bytes of each array at a time
    // (whole 128-byte lines for 8 lanes x 4 entries).  Entries past the end of the range: (last column, 0), taken
    // one by one so that nothing past the arrays is touched.
#define PSP_FETCH(base, c_out, v_out)                                                        \
    {                                                                                        \
        const int p0_ = (base) + sub * U;                                                    \
        if (p0_ + U <= b) {                                                                  \
            psp_load_words<U>(colIdx + p0_, c_out);                                          \
            int w_[U * NR];                                                                  \
            psp_load_words<U * NR>((const int *)val + (size_t)p0_ * NR, w_);                 \
            _Pragma("unroll") for (int u_ = 0; u_ < U; u_++)                                 \
                _Pragma("unroll") for (int r_ = 0; r_ < NR; r_++) v_out[u_][r_] = __int_as_float(w_[u_ * NR + r_]); \
        } else {                                                                             \
            _Pragma("unroll") for (int u_ = 0; u_ < U; u_++)                                 \
            {                                                                                \
                const bool ok_ = p0_ + u_ < b;                                               \
                const int pp_ = ok_ ? p0_ + u_ : b - 1;                                      \
                c_out[u_] = colIdx[pp_];                                                     \
                _Pragma("unroll") for (int r_ = 0; r_ < NR; r_++)                            \
                {                                                                            \
                    const float t_ = val[(size_t)pp_ * NR + r_];                             \
                    v_out[u_][r_] = ok_ ? t_ : 0.0f;                                         \
                }                                                                            \
            }                                                                                \
        }                                                                                    \
    }

    int c_cur[U], c_nxt[U];
    float v_cur[U][NR], v_nxt[U][NR];
#pragma unroll
    for (int u = 0; u < U; u++) {
        c_cur[u] = c_nxt[u] = 0;
#pragma unroll
        for (int r = 0; r < NR; r++) v_cur[u][r] = v_nxt[u][r] = 0.0f;
    }
    if (busy) PSP_FETCH(a, c_cur, v_cur);

    // The entry just added closed its segment and the group's range goes on: move to the next filled segment
    // (the table holds filled segments only) and, when that belongs to another row, hand the finished row on.
    auto next_segment = [&]() {
        const int2 nx = w_seg[++cur];
        row_end = nx.x;
        const int nkey = nx.y;
        if (nkey != mykey) {
            if (first_run && head_valid) {
#pragma unroll
                for (int r = 0; r < NR; r++)
#pragma unroll
                    for (int i = 0; i < C; i++)
#pragma unroll
                        for (int e = 0; e < V; e++) head[r][i][e] = acc[r][i][e];
                head_l = acc_l;
                flags = F_HEAD | F_CLOSED;
            } else {
                write_out(mykey, first_run && ext_head);
            }
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int i = 0; i < C; i++)
#pragma unroll
                    for (int e = 0; e < V; e++) acc[r][i][e] = 0.0f;
            acc_l = 0.0f;
            first_run = false;
            mykey = nkey;
            if constexpr (SM) m_cur = s_m[wave][cur];
        }
    };

    // The walk goes over batches of U entries, whatever rows they belong to.  GATHER takes the next U (column, value)
    // pairs of the group from the lanes that hold them and issues the feature loads; CONSUME adds a batch entry by
    // entry and closes a row where one ends.  Every lane group of the wavefront issues the same loads at the same time
    // (nothing before them depends on the row lengths), and only the short row-closing part diverges between groups.
    // Entries past the group's range (last, partial batch) are loaded from a valid address but never added, so values
    // of other rows cannot leak in.
    // !SINGLE: two register sets alternate, the loads of batch t+1 are issued before batch t is added.
    // SINGLE: one register set -- gather a batch, add it, gather the next.  What the second set buys is small: the
    // wait in front of a batch's additions is placed for the path on which the next gather was skipped, so behind a
    // gather that was issued it also covers that gather's loads, and a wavefront has one batch in flight beyond the one
    // it waits for only while it issues.  The registers of the second set cost more: without it the kernel with four
    // entries in flight keeps 7 wavefronts per SIMD instead of 5, and is 15-20 % faster on graphs whose gathers mostly
    // hit (block model, stencil), 2-8 % on the R-MAT graph.  With one entry in flight, or lane groups of 2 or 4 lanes
    // with two, the second set still pays (psp_spmm_single_set).
    int pos = a;      // first entry of the next batch to gather
    int cbase = a;    // first entry of the chunk c_cur / v_cur hold (lane `sub` holds entries cbase + sub*U ..)
    int jb = 0;       // batch of that chunk the next gather takes: the one lane `jb` of the group holds
    const int chunk = L * U;
    if (busy && a + chunk < b) PSP_FETCH(a + chunk, c_nxt, v_nxt);

#define PSP_DECLARE(S)      \
    int S##_ck[U], S##_pos; \
    float S##_vk[U][NR];    \
    vec_t S##_x[U][C];
#define PSP_GATHER(S)                                                                                  \
    {                                                                                                  \
        if (jb == L) { /* the chunk is used up: the prefetched one becomes current, the next is requested */ \
            _Pragma("unroll") for (int u = 0; u < U; u++)                                              \
            {                                                                                          \
                c_cur[u] = c_nxt[u];                                                                   \
                _Pragma("unroll") for (int r = 0; r < NR; r++) v_cur[u][r] = v_nxt[u][r];              \
            }                                                                                          \
            cbase += chunk;                                                                            \
            if (cbase + chunk < b) PSP_FETCH(cbase + chunk, c_nxt, v_nxt);                             \
            jb = 0;                                                                                    \
        }                                                                                              \
        S##_pos = pos;                                                                                 \
        const int src = grp_base + jb;                                                                 \
        _Pragma("unroll") for (int u = 0; u < U; u++)                                                  \
        {                                                                                              \
            S##_ck[u] = psp_bperm_i(src, c_cur[u]);                                                    \
            _Pragma("unroll") for (int r = 0; r < NR; r++) S##_vk[u][r] = psp_bperm_f(src, v_cur[u][r]); \
        }                                                                                              \
        _Pragma("unroll") for (int u = 0; u < U; u++)                                                  \
        {                                                                                              \
            const float *xr = X + (size_t)S##_ck[u] * (size_t)N;                                       \
            _Pragma("unroll") for (int i = 0; i < C; i++) S##_x[u][i] = *(const vec_t *)(xr + off[i]); \
        }                                                                                              \
        pos += U;                                                                                      \
        jb++;                                                                                          \
    }
#define PSP_CONSUME(S)                                                                                 \
    {                                                                                                  \
        if (ACT && relu_x) {                                                                           \
            _Pragma("unroll") for (int u = 0; u < U; u++)                                              \
                _Pragma("unroll") for (int i = 0; i < C; i++) psp_relu_vec<V>(S##_x[u][i]);            \
        }                                                                                              \
        _Pragma("unroll") for (int u = 0; u < U; u++)                                                  \
        {                                                                                              \
            const int p1 = S##_pos + u + 1;                                                            \
            if (p1 <= b) {                                                                             \
                if constexpr (SM) {                                                                    \
                    S##_vk[u][0] = __expf(S##_vk[u][0] - m_cur);                                       \
                    acc_l += S##_vk[u][0];                                                             \
                }                                                                                      \
                _Pragma("unroll") for (int r = 0; r < NR; r++)                                         \
                {                                                                                      \
                    /* 2x1 blocks: a zero entry is skipped (SpMM_kernel.cu:1399,1405) */               \
                    if (NR == 1 || S##_vk[u][r] != 0.0f) {                                             \
                        _Pragma("unroll") for (int i = 0; i < C; i++)                                  \
                            _Pragma("unroll") for (int e = 0; e < V; e++)                              \
                                acc[r][i][e] = __builtin_fmaf(S##_vk[u][r], psp_elem<V>(S##_x[u][i], e), acc[r][i][e]); \
                    }                                                                                  \
                }                                                                                      \
                if (p1 == row_end && p1 < b) next_segment();                                           \
            }                                                                                          \
        }                                                                                              \
    }

    if constexpr (SINGLE) {
        if (busy) {
            PSP_DECLARE(A)
            do {
                PSP_GATHER(A)
                PSP_CONSUME(A)
            } while (pos < b);
        }
    } else if (busy) {
        PSP_DECLARE(A)
        PSP_DECLARE(B)
        PSP_GATHER(A)
        while (true) {
            bool more = pos < b;
            if (more) PSP_GATHER(B)
            PSP_CONSUME(A)
            if (!more) break;
            more = pos < b;
            if (more) PSP_GATHER(A)
            PSP_CONSUME(B)
            if (!more) break;
        }
    }
#undef PSP_DECLARE
#undef PSP_GATHER
#undef PSP_CONSUME
#undef PSP_FETCH

    // ---- the row this group stopped in ----------------------------------------------------------------
    if (busy) {
        bool goes_on = false;  // does the row continue in the next group?
        if (b < P1) {
            if (b < row_end) goes_on = true;
            else if (SPLIT) goes_on = w_seg[cur + 1].y == mykey;
        }
        if (SPLIT && b == P1) ext_tail = tr_next == mykey;
        const bool partial_head = first_run && head_valid;
        if (goes_on) {
            if (partial_head) {
                // the whole range lies inside one row that began earlier and goes on
#pragma unroll
                for (int r = 0; r < NR; r++)
#pragma unroll
                    for (int i = 0; i < C; i++)
#pragma unroll
                        for (int e = 0; e < V; e++) head[r][i][e] = acc[r][i][e];
                head_l = acc_l;
                flags = F_HEAD;
            } else {
                has_tail = true;
                tail_shared = first_run && ext_head;
            }
        } else if (partial_head) {
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int i = 0; i < C; i++)
#pragma unroll
                    for (int e = 0; e < V; e++) head[r][i][e] = acc[r][i][e];
            head_l = acc_l;
            flags = F_HEAD | F_CLOSED | (ext_tail ? F_SHARED : 0);
        } else {
            write_out(mykey, (first_run && ext_head) || ext_tail);
        }
    }

    // ---- rows cut by group boundaries: the group holding the start adds the following groups' heads ---
    // (all lanes take part in every ds_bpermute; only groups with an open tail accumulate)
    for (int d = 1; __ballot(has_tail) != 0ull; d++) {
        const int src = lane + (d << logL);
        const int src_c = src & (PSP_WAVE - 1);
        const int hf_any = psp_bperm_i(src_c, flags);  // executed by every lane, then masked
        const int hf = (src < PSP_WAVE) ? hf_any : 0;
        if constexpr (SM) {
            const float hl = psp_bperm_f(src_c, head_l);
            if (has_tail && (hf & F_HEAD)) acc_l += hl;
        }
#pragma unroll
        for (int r = 0; r < NR; r++)
#pragma unroll
            for (int i = 0; i < C; i++)
#pragma unroll
                for (int e = 0; e < V; e++) {
                    const float h = psp_bperm_f(src_c, head[r][i][e]);
                    if (has_tail && (hf & F_HEAD)) acc[r][i][e] += h;
                }
        if (has_tail && (!(hf & F_HEAD) || (hf & F_CLOSED) || src >= PSP_WAVE)) {
            write_out(mykey, tail_shared || (hf & F_SHARED));
            has_tail = false;
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
                                  int, int, int, int, int, int, int, const float *, float *, int, int);
#define PSP_SPMM_TAIL_ROWS_MAX 16  // more rows than this past the matrix are cleared by a fill launch

// One register set or two (template parameter SINGLE)?  Measured on the block model, the stencil and the R-MAT graph at
// N = 16 ... 256, all layouts: four or more entries in flight -- one set, everywhere (-8 ... -25 %; these kernels always
// have lane groups of at least four lanes); two entries -- one set from 8 lanes per row on (-0 ... -13 %; +2 ... +20 %
// with 2 or 4 lanes); one entry in flight -- two sets (one set: +2 ... +31 %).
static inline bool psp_spmm_single_set(int U, int lanes_per_row) { return U >= 4 || (U == 2 && lanes_per_row >= 8); }

// only the variants psp_spmm_single_set can ask for are instantiated
template <int C, int V, int U, int NR, bool SPLIT, bool SM, bool ACT>
static psp_spmm_kernel_t psp_spmm_pick(bool single)
{
    if constexpr (U >= 4) return psp_spmm_kernel<C, V, U, NR, SPLIT, SM, ACT, true>;
    else if constexpr (U == 2)
        return single ? psp_spmm_kernel<C, V, U, NR, SPLIT, SM, ACT, true> : psp_spmm_kernel<C, V, U, NR, SPLIT, SM, ACT, false>;
    else return psp_spmm_kernel<C, V, U, NR, SPLIT, SM, ACT, false>;
}

// softmax-weighted variants exist for CSR layouts, float4 columns and up to 4 vectors per lane
template <int NR, bool SPLIT>
static psp_spmm_kernel_t psp_spmm_lookup(int C, int V, int U, int lanes_per_row, bool softmax, bool act = false)
{
    const bool single = psp_spmm_single_set(U, lanes_per_row);
#define PSP_CASE(C_, U_)                                                        \
    if (C == C_ && U == U_) {                                                   \
        if (act) {                                                              \
            if constexpr (NR <= 2) {                                            \
                if (V == 4) return psp_spmm_pick<C_, 4, U_, NR, SPLIT, false, true>(single); \
                if (V == 2) return psp_spmm_pick<C_, 2, U_, NR, SPLIT, false, true>(single); \
                return psp_spmm_pick<C_, 1, U_, NR, SPLIT, false, true>(single); \
            }                                                                   \
            return nullptr;                                                     \
        }                                                                       \
        if (softmax) {                                                          \
            if constexpr (NR == 1 && C_ <= 4) {                                 \
                if (V == 4) return psp_spmm_pick<C_, 4, U_, 1, SPLIT, true, false>(single); \
            }                                                                   \
            return nullptr;                                                     \
        }                                                                       \
        if (V == 4) return psp_spmm_pick<C_, 4, U_, NR, SPLIT, false, false>(single); \
        if (V == 2) return psp_spmm_pick<C_, 2, U_, NR, SPLIT, false, false>(single); \
        return psp_spmm_pick<C_, 1, U_, NR, SPLIT, false, false>(single);       \
    }
    PSP_SPMM_FOR_EACH_CU(PSP_CASE)
#undef PSP_CASE
    return nullptr;
}

// nrows: rows / block-rows / segments.  Y rows covered: nrows*NR (plain) or all of rows_out (split, cleared first).
template <int NR, bool SPLIT>
int psp_spmm_launch(const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                    const float *X, float *Y, int nrows, int N, int rows_out, int CF, int blkWarpNum,
                    hipStream_t stream, const float *row_max, float *row_sum, int relu_x = 0);
