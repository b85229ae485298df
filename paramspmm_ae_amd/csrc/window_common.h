// Shared by the kernels that walk the windowed CSR layout (spmm_window.hip, sddmm_window.hip): the layout's constants,
// moves inside a lane group, and the sizing of a launch of persistent workgroups.
#pragma once
#include "psp_common.h"
#include <cstdlib>

typedef float psp_f32x4 __attribute__((ext_vector_type(4)));

#define PSPW_BLOCK PSP_WINDOW_BLOCK
#define PSPW_HALO PSP_WINDOW_HALO
// pieces of PSPW_BLOCK rows that cover a block's whole window (loaded before the first block of a run)
#define PSPW_FIRST_PIECES ((PSPW_BLOCK + 2 * PSPW_HALO + PSPW_BLOCK - 1) / PSPW_BLOCK)
#define PSPW_UR 4        // remote entries per row whose X tiles are prefetched into registers
#define PSPW_LOCAL 32    // local entries per row fetched up front (T = 32 / L chunks)

// slot of matrix row g (>= -PSPW_HALO) in a ring of RING rows
template <int RING> __device__ __forceinline__ int pspw_slot(int g) { return (int)((unsigned)(g + RING) % (unsigned)RING); }

// value of lane j of the caller's lane group (L = 4 or 8 consecutive lanes), j a compile-time constant: DPP moves on
// the vector ALU, which this kernel leaves idle, instead of ds_bpermute on the LDS pipeline, which it keeps busy
template <int L, int J> __device__ __forceinline__ int pspw_bcast(int x, int sub)
{
    constexpr int q = J & 3;
    const int t = __builtin_amdgcn_mov_dpp(x, q * 0x55, 0xf, 0xf, true);  // quad_perm: every lane of a quad reads lane q
    if constexpr (L == 4) return t;
    else {
        const int u = __builtin_amdgcn_mov_dpp(t, 0x141, 0xf, 0xf, true);  // row_half_mirror: lane k of 8 reads lane 7 - k
        // lanes 0..3 of the group hold x[q] in t and x[4 + q] in u; lanes 4..7 the other way round
        return ((sub < 4) == (J < 4)) ? t : u;
    }
}
template <int L, int J> __device__ __forceinline__ float pspw_bcast_f(float x, int sub)
{
    return __int_as_float(pspw_bcast<L, J>(__float_as_int(x), sub));
}
// the same for one of the first four lanes, u being the index of an unrolled loop
template <int L> __device__ __forceinline__ int pspw_bcast_u(int x, int u, int sub)
{
    switch (u) {
    case 0: return pspw_bcast<L, 0>(x, sub);
    case 1: return pspw_bcast<L, 1>(x, sub);
    case 2: return pspw_bcast<L, 2>(x, sub);
    default: return pspw_bcast<L, 3>(x, sub);
    }
}
// A lane group keeps the (column, value) pairs of a row's first L remote entries in registers, entry e in lane e.  The X
// rows of the first PSPW_UR = 4 are gathered a block ahead; groups of 8 lanes gather the other four together, in a
// second round, when some row of the wavefront has that many.  (Groups of 4 lanes -- 16 rows per wavefront, of which
// some row nearly always has a fifth entry -- were slower with a second round than with the plain loop.)
// Entry e (a constant after unrolling) for every lane of the group:
template <int L> __device__ __forceinline__ int pspw_remote(int x, int e, int sub)
{
    switch (e) {
    case 0: return pspw_bcast<L, 0>(x, sub);
    case 1: return pspw_bcast<L, 1>(x, sub);
    case 2: return pspw_bcast<L, 2>(x, sub);
    case 3: return pspw_bcast<L, 3>(x, sub);
    case 4: return pspw_bcast<L, 4>(x, sub);
    case 5: return pspw_bcast<L, 5>(x, sub);
    case 6: return pspw_bcast<L, 6>(x, sub);
    default: return pspw_bcast<L, 7>(x, sub);
    }
}
template <int L> __device__ __forceinline__ float pspw_remote_f(float x, int e, int sub)
{
    return __int_as_float(pspw_remote<L>(__float_as_int(x), e, sub));
}

// the same for any lane of the group
template <int L> __device__ __forceinline__ float pspw_bcast_any_f(float x, int j, int sub)
{
    const int v = __float_as_int(x);
    switch (j) {
    case 0: return __int_as_float(pspw_bcast<L, 0>(v, sub));
    case 1: return __int_as_float(pspw_bcast<L, 1>(v, sub));
    case 2: return __int_as_float(pspw_bcast<L, 2>(v, sub));
    case 3: return __int_as_float(pspw_bcast<L, 3>(v, sub));
    case 4: return __int_as_float(pspw_bcast<L, 4>(v, sub));
    case 5: return __int_as_float(pspw_bcast<L, 5>(v, sub));
    case 6: return __int_as_float(pspw_bcast<L, 6>(v, sub));
    default: return __int_as_float(pspw_bcast<L, 7>(v, sub));
    }
}

// Blocks one workgroup walks in a row.  Measured on a community-ordered block model (10^6 rows) with runs of 2 .. 64
// blocks at every width: the longer the run the better -- a run pays for its first window (192 rows instead of 64)
// and for the one wait the pipeline cannot hide -- up to the point where the launch has exactly as many workgroups as
// the GPU holds at once.  One workgroup more than that and the launch takes half as long again (the late workgroup
// starts when the first one ends, and every workgroup runs for the whole launch); fewer and CUs idle.  So the launch
// is sized from the occupancy the runtime reports for the kernel: at most that many workgroups (a multiple of the
// 8 XCDs per column tile, so that the grid holds no empty ones), each with an equal share of the blocks.
// PSP_WINDOW_RUN overrides the choice.
static int pspw_run_length(int nblocks, int tiles, int slot_key, const void *kernel, int threads, int lds)
{
    static const int forced = [] {
        const char *e = getenv("PSP_WINDOW_RUN");
        return e ? atoi(e) : 0;
    }();
    if (forced > 0) return forced;
    static int slots_of[16];  // workgroups the current GPU holds at once, per kernel of the including file (0 = not asked yet)
    if (slots_of[slot_key] == 0) {
        int dev = 0, cus = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, (size_t)lds) != hipSuccess || per_cu <= 0)
            per_cu = 1;
        slots_of[slot_key] = cus * per_cu;
    }
    int nruns = slots_of[slot_key] / tiles / PSP_XCDS * PSP_XCDS;
    if (nruns < PSP_XCDS) nruns = PSP_XCDS;
    const int run = (nblocks + nruns - 1) / nruns;
    return run < 1 ? 1 : run;
}


// Sum over the L lanes of a lane group of L values at once: lane s returns the sum, over the group, of p[s].  Halving
// steps -- a lane keeps the half of the values its partner does not, adds what the partner sends for that half -- so
// L values cost L - 1 DPP additions instead of L log2(L).  (Partners: 7 - s for the step over 8 lanes, then s ^ 2 and
// s ^ 1 inside the quad; the pairs {s, 7 - s} of a quad are exactly the other quad.)
template <int L> __device__ __forceinline__ float pspw_reduce_transposed(const float (&p)[L], int sub)
{
    float q[4];
    if constexpr (L == 8) {
        const bool hi = sub >= 4;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float keep = hi ? p[4 + i] : p[i], send = hi ? p[i] : p[4 + i];
            q[i] = keep + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(send), 0x141, 0xf, 0xf, true));
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = p[i];
    }
    const bool b1 = (sub & 2) != 0, b0 = (sub & 1) != 0;
    float r[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float keep = b1 ? q[2 + i] : q[i], send = b1 ? q[i] : q[2 + i];
        r[i] = keep + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(send), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
    }
    const float keep = b0 ? r[1] : r[0], send = b0 ? r[0] : r[1];
    return keep + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(send), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
}
// the same for four values: lane s returns the group's sum of p[s & 3]
template <int L> __device__ __forceinline__ float pspw_reduce_transposed4(const float (&p)[4], int sub)
{
    float q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        q[i] = p[i];
        if constexpr (L == 8) q[i] += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(p[i]), 0x141, 0xf, 0xf, true));
    }
    return pspw_reduce_transposed<4>(q, sub);
}
// sum of x over the lane group, in every lane
template <int L> __device__ __forceinline__ float pspw_reduce_all(float x)
{
    if constexpr (L == 8) x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xf, 0xf, true));
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xf, 0xf, true));
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xf, 0xf, true));
    return x;
}
