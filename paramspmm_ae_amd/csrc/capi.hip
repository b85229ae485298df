// extern "C" surface of libparamsp_hip.so (declared in include/paramsp.h), the small utility kernels
// (zero fill, genmask, segment softmax) and the host-side PCSR index construction.
#include <algorithm>
#include <mutex>
#include <thread>
#include <vector>
#include <string.h>
#include <stdlib.h>
#include "psp_common.h"
#include "spmm_kernel.h"
#include "sddmm_kernel.h"

// ------------------------------------------------------------------------------------------------
// errors
// ------------------------------------------------------------------------------------------------
static thread_local char g_err[512] = "";

int psp_fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Library-wide options: defaults, overridden once by the environment (PSP_XCD_STRIPE_ROWS, PSP_ALIGN_PCT,
// PSP_SPLIT_CLEAR_MIN, PSP_WHOLE_ROWS, PSP_DENSE_SPLIT) when the library is first used, and afterwards only through psp_set_option.
psp_options &psp_opts(void)
{
    static psp_options o = [] {
        psp_options d;
        d.stripe_rows = 8192;
        d.align_pct = 50;
        d.split_clear_min = (long long)4 << 20;
        d.whole_rows = 0;
        d.dense_split = 1;
        if (const char *e = getenv("PSP_XCD_STRIPE_ROWS")) {
            if (atoi(e) > 0) d.stripe_rows = atoi(e);
        }
        if (const char *e = getenv("PSP_ALIGN_PCT")) {
            if (atoi(e) >= 0) d.align_pct = atoi(e);
        }
        if (const char *e = getenv("PSP_SPLIT_CLEAR_MIN")) {
            if (atoll(e) >= 0) d.split_clear_min = atoll(e);
        }
        if (const char *e = getenv("PSP_WHOLE_ROWS")) d.whole_rows = atoi(e) != 0;
        if (const char *e = getenv("PSP_DENSE_SPLIT")) d.dense_split = atoi(e) != 0;
        return d;
    }();
    return o;
}
int psp_stripe_rows(void) { return psp_opts().stripe_rows; }

PSP_EXPORT int psp_set_option(const char *name, long long value)
{
    PSP_REQUIRE(name != nullptr, "set_option: name is null");
    psp_options &o = psp_opts();
    if (!strcmp(name, "xcd_stripe_rows")) {
        PSP_REQUIRE(value >= 1 && value <= (1 << 30), "set_option: xcd_stripe_rows must be positive");
        o.stripe_rows = (int)value;
    } else if (!strcmp(name, "align_pct")) {
        PSP_REQUIRE(value >= 0 && value <= 100000, "set_option: align_pct must be 0..100000");
        o.align_pct = (int)value;
    } else if (!strcmp(name, "split_clear_min")) {
        PSP_REQUIRE(value >= 0, "set_option: split_clear_min must not be negative");
        o.split_clear_min = value;
    } else if (!strcmp(name, "whole_rows")) {
        PSP_REQUIRE(value == 0 || value == 1, "set_option: whole_rows is 0 or 1");
        o.whole_rows = (int)value;
    } else if (!strcmp(name, "dense_split")) {
        PSP_REQUIRE(value == 0 || value == 1, "set_option: dense_split is 0 or 1");
        o.dense_split = (int)value;
    } else {
        return psp_fail(PSP_ERR_ARG, "set_option: unknown option '%s'", name);
    }
    return PSP_OK;
}

PSP_EXPORT long long psp_get_option(const char *name)
{
    if (!name) return psp_fail(PSP_ERR_ARG, "get_option: name is null");
    const psp_options &o = psp_opts();
    if (!strcmp(name, "xcd_stripe_rows")) return o.stripe_rows;
    if (!strcmp(name, "align_pct")) return o.align_pct;
    if (!strcmp(name, "split_clear_min")) return o.split_clear_min;
    if (!strcmp(name, "whole_rows")) return o.whole_rows;
    if (!strcmp(name, "dense_split")) return o.dense_split;
    return psp_fail(PSP_ERR_ARG, "get_option: unknown option '%s'", name);
}

PSP_EXPORT const char *psp_last_error(void) { return g_err; }
PSP_EXPORT int psp_version(void) { return PSP_ABI_VERSION; }

// ------------------------------------------------------------------------------------------------
// (N, CF, blkWarpNum) -> wave64 launch plan
// ------------------------------------------------------------------------------------------------
static bool psp_cu_pair_exists(int C, int U)
{
#define PSP_HAS(C_, U_) \
    if (C == C_ && U == U_) return true;
    PSP_SPMM_FOR_EACH_CU(PSP_HAS)
#undef PSP_HAS
    return false;
}

PSP_EXPORT int psp_spmm_plan_for(int N, int CF, int blkWarpNum, psp_spmm_plan *plan)
{
    PSP_REQUIRE(plan != nullptr, "plan is null");
    PSP_REQUIRE(N >= 1, "feature dimension must be positive (got %d)", N);
    const int stripe_rows = ((blkWarpNum & PSP_BW_STRIPE_MASK) >> PSP_BW_STRIPE_SHIFT) * 256;  // 0: the library option
    blkWarpNum &= ~PSP_BW_STRIPE_MASK;
    PSP_REQUIRE(blkWarpNum == 4 || blkWarpNum == 8, "blkWarpNum must be 4 or 8 (got %d)", blkWarpNum);
    const int V = (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
    const int nvec = N / V;
    int C, L, U, logW = -1;
    if (CF & PSP_CF_NATIVE) {
        // native configuration: every field of the wave64 mapping chosen by the caller (the sweep / the decider)
        PSP_REQUIRE((CF & ~(PSP_CF_NATIVE | 0xfff)) == 0, "CF 0x%x: unknown bits in a native configuration", CF);
        C = (CF & 7) + 1;
        const int logL = (CF >> 3) & 7, logU = (CF >> 6) & 3, wsel = (CF >> 8) & 7;
        PSP_REQUIRE(logL <= 6, "native configuration: 2^%d lanes per row exceed the wavefront", logL);
        L = 1 << logL;
        U = 1 << logU;
        PSP_REQUIRE(U <= L, "native configuration: %d entries in flight need at least as many lanes per row (got %d)", U, L);
        C = std::min(C, nvec);
        PSP_REQUIRE(psp_cu_pair_exists(C, U), "native configuration: no kernel for %d vectors per lane with %d entries in flight", C, U);
        if (wsel) logW = wsel - 1;
    } else {
        PSP_REQUIRE(CF >= 1 && CF <= 8, "CF must be 1..8 (got %d)", CF);
        // A lane group owns a tile of 32*CF columns, as the reference's warp does (CF columns per lane of a 32-lane
        // warp, SpMM_kernel.cu:162-165); the remaining columns go to further column tiles (grid.y).  Natively the
        // 32-column slab is 8 lanes x float4 (16 x float2 / 32 x float when N is not a multiple of 4) and CF is the
        // number of such vectors per lane, so a wavefront carries 8 rows whatever CF is.
        C = std::min(CF, nvec);
        L = 32 / V;
        while (L > 1 && (L / 2) * C >= nvec) L >>= 1;  // one tile already covers N: no wider than needed
        U = C == 1 ? 4 : C <= 4 ? 2 : 1;  // feature vectors in flight per lane: U entries x C vectors
        while (U > L) U >>= 1;
    }
    plan->vec = V;
    plan->coarsen = C;
    plan->lanes_per_row = L;
    plan->rows_per_wave = PSP_WAVE / L;
    plan->unroll = U;
    plan->col_tiles = psp_ceil_div(nvec, L * C);
    plan->waves_per_block = blkWarpNum;
    plan->log_segs_per_wave = logW;
    plan->even_split = (CF & PSP_CF_NATIVE) && (CF & PSP_CF_EVEN_SPLIT) ? 1 : 0;
    plan->xcd_stripe_rows = stripe_rows;
    return PSP_OK;
}

PSP_EXPORT int psp_spmm_register_sets(int unroll, int lanes_per_row) { return psp_spmm_single_set(unroll, lanes_per_row) ? 1 : 2; }

// ------------------------------------------------------------------------------------------------
// zero fill
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) psp_zero_kernel(float *__restrict__ p, size_t n)
{
    // n4 float4 stores from a 16-byte aligned start, scalar head and tail
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t head = std::min<size_t>(n, (size_t)((16 - ((uintptr_t)p & 15)) & 15) / 4);
    float *q = p + head;
    const size_t n4 = (n - head) / 4;
    psp_f32x4 z = {0.f, 0.f, 0.f, 0.f};
    for (size_t i = tid; i < n4; i += stride) ((psp_f32x4 *)q)[i] = z;
    if (tid < head) p[tid] = 0.f;
    const size_t tail0 = head + n4 * 4;
    if (tid < n - tail0) p[tail0 + tid] = 0.f;
}

int psp_zero_f32(float *p, size_t n, hipStream_t stream)
{
    if (n == 0) return PSP_OK;
    const size_t want = (n / 4 + 255) / 256 + 1;
    const int blocks = (int)std::min<size_t>(want, 256 * 32);
    hipLaunchKernelGGL(psp_zero_kernel, dim3(blocks), dim3(256), 0, stream, p, n);
    return psp_check_launch("zero fill");
}

__global__ void __launch_bounds__(256) psp_fill_kernel(float *__restrict__ p, size_t n, float value)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = value;
}

int psp_fill_f32(float *p, size_t n, float value, hipStream_t stream)
{
    if (n == 0) return PSP_OK;
    const int blocks = (int)std::min<size_t>((n + 255) / 256, 256 * 32);
    hipLaunchKernelGGL(psp_fill_kernel, dim3(blocks), dim3(256), 0, stream, p, n, value);
    return psp_check_launch("fill");
}

__global__ void __launch_bounds__(256) psp_row_scale_kernel(float *__restrict__ Y, const float *__restrict__ s, int rows, int N)
{
    // 16 lanes per row: almost every row has s == 0 and costs one load
    const long long g = ((long long)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int sub = threadIdx.x & 15;
    if (g >= rows) return;
    const float w = s[g];
    if (w == 0.0f) return;
    const float inv = 1.0f / w;
    float *yr = Y + g * N;
    for (int c = sub; c < N; c += 16) yr[c] *= inv;
}

int psp_row_scale(float *Y, const float *s, int rows, int N, hipStream_t stream)
{
    if (rows == 0 || N == 0) return PSP_OK;
    hipLaunchKernelGGL(psp_row_scale_kernel, dim3(psp_ceil_div((long long)rows * 16, 256)), dim3(256), 0, stream, Y, s, rows, N);
    return psp_check_launch("row scale");
}

// ------------------------------------------------------------------------------------------------
// selective clear for row-split SpMM: the rows the SpMM kernel adds to rather than stores (a row continuing across
// two wavefronts, a row with an empty segment) and the rows no segment targets.
//
// The first `seg_blocks` workgroups walk the segments, one lane per segment (coalesced loads of target_row and
// rowPtr_split, no search): a wavefront clears the rows its 64 segments flag, and the run of untargeted rows in front
// of each segment's row (after the last segment too) -- up to PSP_CLEAR_CAP rows of it.  Hub rows of a thousand
// segments cost nothing extra this way (a workgroup per 256 target rows, which this replaces, spent 85 us scanning
// the segments of the R-MAT graph's first 256 rows while the rest of the grid had long finished).
// The remaining workgroups sweep what is left of long runs: one wavefront per PSP_CLEAR_CAP target rows finds the
// segment its rows start at (a 64-ary search in target_row, one independent load per lane and round) and clears the
// rows of its block that lie in a run beyond the run's first PSP_CLEAR_CAP rows.  A run that reaches past its cap
// into a block contains the block's first row, so that one search finds it; a run of 10^5 untargeted rows spreads
// over hundreds of wavefronts.
// ------------------------------------------------------------------------------------------------
#define PSP_CLEAR_CAP 256

__device__ __forceinline__ void psp_wave_clear(float *__restrict__ Y, size_t b0, size_t b1, int lane, bool vec4)
{
    if (vec4) {
        const psp_f32x4 z = {0.f, 0.f, 0.f, 0.f};
        for (size_t j = b0 + 4 * (size_t)lane; j < b1; j += 256) *(psp_f32x4 *)(Y + j) = z;
    } else {
        for (size_t j = b0 + lane; j < b1; j += 64) Y[j] = 0.0f;
    }
}

__global__ void __launch_bounds__(256)
psp_split_clear_kernel(const int *__restrict__ rowPtr_split, const int *__restrict__ target_row, float *__restrict__ Y,
                       int nseg, int N, int nr, int rows_out, int logW, int seg_blocks)
{
    const int ntargets = (rows_out + nr - 1) / nr;
    const int lane = threadIdx.x & 63;
    const size_t per_target = (size_t)nr * N, total = (size_t)rows_out * N;  // the last target row may be cut by rows_out
    const bool vec4 = (per_target & 3) == 0 && (total & 3) == 0 && ((uintptr_t)Y & 15) == 0;
    if ((int)blockIdx.x < seg_blocks) {
        // lane s < nseg: segment s; lane s == nseg: a virtual segment that targets the row past the last one, so that
        // the untargeted rows at the end are the run in front of it
        const int s = blockIdx.x * 256 + threadIdx.x;
        const bool in = s < nseg;
        const int t = in ? target_row[s] : ntargets;
        const int tp = s == 0 ? -1 : (s <= nseg ? target_row[s - 1] : ntargets);
        bool added = false;
        if (in) {
            const bool boundary = s > 0 && (s & ((1 << logW) - 1)) == 0 && tp == t;  // continues across two wavefronts
            const bool empty = rowPtr_split[s] == rowPtr_split[s + 1];
            added = boundary || empty;
        }
        const int run = s <= nseg ? min(t - tp - 1, PSP_CLEAR_CAP) : 0;  // untargeted rows right in front of row t
        unsigned long long m = __ballot(added);
        while (m) {  // wave-uniform
            const int b = __ffsll((long long)m) - 1;
            m &= m - 1;
            const size_t b0 = (size_t)__shfl(t, b) * per_target;
            psp_wave_clear(Y, b0, min(total, b0 + per_target), lane, vec4);
        }
        m = __ballot(run > 0);
        while (m) {
            const int b = __ffsll((long long)m) - 1;
            m &= m - 1;
            const size_t b0 = (size_t)(__shfl(tp, b) + 1) * per_target;
            psp_wave_clear(Y, b0, min(total, b0 + (size_t)__shfl(run, b) * per_target), lane, vec4);
        }
        return;
    }
    const int u0 = (((int)blockIdx.x - seg_blocks) * 4 + (int)(threadIdx.x >> 6)) * PSP_CLEAR_CAP;
    if (u0 >= ntargets) return;  // wave-uniform
    int lo = 0, hi = nseg;  // target_row[i] < u0 for i < lo, >= u0 for i >= hi
    while (lo < hi) {
        const int step = (hi - lo + 63) >> 6;
        const int i = lo + lane * step;
        // probes are ascending and a probe past the range counts as >= u0: false up to some lane, true from there on
        const bool ge = i >= hi || target_row[i] >= u0;
        const unsigned long long m = __ballot(ge);
        const int f = m ? __ffsll((long long)m) - 1 : 64;
        const int nlo = f == 0 ? lo : lo + (f - 1) * step + 1;
        const int nhi = f == 64 ? hi : lo + f * step;
        lo = min(nlo, hi);
        hi = min(nhi, hi);
    }
    const int tp = lo > 0 ? target_row[lo - 1] : -1;      // last targeted row in front of the block
    const int tn = lo < nseg ? target_row[lo] : ntargets;  // first targeted row at or after the block's first row
    const int r0 = max(u0, tp + 1 + PSP_CLEAR_CAP), r1 = min(min(u0 + PSP_CLEAR_CAP, tn), ntargets);
    if (r0 < r1) psp_wave_clear(Y, (size_t)r0 * per_target, min(total, (size_t)r1 * per_target), lane, vec4);
}

int psp_split_clear(const int *rowPtr_split, const int *target_row, float *Y, int nseg, int N, int nr, int rows_out,
                    int logW, hipStream_t stream)
{
    const int ntargets = (rows_out + nr - 1) / nr;
    if (ntargets == 0 || N == 0) return PSP_OK;
    const int seg_blocks = nseg / 256 + 1;  // one lane more than there are segments
    const int sweep_blocks = psp_ceil_div(ntargets, 4 * PSP_CLEAR_CAP);
    hipLaunchKernelGGL(psp_split_clear_kernel, dim3(seg_blocks + sweep_blocks), dim3(256), 0, stream, rowPtr_split, target_row,
                       Y, nseg, N, nr, rows_out, logW, seg_blocks);
    return psp_check_launch("split clear kernel");
}

// ------------------------------------------------------------------------------------------------
// genmask (SDDMM/sddmm_kernel.cu:78-141): one lane per block-row walks its blocks in storage order
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
psp_genmask_kernel(const int *__restrict__ rowPtr_b, const int *__restrict__ rowPtr,
                   const float *__restrict__ val_b, int *__restrict__ mask, int nblkrows)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nblkrows) return;
    const int lb = rowPtr_b[t], hb = rowPtr_b[t + 1];
    if (lb == hb) return;
    int cnt0 = rowPtr[2 * t], cnt1 = rowPtr[2 * t + 1];
    for (int i = lb; i < hb; i++) {
        const psp_f32x2 v = ((const psp_f32x2 *)val_b)[i];
        if (v[0] != 0.0f) mask[cnt0++] = 2 * i;
        if (v[1] != 0.0f) mask[cnt1++] = 2 * i + 1;
    }
}

PSP_EXPORT int psp_genmask(const int *rowPtr_b, const int *rowPtr, const float *val_b, int nblkrows, int nnz,
                           int *mask, psp_stream_t stream)
{
    PSP_REQUIRE(nblkrows >= 0 && nnz >= 0, "genmask: negative size");
    if (nnz == 0 || nblkrows == 0) return PSP_OK;
    PSP_REQUIRE(rowPtr_b && rowPtr && val_b && mask, "genmask: null pointer");
    // slots no non-zero block entry maps to stay zero, as in the reference (mask = zeros, sddmm_kernel.cu:126)
    int rc = psp_zero_f32((float *)mask, (size_t)nnz, (hipStream_t)stream);
    if (rc != PSP_OK) return rc;
    hipLaunchKernelGGL(psp_genmask_kernel, dim3(psp_ceil_div(nblkrows, 256)), dim3(256), 0, (hipStream_t)stream,
                       rowPtr_b, rowPtr, val_b, mask, nblkrows);
    return psp_check_launch("genmask kernel");
}

// ------------------------------------------------------------------------------------------------
// segment softmax.  Short rows: 16 lanes per row, three sweeps over the row (max, sum, write); rows of up to 64
// entries never re-read memory.  Rows longer than PSP_SOFTMAX_LONG (128) entries are handled in one of two ways:
//   * without workspace (psp_segment_softmax_f32): the workgroup that met the row takes it with all 256 lanes;
//     a hub row of 10^5 entries then runs on one workgroup -- correct, but it becomes the tail of the launch;
//   * with workspace (psp_segment_softmax_ws_f32): the short-row kernel only resets the row's (max, sum) pair in
//     the workspace; three further launches walk the entry array in chunks of PSP_SOFTMAX_CHUNK entries, every
//     workgroup finding the long rows that cross its chunk and, one wavefront per row, contributing to their max
//     (atomic max), their sum (atomic add) and finally writing its part of the result -- a hub row spreads over
//     the whole GPU and rows of a few hundred entries no longer crawl along on 16 lanes.
// ------------------------------------------------------------------------------------------------
#define PSP_SOFTMAX_LONG 128
#define PSP_SOFTMAX_CHUNK 4096
#define PSP_SOFTMAX_NEG (-3.402823466e+38f)

__device__ __forceinline__ float psp_max16(float v)
{
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0xB1, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x4E, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x141, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x140, 0xF, 0xF, false)));
    return v;
}

// 256-lane reductions through LDS (4 wavefronts); every lane of the workgroup must call them
__device__ __forceinline__ float psp_block_max(float v, float *s_red)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v = fmaxf(v, __shfl_xor(v, d));
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = v;
    __syncthreads();
    v = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    __syncthreads();
    return v;
}
__device__ __forceinline__ float psp_block_sum(float v, float *s_red)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v += __shfl_xor(v, d);
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = v;
    __syncthreads();
    v = s_red[0] + s_red[1] + s_red[2] + s_red[3];
    __syncthreads();
    return v;
}

// WS: long rows are left to the chunk kernels, only their workspace pair is reset here
template <bool WS>
__global__ void __launch_bounds__(256)
psp_segment_softmax_kernel(const int *__restrict__ rowPtr, const float *in, float *out, int M, float *__restrict__ ws)
{
    __shared__ int s_long[16];    // rows of this workgroup left to the long-row loop
    __shared__ int s_nlong;
    __shared__ float s_red[4];    // one slot per wavefront
    const float NEG = PSP_SOFTMAX_NEG;
    if (threadIdx.x == 0) s_nlong = 0;
    __syncthreads();

    const int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int sub = threadIdx.x & 15;
    int lb = 0, hb = 0;
    if (row < M) {
        lb = rowPtr[row];
        hb = rowPtr[row + 1];
    }
    if (hb - lb > PSP_SOFTMAX_LONG) {
        if (WS) {
            if (sub == 0) {
                ws[2 * (size_t)row] = NEG;
                ws[2 * (size_t)row + 1] = 0.0f;
            }
        } else if (sub == 0) {
            s_long[atomicAdd(&s_nlong, 1)] = row;
        }
    } else if (lb < hb) {  // a 16-lane group is uniform here
        // the first 64 entries of the row stay in registers (four independent loads per lane): rows up to that
        // length are read once; longer ones sweep the rest three times
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int p = lb + sub + 16 * j;
            v[j] = p < hb ? in[p] : NEG;
        }
        float mx = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
        for (int p = lb + 64 + sub; p < hb; p += 16) mx = fmaxf(mx, in[p]);
        mx = psp_max16(mx);
        float ex[4], s = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            ex[j] = __expf(v[j] - mx);  // exactly 0 for the padding value
            s += ex[j];
        }
        for (int p = lb + 64 + sub; p < hb; p += 16) s += __expf(in[p] - mx);
        s = psp_group_sum<4>(s);
        const float inv = 1.0f / s;
        // every entry is read and written by the same lane, reads first, so in == out is fine
        for (int p = lb + 64 + sub; p < hb; p += 16) out[p] = __expf(in[p] - mx) * inv;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int p = lb + sub + 16 * j;
            if (p < hb) out[p] = ex[j] * inv;
        }
    }
    if (WS) return;
    __syncthreads();

    const int nlong = s_nlong;  // workgroup-uniform
    for (int i = 0; i < nlong; i++) {
        const int r = s_long[i];
        const int a = rowPtr[r], b = rowPtr[r + 1];
        float mx = NEG;
        for (int p = a + threadIdx.x; p < b; p += 256) mx = fmaxf(mx, in[p]);
        mx = psp_block_max(mx, s_red);
        float s = 0.0f;
        for (int p = a + threadIdx.x; p < b; p += 256) s += __expf(in[p] - mx);
        const float inv = 1.0f / psp_block_sum(s, s_red);
        for (int p = a + threadIdx.x; p < b; p += 256) out[p] = __expf(in[p] - mx) * inv;
    }
}

// PASS 0: row maxima, 1: sums of exp(x - max), 2: results.  One workgroup per chunk of the entry array.
template <int PASS>
__global__ void __launch_bounds__(256)
psp_softmax_long_kernel(const int *__restrict__ rowPtr, const float *in, float *out, int M, int nnz, float *ws)
{
    __shared__ int s_rows[PSP_SOFTMAX_CHUNK / PSP_SOFTMAX_LONG + 4];  // long rows that cross this chunk
    __shared__ int s_n;
    const int c0 = blockIdx.x * PSP_SOFTMAX_CHUNK;
    const int c1 = min(nnz, c0 + PSP_SOFTMAX_CHUNK);
    if (threadIdx.x == 0) s_n = 0;
    __syncthreads();
    // rows that hold entries of [c0, c1): from the first row ending after c0 to the last row starting before c1
    int lo = 0, hi = M;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (rowPtr[mid + 1] > c0) hi = mid; else lo = mid + 1;
    }
    const int r_first = lo;
    hi = M;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (rowPtr[mid] >= c1) hi = mid; else lo = mid + 1;
    }
    const int r_end = lo;  // first row starting at or after c1
    for (int r = r_first + threadIdx.x; r < r_end; r += 256)
        if (rowPtr[r + 1] - rowPtr[r] > PSP_SOFTMAX_LONG) s_rows[atomicAdd(&s_n, 1)] = r;
    __syncthreads();
    const int n = s_n;  // workgroup-uniform, at most CHUNK/LONG + 2
    // one wavefront per (row, chunk) intersection
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x >> 6; i < n; i += 4) {
        const int r = s_rows[i];
        const int a = max(rowPtr[r], c0), b = min(rowPtr[r + 1], c1);
        if (PASS == 0) {
            float mx = PSP_SOFTMAX_NEG;
            for (int p = a + lane; p < b; p += 64) mx = fmaxf(mx, in[p]);
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
            if (lane == 0) psp_atomic_max_f32(ws + 2 * (size_t)r, mx);
        } else if (PASS == 1) {
            const float mx = ws[2 * (size_t)r];
            float s = 0.0f;
            for (int p = a + lane; p < b; p += 64) s += __expf(in[p] - mx);
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) s += __shfl_xor(s, d);
            if (lane == 0) atomicAdd(ws + 2 * (size_t)r + 1, s);
        } else {
            const float mx = ws[2 * (size_t)r], inv = 1.0f / ws[2 * (size_t)r + 1];
            for (int p = a + lane; p < b; p += 64) out[p] = __expf(in[p] - mx) * inv;
        }
    }
}

PSP_EXPORT int psp_segment_softmax_f32(const int *rowPtr, const float *in, float *out, int M, psp_stream_t stream)
{
    PSP_REQUIRE(M >= 0, "segment_softmax: negative row count");
    if (M == 0) return PSP_OK;
    PSP_REQUIRE(rowPtr && in && out, "segment_softmax: null pointer");
    hipLaunchKernelGGL(psp_segment_softmax_kernel<false>, dim3(psp_ceil_div((long long)M * 16, 256)), dim3(256), 0,
                       (hipStream_t)stream, rowPtr, in, out, M, (float *)nullptr);
    return psp_check_launch("segment softmax kernel");
}

PSP_EXPORT int psp_segment_softmax_ws_f32(const int *rowPtr, const float *in, float *out, int M, int nnz,
                                          float *workspace, psp_stream_t stream)
{
    PSP_REQUIRE(M >= 0 && nnz >= 0, "segment_softmax_ws: negative size");
    if (M == 0 || nnz == 0) return PSP_OK;
    PSP_REQUIRE(rowPtr && in && out && workspace, "segment_softmax_ws: null pointer");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(psp_segment_softmax_kernel<true>, dim3(psp_ceil_div((long long)M * 16, 256)), dim3(256), 0, st,
                       rowPtr, in, out, M, workspace);
    const dim3 grid(psp_ceil_div(nnz, PSP_SOFTMAX_CHUNK));
    hipLaunchKernelGGL(psp_softmax_long_kernel<0>, grid, dim3(256), 0, st, rowPtr, in, out, M, nnz, workspace);
    hipLaunchKernelGGL(psp_softmax_long_kernel<1>, grid, dim3(256), 0, st, rowPtr, in, out, M, nnz, workspace);
    hipLaunchKernelGGL(psp_softmax_long_kernel<2>, grid, dim3(256), 0, st, rowPtr, in, out, M, nnz, workspace);
    return psp_check_launch("segment softmax kernels");
}

// ------------------------------------------------------------------------------------------------
// The same softmax for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that
// forbid hipMalloc): the (max, sum) pairs of the long rows live in a fixed array inside the library's device image
// instead of a caller's workspace.  Every GPU holds its own copy of the array at its own address, so the address
// is looked up once per device (hipGetSymbolAddress, no allocation) and the kernels receive it as an argument like
// any workspace.  In host code the array's name is only a handle for that lookup, never a device address.
// ------------------------------------------------------------------------------------------------
#define PSP_STATIC_SOFTMAX_MAX_ROWS PSP_SEGMENT_SOFTMAX_STATIC_MAX_ROWS  // include/paramsp.h
#define PSP_MAX_DEVICES 64
static __device__ __align__(256) float psp_softmax_scratch[2 * PSP_STATIC_SOFTMAX_MAX_ROWS];  // 16 MiB per GPU
static float *g_softmax_scratch[PSP_MAX_DEVICES];  // device address of the array on each GPU, null = not looked up
static std::mutex g_softmax_scratch_lock;

static int psp_softmax_scratch_ptr(float **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return psp_fail(PSP_ERR_LAUNCH, "segment_softmax_static: hipGetDevice: %s", hipGetErrorString(e));
    PSP_REQUIRE(dev >= 0 && dev < PSP_MAX_DEVICES, "segment_softmax_static: device %d outside 0..%d", dev, PSP_MAX_DEVICES - 1);
    std::lock_guard<std::mutex> hold(g_softmax_scratch_lock);
    if (!g_softmax_scratch[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(psp_softmax_scratch));
        if (e != hipSuccess || !p)
            return psp_fail(PSP_ERR_LAUNCH, "segment_softmax_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
        g_softmax_scratch[dev] = (float *)p;
    }
    *out = g_softmax_scratch[dev];
    return PSP_OK;
}

PSP_EXPORT int psp_segment_softmax_static_f32(const int *rowPtr, const float *in, float *out, int M, int nnz,
                                              psp_stream_t stream)
{
    PSP_REQUIRE(M >= 0 && nnz >= 0, "segment_softmax_static: negative size");
    PSP_REQUIRE(M <= PSP_STATIC_SOFTMAX_MAX_ROWS,
                "segment_softmax_static: %d rows exceed the built-in scratch of %d rows; use psp_segment_softmax_ws_f32", M,
                PSP_STATIC_SOFTMAX_MAX_ROWS);
    // The address lookup of the first call on a device is host work that does not belong under stream capture: an
    // empty call (M = 0) performs it and launches nothing, which is how a caller prepares a device before capturing.
    float *scratch = nullptr;
    const int rc = psp_softmax_scratch_ptr(&scratch);
    if (rc != PSP_OK) return rc;
    if (M == 0 || nnz == 0) return PSP_OK;
    PSP_REQUIRE(rowPtr && in && out, "segment_softmax_static: null pointer");
    // Nothing has to start at zero: the first kernel resets the pair of every long row of this call, and pairs of
    // other rows (left by earlier calls) are never read.
    return psp_segment_softmax_ws_f32(rowPtr, in, out, M, nnz, scratch, stream);
}

PSP_EXPORT int psp_sddmm_vec_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *A,
                                 const float *B, float *out, int Mb, int K, int vec_size, int blkWarpNum,
                                 psp_stream_t stream)
{
    if (vec_size == 2)
        return psp_sddmm_launch<2, false>(rowPtr_b, colIdx_b, val_b, nullptr, A, B, nullptr, out, Mb, K, blkWarpNum,
                                          (hipStream_t)stream, nullptr);
    PSP_REQUIRE(vec_size == 3, "sddmm_vec: block height %d is not built (2 and 3 are)", vec_size);
    return psp_sddmm_launch<3, false>(rowPtr_b, colIdx_b, val_b, nullptr, A, B, nullptr, out, Mb, K, blkWarpNum,
                                      (hipStream_t)stream, nullptr);
}

PSP_EXPORT int psp_sddmm_vec_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                                       const int *target_row, const float *A, const float *B, float *out, int Sb,
                                       int K, int vec_size, int blkWarpNum, psp_stream_t stream)
{
    if (vec_size == 2)
        return psp_sddmm_launch<2, true>(rowPtr_bs, colIdx_b, val_b, target_row, A, B, nullptr, out, Sb, K, blkWarpNum,
                                         (hipStream_t)stream, nullptr);
    PSP_REQUIRE(vec_size == 3, "sddmm_vec_split: block height %d is not built (2 and 3 are)", vec_size);
    return psp_sddmm_launch<3, true>(rowPtr_bs, colIdx_b, val_b, target_row, A, B, nullptr, out, Sb, K, blkWarpNum,
                                     (hipStream_t)stream, nullptr);
}

// ------------------------------------------------------------------------------------------------
// host: row split (SpMM/SpMM.cpp:15-75)
// ------------------------------------------------------------------------------------------------
PSP_EXPORT int psp_split_csr_count(const int *rowPtr, int nrows, int g)
{
    PSP_REQUIRE(rowPtr && nrows >= 0, "split_csr: bad rowPtr / nrows");
    PSP_REQUIRE(g >= 1, "split_csr: granularity must be positive (got %d)", g);
    long long S = 0;
    for (int i = 0; i < nrows; i++) {
        const int k = rowPtr[i + 1] - rowPtr[i];
        PSP_REQUIRE(k >= 0, "split_csr: rowPtr decreases at row %d", i);
        S += (k + g - 1) / g;
    }
    if (S > 0x7fffffffLL) return psp_fail(PSP_ERR_RANGE, "split_csr: %lld segments do not fit int32", S);
    return (int)S;
}

static void split_rows(const int *rowPtr, int r0, int r1, int g, int off, int *rowPtr_split, int *target_row)
{
    for (int i = r0; i < r1; i++) {
        const int hb = rowPtr[i + 1];
        for (int lb = rowPtr[i]; lb < hb; lb += g) {
            target_row[off] = i;
            rowPtr_split[off + 1] = std::min(lb + g, hb);
            off++;
        }
    }
}

PSP_EXPORT int psp_split_csr(const int *rowPtr, int nrows, int g, int *rowPtr_split, int *target_row)
{
    const int S = psp_split_csr_count(rowPtr, nrows, g);
    if (S < 0) return S;
    PSP_REQUIRE(rowPtr_split && (target_row || S == 0), "split_csr: null output");
    rowPtr_split[0] = 0;
    split_rows(rowPtr, 0, nrows, g, 0, rowPtr_split, target_row);
    return S;
}

PSP_EXPORT int psp_split_csr_par(const int *rowPtr, const int *row_split_offset, int nrows, int g,
                                 int *rowPtr_split, int *target_row)
{
    PSP_REQUIRE(rowPtr && row_split_offset && nrows >= 0, "split_csr_par: bad input");
    PSP_REQUIRE(g >= 1, "split_csr_par: granularity must be positive (got %d)", g);
    const int S = row_split_offset[nrows];
    PSP_REQUIRE(S >= 0 && rowPtr_split && (target_row || S == 0), "split_csr_par: bad output");
    // the offsets must be the exclusive prefix of ceil(nnz_i / g): rows write disjoint ranges only then
    for (int i = 0; i < nrows; i++) {
        const int k = rowPtr[i + 1] - rowPtr[i];
        PSP_REQUIRE(k >= 0 && row_split_offset[i + 1] - row_split_offset[i] == (k + g - 1) / g,
                    "split_csr_par: row_split_offset is not the prefix sum of ceil(nnz/g) at row %d", i);
    }
    rowPtr_split[0] = 0;
    unsigned hw = std::thread::hardware_concurrency();
    int nthreads = (int)std::min<unsigned>(hw ? hw : 1, 16);
    if (nrows < (1 << 16)) nthreads = 1;
    if (nthreads <= 1) {
        split_rows(rowPtr, 0, nrows, g, 0, rowPtr_split, target_row);
        return S;
    }
    std::vector<std::thread> pool;
    const int per = (nrows + nthreads - 1) / nthreads;
    for (int t = 0; t < nthreads; t++) {
        const int r0 = std::min(nrows, t * per), r1 = std::min(nrows, r0 + per);
        if (r0 == r1) continue;
        pool.emplace_back(split_rows, rowPtr, r0, r1, g, row_split_offset[r0], rowPtr_split, target_row);
    }
    for (auto &th : pool) th.join();
    return S;
}

// ------------------------------------------------------------------------------------------------
// host: BCSR 2x1 in first-encounter block order (what SciPy's tobsr produces, graph_input.py:245-256)
// ------------------------------------------------------------------------------------------------
static int bcsr_walk(const int *rowPtr, const int *colIdx, const float *val, int nrows, int ncols,
                     int *rowPtr_b, int *colIdx_b, float *val_b, int R = 2)
{
    const int nbr = (nrows + R - 1) / R;
    std::vector<int> slot((size_t)std::max(ncols, 1), -1);
    long long nblk = 0;
    if (rowPtr_b) rowPtr_b[0] = 0;
    for (int t = 0; t < nbr; t++) {
        const long long first = nblk;
        for (int k = 0; k < R; k++) {
            const int r = R * t + k;
            if (r >= nrows) break;
            for (int p = rowPtr[r]; p < rowPtr[r + 1]; p++) {
                const int c = colIdx[p];
                if (c < 0 || c >= ncols) return psp_fail(PSP_ERR_ARG, "bcsr: column %d out of range at entry %d", c, p);
                if (slot[c] < first) {
                    if (nblk >= 0x7fffffffLL / R) return psp_fail(PSP_ERR_RANGE, "bcsr: block count overflows int32");
                    slot[c] = (int)nblk;
                    if (colIdx_b) {
                        colIdx_b[nblk] = c;
                        for (int q = 0; q < R; q++) val_b[(size_t)R * nblk + q] = 0.0f;
                    }
                    nblk++;
                }
                if (colIdx_b) val_b[(size_t)R * slot[c] + k] += val[p];
            }
        }
        if (rowPtr_b) rowPtr_b[t + 1] = (int)nblk;
    }
    return (int)nblk;
}

PSP_EXPORT int psp_bcsr_count(const int *rowPtr, const int *colIdx, int nrows, int ncols)
{
    PSP_REQUIRE(rowPtr && nrows >= 0 && ncols >= 0, "bcsr_count: bad input");
    PSP_REQUIRE(colIdx || rowPtr[nrows] == 0, "bcsr_count: colIdx is null");
    return bcsr_walk(rowPtr, colIdx, nullptr, nrows, ncols, nullptr, nullptr, nullptr);
}

PSP_EXPORT int psp_bcsr_build(const int *rowPtr, const int *colIdx, const float *val, int nrows, int ncols,
                              int *rowPtr_b, int *colIdx_b, float *val_b)
{
    PSP_REQUIRE(rowPtr && nrows >= 0 && ncols >= 0 && rowPtr_b, "bcsr_build: bad input");
    const bool empty = rowPtr[nrows] == 0;
    PSP_REQUIRE(empty || (colIdx && val && colIdx_b && val_b), "bcsr_build: null pointer");
    if (empty) {
        for (int t = 0; t <= (nrows + 1) / 2; t++) rowPtr_b[t] = 0;
        return 0;
    }
    return bcsr_walk(rowPtr, colIdx, val, nrows, ncols, rowPtr_b, colIdx_b, val_b);
}

PSP_EXPORT int psp_vbsr_count(const int *rowPtr, const int *colIdx, int nrows, int ncols, int R)
{
    PSP_REQUIRE(rowPtr && nrows >= 0 && ncols >= 0, "vbsr_count: bad input");
    PSP_REQUIRE(R >= 1 && R <= 8, "vbsr_count: block height %d out of range (1..8)", R);
    PSP_REQUIRE(colIdx || rowPtr[nrows] == 0, "vbsr_count: colIdx is null");
    return bcsr_walk(rowPtr, colIdx, nullptr, nrows, ncols, nullptr, nullptr, nullptr, R);
}

PSP_EXPORT int psp_vbsr_build(const int *rowPtr, const int *colIdx, const float *val, int nrows, int ncols, int R,
                              int *rowPtr_b, int *colIdx_b, float *val_b)
{
    PSP_REQUIRE(rowPtr && nrows >= 0 && ncols >= 0 && rowPtr_b, "vbsr_build: bad input");
    PSP_REQUIRE(R >= 1 && R <= 8, "vbsr_build: block height %d out of range (1..8)", R);
    const bool empty = rowPtr[nrows] == 0;
    PSP_REQUIRE(empty || (colIdx && val && colIdx_b && val_b), "vbsr_build: null pointer");
    if (empty) {
        for (int t = 0; t <= (nrows + R - 1) / R; t++) rowPtr_b[t] = 0;
        return 0;
    }
    return bcsr_walk(rowPtr, colIdx, val, nrows, ncols, rowPtr_b, colIdx_b, val_b, R);
}

// ------------------------------------------------------------------------------------------------
// device entry points
// ------------------------------------------------------------------------------------------------
PSP_EXPORT int psp_spmm_csr_f32(const int *rowPtr, const int *colIdx, const float *val, const float *X, float *Y,
                                int M, int N, int rows_out, int CF, int blkWarpNum, psp_stream_t stream)
{
    return psp_spmm_launch<1, false>(rowPtr, colIdx, val, nullptr, X, Y, M, N, rows_out, CF, blkWarpNum,
                                         (hipStream_t)stream, nullptr, nullptr);
}

PSP_EXPORT int psp_spmm_csr_softmax_f32(const int *rowPtr, const int *colIdx, const float *e, const float *row_max,
                                        const float *X, float *Y, int M, int N, int rows_out, int CF, int blkWarpNum,
                                        psp_stream_t stream)
{
    PSP_REQUIRE(row_max || M == 0, "spmm softmax: row_max is null");
    return psp_spmm_launch<1, false>(rowPtr, colIdx, e, nullptr, X, Y, M, N, rows_out, CF, blkWarpNum,
                                     (hipStream_t)stream, row_max, nullptr);
}

PSP_EXPORT int psp_spmm_csr_split_f32(const int *rowPtr_split, const int *colIdx, const float *val,
                                      const int *target_row, const float *X, float *Y, int S, int N, int rows_out,
                                      int CF, int blkWarpNum, psp_stream_t stream)
{
    return psp_spmm_launch<1, true>(rowPtr_split, colIdx, val, target_row, X, Y, S, N, rows_out, CF, blkWarpNum,
                                        (hipStream_t)stream, nullptr, nullptr);
}

PSP_EXPORT int psp_spmm_csr_split_softmax_f32(const int *rowPtr_split, const int *colIdx, const float *e,
                                              const int *target_row, const float *row_max, float *row_sum,
                                              const float *X, float *Y, int S, int N, int rows_out, int CF,
                                              int blkWarpNum, psp_stream_t stream)
{
    PSP_REQUIRE(row_max || S == 0, "spmm softmax: row_max is null");
    return psp_spmm_launch<1, true>(rowPtr_split, colIdx, e, target_row, X, Y, S, N, rows_out, CF, blkWarpNum,
                                    (hipStream_t)stream, row_max, row_sum);
}

PSP_EXPORT int psp_spmm_bcsr_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *X,
                                 float *Y, int Mb, int N, int rows_out, int CF, int blkWarpNum, psp_stream_t stream)
{
    return psp_spmm_launch<2, false>(rowPtr_b, colIdx_b, val_b, nullptr, X, Y, Mb, N, rows_out, CF, blkWarpNum,
                                        (hipStream_t)stream, nullptr, nullptr);
}

PSP_EXPORT int psp_spmm_bcsr_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                                       const int *target_row, const float *X, float *Y, int Sb, int N,
                                       int rows_out, int CF, int blkWarpNum, psp_stream_t stream)
{
    return psp_spmm_launch<2, true>(rowPtr_bs, colIdx_b, val_b, target_row, X, Y, Sb, N, rows_out, CF, blkWarpNum,
                                       (hipStream_t)stream, nullptr, nullptr);
}

PSP_EXPORT int psp_spmm_vec_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *X, float *Y,
                                int Mb, int N, int rows_out, int vec_size, int CF, int blkWarpNum, psp_stream_t stream)
{
    if (vec_size == 2)
        return psp_spmm_launch<2, false>(rowPtr_b, colIdx_b, val_b, nullptr, X, Y, Mb, N, rows_out, CF, blkWarpNum,
                                         (hipStream_t)stream, nullptr, nullptr);
    PSP_REQUIRE(vec_size == 3, "spmm_vec: block height %d is not built (2 and 3 are)", vec_size);
    return psp_spmm_launch<3, false>(rowPtr_b, colIdx_b, val_b, nullptr, X, Y, Mb, N, rows_out, CF, blkWarpNum,
                                     (hipStream_t)stream, nullptr, nullptr);
}

PSP_EXPORT int psp_spmm_vec_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                                      const int *target_row, const float *X, float *Y, int Sb, int N, int rows_out,
                                      int vec_size, int CF, int blkWarpNum, psp_stream_t stream)
{
    if (vec_size == 2)
        return psp_spmm_launch<2, true>(rowPtr_bs, colIdx_b, val_b, target_row, X, Y, Sb, N, rows_out, CF, blkWarpNum,
                                        (hipStream_t)stream, nullptr, nullptr);
    PSP_REQUIRE(vec_size == 3, "spmm_vec_split: block height %d is not built (2 and 3 are)", vec_size);
    return psp_spmm_launch<3, true>(rowPtr_bs, colIdx_b, val_b, target_row, X, Y, Sb, N, rows_out, CF, blkWarpNum,
                                    (hipStream_t)stream, nullptr, nullptr);
}

// Y[i] = Y[i] where mask[i] > 0, else 0 (float4 pieces; n a multiple of 4 is not required)
__global__ void __launch_bounds__(256) psp_mask_kernel(float *__restrict__ Y, const float *__restrict__ mask, size_t n)
{
    const size_t n4 = n / 4;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        psp_f32x4 y = ((const psp_f32x4 *)Y)[i];
        const psp_f32x4 m = __builtin_nontemporal_load((const psp_f32x4 *)mask + i);
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = m[e] > 0.0f ? y[e] : 0.0f;
        ((psp_f32x4 *)Y)[i] = y;
    }
    const size_t t = n4 * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n) Y[t] = mask[t] > 0.0f ? Y[t] : 0.0f;
}

PSP_EXPORT int psp_spmm_act_f32(int fmt, const int *rowPtr, const int *colIdx, const float *val, const int *target_row,
                                const float *X, float *Y, int nseg, int N, int rows_out, int CF, int blkWarpNum,
                                int relu_x, const float *mask, psp_stream_t stream)
{
    PSP_REQUIRE(fmt >= 0 && fmt <= 3, "spmm_act: format code %d (0 csr, 1 csr_split, 2 bcsr, 3 bcsr_split)", fmt);
    PSP_REQUIRE(((fmt & 1) != 0) == (target_row != nullptr) || nseg == 0, "spmm_act: target_row and the format code disagree");
    PSP_REQUIRE((((size_t)mask | (size_t)Y) & 15) == 0, "spmm_act: Y and mask must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const int rx = relu_x != 0;
    int rc;
    switch (fmt) {
    case 0: rc = psp_spmm_launch<1, false>(rowPtr, colIdx, val, nullptr, X, Y, nseg, N, rows_out, CF, blkWarpNum, st, nullptr, nullptr, rx); break;
    case 1: rc = psp_spmm_launch<1, true>(rowPtr, colIdx, val, target_row, X, Y, nseg, N, rows_out, CF, blkWarpNum, st, nullptr, nullptr, rx); break;
    case 2: rc = psp_spmm_launch<2, false>(rowPtr, colIdx, val, nullptr, X, Y, nseg, N, rows_out, CF, blkWarpNum, st, nullptr, nullptr, rx); break;
    default: rc = psp_spmm_launch<2, true>(rowPtr, colIdx, val, target_row, X, Y, nseg, N, rows_out, CF, blkWarpNum, st, nullptr, nullptr, rx); break;
    }
    if (rc != PSP_OK || mask == nullptr) return rc;
    // The mask is a pass of its own over Y (see spmm_kernel.h: applied where the kernel closes a row it was slower).
    const size_t n = (size_t)rows_out * (size_t)N;
    if (n == 0) return PSP_OK;
    const size_t want = (n / 4 + 255) / 256 + 1;
    hipLaunchKernelGGL(psp_mask_kernel, dim3((unsigned)std::min<size_t>(want, 256 * 32)), dim3(256), 0, st, Y, mask, n);
    return psp_check_launch("mask pass");
}

PSP_EXPORT int psp_sddmm_csr_f32(const int *rowPtr, const int *colIdx, const float *A, const float *B,
                                 const float *scale, float *out, int M, int K, int blkWarpNum, psp_stream_t stream)
{
    return psp_sddmm_launch<1, false>(rowPtr, colIdx, nullptr, nullptr, A, B, scale, out, M, K, blkWarpNum,
                                          (hipStream_t)stream, nullptr);
}

PSP_EXPORT int psp_sddmm_csr_rowmax_f32(const int *rowPtr, const int *colIdx, const float *A, const float *B,
                                        const float *scale, float *out, float *row_max, int M, int K, int blkWarpNum,
                                        psp_stream_t stream)
{
    PSP_REQUIRE(M >= 0 && (row_max || M == 0), "sddmm rowmax: row_max is null");
    int rc = psp_fill_f32(row_max, (size_t)M, PSP_F32_LOWEST, (hipStream_t)stream);
    if (rc != PSP_OK) return rc;
    return psp_sddmm_launch<1, false>(rowPtr, colIdx, nullptr, nullptr, A, B, scale, out, M, K, blkWarpNum,
                                          (hipStream_t)stream, row_max);
}

PSP_EXPORT int psp_sddmm_csr_split_f32(const int *rowPtr_split, const int *colIdx, const int *target_row,
                                       const float *A, const float *B, const float *scale, float *out, int S,
                                       int K, int blkWarpNum, psp_stream_t stream)
{
    return psp_sddmm_launch<1, true>(rowPtr_split, colIdx, nullptr, target_row, A, B, scale, out, S, K,
                                         blkWarpNum, (hipStream_t)stream, nullptr);
}

PSP_EXPORT int psp_sddmm_csr_split_rowmax_f32(const int *rowPtr_split, const int *colIdx, const int *target_row,
                                              const float *A, const float *B, const float *scale, float *out,
                                              float *row_max, int S, int rows, int K, int blkWarpNum,
                                              psp_stream_t stream)
{
    PSP_REQUIRE(rows >= 0 && (row_max || rows == 0), "sddmm rowmax: row_max is null");
    int rc = psp_fill_f32(row_max, (size_t)rows, PSP_F32_LOWEST, (hipStream_t)stream);
    if (rc != PSP_OK) return rc;
    return psp_sddmm_launch<1, true>(rowPtr_split, colIdx, nullptr, target_row, A, B, scale, out, S, K,
                                         blkWarpNum, (hipStream_t)stream, row_max);
}

PSP_EXPORT int psp_sddmm_bcsr_f32(const int *rowPtr_b, const int *colIdx_b, const float *val_b, const float *A,
                                  const float *B, float *out, int Mb, int K, int blkWarpNum, psp_stream_t stream)
{
    return psp_sddmm_launch<2, false>(rowPtr_b, colIdx_b, val_b, nullptr, A, B, nullptr, out, Mb, K, blkWarpNum,
                                         (hipStream_t)stream, nullptr);
}

PSP_EXPORT int psp_sddmm_bcsr_split_f32(const int *rowPtr_bs, const int *colIdx_b, const float *val_b,
                                        const int *target_row, const float *A, const float *B, float *out, int Sb,
                                        int K, int blkWarpNum, psp_stream_t stream)
{
    return psp_sddmm_launch<2, true>(rowPtr_bs, colIdx_b, val_b, target_row, A, B, nullptr, out, Sb, K,
                                        blkWarpNum, (hipStream_t)stream, nullptr);
}
