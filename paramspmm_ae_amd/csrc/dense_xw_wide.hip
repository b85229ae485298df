// Y[n,K2] = X[n,K1] * W  or  X * W^T  for tall-skinny X and a weight matrix of 64 or 128 output columns: the dense
// products of the wide GCN / GIN layers (torch::mm(H, W) and torch::mm(AG, W.t()) in SpCONV/SpCONV.h:43-71), with the
// ReLU between two layers folded in like the narrow kernel of dense_xw.hip does.  At 128 x 128 the product is 32 kflop
// per row against 1 KB of traffic: matrix-core time and memory time are about equal, so this one runs on the matrix
// cores (v_mfma_f32_16x16x4_f32, fp32 in, fp32 accumulate).
//
// The product is formed transposed, Y^T = W^T X^T, so that a lane ends up with consecutive elements of one output row:
//   * MFMA operand B (4 x 16) is a piece of X^T: lane (r, q) = (lane % 16, lane / 16) supplies X[row r][k]; it loads
//     its row 16 bytes at a time, float4 t covering columns 16t + 4q .. 16t + 4q + 3, so the four q-lanes of a row
//     read 64 contiguous bytes.  Element e of float4 t is used in contraction step (t, e), where the lane's column
//     16t + 4q + e stands for index k = q of the instruction: which four columns a step contracts is free as long as
//     operand A follows the same rule;
//   * operand A (16 x 4) is a piece of W^T read from LDS: lane (r, q) supplies W[16t + 4q + e][16j + r] for column
//     tile j (T = K2 / 16 tiles).  LDS holds the columns of W permuted -- column 16j + r at position
//     ((j / 4) * 16 + r) * 4 + j % 4 -- so a lane fetches four tiles with one 16-byte read and the sixteen r-lanes of
//     such a read cover 256 contiguous bytes (no bank conflicts): two reads per step serve eight MFMAs (sixteen with
//     the two row blocks a wavefront works on);
//   * result lane (r, q), tile j, element i is Y[row r][16j + 4q + i]: one 16-byte store per tile, the four q-lanes
//     of a row writing 64 contiguous bytes.
// W (K1 rows of K2 + 4 floats: 66 KB at 128 x 128) is staged into LDS once per workgroup, transposed on the way in for
// the X * W^T form.  That is more than the 64 KB a workgroup gets on earlier CDNA parts: the kernel is built for
// gfx950 only, whose CUs have 160 KB, and two workgroups per CU (the launch shape) need 132 KB of it.  The grid is sized
// to the GPU and every wavefront walks blocks of 32 rows with the next block's loads in flight.
#include "psp_common.h"
#include "bf16_split.h"
#include <cstdlib>

typedef float psp_f32x4 __attribute__((ext_vector_type(4)));

#define XWW_ROWS 32  // rows per wavefront and step: two MFMA row blocks share every operand read from LDS

template <int K1, int K2, bool RELU_X, bool MASK>
// (the bound of 512 lanes leaves the register allocator 256 registers per lane; launched with 256)
__global__ void __launch_bounds__(512)
psp_xw_wide_kernel(const float *__restrict__ X, const float *__restrict__ W, float *__restrict__ Y, long long n,
                   const float *__restrict__ mask, int transW, long long nblocks)
{
    constexpr int T = K2 / 16;   // column tiles
    constexpr int KT = K1 / 16;  // float4 loads per lane and row block
    constexpr int S = K2 + 4;    // LDS row stride: the four k-rows a step reads fall into different bank halves
    static_assert(T % 4 == 0 && K1 % 16 == 0, "widths: K2 a multiple of 64, K1 a multiple of 16");  // T % 4: 16-byte LDS reads
    // two workgroups share a CU's 160 KB of LDS
    static_assert(sizeof(float) * K1 * S <= 80 * 1024, "W does not fit half of a gfx950 CU's LDS");
    __shared__ float Ws[K1 * S];

    for (int idx = threadIdx.x; idx < K1 * K2; idx += blockDim.x) {
        int k, c;
        if (transW) {  // W is [K2, K1]
            c = idx / K1;
            k = idx - c * K1;
        } else {  // W is [K1, K2]
            k = idx / K2;
            c = idx - k * K2;
        }
        Ws[k * S + (((c >> 6) * 16 + (c & 15)) << 2) + ((c >> 4) & 3)] = W[idx];
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int waves = blockDim.x >> 6;
    const long long stride = (long long)gridDim.x * waves;
    long long blk = (long long)blockIdx.x * waves + wave;
    if (blk >= nblocks) return;

    psp_f32x4 xa[2][KT], xb[2][KT];
    auto load_block = [&](long long b, psp_f32x4 (&x)[2][KT]) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            long long row = b * XWW_ROWS + 16 * h + r;
            if (row >= n) row = n - 1;  // loaded and computed, never stored
            const psp_f32x4 *xr = (const psp_f32x4 *)(X + row * K1) + q;
#pragma unroll
            for (int t = 0; t < KT; t++) x[h][t] = xr[4 * t];
        }
    };
    auto compute_block = [&](long long b, psp_f32x4 (&x)[2][KT]) {
        if constexpr (RELU_X) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int e = 0; e < 4; e++) x[h][t][e] = x[h][t][e] < 0.0f ? 0.0f : x[h][t][e];  // NaN stays NaN
        }
        psp_f32x4 acc[2][T];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < T; j++) acc[h][j] = psp_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < KT; t++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const psp_f32x4 *wr = (const psp_f32x4 *)(Ws + (16 * t + 4 * q + e) * S) + r;
                psp_f32x4 a4[T / 4];
#pragma unroll
                for (int v = 0; v < T / 4; v++) a4[v] = wr[16 * v];
#pragma unroll
                for (int j = 0; j < T; j++) {
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j / 4][j % 4], x[h][t][e], acc[h][j], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const long long row = b * XWW_ROWS + 16 * h + r;
            if (row >= n) continue;
            psp_f32x4 *yr = (psp_f32x4 *)(Y + row * K2) + q;
            const psp_f32x4 *mr = (const psp_f32x4 *)(mask + row * K2) + q;
#pragma unroll
            for (int j = 0; j < T; j++) {
                psp_f32x4 o = acc[h][j];
                if constexpr (MASK) {
                    const psp_f32x4 m = mr[4 * j];
#pragma unroll
                    for (int c = 0; c < 4; c++) o[c] = m[c] > 0.0f ? o[c] : 0.0f;
                }
                yr[4 * j] = o;
            }
        }
    };

    // two register sets alternate: the next block's rows are requested before the current block is multiplied
    load_block(blk, xa);
    while (true) {
        long long nxt = blk + stride;
        if (nxt < nblocks) load_block(nxt, xb);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(blk, xa);
        if (nxt >= nblocks) break;
        blk = nxt;
        nxt = blk + stride;
        if (nxt < nblocks) load_block(nxt, xa);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(blk, xb);
        if (nxt >= nblocks) break;
        blk = nxt;
    }
}

// ---- the 128 x 128 product on the bf16 matrix-core path -----------------------------------------------------------------
// At 128 x 128 the fp32 instruction above needs as long for its 32 kflop per row as the memory system needs for the row's
// 1 KB.  gfx950 multiplies bf16 sixteen times as fast, and an fp32 number is the exact sum of three bf16 numbers
// (x = hi + mid + lo, 8 + 8 + 8 significant bits), so x w = sum of nine bf16 products, of which the six with at least
// 16 significant bits between them (hi hi, hi mid, mid hi, mid mid, hi lo, lo hi) carry the product to 2^-23 of |x||w|
// -- the rounding level of an fp32 product -- and are accumulated in fp32 by v_mfma_f32_16x16x32_bf16.  Six instructions
// of 16 cycles replace eight of 32: the kernel is bound by its 1 KB per row again.  Same transposed form and the same
// lane roles as above; a contraction step covers 32 columns: lane (r, q) supplies the eight values of its float4 pair
// (2s, 2s + 1), i.e. columns 32s + 16 (i / 4) + 4q + i % 4 stand for k = 8q + i, and the W fragments in LDS follow the same
// rule: [s][tile j][hi | mid | lo][lane][8 bf16], one 16-byte read per fragment.  An infinite input turns its products
// into NaN (inf - inf in the split) instead of +-inf; NaN stays NaN.

template <bool RELU_X, bool MASK>
__global__ void __launch_bounds__(512)
psp_xw_wide_split_kernel(const float *__restrict__ X, const float *__restrict__ W, float *__restrict__ Y, long long n,
                         const float *__restrict__ mask, int transW, long long nblocks)
{
    constexpr int K1 = 128, K2 = 128;
    constexpr int T = K2 / 16;   // column tiles
    constexpr int KT = K1 / 16;  // float4 loads per lane and row block
    constexpr int KS = K1 / 32;  // contraction steps
    extern __shared__ __align__(16) unsigned short Wb[];  // [KS][T][3][64][8]

    for (int idx = threadIdx.x; idx < K1 * K2; idx += blockDim.x) {
        const int i = idx & 7, l = (idx >> 3) & 63, sj = idx >> 9;  // sj = s * T + j
        const int j = sj % T, st = sj / T;
        const int r_ = l & 15, q_ = l >> 4;
        const int k = 32 * st + 16 * (i >> 2) + 4 * q_ + (i & 3), c = 16 * j + r_;
        const float w = transW ? W[c * K1 + k] : W[k * K2 + c];
        unsigned hi, mid, lo;
        psp_split3(w, 0.0f, hi, mid, lo);
        unsigned short *at = Wb + ((size_t)(sj * 3) * 64 + l) * 8 + i;
        at[0] = (unsigned short)hi;
        at[64 * 8] = (unsigned short)mid;
        at[2 * 64 * 8] = (unsigned short)lo;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int waves = blockDim.x >> 6;
    const long long stride = (long long)gridDim.x * waves;
    long long blk = (long long)blockIdx.x * waves + wave;
    if (blk >= nblocks) return;

    psp_f32x4 xa[2][KT], xb[2][KT];
    auto load_block = [&](long long b, psp_f32x4 (&x)[2][KT]) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            long long row = b * XWW_ROWS + 16 * h + r;
            if (row >= n) row = n - 1;  // loaded and computed, never stored
            const psp_f32x4 *xr = (const psp_f32x4 *)(X + row * K1) + q;
#pragma unroll
            for (int t = 0; t < KT; t++) x[h][t] = xr[4 * t];
        }
    };
    auto compute_block = [&](long long b, psp_f32x4 (&x)[2][KT]) {
        psp_f32x4 acc[2][T];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < T; j++) acc[h][j] = psp_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < KS; st++) {
            psp_u32x4 xh[2], xm[2], xl[2];
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float a = x[h][2 * st + (g >> 1)][2 * (g & 1)], c = x[h][2 * st + (g >> 1)][2 * (g & 1) + 1];
                    if constexpr (RELU_X) {
                        a = a < 0.0f ? 0.0f : a;  // NaN stays NaN
                        c = c < 0.0f ? 0.0f : c;
                    }
                    unsigned h_, m_, l_;
                    psp_split3(a, c, h_, m_, l_);
                    xh[h][g] = h_, xm[h][g] = m_, xl[h][g] = l_;
                }
            const psp_u32x4 *wf = (const psp_u32x4 *)Wb + (size_t)(st * T * 3) * 64 + lane;
#pragma unroll
            for (int jp = 0; jp < T; jp += 2) {
                psp_u32x4 w[2][3];
#pragma unroll
                for (int u = 0; u < 2; u++)
#pragma unroll
                    for (int p = 0; p < 3; p++) w[u][p] = wf[((jp + u) * 3 + p) * 64];
                // small terms first; four independent accumulators between two instructions on the same one
#define XWS_TERM(WP_, XV_)                                                                                          \
    _Pragma("unroll") for (int u = 0; u < 2; u++) _Pragma("unroll") for (int h = 0; h < 2; h++)                       \
        acc[h][jp + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(psp_bf16x8, w[u][WP_]),           \
                                                                 __builtin_bit_cast(psp_bf16x8, XV_[h]), acc[h][jp + u], 0, 0, 0);
                XWS_TERM(2, xh)
                XWS_TERM(0, xl)
                XWS_TERM(1, xm)
                XWS_TERM(1, xh)
                XWS_TERM(0, xm)
                XWS_TERM(0, xh)
#undef XWS_TERM
            }
        }
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const long long row = b * XWW_ROWS + 16 * h + r;
            if (row >= n) continue;
            psp_f32x4 *yr = (psp_f32x4 *)(Y + row * K2) + q;
            const psp_f32x4 *mr = (const psp_f32x4 *)(mask + row * K2) + q;
#pragma unroll
            for (int j = 0; j < T; j++) {
                psp_f32x4 o = acc[h][j];
                if constexpr (MASK) {
                    const psp_f32x4 m = mr[4 * j];
#pragma unroll
                    for (int c = 0; c < 4; c++) o[c] = m[c] > 0.0f ? o[c] : 0.0f;
                }
                yr[4 * j] = o;
            }
        }
    };

    load_block(blk, xa);
    while (true) {
        long long nxt = blk + stride;
        if (nxt < nblocks) load_block(nxt, xb);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(blk, xa);
        if (nxt >= nblocks) break;
        blk = nxt;
        nxt = blk + stride;
        if (nxt < nblocks) load_block(nxt, xa);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(blk, xb);
        if (nxt >= nblocks) break;
        blk = nxt;
    }
}

typedef void (*psp_xw_wide_kernel_t)(const float *, const float *, float *, long long, const float *, int, long long);

static psp_xw_wide_kernel_t xw_wide_lookup(int K1, int K2, bool relu_x, bool mask)
{
#define XWW_CASE(A_, B_)                                                   \
    if (K1 == A_ && K2 == B_) {                                            \
        if (mask) return psp_xw_wide_kernel<A_, B_, false, true>;          \
        return relu_x ? psp_xw_wide_kernel<A_, B_, true, false> : psp_xw_wide_kernel<A_, B_, false, false>; \
    }
    XWW_CASE(16, 64) XWW_CASE(32, 64) XWW_CASE(64, 64) XWW_CASE(128, 64)
    XWW_CASE(16, 128) XWW_CASE(32, 128) XWW_CASE(64, 128) XWW_CASE(128, 128)
#undef XWW_CASE
    return nullptr;
}

bool psp_xw_wide_supported(int K1, int K2)
{
    if (xw_wide_lookup(K1, K2, false, false) == nullptr) return false;
    // the staged W must fit what the device grants one workgroup (160 KB per CU on gfx950)
    static int lds_of[64];  // per device, looked up once (0 = not yet; races write the same value)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    int lds = lds_of[dev];
    if (lds == 0) {
        if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return false;
        lds_of[dev] = lds;
    }
    return (size_t)lds >= sizeof(float) * (size_t)K1 * (size_t)(K2 + 4);
}

// called by psp_gemm_xw_act_f32 for the widths the one-lane-per-row kernel does not cover; arguments are checked there
int psp_xw_wide_launch(const float *X, const float *W, float *Y, long long n, int K1, int K2, int transW, int relu_x,
                       const float *mask, hipStream_t stream)
{
    psp_xw_wide_kernel_t k = xw_wide_lookup(K1, K2, relu_x != 0, mask != nullptr);
    if (!k) return psp_fail(PSP_ERR_ARG, "gemm_xw: unsupported widths %d x %d", K1, K2);
    const long long nblocks = (n + XWW_ROWS - 1) / XWW_ROWS;
    if (K1 == 128 && K2 == 128 && psp_opts().dense_split) {
        psp_xw_wide_kernel_t ks = mask ? psp_xw_wide_split_kernel<false, true>
                                       : (relu_x ? psp_xw_wide_split_kernel<true, false> : psp_xw_wide_split_kernel<false, false>);
        const int lds = (K1 / 32) * (K2 / 16) * 3 * 64 * 16;  // 96 KB: one workgroup of eight wavefronts per CU
        static bool raised[3];
        const int which = mask ? 0 : (relu_x ? 1 : 2);
        if (!raised[which]) {
            const hipError_t e = hipFuncSetAttribute((const void *)ks, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
            if (e != hipSuccess) return psp_fail(PSP_ERR_LAUNCH, "gemm_xw: %d bytes of LDS refused: %s", lds, hipGetErrorString(e));
            raised[which] = true;
        }
        // eight wavefronts per workgroup, one workgroup per CU (measured against four and six: 267 / 278 / 283 us at 10^6 rows)
        const int wv = 8;
        const long long want_s = (nblocks + wv - 1) / wv;
        const int grid_s = (int)(want_s < 256 ? want_s : 256);
        hipLaunchKernelGGL(ks, dim3(grid_s), dim3(64 * wv), lds, stream, X, W, Y, n, mask, transW, nblocks);
        return psp_check_launch("gemm_xw wide split kernel");
    }
    // 4 wavefronts per workgroup, two workgroups per CU (two copies of W in LDS side by side); measured against 6 and 8
    // wavefronts per workgroup and one to four workgroups per CU at 10^6 rows: nothing faster
    const int waves = 4;
    const long long want = (nblocks + waves - 1) / waves;
    const int grid = (int)(want < 512 ? want : 512);
    hipLaunchKernelGGL(k, dim3(grid), dim3(64 * waves), 0, stream, X, W, Y, n, mask, transW, nblocks);
    return psp_check_launch("gemm_xw wide kernel");
}
