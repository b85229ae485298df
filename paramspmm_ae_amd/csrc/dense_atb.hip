// C[K1,K2] = A^T * B for tall-skinny A [n,K1], B [n,K2] (n ~ 10^6, K1,K2 multiples of 16 up to 128): the weight-gradient product
// H^T * (A dY) of the fused GCN layer (SpCONV/SpCONV.h:70 calls torch::mm(H.t(), AG)).  The product is a
// reduction over n with a tiny output; a general GEMM picks tiles for large outputs and runs it 20-40 times
// slower than the memory traffic allows.  HBM-bound up to about 64 x 64: 4 n (K1 + K2) bytes.
// Two kernels:
//   psp_atb_mfma_kernel  the matrix cores (v_mfma_f32_16x16x4_f32) fed straight from coalesced loads, for the shapes
//                        whose accumulators fit a wavefront (or a workgroup's four); partial products either meet in
//                        a caller's workspace and are added by psp_atb_reduce_kernel in a fixed order, or go to C
//                        with atomics.
//   psp_atb_kernel       the remaining shapes: every workgroup streams a band of rows through LDS, keeps a
//                        K1/16 x K2/16 register tile per lane (vector FMAs) and adds its partial product to C with
//                        fp32 atomics.
#include "psp_common.h"
#include "spmm_kernel.h"
#include "bf16_split.h"

// RELU_A (both kernels): A enters the product as max(a, 0) -- the weight gradient of a layer whose input is the
// activation of the previous layer's output, without that activation ever being stored.
template <int K1, int K2, bool RELU_A>
__global__ void __launch_bounds__(256)
psp_atb_kernel(const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, long long n,
               long long rows_per_block)
{
    constexpr int RM = K1 / 16, RN = K2 / 16;
    constexpr int ATB_ROWS = (K1 + K2 > 128) ? 32 : 64;  // at most 32 KB of LDS per workgroup
    __shared__ float sA[ATB_ROWS][K1];
    __shared__ float sB[ATB_ROWS][K2];
    const int t = threadIdx.x;
    const int ti = t >> 4, tj = t & 15;
    float acc[RM][RN];
#pragma unroll
    for (int a = 0; a < RM; a++)
#pragma unroll
        for (int b = 0; b < RN; b++) acc[a][b] = 0.0f;

    const long long r_begin = (long long)blockIdx.x * rows_per_block;
    const long long r_end = r_begin + rows_per_block < n ? r_begin + rows_per_block : n;
    for (long long base = r_begin; base < r_end; base += ATB_ROWS) {
        // stage ATB_ROWS rows of A and B; rows past the end contribute zeros
        for (int v = t; v < ATB_ROWS * K1 / 4; v += 256) {
            const int r = v / (K1 / 4), c4 = v % (K1 / 4);
            psp_f32x4 x = {0.f, 0.f, 0.f, 0.f};
            if (base + r < r_end) x = *(const psp_f32x4 *)(A + (base + r) * K1 + c4 * 4);
            if constexpr (RELU_A) {
#pragma unroll
                for (int e = 0; e < 4; e++) x[e] = x[e] < 0.0f ? 0.0f : x[e];
            }
            *(psp_f32x4 *)&sA[r][c4 * 4] = x;
        }
        for (int v = t; v < ATB_ROWS * K2 / 4; v += 256) {
            const int r = v / (K2 / 4), c4 = v % (K2 / 4);
            psp_f32x4 x = {0.f, 0.f, 0.f, 0.f};
            if (base + r < r_end) x = *(const psp_f32x4 *)(B + (base + r) * K2 + c4 * 4);
            *(psp_f32x4 *)&sB[r][c4 * 4] = x;
        }
        __syncthreads();
#pragma unroll 8
        for (int r = 0; r < ATB_ROWS; r++) {
            float av[RM], bv[RN];
#pragma unroll
            for (int a = 0; a < RM; a++) av[a] = sA[r][ti + 16 * a];
#pragma unroll
            for (int b = 0; b < RN; b++) bv[b] = sB[r][tj + 16 * b];
#pragma unroll
            for (int a = 0; a < RM; a++)
#pragma unroll
                for (int b = 0; b < RN; b++) acc[a][b] = __builtin_fmaf(av[a], bv[b], acc[a][b]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < RM; a++)
#pragma unroll
        for (int b = 0; b < RN; b++) unsafeAtomicAdd(&C[(ti + 16 * a) * K2 + tj + 16 * b], acc[a][b]);
}

// The same product on the matrix cores.  v_mfma_f32_16x16x4_f32 contracts four rows at a time; operand lane l holds
// one element of row l / 16 of the four, for output index l % 16.  Which column of A (of B) an output index stands for
// is free as long as the epilogue knows, so a lane loads V consecutive floats of its row (V = 4, 2 or 1) and feeds
// them to V different tiles: tile m, index i is column (m / V) * 16 V + V i + (m % V).  One wave-wide load is then a
// contiguous kilobyte (V = 4) that fills four tiles' operands, with no staging and no repeated loads.
// Wavefronts take U-group chunks round-robin, so the whole grid reads one contiguous window at a time.
//   JSPLIT = 1 (up to sixteen 16x16 output tiles): each wavefront owns its chunks and all tiles; the workgroup's four
//              partial products are added in LDS.
//   JSPLIT = 4 (wider outputs, K2 a multiple of 64): the four wavefronts of a workgroup share their chunks and own a
//              quarter of B's columns each; A is loaded by all four (the repeats are L1 / L2 hits).
typedef float psp_mfma_acc __attribute__((ext_vector_type(4)));

template <int V> __device__ __forceinline__ void psp_atb_load(const float *p, float *out)
{
    if (V == 4) {
        const psp_f32x4 x = *(const psp_f32x4 *)p;
        out[0] = x[0], out[1] = x[1], out[2] = x[2], out[3] = x[3];
    } else if (V == 2) {
        const psp_f32x2 x = *(const psp_f32x2 *)p;
        out[0] = x[0], out[1] = x[1];
    } else {
        out[0] = *p;
    }
}
// column of a (sub)matrix that index i of tile m stands for
template <int V> __device__ __forceinline__ int psp_atb_col(int m, int i) { return (m / V) * 16 * V + V * i + (m % V); }

template <int K1, int K2, int JSPLIT, bool RELU_A>
__global__ void __launch_bounds__(256)
psp_atb_mfma_kernel(const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, long long n,
                    float *__restrict__ partial)
{
    constexpr int RM = K1 / 16, RN = K2 / 16, RNW = RN / JSPLIT;
    constexpr int VA = RM % 4 == 0 ? 4 : RM % 2 == 0 ? 2 : 1, VB = RNW % 4 == 0 ? 4 : RNW % 2 == 0 ? 2 : 1;
    constexpr int U = (RM + RNW <= 2) ? 8 : (RM + RNW <= 4) ? 4 : 2;
    static_assert(RN % JSPLIT == 0 && RM * RNW <= 16, "tile split does not fit the register budget");
    __shared__ float red[JSPLIT == 1 ? RM * RN * 256 : 1];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int col0 = JSPLIT == 1 ? 0 : w * (K2 / JSPLIT);  // first column of B (and C) of this wavefront
    psp_mfma_acc acc[RM][RNW];
#pragma unroll
    for (int m = 0; m < RM; m++)
#pragma unroll
        for (int q = 0; q < RNW; q++) acc[m][q] = psp_mfma_acc{0.f, 0.f, 0.f, 0.f};

    const long long groups = (n + 3) >> 2;
    const long long chunk0 = JSPLIT == 1 ? (long long)blockIdx.x * 4 + w : (long long)blockIdx.x;
    const long long step = (long long)gridDim.x * (JSPLIT == 1 ? 4 : 1) * U;
    // Chunks of U whole groups go through two register buffers in turn: the loads of one chunk are in flight while the
    // MFMAs of the other run (the loop body has no branch, so the compiler waits for exactly the older buffer).
    float a0[U][RM], b0[U][RNW], a1[U][RM], b1[U][RNW];
    auto fetch = [&](long long g, float (&fa)[U][RM], float (&fb)[U][RNW]) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const long long row = (g + u) * 4 + kk;
#pragma unroll
            for (int t = 0; t < RM / VA; t++) psp_atb_load<VA>(A + row * K1 + t * 16 * VA + VA * c, &fa[u][t * VA]);
            if constexpr (RELU_A) {
#pragma unroll
                for (int m = 0; m < RM; m++) fa[u][m] = fa[u][m] < 0.0f ? 0.0f : fa[u][m];
            }
#pragma unroll
            for (int t = 0; t < RNW / VB; t++) psp_atb_load<VB>(B + row * K2 + col0 + t * 16 * VB + VB * c, &fb[u][t * VB]);
        }
    };
    auto multiply = [&](const float (&fa)[U][RM], const float (&fb)[U][RNW]) {
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int m = 0; m < RM; m++)
#pragma unroll
                for (int q = 0; q < RNW; q++)
                    acc[m][q] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[u][m], fb[u][q], acc[m][q], 0, 0, 0);
    };
    const long long whole_chunks = n / (4 * U);  // chunks all of whose rows exist
    const long long stride = step / U;           // wavefronts (JSPLIT = 1) or workgroups sharing the chunks
    const long long count = whole_chunks > chunk0 ? (whole_chunks - chunk0 + stride - 1) / stride : 0;
    long long g = chunk0 * U;
    if (count > 0) {
        fetch(g, a0, b0);
        long long k = 0;
        for (; k + 2 < count; k += 2) {
            // the scheduling barriers keep the compiler from sinking a chunk's loads below the other chunk's MFMAs
            fetch(g + step, a1, b1);
            __builtin_amdgcn_sched_barrier(0);
            multiply(a0, b0);
            __builtin_amdgcn_sched_barrier(0);
            fetch(g + 2 * step, a0, b0);
            __builtin_amdgcn_sched_barrier(0);
            multiply(a1, b1);
            __builtin_amdgcn_sched_barrier(0);
            g += 2 * step;
        }
        if (count - k == 2) {
            fetch(g + step, a1, b1);
            multiply(a0, b0);
            multiply(a1, b1);
        } else {
            multiply(a0, b0);
        }
    }
    // the one chunk that holds the matrix's last rows is partial (unless n is a multiple of 4 U): rows past n are zeros
    if (whole_chunks * U < groups && whole_chunks % stride == chunk0) {
        const long long gt = whole_chunks * U;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const long long row = (gt + u) * 4 + kk;
#pragma unroll
            for (int m = 0; m < RM; m++) {
                a0[u][m] = row < n ? A[row * K1 + psp_atb_col<VA>(m, c)] : 0.f;
                if (RELU_A) a0[u][m] = a0[u][m] < 0.0f ? 0.0f : a0[u][m];
            }
#pragma unroll
            for (int q = 0; q < RNW; q++) b0[u][q] = row < n ? B[row * K2 + col0 + psp_atb_col<VB>(q, c)] : 0.f;
        }
        multiply(a0, b0);
    }
    // the accumulator's register v of lane l is element [4 * (l / 16) + v][l % 16] of its tile.  With `partial` the
    // workgroup stores its K1 x K2 partial product there (row-major, one slot per workgroup) for the reduction kernel;
    // without it the partial product is added to C with atomics.
    float *dst = partial ? partial + (size_t)blockIdx.x * (K1 * K2) : C;
    if (JSPLIT == 1) {
        // the four wavefronts add their tiles one after the other, so the sum has a fixed order
        for (int turn = 0; turn < 4; turn++) {
            if (w == turn) {
#pragma unroll
                for (int m = 0; m < RM; m++)
#pragma unroll
                    for (int q = 0; q < RN; q++)
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            float *r = &red[((m * RN + q) * 4 + v) * 64 + lane];
                            *r = turn == 0 ? acc[m][q % RNW][v] : *r + acc[m][q % RNW][v];
                        }
            }
            __syncthreads();
        }
        for (int e = threadIdx.x; e < RM * RN * 256; e += 256) {
            const int l = e & 63, v = (e >> 6) & 3, tile = e >> 8;
            const int m = tile / RN, q = tile % RN;
            float *d = &dst[psp_atb_col<VA>(m, 4 * (l >> 4) + v) * K2 + psp_atb_col<VB>(q, l & 15)];
            if (partial) *d = red[e];
            else unsafeAtomicAdd(d, red[e]);
        }
    } else {
#pragma unroll
        for (int m = 0; m < RM; m++)
#pragma unroll
            for (int q = 0; q < RNW; q++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    float *d = &dst[psp_atb_col<VA>(m, 4 * kk + v) * K2 + col0 + psp_atb_col<VB>(q, c)];
                    if (partial) *d = acc[m][q][v];
                    else unsafeAtomicAdd(d, acc[m][q][v]);
                }
    }
}

// The 128 x 128 product on the bf16 matrix-core path (option dense_split).  At that shape the fp32 instruction above
// needs as long for its flops as the memory system needs for the two operands; with every fp32 operand taken apart
// into its three bf16 terms (exact: 8 + 8 + 8 significant bits) and the six term products that matter (error 2^-23 of
// |a||b| per product) accumulated in fp32 by v_mfma_f32_16x16x32_bf16, the kernel is bound by its traffic again.
// The instruction contracts 32 rows; operand lane (c, kk) = (lane % 16, lane / 16) supplies eight of them, rows
// 8 kk + i of the chunk, for output index c.  A lane loads, from each of its eight rows, two float4 of A (columns
// 64 t + 4 c ..: tile 4 t + e takes element e) and one float2 of its wavefront's quarter of B (columns col0 + 2 c + q:
// tile q), so one load instruction covers 256 (128) contiguous bytes of four rows.  The four wavefronts of a workgroup
// share a chunk and own a quarter of B's columns each, as in the JSPLIT = 4 form above.  Rows past n enter as zeros.
#define ATB_SPLIT_WGS 512  // two workgroups per CU (three, at 168 registers with spills, were slower): as many partial products to add

template <bool RELU_A>
__global__ void __launch_bounds__(256, 2)
psp_atb_split_kernel(const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, long long n,
                     float *__restrict__ partial)
{
    constexpr int K1 = 128, K2 = 128, RM = 8, RNW = 2;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int col0 = w * 32;
    psp_mfma_acc acc[RM][RNW];
#pragma unroll
    for (int m = 0; m < RM; m++)
#pragma unroll
        for (int q = 0; q < RNW; q++) acc[m][q] = psp_mfma_acc{0.f, 0.f, 0.f, 0.f};

    const long long chunks = (n + 31) >> 5;
    psp_f32x4 a0[8][2];
    psp_f32x2 b0[8];
    // unconditional loads from clamped rows; what lies past n is cleared where it is used
    auto fetch = [&](long long ch, psp_f32x4 (&fa)[8][2], psp_f32x2 (&fb)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            long long row = ch * 32 + 8 * kk + i;
            row = row < n ? row : n - 1;
            fa[i][0] = *(const psp_f32x4 *)(A + row * K1 + 4 * c);
            fa[i][1] = *(const psp_f32x4 *)(A + row * K1 + 64 + 4 * c);
            fb[i] = *(const psp_f32x2 *)(B + row * K2 + col0 + 2 * c);
        }
    };
    auto multiply = [&](long long ch, psp_f32x4 (&fa)[8][2], psp_f32x2 (&fb)[8]) {
        if (ch * 32 + 32 > n) {  // the last chunk of the matrix
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (ch * 32 + 8 * kk + i >= n) {
                    fa[i][0] = fa[i][1] = psp_f32x4{0.f, 0.f, 0.f, 0.f};
                    fb[i] = psp_f32x2{0.f, 0.f};
                }
        }
        psp_u32x4 bh[RNW], bm[RNW], bl[RNW];
#pragma unroll
        for (int q = 0; q < RNW; q++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                unsigned h_, m_, l_;
                psp_split3(fb[2 * g][q], fb[2 * g + 1][q], h_, m_, l_);
                bh[q][g] = h_, bm[q][g] = m_, bl[q][g] = l_;
            }
#pragma unroll
        for (int m = 0; m < RM; m++) {
            psp_u32x4 ah, am, al;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                float x = fa[2 * g][m >> 2][m & 3], y = fa[2 * g + 1][m >> 2][m & 3];
                if constexpr (RELU_A) {
                    x = x < 0.0f ? 0.0f : x;
                    y = y < 0.0f ? 0.0f : y;
                }
                unsigned h_, m_, l_;
                psp_split3(x, y, h_, m_, l_);
                ah[g] = h_, am[g] = m_, al[g] = l_;
            }
            // small terms first; the two column tiles alternate, so no instruction waits for the one before it
#define ATBS_TERM(AV_, BV_)                                                                                            \
    _Pragma("unroll") for (int q = 0; q < RNW; q++) acc[m][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(               \
        __builtin_bit_cast(psp_bf16x8, AV_), __builtin_bit_cast(psp_bf16x8, BV_[q]), acc[m][q], 0, 0, 0);
            ATBS_TERM(al, bh)
            ATBS_TERM(ah, bl)
            ATBS_TERM(am, bm)
            ATBS_TERM(am, bh)
            ATBS_TERM(ah, bm)
            ATBS_TERM(ah, bh)
#undef ATBS_TERM
        }
    };
    // one set of operand registers: two workgroups share a CU (256 registers per lane each), and while one waits for
    // its chunk the other takes its own apart and multiplies
    for (long long ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
        fetch(ch, a0, b0);
        multiply(ch, a0, b0);
    }
    // accumulator register v of lane (c, kk), tile (m, q) is C[64 (m / 4) + 4 (4 kk + v) + m % 4][col0 + 2 c + q]
    float *dst = partial ? partial + (size_t)blockIdx.x * (K1 * K2) : C;
#pragma unroll
    for (int m = 0; m < RM; m++)
#pragma unroll
        for (int q = 0; q < RNW; q++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float *d = &dst[(64 * (m >> 2) + 4 * (4 * kk + v) + (m & 3)) * K2 + col0 + 2 * c + q];
                if (partial) *d = acc[m][q][v];
                else unsafeAtomicAdd(d, acc[m][q][v]);
            }
}

// C[e] = sum over the P workgroup slots of partial[p][e].  A workgroup of 1024 lanes takes 16 elements; lane t adds the
// slots t / 16, t / 16 + 64, ... of element t % 16 (all loads independent, so one memory latency covers them), then
// the 64 sums of an element meet in LDS.
__global__ void __launch_bounds__(1024)
psp_atb_reduce_kernel(const float *__restrict__ partial, float *__restrict__ C, int P, int E)
{
    __shared__ float part[64][17];
    const int el = threadIdx.x & 15, sg = threadIdx.x >> 4;
    const int e = blockIdx.x * 16 + el;
    float s = 0.f;
    if (e < E) {
#pragma unroll 16
        for (int p = sg; p < P; p += 64) s += partial[(size_t)p * E + e];
    }
    part[sg][el] = s;
    __syncthreads();
    if (threadIdx.x < 16 && e < E) {
        float t = 0.f;
#pragma unroll
        for (int g = 0; g < 64; g++) t += part[g][threadIdx.x];
        C[e] = t;
    }
}

typedef void (*psp_atb_kernel_t)(const float *, const float *, float *, long long, long long);
typedef void (*psp_atb_mfma_kernel_t)(const float *, const float *, float *, long long, float *);

static psp_atb_kernel_t atb_lookup(int K1, int K2, bool relu_a = false)
{
#define ATB_CASE(a, b) \
    if (K1 == a && K2 == b) return relu_a ? psp_atb_kernel<a, b, true> : psp_atb_kernel<a, b, false>;
#define ATB_ROW(a) ATB_CASE(a, 16) ATB_CASE(a, 32) ATB_CASE(a, 48) ATB_CASE(a, 64) ATB_CASE(a, 80) ATB_CASE(a, 96) ATB_CASE(a, 112) ATB_CASE(a, 128)
    ATB_ROW(16) ATB_ROW(32) ATB_ROW(48) ATB_ROW(64) ATB_ROW(80) ATB_ROW(96) ATB_ROW(112) ATB_ROW(128)
#undef ATB_ROW
#undef ATB_CASE
    return nullptr;
}

// *jsplit receives the kernel's JSPLIT
static psp_atb_mfma_kernel_t atb_mfma_lookup(int K1, int K2, int *jsplit, bool relu_a = false)
{
    *jsplit = 1;
#define ATB_MFMA(a, b) \
    if (K1 == a && K2 == b) return relu_a ? psp_atb_mfma_kernel<a, b, 1, true> : psp_atb_mfma_kernel<a, b, 1, false>;
    ATB_MFMA(16, 16) ATB_MFMA(16, 32) ATB_MFMA(16, 48) ATB_MFMA(16, 64) ATB_MFMA(16, 80) ATB_MFMA(16, 96) ATB_MFMA(16, 112) ATB_MFMA(16, 128)
    ATB_MFMA(32, 16) ATB_MFMA(32, 32) ATB_MFMA(32, 48) ATB_MFMA(32, 64) ATB_MFMA(32, 80) ATB_MFMA(32, 96) ATB_MFMA(32, 112) ATB_MFMA(32, 128)
    ATB_MFMA(48, 16) ATB_MFMA(48, 32) ATB_MFMA(48, 48) ATB_MFMA(48, 64) ATB_MFMA(48, 80)
    ATB_MFMA(64, 16) ATB_MFMA(64, 32) ATB_MFMA(64, 48) ATB_MFMA(64, 64)
    ATB_MFMA(80, 16) ATB_MFMA(80, 32) ATB_MFMA(80, 48)
    ATB_MFMA(96, 16) ATB_MFMA(96, 32) ATB_MFMA(112, 16) ATB_MFMA(112, 32) ATB_MFMA(128, 16) ATB_MFMA(128, 32)
#undef ATB_MFMA
    *jsplit = 4;
#define ATB_MFMA4(a, b) \
    if (K1 == a && K2 == b) return relu_a ? psp_atb_mfma_kernel<a, b, 4, true> : psp_atb_mfma_kernel<a, b, 4, false>;
    ATB_MFMA4(64, 128) ATB_MFMA4(80, 64) ATB_MFMA4(96, 64) ATB_MFMA4(112, 64) ATB_MFMA4(128, 64)
    ATB_MFMA4(80, 128) ATB_MFMA4(96, 128) ATB_MFMA4(112, 128) ATB_MFMA4(128, 128)
#undef ATB_MFMA4
    return nullptr;
}

// Workgroups of the MFMA kernel: about four per CU, fewer when there are not that many 8-group chunks.
static long long atb_mfma_grid(long long n, int jsplit, int E)
{
    const long long chunks = ((n + 3) / 4 + 7) / 8;
    const long long max_wgs = 1024;
    long long wgs = jsplit == 1 ? (chunks + 3) / 4 : chunks;
    if (wgs > max_wgs) wgs = max_wgs;
    return wgs < 1 ? 1 : wgs;
}

PSP_EXPORT int psp_gemm_atb_supported(int K1, int K2) { return atb_lookup(K1, K2) != nullptr; }

static int atb_atomic(const float *A, const float *B, float *C, long long n, int K1, int K2, bool relu_a, hipStream_t stream)
{
    PSP_REQUIRE(n >= 0 && K1 >= 1 && K2 >= 1, "gemm_atb: bad size");
    psp_atb_kernel_t k = atb_lookup(K1, K2, relu_a);
    PSP_REQUIRE(k != nullptr, "gemm_atb: K1 and K2 must be multiples of 16 up to 128 (got %d, %d)", K1, K2);
    PSP_REQUIRE(C != nullptr && (n == 0 || (A && B)), "gemm_atb: null pointer");
    int rc = psp_zero_f32(C, (size_t)K1 * K2, stream);
    if (rc != PSP_OK || n == 0) return rc;
    int jsplit = 1;
    if (psp_atb_mfma_kernel_t km = atb_mfma_lookup(K1, K2, &jsplit, relu_a)) {
        long long wgs = atb_mfma_grid(n, jsplit, K1 * K2);
        if (K1 == 128 && K2 == 128 && psp_opts().dense_split) {
            km = relu_a ? psp_atb_split_kernel<true> : psp_atb_split_kernel<false>;
            wgs = wgs < ATB_SPLIT_WGS ? wgs : ATB_SPLIT_WGS;
        }
        hipLaunchKernelGGL(km, dim3((unsigned)wgs), dim3(256), 0, stream, A, B, C, n, (float *)nullptr);
        return psp_check_launch("gemm_atb mfma kernel");
    }
    // about 8 workgroups per CU, each on a contiguous band of whole 64-row tiles
    const int ATB_ROWS = 64;
    long long blocks = (n + ATB_ROWS - 1) / ATB_ROWS;
    if (blocks > 2048) blocks = 2048;
    long long rows_per_block = ((n + blocks - 1) / blocks + ATB_ROWS - 1) / ATB_ROWS * ATB_ROWS;
    blocks = (n + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), 0, stream, A, B, C, n, rows_per_block);
    return psp_check_launch("gemm_atb kernel");
}

PSP_EXPORT int psp_gemm_atb_f32(const float *A, const float *B, float *C, long long n, int K1, int K2,
                                psp_stream_t stream)
{
    return atb_atomic(A, B, C, n, K1, K2, false, (hipStream_t)stream);
}

PSP_EXPORT long long psp_gemm_atb_workspace_floats(long long n, int K1, int K2)
{
    int jsplit = 1;
    if (n <= 0 || !atb_mfma_lookup(K1, K2, &jsplit)) return 0;
    return atb_mfma_grid(n, jsplit, K1 * K2) * K1 * K2;
}

PSP_EXPORT int psp_gemm_atb_ws_act_f32(const float *A, const float *B, float *C, long long n, int K1, int K2, int relu_a,
                                       float *workspace, long long workspace_floats, psp_stream_t stream)
{
    int jsplit = 1;
    psp_atb_mfma_kernel_t km = atb_mfma_lookup(K1, K2, &jsplit, relu_a != 0);
    if (!km || n <= 0) return atb_atomic(A, B, C, n, K1, K2, relu_a != 0, (hipStream_t)stream);  // shapes of the LDS-tiled kernel; n = 0
    PSP_REQUIRE(A && B && C, "gemm_atb_ws: null pointer");
    long long wgs = atb_mfma_grid(n, jsplit, K1 * K2);
    PSP_REQUIRE(workspace && workspace_floats >= wgs * K1 * K2, "gemm_atb_ws: the workspace holds %lld floats, %lld needed",
                workspace_floats, wgs * K1 * K2);
    if (K1 == 128 && K2 == 128 && psp_opts().dense_split) {
        km = relu_a ? psp_atb_split_kernel<true> : psp_atb_split_kernel<false>;
        wgs = wgs < ATB_SPLIT_WGS ? wgs : ATB_SPLIT_WGS;  // (uses the first slots of the workspace)
    }
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(km, dim3((unsigned)wgs), dim3(256), 0, st, A, B, C, n, workspace);
    int rc = psp_check_launch("gemm_atb mfma kernel");
    if (rc != PSP_OK) return rc;
    hipLaunchKernelGGL(psp_atb_reduce_kernel, dim3((unsigned)((K1 * K2 + 15) / 16)), dim3(1024), 0, st, workspace, C, (int)wgs,
                       K1 * K2);
    return psp_check_launch("gemm_atb reduce kernel");
}

PSP_EXPORT int psp_gemm_atb_ws_f32(const float *A, const float *B, float *C, long long n, int K1, int K2,
                                   float *workspace, long long workspace_floats, psp_stream_t stream)
{
    return psp_gemm_atb_ws_act_f32(A, B, C, n, K1, K2, 0, workspace, workspace_floats, stream);
}
