// Mean negative log-likelihood over the rows of a log-probability matrix, forward and backward: the loss at the
// end of the reference's training step, F.nll_loss(model(), labels) in GNN.py:131-146.  PyTorch's kernels for it
// reduce the whole batch in a single workgroup; on 10^6 nodes they take 1.0 ms + 0.7 ms per step, more than a third
// of a 16-wide GCN epoch.  These run at the speed of reading the labels and writing the gradient.
//
// Rows whose label lies outside [0, C) do not count (PyTorch's ignore_index behaves the same way for its one
// ignored value, -100, and raises a device assertion for any other stray label); the mean is over the rows that
// count, and the number of stray labels other than -100 is reported in stats[2] so that a caller can check.
// No atomics: the result is the same bit for bit on every run.
#include "psp_common.h"

#define PSP_NLL_MAX_BLOCKS 1024
// stats layout (floats): [0] sum of logp[i, label_i], [1] number of rows that count, [2] number of labels that are
// out of range without being PyTorch's ignore_index (-100), then one partial sum and one partial count per workgroup
#define PSP_NLL_STATS_FLOATS (3 + 3 * PSP_NLL_MAX_BLOCKS)

// every workgroup stores its partial sum, its row count and its count of stray labels in its own slots: no atomics
__global__ void __launch_bounds__(256) nll_sum_kernel(const float *__restrict__ logp, const long long *__restrict__ labels,
                                                      long long n, int C, float *__restrict__ stats)
{
    __shared__ float s_sum[4];
    __shared__ int s_cnt[4], s_bad[4];
    float sum = 0.0f;
    int cnt = 0, bad = 0;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long y = labels[i];
        if (y >= 0 && y < C) {
            sum += logp[i * C + y];
            cnt++;
        } else if (y != -100) {
            bad++;
        }
    }
#pragma unroll
    for (int d = 1; d < PSP_WAVE; d <<= 1) {
        sum += __shfl_xor(sum, d);
        cnt += __shfl_xor(cnt, d);
        bad += __shfl_xor(bad, d);
    }
    if ((threadIdx.x & 63) == 0) {
        s_sum[threadIdx.x >> 6] = sum;
        s_cnt[threadIdx.x >> 6] = cnt;
        s_bad[threadIdx.x >> 6] = bad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        stats[3 + blockIdx.x] = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);
        ((int *)stats)[3 + PSP_NLL_MAX_BLOCKS + blockIdx.x] = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
        ((int *)stats)[3 + 2 * PSP_NLL_MAX_BLOCKS + blockIdx.x] = s_bad[0] + s_bad[1] + s_bad[2] + s_bad[3];
    }
}

// one workgroup adds the partial results in a fixed order (the loss repeats bit for bit from run to run and between
// replays of a recorded step); the row count is an exact integer until it is stored
__global__ void __launch_bounds__(256) nll_finish_kernel(float *__restrict__ stats, float *__restrict__ loss, int blocks)
{
    __shared__ float s_sum[256];
    __shared__ long long s_cnt[256], s_bad[256];
    float sum = 0.0f;
    long long cnt = 0, bad = 0;
    for (int b = threadIdx.x; b < blocks; b += 256) {
        sum += stats[3 + b];
        cnt += ((const int *)stats)[3 + PSP_NLL_MAX_BLOCKS + b];
        bad += ((const int *)stats)[3 + 2 * PSP_NLL_MAX_BLOCKS + b];
    }
    s_sum[threadIdx.x] = sum;
    s_cnt[threadIdx.x] = cnt;
    s_bad[threadIdx.x] = bad;
    __syncthreads();
    for (int d = 128; d >= 1; d >>= 1) {
        if ((int)threadIdx.x < d) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + d];
            s_cnt[threadIdx.x] += s_cnt[threadIdx.x + d];
            s_bad[threadIdx.x] += s_bad[threadIdx.x + d];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const double count = (double)s_cnt[0];
        stats[0] = s_sum[0];
        stats[1] = (float)count;
        stats[2] = (float)s_bad[0];
        *loss = (float)(-(double)s_sum[0] / count);
    }
}

// grad[i, c] = -g / count at c = label_i, 0 elsewhere; V consecutive columns per lane
template <int V>
__global__ void __launch_bounds__(256) nll_backward_kernel(const long long *__restrict__ labels, const float *__restrict__ grad_loss,
                                                           const float *__restrict__ stats, long long n, int C,
                                                           float *__restrict__ grad)
{
    const float w = -grad_loss[0] / stats[1];
    const long long total = n * C / V;
    for (long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long long)gridDim.x * blockDim.x) {
        const long long e = t * V;
        const long long row = e / C;
        const int c0 = (int)(e - row * C);
        const long long y = labels[row];  // V divides C, so the V columns belong to one row
        float v[V];
#pragma unroll
        for (int k = 0; k < V; k++) v[k] = (y == c0 + k) ? w : 0.0f;
        if (V == 4) *(float4 *)(grad + e) = make_float4(v[0], v[1], v[2], v[3]);
        else grad[e] = v[0];
    }
}

// ---- the same loss from the logits: log-softmax and the mean NLL in one pass ------------------------------------------------
// F.nll_loss(F.log_softmax(x, 1), labels) (GNN.py:61,78,101 and 131-146) reads and writes the [n, C] matrix five times
// (softmax forward, the loss, its gradient, softmax backward); from the logits it is one read forward and one read and
// one write backward.  A lane owns a row and holds its C logits in registers (C a multiple of 4 up to 64).
//   forward:  logp[y] = x[y] - max - log(sum exp(x - max)), summed per workgroup as above;
//   backward: grad[c] = (exp(x[c] - lse) - [c == y]) g / count for rows that count, 0 for the others.
template <int C4>
__global__ void __launch_bounds__(256) xent_sum_kernel(const float *__restrict__ x, const long long *__restrict__ labels,
                                                       long long n, float *__restrict__ stats)
{
    constexpr int C = C4 * 4;
    __shared__ float s_sum[4];
    __shared__ int s_cnt[4], s_bad[4];
    float sum = 0.0f;
    int cnt = 0, bad = 0;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long y = labels[i];
        float4 v[C4];
#pragma unroll
        for (int k = 0; k < C4; k++) v[k] = ((const float4 *)(x + i * C))[k];
        if (y >= 0 && y < C) {
            float mx = v[0].x, xy = 0.0f;
#pragma unroll
            for (int k = 0; k < C4; k++) {
                mx = fmaxf(fmaxf(mx, v[k].x), fmaxf(v[k].y, fmaxf(v[k].z, v[k].w)));
                const float e[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
                for (int c = 0; c < 4; c++) xy = (4 * k + c == (int)y) ? e[c] : xy;
            }
            float se = 0.0f;
#pragma unroll
            for (int k = 0; k < C4; k++) se += (__expf(v[k].x - mx) + __expf(v[k].y - mx)) + (__expf(v[k].z - mx) + __expf(v[k].w - mx));
            sum += (xy - mx) - __logf(se);
            cnt++;
        } else if (y != -100) {
            bad++;
        }
    }
#pragma unroll
    for (int d = 1; d < PSP_WAVE; d <<= 1) {
        sum += __shfl_xor(sum, d);
        cnt += __shfl_xor(cnt, d);
        bad += __shfl_xor(bad, d);
    }
    if ((threadIdx.x & 63) == 0) {
        s_sum[threadIdx.x >> 6] = sum;
        s_cnt[threadIdx.x >> 6] = cnt;
        s_bad[threadIdx.x >> 6] = bad;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        stats[3 + blockIdx.x] = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);
        ((int *)stats)[3 + PSP_NLL_MAX_BLOCKS + blockIdx.x] = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
        ((int *)stats)[3 + 2 * PSP_NLL_MAX_BLOCKS + blockIdx.x] = s_bad[0] + s_bad[1] + s_bad[2] + s_bad[3];
    }
}

template <int C4>
__global__ void __launch_bounds__(256) xent_backward_kernel(const float *__restrict__ x, const long long *__restrict__ labels,
                                                            const float *__restrict__ grad_loss, const float *__restrict__ stats,
                                                            long long n, float *__restrict__ grad)
{
    constexpr int C = C4 * 4;
    const float w = grad_loss[0] / stats[1];
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long y = labels[i];
        float4 v[C4];
#pragma unroll
        for (int k = 0; k < C4; k++) v[k] = ((const float4 *)(x + i * C))[k];
        const bool counts = y >= 0 && y < C;
        float mx = v[0].x;
#pragma unroll
        for (int k = 0; k < C4; k++) mx = fmaxf(fmaxf(mx, v[k].x), fmaxf(v[k].y, fmaxf(v[k].z, v[k].w)));
        float se = 0.0f;
#pragma unroll
        for (int k = 0; k < C4; k++) {
            v[k].x = __expf(v[k].x - mx), v[k].y = __expf(v[k].y - mx), v[k].z = __expf(v[k].z - mx), v[k].w = __expf(v[k].w - mx);
            se += (v[k].x + v[k].y) + (v[k].z + v[k].w);
        }
        const float scale = counts ? w / se : 0.0f;  // rows that do not count get a zero gradient (not NaN: 0 * p)
#pragma unroll
        for (int k = 0; k < C4; k++) {
            float4 o;
            o.x = counts ? v[k].x * scale - ((4 * k + 0 == (int)y) ? w : 0.0f) : 0.0f;
            o.y = counts ? v[k].y * scale - ((4 * k + 1 == (int)y) ? w : 0.0f) : 0.0f;
            o.z = counts ? v[k].z * scale - ((4 * k + 2 == (int)y) ? w : 0.0f) : 0.0f;
            o.w = counts ? v[k].w * scale - ((4 * k + 3 == (int)y) ? w : 0.0f) : 0.0f;
            ((float4 *)(grad + i * C))[k] = o;
        }
    }
}

PSP_EXPORT int psp_softmax_nll_supported(int C) { return C >= 4 && C % 4 == 0 && C <= 64; }

#define XENT_DISPATCH(KERNEL, ...)                                                                     \
    switch (C / 4) {                                                                                    \
    case 1: hipLaunchKernelGGL(KERNEL<1>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 2: hipLaunchKernelGGL(KERNEL<2>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 3: hipLaunchKernelGGL(KERNEL<3>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 4: hipLaunchKernelGGL(KERNEL<4>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 5: hipLaunchKernelGGL(KERNEL<5>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 6: hipLaunchKernelGGL(KERNEL<6>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 7: hipLaunchKernelGGL(KERNEL<7>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 8: hipLaunchKernelGGL(KERNEL<8>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 9: hipLaunchKernelGGL(KERNEL<9>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;           \
    case 10: hipLaunchKernelGGL(KERNEL<10>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    case 11: hipLaunchKernelGGL(KERNEL<11>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    case 12: hipLaunchKernelGGL(KERNEL<12>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    case 13: hipLaunchKernelGGL(KERNEL<13>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    case 14: hipLaunchKernelGGL(KERNEL<14>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    case 15: hipLaunchKernelGGL(KERNEL<15>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    default: hipLaunchKernelGGL(KERNEL<16>, dim3(blocks), dim3(256), 0, st, __VA_ARGS__); break;         \
    }

PSP_EXPORT int psp_softmax_nll_mean_f32(const float *logits, const long long *labels, long long n, int C, float *loss,
                                        float *stats, psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && psp_softmax_nll_supported(C), "softmax_nll: C must be a multiple of 4 up to 64 (n %lld, C %d)", n, C);
    PSP_REQUIRE(loss && stats && (n == 0 || (logits && labels)), "softmax_nll: null pointer");
    PSP_REQUIRE(((size_t)logits & 15) == 0, "softmax_nll: the logits must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    int blocks = 0;
    if (n > 0) {
        blocks = psp_ceil_div(n, 256);
        if (blocks > PSP_NLL_MAX_BLOCKS) blocks = PSP_NLL_MAX_BLOCKS;
        XENT_DISPATCH(xent_sum_kernel, logits, labels, n, stats)
    }
    hipLaunchKernelGGL(nll_finish_kernel, dim3(1), dim3(256), 0, st, stats, loss, blocks);
    return psp_check_launch("softmax nll kernels");
}

PSP_EXPORT int psp_softmax_nll_mean_backward_f32(const float *logits, const long long *labels, const float *grad_loss,
                                                 const float *stats, long long n, int C, float *grad_logits, psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && psp_softmax_nll_supported(C), "softmax_nll backward: C must be a multiple of 4 up to 64 (n %lld, C %d)", n, C);
    if (n == 0) return PSP_OK;
    PSP_REQUIRE(logits && labels && grad_loss && stats && grad_logits, "softmax_nll backward: null pointer");
    PSP_REQUIRE((((size_t)logits | (size_t)grad_logits) & 15) == 0, "softmax_nll backward: the matrices must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    int blocks = psp_ceil_div(n, 256);
    if (blocks > 16384) blocks = 16384;
    XENT_DISPATCH(xent_backward_kernel, logits, labels, grad_loss, stats, n, grad_logits)
    return psp_check_launch("softmax nll backward kernel");
}

PSP_EXPORT int psp_nll_loss_stats_floats(void) { return PSP_NLL_STATS_FLOATS; }

PSP_EXPORT int psp_nll_loss_mean_f32(const float *logp, const long long *labels, long long n, int C, float *loss,
                                     float *stats, psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && C >= 1, "nll_loss: bad shape (n %lld, C %d)", n, C);
    PSP_REQUIRE(loss && stats && (n == 0 || (logp && labels)), "nll_loss: null pointer");
    hipStream_t st = (hipStream_t)stream;
    int blocks = 0;
    if (n > 0) {
        blocks = psp_ceil_div(n, 256 * 4);
        if (blocks > PSP_NLL_MAX_BLOCKS) blocks = PSP_NLL_MAX_BLOCKS;
        hipLaunchKernelGGL(nll_sum_kernel, dim3(blocks), dim3(256), 0, st, logp, labels, n, C, stats);
    }
    hipLaunchKernelGGL(nll_finish_kernel, dim3(1), dim3(256), 0, st, stats, loss, blocks);
    return psp_check_launch("nll loss kernels");
}

PSP_EXPORT int psp_nll_loss_mean_backward_f32(const long long *labels, const float *grad_loss, const float *stats,
                                              long long n, int C, float *grad_logp, psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && C >= 1, "nll_loss backward: bad shape (n %lld, C %d)", n, C);
    if (n == 0) return PSP_OK;
    PSP_REQUIRE(labels && grad_loss && stats && grad_logp, "nll_loss backward: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const bool vec = C % 4 == 0 && ((size_t)grad_logp & 15) == 0;
    long long work = n * C / (vec ? 4 : 1);
    int blocks = psp_ceil_div(work, 256);
    if (blocks > 16384) blocks = 16384;
    if (vec) hipLaunchKernelGGL(nll_backward_kernel<4>, dim3(blocks), dim3(256), 0, st, labels, grad_loss, stats, n, C, grad_logp);
    else hipLaunchKernelGGL(nll_backward_kernel<1>, dim3(blocks), dim3(256), 0, st, labels, grad_loss, stats, n, C, grad_logp);
    return psp_check_launch("nll loss backward kernel");
}
