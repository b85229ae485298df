// Mean negative log-likelihood over the rows of a log-probability matrix, forward and backward: the loss at the
// end of the reference's training step, F.nll_loss(model(), labels) in GNN.py:131-146.  PyTorch's kernels for it
// reduce the whole batch in a single workgroup; on 10^6 nodes they take 1.0 ms + 0.7 ms per step, more than a third
// of a 16-wide GCN epoch.  These run at the speed of reading the labels and writing the gradient.
//
// Rows whose label lies outside [0, C) do not count (PyTorch's ignore_index behaves the same way for its one
// ignored value); the mean is over the rows that count.
#include "psp_common.h"

// stats[0] += sum of logp[i, label_i], stats[1] += number of rows that count
__global__ void __launch_bounds__(256) nll_sum_kernel(const float *__restrict__ logp, const long long *__restrict__ labels,
                                                      long long n, int C, float *__restrict__ stats)
{
    __shared__ float s_sum[4], s_cnt[4];
    float sum = 0.0f, cnt = 0.0f;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long y = labels[i];
        if (y >= 0 && y < C) {
            sum += logp[i * C + y];
            cnt += 1.0f;
        }
    }
#pragma unroll
    for (int d = 1; d < PSP_WAVE; d <<= 1) {
        sum += __shfl_xor(sum, d);
        cnt += __shfl_xor(cnt, d);
    }
    if ((threadIdx.x & 63) == 0) {
        s_sum[threadIdx.x >> 6] = sum;
        s_cnt[threadIdx.x >> 6] = cnt;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicAdd(stats, s_sum[0] + s_sum[1] + s_sum[2] + s_sum[3]);
        atomicAdd(stats + 1, s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3]);
    }
}

__global__ void nll_finish_kernel(const float *__restrict__ stats, float *__restrict__ loss)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) *loss = -stats[0] / stats[1];
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

PSP_EXPORT int psp_nll_loss_mean_f32(const float *logp, const long long *labels, long long n, int C, float *loss,
                                     float *stats, psp_stream_t stream)
{
    PSP_REQUIRE(n >= 0 && C >= 1, "nll_loss: bad shape (n %lld, C %d)", n, C);
    PSP_REQUIRE(loss && stats && (n == 0 || (logp && labels)), "nll_loss: null pointer");
    hipStream_t st = (hipStream_t)stream;
    int rc = psp_zero_f32(stats, 2, st);
    if (rc != PSP_OK) return rc;
    if (n > 0) {
        int blocks = psp_ceil_div(n, 256 * 4);
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(nll_sum_kernel, dim3(blocks), dim3(256), 0, st, logp, labels, n, C, stats);
    }
    hipLaunchKernelGGL(nll_finish_kernel, dim3(1), dim3(64), 0, st, stats, loss);
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
