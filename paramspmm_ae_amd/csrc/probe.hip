// Measurement aid: the gather ceiling of a sparse pattern.  psp_probe_gather_f32 walks the same colIdx stream as
// an SpMM and loads the same X row tiles (lane groups of 2^logL lanes, one float4 per lane, column tiles in
// grid.y), but has no rows: no row pointer, no multiplications, no row stores -- every lane only adds what it
// loads and stores one float4 when its wavefront is done.  Its time is what the memory system needs for the
// gathers alone, U loads in flight per lane (bench.py tries U = 4 and 8 with several wavefront shares and keeps the
// fastest); an SpMM that walks the same pattern the same way cannot be faster.
#include "psp_common.h"

typedef float psp_f32x4 __attribute__((ext_vector_type(4)));
typedef int psp_i32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef int psp_i32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));

template <int U>
__global__ void __launch_bounds__(256)
psp_probe_gather_kernel(const int *__restrict__ colIdx, long long nnz, const float *__restrict__ X, int N, int logL,
                        int per_wave, float *__restrict__ out)
{
    const int L = 1 << logL;
    const int lane = threadIdx.x & 63;
    const int sub = lane & (L - 1), grp = lane >> logL, grp_base = lane - sub;
    const long long wave = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const long long e0 = wave * per_wave;
    if (e0 >= nnz) return;
    const long long e1 = e0 + per_wave < nnz ? e0 + per_wave : nnz;
    const int q = per_wave >> (6 - logL);  // entries per lane group
    long long a = e0 + (long long)grp * q, b = a + q;
    if (a > e1) a = e1;
    if (b > e1) b = e1;
    // A lane whose columns lie past N stays active -- ds_bpermute reads 0 from an inactive lane, which would turn
    // the entries those lanes fetched into gathers of X row 0 -- and loads the last valid vector instead, as the SpMM
    // kernel does; what it loads is not added.
    const int col_own = (blockIdx.y << logL) * 4 + sub * 4;  // this lane's first column
    const bool live = col_own < N;
    const int col0 = live ? col_own : N - 4;
    psp_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    {
        // lane `sub` takes the U consecutive entries base + sub*U .. (one 4U-byte load, whole lines per group), as
        // the SpMM kernel does
        for (long long base = a; base < b; base += L * U) {
            int c[U];
            const long long p0 = base + (long long)sub * U;
            if (p0 + U <= b) {
                if constexpr (U == 1) c[0] = colIdx[p0];
                else if constexpr (U == 2) {
                    const psp_i32x2_a4 t = *(const psp_i32x2_a4 *)(colIdx + p0);
                    c[0] = t[0];
                    c[1] = t[1];
                } else {
#pragma unroll
                    for (int h = 0; h < U; h += 4) {
                        const psp_i32x4_a4 t = *(const psp_i32x4_a4 *)(colIdx + p0 + h);
#pragma unroll
                        for (int e = 0; e < 4; e++) c[h + e] = t[e];
                    }
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; u++) c[u] = colIdx[p0 + u < b ? p0 + u : b - 1];
            }
            psp_f32x4 x[U];
            for (int j = 0; j < L; j++) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int ck = __builtin_amdgcn_ds_bpermute((grp_base + j) << 2, c[u]);
                    x[u] = *(const psp_f32x4 *)(X + (size_t)ck * (size_t)N + col0);
                }
#pragma unroll
                for (int u = 0; u < U; u++)
                    if (live && base + (long long)j * U + u < b) acc += x[u];
            }
        }
    }
    const size_t slot = ((size_t)blockIdx.y * gridDim.x * (blockDim.x >> 6) + (size_t)wave) * 64 + lane;
    __builtin_nontemporal_store(acc, (psp_f32x4 *)out + slot);
}

PSP_EXPORT long long psp_probe_gather_out_floats(long long nnz, int N, int lanes_per_row, int entries_per_wave)
{
    if (nnz <= 0 || N <= 0 || lanes_per_row <= 0 || entries_per_wave <= 0) return 0;
    const long long waves = (nnz + entries_per_wave - 1) / entries_per_wave;
    const long long blocks = (waves + 3) / 4;
    const long long tiles = (N / 4 + lanes_per_row - 1) / lanes_per_row;
    return blocks * 4 * tiles * 64 * 4;
}

PSP_EXPORT int psp_probe_gather_f32(const int *colIdx, long long nnz, const float *X, int N, int lanes_per_row,
                                    int unroll, int entries_per_wave, float *out, long long out_floats,
                                    psp_stream_t stream)
{
    PSP_REQUIRE(nnz >= 0 && N >= 4 && N % 4 == 0, "probe_gather: N must be a positive multiple of 4 (got %d)", N);
    PSP_REQUIRE(lanes_per_row >= 1 && lanes_per_row <= 64 && (lanes_per_row & (lanes_per_row - 1)) == 0,
                "probe_gather: lanes_per_row must be a power of two up to 64");
    PSP_REQUIRE(unroll == 1 || unroll == 2 || unroll == 4 || unroll == 8, "probe_gather: unroll must be 1, 2, 4 or 8");
    PSP_REQUIRE(entries_per_wave >= 64 && entries_per_wave % 64 == 0 && entries_per_wave <= (1 << 20),
                "probe_gather: entries_per_wave must be a multiple of 64");
    if (nnz == 0) return PSP_OK;
    PSP_REQUIRE(colIdx && X && out, "probe_gather: null pointer");
    PSP_REQUIRE(out_floats >= psp_probe_gather_out_floats(nnz, N, lanes_per_row, entries_per_wave),
                "probe_gather: out holds %lld floats, %lld needed", out_floats,
                psp_probe_gather_out_floats(nnz, N, lanes_per_row, entries_per_wave));
    int logL = 0;
    while ((1 << logL) < lanes_per_row) logL++;
    const long long waves = (nnz + entries_per_wave - 1) / entries_per_wave;
    const long long blocks = (waves + 3) / 4;
    PSP_REQUIRE(blocks <= 0x7fffffffLL, "probe_gather: too many workgroups");
    const int tiles = (N / 4 + lanes_per_row - 1) / lanes_per_row;
    dim3 grid((unsigned)blocks, tiles, 1), block(256, 1, 1);
    hipStream_t st = (hipStream_t)stream;
#define PSP_PROBE(U_) \
    hipLaunchKernelGGL(psp_probe_gather_kernel<U_>, grid, block, 0, st, colIdx, nnz, X, N, logL, entries_per_wave, out)
    if (unroll == 1) PSP_PROBE(1);
    else if (unroll == 2) PSP_PROBE(2);
    else if (unroll == 4) PSP_PROBE(4);
    else PSP_PROBE(8);
#undef PSP_PROBE
    return psp_check_launch("probe gather kernel");
}
