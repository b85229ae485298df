// Shared by the translation units of libparamsp_hip.so (gfx950 only, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdarg.h>
#include "paramsp.h"

#define PSP_WAVE 64
#define PSP_XCDS 8  // MI355X: 8 accelerator complex dies, each with its own L2

#define PSP_EXPORT extern "C" __attribute__((visibility("default")))

// thread-local text of the last failure (psp_last_error)
int psp_fail(int code, const char *fmt, ...);

#define PSP_REQUIRE(cond, ...) \
    do {                       \
        if (!(cond)) return psp_fail(PSP_ERR_ARG, __VA_ARGS__); \
    } while (0)

static inline int psp_check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return psp_fail(PSP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return PSP_OK;
}

static inline int psp_ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

// Workgroups are handed to the 8 XCDs round-robin by linear workgroup id.  To give each XCD (one L2) runs of
// neighbouring sparse rows -- so that rows which gather the same rows of X find them in the same L2 -- the
// logical tiles are dealt out in stripes: XCD x works on tiles [s*8*G + x*G, s*8*G + (x+1)*G) for s = 0,1,..
// (G = tiles per stripe).  Stripes are short enough (a few thousand rows) that a matrix whose long rows
// cluster in one index range still spreads over all XCDs.  G = 1 is the identity mapping.
struct psp_grid1d {
    int real;    // logical tiles
    int stripe;  // G: consecutive tiles that go to one XCD
    int launch;  // workgroups launched (>= real, a multiple of 8*G)
};
static inline psp_grid1d psp_xcd_grid(int tiles, int stripe)
{
    psp_grid1d g;
    g.real = tiles;
    const int band = (tiles + PSP_XCDS - 1) / PSP_XCDS;  // one stripe per XCD is the widest useful setting
    g.stripe = stripe < 1 ? 1 : (stripe > band ? (band < 1 ? 1 : band) : stripe);
    const int round = PSP_XCDS * g.stripe;
    g.launch = (tiles + round - 1) / round * round;
    return g;
}
__device__ __forceinline__ int psp_xcd_tile(int stripe)
{
    const int xcd = blockIdx.x % PSP_XCDS, idx = blockIdx.x / PSP_XCDS;
    return ((idx / stripe) * PSP_XCDS + xcd) * stripe + idx % stripe;
}
// library-wide options (psp_set_option); the environment is consulted once, when they are first needed
struct psp_options {
    int stripe_rows;            // rows (or segments) one XCD stripe should span
    int align_pct;              // whole segments per lane group when that costs at most this many percent more steps
    long long split_clear_min;  // row-split outputs of at least this many floats are cleared selectively
    int whole_rows;             // SpMM: a lane group always takes whole segments (reference summation order)
    int dense_split;            // 128 x 128 layer products: fp32 operands as three bf16 terms on the bf16 matrix-core path
};
psp_options &psp_opts(void);
int psp_stripe_rows(void);

// zero-fill used instead of hipMemsetAsync (callers may capture these launches in a HIP graph)
int psp_zero_f32(float *p, size_t n, hipStream_t stream);
// the same for an arbitrary value
int psp_fill_f32(float *p, size_t n, float value, hipStream_t stream);

// Y[r, :] /= s[r] for every row with s[r] != 0 (rows of the softmax-weighted row-split SpMM that several
// wavefronts accumulated without normalising)
int psp_row_scale(float *Y, const float *s, int rows, int N, hipStream_t stream);

#define PSP_F32_LOWEST (-3.402823466e+38f)

#ifdef __HIPCC__
// float maximum through the integer atomics: the order of non-negative floats is that of their bit patterns read
// as signed integers, the order of negative floats is the reverse of their patterns read as unsigned
__device__ __forceinline__ void psp_atomic_max_f32(float *addr, float v)
{
    if (v >= 0.0f) atomicMax((int *)addr, __float_as_int(v));
    else atomicMin((unsigned int *)addr, __float_as_uint(v));
}
#endif

// Row-split SpMM: clears exactly the rows of Y the SpMM kernel will not plainly store -- rows whose segments sit
// in two wavefronts (each wavefront owns 2^logW consecutive segments), rows of empty segments, and rows no segment
// targets.  nr = matrix rows per target row (2 for 2x1 blocks).
int psp_split_clear(const int *rowPtr_split, const int *target_row, float *Y, int nseg, int N, int nr, int rows_out,
                    int logW, hipStream_t stream);
