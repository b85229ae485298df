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

// Workgroups are handed to the 8 XCDs round-robin by linear workgroup id.  Launching
// PSP_XCDS*chunk workgroups and giving workgroup b the logical tile (b%8)*chunk + b/8 makes each XCD
// (one L2) work on one contiguous band of sparse rows, so neighbouring rows that gather the same rows
// of X find them in the same L2.
struct psp_grid1d {
    int real;   // logical tiles
    int chunk;  // tiles per XCD
    int launch; // workgroups launched (>= real)
};
static inline psp_grid1d psp_xcd_grid(int tiles)
{
    psp_grid1d g;
    g.real = tiles;
    g.chunk = (tiles + PSP_XCDS - 1) / PSP_XCDS;
    g.launch = g.chunk * PSP_XCDS;
    return g;
}
__device__ __forceinline__ int psp_xcd_tile(int chunk) { return (blockIdx.x % PSP_XCDS) * chunk + blockIdx.x / PSP_XCDS; }

// zero-fill used instead of hipMemsetAsync (callers may capture these launches in a HIP graph)
int psp_zero_f32(float *p, size_t n, hipStream_t stream);
