// SDDMM kernels of the bcsr format (instantiations only; the template lives in sddmm_kernel.h).
#include "sddmm_launch_impl.h"
template int psp_sddmm_launch<2, false>(const int *, const int *, const float *, const int *, const float *,
                                      const float *, const float *, float *, int, int, int, hipStream_t, float *);
