// SpMM kernels of the 3x1-block format (instantiations only; the template lives in spmm_kernel.h).
#include "spmm_launch_impl.h"
template int psp_spmm_launch<3, false>(const int *, const int *, const float *, const int *, const float *, float *,
                                     int, int, int, int, int, hipStream_t, const float *, float *, int);
