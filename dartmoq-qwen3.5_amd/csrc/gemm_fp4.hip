// dmq_gemm_gf_kernel instantiations for the FP4 precision mode.
#include "gemm_dispatch.h"

int dmq_gemm_launch_fp4(const GemmLaunch& L) { return dmq_gemm_launch_mode<DMQ_MODE_FP4>(L); }
