// dmq_gemm_gf_kernel instantiations for the FP8 precision mode.
#include "gemm_dispatch.h"

int dmq_gemm_launch_fp8(const GemmLaunch& L) { return dmq_gemm_launch_mode<DMQ_MODE_FP8>(L); }
