// dmq_gemm_gf_kernel instantiations for the A8 precision mode.
#include "gemm_dispatch.h"

int dmq_gemm_launch_a8(const GemmLaunch& L) { return dmq_gemm_launch_mode<DMQ_MODE_A8>(L); }
