// dmq_gemm_gf_kernel instantiations for the A16 precision mode.
#include "gemm_dispatch.h"

int dmq_gemm_launch_a16(const GemmLaunch& L) { return dmq_gemm_launch_mode<DMQ_MODE_A16>(L); }
