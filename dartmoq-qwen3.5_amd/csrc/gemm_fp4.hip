// dmq_gemm_gf_kernel instantiations for the FP4 (MX e2m1) precision mode.
// Weights arrive already folded to packed e2m1 (64 bytes per row and group), so the
// kernel does not depend on the original index bit width.
#include "gemm_dispatch.h"

int dmq_gemm_launch_fp4(const GemmLaunch& L) { return dmq_gemm_launch_tt<DMQ_MODE_FP4, 4>(L); }
