// dmq_gemm_gf_kernel instantiations for the A16 precision mode.
#include "gemm_dispatch.h"

int dmq_gemm_launch_a16(const GemmLaunch& L) { return dmq_gemm_launch_mode<DMQ_MODE_A16>(L); }

#ifdef DMQ_TRACE
extern "C" int dmq_trace_read(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(dmq_trace_buf), sizeof(long long) * 256);
}
extern "C" int dmq_trace_read_wg(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(dmq_wg_buf), sizeof(long long) * DMQ_WG_SLOTS * 4);
}
extern "C" int dmq_trace_reset_wg(void) {
  void* p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(dmq_wg_buf)) != hipSuccess) return 1;
  return (int)hipMemset(p, 0, sizeof(long long) * DMQ_WG_SLOTS * 4);
}
#endif
