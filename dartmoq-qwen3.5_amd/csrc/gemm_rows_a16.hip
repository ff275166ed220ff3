// dmq_gemm_rows_kernel instantiations and their host launcher.
#include "gemm_rows.h"
#include "gemm_dispatch.h"

// one workgroup per CU (the kernel takes a CU's registers and most of its LDS), a multiple of the
// XCD count
static int dmq_rows_grid(int* grid) {
  static int cached[64];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return DMQ_ERR_HIP;
  if (!cached[dev]) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < DMQ_XCDS)
      return DMQ_ERR_HIP;
    cached[dev] = cus / DMQ_XCDS * DMQ_XCDS;
  }
  *grid = cached[dev];
  return DMQ_OK;
}

template <int EPI>
static int dmq_rows_launch_epi(const GemmParams& p, int* queue, int nbl, hipStream_t stream) {
  static bool attr_set = false;      // the kernel needs more than the default 64 KiB of LDS
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&dmq_gemm_rows_kernel<EPI>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, DMQ_ROWS_LDS) != hipSuccess)
      return DMQ_ERR_HIP;
    attr_set = true;
  }
  int grid = 0;
  const int rc = dmq_rows_grid(&grid);
  if (rc) return rc;
  hipLaunchKernelGGL((dmq_gemm_rows_kernel<EPI>), dim3(grid), dim3(256), DMQ_ROWS_LDS, stream, p, queue, nbl);
  return dmq_check_launch();
}

int dmq_gemm_rows_launch(const GemmParams& p, int epi, int* queue, int nbl, hipStream_t stream) {
  switch (epi) {
    case DMQ_EPI_STORE: return dmq_rows_launch_epi<DMQ_EPI_STORE>(p, queue, nbl, stream);
    case DMQ_EPI_SILU: return dmq_rows_launch_epi<DMQ_EPI_SILU>(p, queue, nbl, stream);
    case DMQ_EPI_SCATTER: return dmq_rows_launch_epi<DMQ_EPI_SCATTER>(p, queue, nbl, stream);
    case DMQ_EPI_SILU_ROT: return dmq_rows_launch_epi<DMQ_EPI_SILU_ROT>(p, queue, nbl, stream);
  }
  return DMQ_ERR_MODE;
}
