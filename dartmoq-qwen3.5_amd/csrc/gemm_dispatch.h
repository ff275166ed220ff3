// Host-side dispatch of dmq_gemm_gf_kernel instantiations for one precision mode.
// Each mode lives in its own translation unit so the modes compile in parallel.
#pragma once
#include "gemm_gf.h"

struct GemmLaunch {
  GemmParams p;
  int bit;
  int epi;
  int tt;          // token tiles per wave: 1, 2 or 4
  int dbg;
  int grid;
  hipStream_t stream;
};

template <int MODE, int BIT, int TT, int EPI, bool DBG>
static int dmq_gemm_launch_one(const GemmLaunch& L) {
  hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, BIT, 4, TT, EPI, DBG>), dim3(L.grid), dim3(256), 0,
                     L.stream, L.p);
  return dmq_check_launch();
}

template <int MODE, int BIT, int TT>
static int dmq_gemm_launch_epi(const GemmLaunch& L) {
  switch (L.epi) {
    case DMQ_EPI_STORE:
      if (MODE == DMQ_MODE_A8 && TT == 1 && L.dbg)
        return dmq_gemm_launch_one<MODE, BIT, TT, DMQ_EPI_STORE, (MODE == DMQ_MODE_A8 && TT == 1)>(L);
      return dmq_gemm_launch_one<MODE, BIT, TT, DMQ_EPI_STORE, false>(L);
    case DMQ_EPI_SILU: return dmq_gemm_launch_one<MODE, BIT, TT, DMQ_EPI_SILU, false>(L);
    case DMQ_EPI_SCATTER: return dmq_gemm_launch_one<MODE, BIT, TT, DMQ_EPI_SCATTER, false>(L);
  }
  return DMQ_ERR_MODE;
}

template <int MODE, int BIT>
static int dmq_gemm_launch_tt(const GemmLaunch& L) {
  if (L.dbg && !(MODE == DMQ_MODE_A8 && L.tt == 1 && L.epi == DMQ_EPI_STORE)) return DMQ_ERR_MODE;
  switch (L.tt) {
    case 1: return dmq_gemm_launch_epi<MODE, BIT, 1>(L);
    case 2: return dmq_gemm_launch_epi<MODE, BIT, 2>(L);
    case 4: return dmq_gemm_launch_epi<MODE, BIT, 4>(L);
  }
  return DMQ_ERR_MODE;
}

template <int MODE>
static int dmq_gemm_launch_bits(const GemmLaunch& L) {
  switch (L.bit) {
    case 1: return dmq_gemm_launch_tt<MODE, 1>(L);
    case 2: return dmq_gemm_launch_tt<MODE, 2>(L);
    case 4: return dmq_gemm_launch_tt<MODE, 4>(L);
  }
  return DMQ_ERR_BIT;
}

// one definition per mode translation unit
int dmq_gemm_launch_a16(const GemmLaunch& L);
int dmq_gemm_launch_a8(const GemmLaunch& L);
int dmq_gemm_launch_fp8(const GemmLaunch& L);
int dmq_gemm_launch_fp4(const GemmLaunch& L);
