// Host-side dispatch of dmq_gemm_gf_kernel instantiations for one precision mode.
// Each mode lives in its own translation unit so the modes compile in parallel.
#pragma once
#include "gemm_gf.h"

struct GemmLaunch {
  GemmParams p;
  int epi;
  int tt;          // activation tiles of 16 rows per wave: 1, 2 or 4
  int ks;          // waves splitting K: 1, 2 or 4
  int dbg;
  int wide;        // 1: the pools of 8-bit indices (ks must be 1 unless nt == 1), 0: the 1/2/4-bit pools,
                   // 2: both in one launch (tt == 1, ks == 1, epilogues other than the plain store)
  int nt;          // n-tiles per wave: 4, or 1 (plain store, tt == 1, ks == 4 only)
  int roomy;       // tt == 1, ks == 1: the two-waves-per-SIMD instance (see ROOMY)
  int mode2;       // -1, or DMQ_MODE_A16 next to a quantized mode (tt == 1, ks == 1, no 8-bit pools: see MODE2)
  int grid;
  hipStream_t stream;
};

// instantiated (tt, ks) pairs: 16-row tiles with K split over the waves (1,4) or not (1,1),
// 32- and 64-row tiles with LDS-staged activations (2,1) (4,1)
static inline bool dmq_gemm_config_ok(int tt, int ks) {
  return (tt == 1 && (ks == 4 || ks == 1)) || (tt == 2 && ks == 1) || (tt == 4 && ks == 1);
}

template <int MODE, int TT, int KS, int EPI, bool DBG>
static int dmq_gemm_launch_one(const GemmLaunch& L) {
  if constexpr (MODE != DMQ_MODE_FP4 && TT == 1 && KS == 1 && !DBG && EPI != DMQ_EPI_STORE) {
    if (L.wide == 2) {
      if (L.mode2 >= 0) return DMQ_ERR_MODE;
      hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, TT, EPI, KS, DBG, 2>), dim3(L.grid), dim3(256), 0,
                         L.stream, L.p);
      return dmq_check_launch();
    }
  }
  if (L.wide == 2) return DMQ_ERR_MODE;
  if constexpr (MODE != DMQ_MODE_FP4 && KS == 1 && !DBG) {
    if (L.wide) {
      if (L.mode2 >= 0) return DMQ_ERR_MODE;
      hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, TT, EPI, KS, DBG, true>), dim3(L.grid), dim3(256), 0,
                         L.stream, L.p);
      return dmq_check_launch();
    }
  }
  if (L.wide) return DMQ_ERR_MODE;
  if constexpr (MODE != DMQ_MODE_A16 && TT <= 2 && KS == 1 && !DBG && EPI != DMQ_EPI_STORE) {
    if (L.mode2 == DMQ_MODE_A16) {     // both instances, picked like those of a single mode
      if (TT == 1 && (L.roomy || MODE == DMQ_MODE_FP4))
        hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, TT, EPI, KS, DBG, false, 4, true, DMQ_MODE_A16>),
                           dim3(L.grid), dim3(256), 0, L.stream, L.p);
      else
        hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, TT, EPI, KS, DBG, false, 4, false, DMQ_MODE_A16>),
                           dim3(L.grid), dim3(256), 0, L.stream, L.p);
      return dmq_check_launch();
    }
  }
  if (L.mode2 >= 0) return DMQ_ERR_MODE;
  if constexpr (MODE != DMQ_MODE_FP4 && TT == 1 && KS == 1 && !DBG) {
    if (L.roomy) {
      hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, TT, EPI, KS, DBG, false, 4, true>), dim3(L.grid),
                         dim3(256), 0, L.stream, L.p);
      return dmq_check_launch();
    }
  }
  hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, TT, EPI, KS, DBG, false>), dim3(L.grid), dim3(256), 0,
                     L.stream, L.p);
  return dmq_check_launch();
}

template <int MODE, int TT, int KS>
static int dmq_gemm_launch_epi(const GemmLaunch& L) {
  switch (L.epi) {
    case DMQ_EPI_STORE:
      if constexpr (MODE == DMQ_MODE_A8 && KS == 1) {      // 16-, 32- and 64-row tiles
        if (L.dbg) return dmq_gemm_launch_one<MODE, TT, KS, DMQ_EPI_STORE, true>(L);
      }
      return dmq_gemm_launch_one<MODE, TT, KS, DMQ_EPI_STORE, false>(L);
    case DMQ_EPI_SILU: return dmq_gemm_launch_one<MODE, TT, KS, DMQ_EPI_SILU, false>(L);
    case DMQ_EPI_SILU_ROT:
      if constexpr (KS == 1) return dmq_gemm_launch_one<MODE, TT, KS, DMQ_EPI_SILU_ROT, false>(L);
      return DMQ_ERR_MODE;
    case DMQ_EPI_SCATTER: return dmq_gemm_launch_one<MODE, TT, KS, DMQ_EPI_SCATTER, false>(L);
  }
  return DMQ_ERR_MODE;
}

// one n-tile per wave, K split over the four waves: the launch of a Linear with few rows
template <int MODE>
static int dmq_gemm_launch_narrow(const GemmLaunch& L) {
  if constexpr (MODE != DMQ_MODE_FP4) {
    if (L.wide)
      hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, 1, DMQ_EPI_STORE, 4, false, true, 1>), dim3(L.grid),
                         dim3(256), 0, L.stream, L.p);
    else
      hipLaunchKernelGGL((dmq_gemm_gf_kernel<MODE, 1, DMQ_EPI_STORE, 4, false, false, 1>), dim3(L.grid),
                         dim3(256), 0, L.stream, L.p);
    return dmq_check_launch();
  }
  return DMQ_ERR_MODE;
}

template <int MODE>
static int dmq_gemm_launch_mode(const GemmLaunch& L) {
  if (L.nt == 1) {
    if (L.tt != 1 || L.ks != 4 || L.epi != DMQ_EPI_STORE || L.dbg) return DMQ_ERR_MODE;
    return dmq_gemm_launch_narrow<MODE>(L);
  }
  if (L.dbg && !(MODE == DMQ_MODE_A8 && L.ks == 1 && L.epi == DMQ_EPI_STORE))
    return DMQ_ERR_MODE;
  if (L.tt == 1 && L.ks == 4) return dmq_gemm_launch_epi<MODE, 1, 4>(L);
  if (L.tt == 1 && L.ks == 1) return dmq_gemm_launch_epi<MODE, 1, 1>(L);
  if (L.tt == 2 && L.ks == 1) return dmq_gemm_launch_epi<MODE, 2, 1>(L);
  if (L.tt == 4 && L.ks == 1) return dmq_gemm_launch_epi<MODE, 4, 1>(L);
  return DMQ_ERR_MODE;
}

// one definition per mode translation unit
int dmq_gemm_launch_a16(const GemmLaunch& L);
int dmq_gemm_launch_a8(const GemmLaunch& L);
int dmq_gemm_launch_fp8(const GemmLaunch& L);
int dmq_gemm_launch_fp4(const GemmLaunch& L);
// persistent launch over work items of 128 rows, fp16 pools of 1/2/4-bit indices (gemm_rows.h);
// nbl: feature blocks per unit; queue: DMQ_ROWS_QUEUE_WORDS zeroed device words
int dmq_gemm_rows_launch(const GemmParams& p, int epi, int* queue, int nbl, hipStream_t stream);

// dot-product launch for work items of at most four rows (csrc/gemv.hip)
#define DMQ_GEMV_MAX_TOKENS 2
#define DMQ_GEMV_CUS 256          // compute units of an MI355X
bool dmq_gemv_shape_ok(int groups, int n_out, int rotate);
int dmq_gemv_planes(int groups);
int dmq_gemv_launch(const GemmParams& p, int silu, int max_items, hipStream_t stream);
