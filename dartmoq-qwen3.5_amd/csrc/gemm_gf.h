// Codebook-dequant GEMM over group-first packed weights (gfx950 MFMA).
//
//   out[r, n] = sum_g  s_a[r, g] * norm[g, n] * sum_{k<128} a[r, g, k] * LUT[idx[g, n, k]]
//
// One launch covers every bit pool of a layer: a work item is (pool, expert, tile of 16*TT
// activation rows) and a workgroup of four waves handles one item for one block of output
// features.  Inside the workgroup the waves split the output features (ROWPARTS) and / or the
// quantization groups (KS way split of K, reduced through LDS at the end); each wave owns NT
// tiles of 16 weight rows and TT tiles of 16 activation rows and walks its share of K one
// group (128 features) at a time:
//
//   * weights are the MFMA "A" operand: lane (n = lane % 16, q = lane / 16) owns the 32
//     features [32q, 32q+32) of row n inside the group, i.e. 4*BIT consecutive packed
//     bytes, fetched with one global load and expanded through the LDS byte table;
//   * activations are the "B" operand: lane (t = lane % 16, q) owns the same 32 features
//     of activation row t (64 B fp16, 32 B int8 / e4m3, 16 B packed e2m1);
//   * the 16x16 result tile has lane (t = lane % 16, q) holding rows n = 4q .. 4q+3, so
//     the per-group epilogue needs 4 consecutive norms and one activation scale per lane
//     and the final store is 4 consecutive output features of one activation row.
//
// The same mapping serves all four precision modes: a group is 4 MFMA steps of K=32
// (fp16, e4m3), 2 steps of K=64 (int8) or 1 MX-scaled step of K=128 (e2m1).
#pragma once
#include "common.h"
#include "lut.h"

#define DMQ_MAX_POOLS 4

struct PoolW {
  const uint8_t* w;            // [G_total, n_total, ppg] packed indices (FP4: folded e2m1, ppg = 64)
  const __half* norms;         // [G_total, n_total] fp16, already divided by sqrt(128)
  const void* lut;             // fp16 / int8 / e4m3 codebook (unused for FP4)
  const int* expert_info;      // [n_experts, 4] token_start, token_count, slice_start, slice_count
  const uint8_t* act;          // activation codes of this pool, row-major
  const void* act_scale;       // A8/FP8: fp16 [rows, stride]; FP4: u8 [rows, stride]
  const int* row_index;        // optional gather: physical activation row of logical row r
  int n_total;
  int bit;
  int mode;                    // items of pools whose mode differs from the kernel's are skipped
  int w_scale_byte;            // FP4: constant e8m0 byte of the weight blocks
};

struct GemmParams {
  PoolW pool[DMQ_MAX_POOLS];
  long act_row_bytes;
  int act_scale_stride;
  int groups;                  // groups contracted per expert (K / 128)
  int n_out;                   // output features per activation row
  int half_width;              // SiLU epilogue: I (gate rows [0,I), up rows [I,2I) of the slice)
  int slice_is_groups;         // 0: slice_start offsets weight rows; 1: offsets groups (down)
  // work list
  const int* items;            // [*, 4] pool, expert index, token tile inside the expert, unused
  const int* n_items;          // device scalar
  int n_blocks;                // workgroups along the output features
  // outputs
  __half* out;                 // STORE / SILU: fp16 [rows, out_stride]
  long out_stride;
  float* out_slots;            // SLOT: fp32 [rows, out_stride] addressed by row_slot[r]
  const float* row_weight;     // SLOT: routing weight of logical row r
  const int* row_slot;         // SLOT: destination row (token * top_k + slot) of logical row r
  int* dbg_acc;                // optional int32 [rows, groups, n_out] per-group accumulators (A8)
};

template <int MODE> struct ModeTraits;
template <> struct ModeTraits<DMQ_MODE_A16> {
  static constexpr int ES = 2, STEPS = 4, ACT_WORDS = 16; using acc_t = float4_t; };
template <> struct ModeTraits<DMQ_MODE_A8> {
  static constexpr int ES = 1, STEPS = 2, ACT_WORDS = 8; using acc_t = int4_t; };
template <> struct ModeTraits<DMQ_MODE_FP8> {
  static constexpr int ES = 1, STEPS = 4, ACT_WORDS = 8; using acc_t = float4_t; };
template <> struct ModeTraits<DMQ_MODE_FP4> {
  static constexpr int ES = 1, STEPS = 1, ACT_WORDS = 4; using acc_t = float4_t; };

// packed weight words a lane holds for one (group, n-tile)
template <int MODE, int BIT> struct WeightWords {
  static constexpr int N = (MODE == DMQ_MODE_FP4) ? 4 : BIT; };

template <int N> __device__ __forceinline__ void dmq_load_words(const uint8_t* p, uint32_t* d) {
  if (N == 1) { d[0] = *(const uint32_t*)p; }
  else if (N == 2) { uint2_t v = *(const uint2_t*)p; d[0] = v.x; d[1] = v.y; }
  else if (N == 4) { uint4_t v = *(const uint4_t*)p; d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w; }
  else {
#pragma unroll
    for (int i = 0; i < N; i += 4) {
      uint4_t v = *(const uint4_t*)(p + 4 * i);
      d[i] = v.x; d[i + 1] = v.y; d[i + 2] = v.z; d[i + 3] = v.w;
    }
  }
}

// Expand the packed bytes of MFMA step `s` into the lane's operand words.
template <int MODE, int BIT>
__device__ __forceinline__ void dmq_dequant_step(const uint8_t* tbl, uint32_t lane_base,
                                                 const uint32_t* pk, int s, uint32_t* w) {
  using T = ModeTraits<MODE>;
  using G = LutGeom<BIT, T::ES>;
  constexpr int BYTES = (4 * BIT) / T::STEPS;           // packed bytes per step
#pragma unroll
  for (int b = 0; b < BYTES; ++b) {
    const int bi = s * BYTES + b;
    const uint32_t byte = (pk[bi >> 2] >> ((bi & 3) * 8)) & 0xffu;
    if (G::EB >= 4) {
      dmq_lut_read<BIT, T::ES>(tbl, lane_base, byte, w + b * (G::EB / 4));
    } else {                                            // two one-byte elements per look-up
      uint32_t v;
      dmq_lut_read<BIT, T::ES>(tbl, lane_base, byte, &v);
      if (b & 1) w[b >> 1] |= v << 16; else w[b >> 1] = v;
    }
  }
}

// LDS needed by the K-split reduction: every wave parks NT*TT tiles of 64 lanes x 4 floats
template <int NT, int TT, int KS> struct RedGeom {
  static constexpr int FLOATS = (KS > 1) ? 4 * NT * TT * 256 : 4; };

template <int MODE, int BIT, int NT, int TT, int EPI, int KS, bool DBG>
__device__ __forceinline__ void dmq_gemm_body(const GemmParams& p, const PoolW& pw, uint8_t* tbl,
                                              float* red, int eidx, int ttile, int nb) {
  using T = ModeTraits<MODE>;
  using acc_t = typename T::acc_t;
  constexpr int WW = WeightWords<MODE, BIT>::N;
  constexpr int AW = T::ACT_WORDS;
  constexpr int ROWPARTS = 4 / KS;                                   // waves along the features
  constexpr int UNIT = (EPI == DMQ_EPI_SILU) ? 2 : 1;                // tiles finalized together
  constexpr int UNITS = NT / UNIT;
  constexpr int FEAT_TILES = NT / UNIT;                              // output tiles per wave
  constexpr int PPG = (MODE == DMQ_MODE_FP4) ? 64 : (DMQ_GS * BIT / 8);
  static_assert(NT % UNIT == 0, "SiLU epilogue pairs gate/up tiles");

  if (MODE != DMQ_MODE_FP4) dmq_lut_build<BIT, T::ES>(tbl, pw.lut);
  __syncthreads();

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const int kpart = wave % KS;
  const int rowpart = wave / KS;
  const uint32_t lane_base = (MODE == DMQ_MODE_FP4) ? 0u : dmq_lut_lane_base<BIT, T::ES>(lane);

  const int token_start = pw.expert_info[4 * eidx + 0];
  const int token_count = pw.expert_info[4 * eidx + 1];
  const int slice_start = pw.expert_info[4 * eidx + 2];

  const int feat0 = (nb * ROWPARTS + rowpart) * (FEAT_TILES * 16);   // first output feature of the wave
  const bool wave_active = feat0 < p.n_out;                          // wave-uniform

  // weight row of each n-tile
  int wrow[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (EPI == DMQ_EPI_SILU) wrow[j] = slice_start + ((j & 1) ? p.half_width : 0) + feat0 + (j >> 1) * 16;
    else wrow[j] = (p.slice_is_groups ? 0 : slice_start) + feat0 + j * 16;
  }
  const int g_base = p.slice_is_groups ? slice_start : 0;
  const int g_lo = (p.groups * kpart) / KS;
  const int g_hi = (p.groups * (kpart + 1)) / KS;

  // activation rows of each token tile
  const int r_first = token_start + ttile * (16 * TT);
  const int r_end = token_start + token_count;
  const uint8_t* arow[TT];
  bool avalid[TT];
  int rlog[TT];
  int rphys[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    rlog[t] = r_first + t * 16 + l16;
    avalid[t] = rlog[t] < r_end;
    rphys[t] = avalid[t] ? (pw.row_index ? pw.row_index[rlog[t]] : rlog[t]) : 0;
    arow[t] = pw.act + (long)rphys[t] * p.act_row_bytes + q * (AW * 4);
  }

  float4_t total_acc[NT][TT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < TT; ++t) total_acc[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};

  if (wave_active && g_lo < g_hi) {
    uint32_t pk_n[NT][WW];
    uint32_t xa_n[TT][AW];

    auto fetch = [&](int g) {
      const long gg = (long)(g_base + g) * pw.n_total;
#pragma unroll
      for (int j = 0; j < NT; ++j)
        dmq_load_words<WW>(pw.w + (gg + wrow[j] + l16) * PPG + q * (WW * 4), pk_n[j]);
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if (avalid[t]) {
          dmq_load_words<AW>(arow[t] + (long)g * (AW * 16), xa_n[t]);
        } else {
#pragma unroll
          for (int i = 0; i < AW; ++i) xa_n[t][i] = 0u;
        }
      }
    };

    fetch(g_lo);
    for (int g = g_lo; g < g_hi; ++g) {
      uint32_t pk[NT][WW];
      uint32_t xa[TT][AW];
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < WW; ++i) pk[j][i] = pk_n[j][i];
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int i = 0; i < AW; ++i) xa[t][i] = xa_n[t][i];

      // per-group scales: 4 consecutive norms per n-tile, one activation scale per token tile
      const long gg = (long)(g_base + g) * pw.n_total;
      float nrm[NT][4];
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        half4_t h = *(const half4_t*)(pw.norms + gg + wrow[j] + 4 * q);
        nrm[j][0] = (float)h[0]; nrm[j][1] = (float)h[1];
        nrm[j][2] = (float)h[2]; nrm[j][3] = (float)h[3];
      }
      float xs[TT];
      int xsb[TT];
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        xs[t] = 1.0f; xsb[t] = 127;
        if (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
          xs[t] = avalid[t] ? (float)((const __half*)pw.act_scale)[(long)rphys[t] * p.act_scale_stride + g]
                            : 0.f;
        } else if (MODE == DMQ_MODE_FP4) {
          if (avalid[t])
            xsb[t] = ((const uint8_t*)pw.act_scale)[(long)rphys[t] * p.act_scale_stride + g * 4 + q];
        }
      }

      if (g + 1 < g_hi) fetch(g + 1);

      acc_t acc[NT][TT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[j][t] = (acc_t){0, 0, 0, 0};

#pragma unroll
      for (int s = 0; s < T::STEPS; ++s) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          if constexpr (MODE == DMQ_MODE_A16) {
            uint32_t wq[4];
            dmq_dequant_step<MODE, BIT>(tbl, lane_base, pk[j], s, wq);
            half8_t a = __builtin_bit_cast(half8_t, (uint4_t){wq[0], wq[1], wq[2], wq[3]});
#pragma unroll
            for (int t = 0; t < TT; ++t) {
              half8_t b = __builtin_bit_cast(half8_t, (uint4_t){xa[t][4 * s], xa[t][4 * s + 1],
                                                                xa[t][4 * s + 2], xa[t][4 * s + 3]});
              acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[j][t], 0, 0, 0);
            }
          } else if constexpr (MODE == DMQ_MODE_A8) {
            uint32_t wq[4];
            dmq_dequant_step<MODE, BIT>(tbl, lane_base, pk[j], s, wq);
            int4_t a = {(int)wq[0], (int)wq[1], (int)wq[2], (int)wq[3]};
#pragma unroll
            for (int t = 0; t < TT; ++t) {
              int4_t b = {(int)xa[t][4 * s], (int)xa[t][4 * s + 1], (int)xa[t][4 * s + 2],
                          (int)xa[t][4 * s + 3]};
              acc[j][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[j][t], 0, 0, 0);
            }
          } else if constexpr (MODE == DMQ_MODE_FP8) {
            uint32_t wq[2];
            dmq_dequant_step<MODE, BIT>(tbl, lane_base, pk[j], s, wq);
            long a = (long)(((uint64_t)wq[1] << 32) | wq[0]);
#pragma unroll
            for (int t = 0; t < TT; ++t) {
              long b = (long)(((uint64_t)xa[t][2 * s + 1] << 32) | xa[t][2 * s]);
              acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, acc[j][t], 0, 0, 0);
            }
          } else {
            int8_t8 a = {(int)pk[j][0], (int)pk[j][1], (int)pk[j][2], (int)pk[j][3], 0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < TT; ++t) {
              int8_t8 b = {(int)xa[t][0], (int)xa[t][1], (int)xa[t][2], (int)xa[t][3], 0, 0, 0, 0};
              acc[j][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                  a, b, acc[j][t], 4, 4, 0, pw.w_scale_byte, 0, xsb[t]);
            }
          }
        }
      }

#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int t = 0; t < TT; ++t) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = (float)acc[j][t][r];
            if (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) v = v * xs[t];
            total_acc[j][t][r] += v * nrm[j][r];
          }
          if (DBG && MODE == DMQ_MODE_A8 && avalid[t]) {
            int4_t* d = (int4_t*)(p.dbg_acc + ((long)rlog[t] * p.groups + g) * p.n_out +
                                  feat0 + j * 16 + 4 * q);
            *d = __builtin_bit_cast(int4_t, acc[j][t]);
          }
        }
    }
  }

  // ------------------------------------------------------------------ K-split reduction
  // unit u (a tile, or a gate/up pair) is finalized by the wave with kpart == owner(u); the
  // other waves of the K group park their partial sums in LDS.
  if (KS > 1) {
    float4_t* red4 = (float4_t*)red;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int owner = ((j / UNIT) * KS) / UNITS;
      if (kpart != owner) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
          red4[((wave * NT + j) * TT + t) * 64 + lane] = total_acc[j][t];
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int owner = ((j / UNIT) * KS) / UNITS;
      if (kpart == owner) {
#pragma unroll
        for (int o = 0; o < KS; ++o) {
          if (o == owner) continue;
          const int src = rowpart * KS + o;
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            float4_t v = red4[((src * NT + j) * TT + t) * 64 + lane];
            total_acc[j][t] += v;
          }
        }
      }
    }
  }
  if (!wave_active) return;

  // ------------------------------------------------------------------ epilogue
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    if (!avalid[t]) continue;
#pragma unroll
    for (int j = 0; j < NT; j += UNIT) {
      if (KS > 1 && kpart != ((j / UNIT) * KS) / UNITS) continue;
      if (EPI == DMQ_EPI_STORE) {
        half4_t h = {(_Float16)total_acc[j][t][0], (_Float16)total_acc[j][t][1],
                     (_Float16)total_acc[j][t][2], (_Float16)total_acc[j][t][3]};
        *(half4_t*)(p.out + (long)rlog[t] * p.out_stride + feat0 + j * 16 + 4 * q) = h;
      } else if (EPI == DMQ_EPI_SILU) {
        half4_t h;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          h[r] = (_Float16)(dmq_silu(total_acc[j][t][r]) * total_acc[j + 1][t][r]);
        *(half4_t*)(p.out + (long)rlog[t] * p.out_stride + feat0 + (j >> 1) * 16 + 4 * q) = h;
      } else {
        const float rw = p.row_weight[rlog[t]];
        float4_t v = total_acc[j][t] * rw;
        *(float4_t*)(p.out_slots + (long)p.row_slot[rlog[t]] * p.out_stride + feat0 + j * 16 + 4 * q) = v;
      }
    }
  }
}

template <int MODE, int TT, int EPI, int KS, bool DBG>
__global__ __launch_bounds__(256)
void dmq_gemm_gf_kernel(GemmParams p) {
  constexpr int NT = 4;
  __shared__ __attribute__((aligned(16))) uint8_t tbl[(MODE == DMQ_MODE_FP4) ? 16 : DMQ_LUT_BYTES];
  __shared__ __attribute__((aligned(16))) float red[RedGeom<NT, TT, KS>::FLOATS];

  const int item = blockIdx.x / p.n_blocks;
  if (item >= p.n_items[0]) return;
  const int nb = blockIdx.x - item * p.n_blocks;
  const int pool = p.items[4 * item + 0];
  const int eidx = p.items[4 * item + 1];
  const int ttile = p.items[4 * item + 2];
  const PoolW& pw = p.pool[pool];
  if (pw.mode != MODE) return;
  if constexpr (MODE == DMQ_MODE_FP4) {
    dmq_gemm_body<MODE, 4, NT, TT, EPI, KS, DBG>(p, pw, tbl, red, eidx, ttile, nb);
    return;
  }
  switch (pw.bit) {
    case 1: dmq_gemm_body<MODE, 1, NT, TT, EPI, KS, DBG>(p, pw, tbl, red, eidx, ttile, nb); break;
    case 2: dmq_gemm_body<MODE, 2, NT, TT, EPI, KS, DBG>(p, pw, tbl, red, eidx, ttile, nb); break;
    default: dmq_gemm_body<MODE, 4, NT, TT, EPI, KS, DBG>(p, pw, tbl, red, eidx, ttile, nb); break;
  }
}
