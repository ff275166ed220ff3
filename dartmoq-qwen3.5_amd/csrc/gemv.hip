// Dequant GEMV for a handful of routed rows (fp16 activations, 1/2/4-bit pools): the gate_up and
// down projections of a decode step of at most four tokens as dot products on the vector ALU.
//
// With one to four rows per expert an MFMA tile is 1/16 to 1/4 full and the 16-row GEMM spends
// about four instructions per weight and lane on a work item that lives a few microseconds; here a
// wave owns four output features (and, for gate_up, their four up features), its 64 lanes split the
// K range of every feature 16 ways (lane = load round x 4 groups, feature, quarter of a group: 32
// weights = 16 BIT / 4 bytes per lane and group), every load of the wave is requested before the
// first is used, a packed byte is expanded through a small table (256 entries of 8 / BIT fp16
// values, one copy) and multiplied with `v_dot2_f32_f16`, the norm is applied to the fp32 sum of a
// (group, quarter) and the sixteen partial sums of a feature meet in four cross-lane adds.  Same
// work list, pools and outputs as dmq_gemm_gf_kernel with the SiLU resp. scatter epilogue (results
// agree to fp32 summation order; the norm is not folded into an fp16 operand here).
#include "gemm_gf.h"
#include "gemm_dispatch.h"

#define DMQ_GEMV_MAX_ROWS 4           // rows of one work item (an expert's rows: one per token)

typedef _Float16 half2_v __attribute__((ext_vector_type(2)));

template <int BIT> struct GemvGeom {
  static constexpr int PPG = 16 * BIT;       // packed bytes of one (group, weight row)
  static constexpr int QB = PPG / 4;         // bytes of a quarter group: a lane's share
  static constexpr int EPB = 8 / BIT;        // weights per packed byte
  static constexpr int ENTRY = EPB * 2;      // bytes of a table entry
};

// 32 weights of one quarter group (packed in `wq`) against the 32 activations `xv`: fp32 sum
template <int BIT>
__device__ __forceinline__ float gemv_quarter(const uint32_t (&wq)[GemvGeom<BIT>::QB / 4], const half8_t (&xv)[4],
                                              const uint8_t* lut) {
  using GG = GemvGeom<BIT>;
  float s = 0.f;
#pragma unroll
  for (int b = 0; b < GG::QB; ++b) {
    const uint32_t byte = (wq[b >> 2] >> ((b & 3) * 8)) & 0xffu;
    if constexpr (BIT == 2) {
      const half4_t c = *(const half4_t*)(lut + byte * 8);
      const half8_t x = xv[b >> 1];
      const int o = (b & 1) * 4;
      s = __builtin_amdgcn_fdot2((half2_v){c[0], c[1]}, (half2_v){x[o], x[o + 1]}, s, false);
      s = __builtin_amdgcn_fdot2((half2_v){c[2], c[3]}, (half2_v){x[o + 2], x[o + 3]}, s, false);
    } else if constexpr (BIT == 4) {
      const half2_v c = *(const half2_v*)(lut + byte * 4);
      const half8_t x = xv[b >> 2];
      const int o = (b & 3) * 2;
      s = __builtin_amdgcn_fdot2(c, (half2_v){x[o], x[o + 1]}, s, false);
    } else {
      const half8_t c = *(const half8_t*)(lut + byte * 16);
      const half8_t x = xv[b];
#pragma unroll
      for (int i = 0; i < 8; i += 2)
        s = __builtin_amdgcn_fdot2((half2_v){c[i], c[i + 1]}, (half2_v){x[i], x[i + 1]}, s, false);
    }
  }
  return s;
}

// One work item x four output features per wave.  NIT = groups / 4 load rounds.
template <int BIT, int NIT, bool SILU>
__device__ __forceinline__ void gemv_body(const GemmParams& p, const PoolW& pw, const uint8_t* xs, const uint8_t* lut,
                                          int token_start, int cnt, int slice_start, int n0) {
  using GG = GemvGeom<BIT>;
  constexpr int WQ = GG::QB / 4;
  constexpr int NM = SILU ? 2 : 1;                       // weight rows per feature: gate and up
  const int lane = threadIdx.x & 63;
  const int f = (lane >> 2) & 3, qtr = lane & 3, gq = lane >> 4;
  const long n_total = pw.n_total;
  long row[NM];
  row[0] = (p.slice_is_groups ? 0 : slice_start) + n0 + f;
  if constexpr (SILU) row[1] = row[0] + p.half_width;
  const int g_base = p.slice_is_groups ? slice_start : 0;
  uint32_t wq[NIT][NM][WQ];
  float nrm[NIT][NM];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const long gg = (long)(g_base + it * 4 + gq) * n_total;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      dmq_load_words<WQ>(pw.w + (gg + row[m]) * GG::PPG + qtr * GG::QB, wq[it][m]);
      nrm[it][m] = __half2float(pw.norms[gg + row[m]]);
    }
  }
  constexpr int kbytes = NIT * 4 * DMQ_GS * 2;           // bytes of one staged activation row
  // one row after the other (at most four): the packed weights stay in registers
  for (int j = 0; j < cnt; ++j) {
    float acc[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) acc[m] = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int g = it * 4 + gq;
      const uint8_t* xp = xs + j * kbytes + (g * DMQ_GS + qtr * 32) * 2;
      half8_t xv[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) xv[c] = *(const half8_t*)(xp + c * 16);
#pragma unroll
      for (int m = 0; m < NM; ++m)
        acc[m] += gemv_quarter<BIT>(wq[it][m], xv, lut) * nrm[it][m];
      // keep the look-ups of one round together: hoisted across rounds they would hold
      // hundreds of registers
      __builtin_amdgcn_sched_barrier(0);
    }
    // the sixteen lanes of a feature differ in bits 0, 1 (quarter) and 4, 5 (group of the round)
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      float v = acc[m];
      v += __shfl_xor(v, 1, 64);
      v += __shfl_xor(v, 2, 64);
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      acc[m] = v;
    }
    if (qtr == 0 && gq == 0) {
      const int rlog = token_start + j;
      if constexpr (SILU) {
        p.out[(long)rlog * p.out_stride + n0 + f] = (__half)(_Float16)(dmq_silu(acc[0]) * acc[NM - 1]);
      } else {
        const float v = acc[0] * p.row_weight[rlog];
        p.out_slots[(long)p.row_slot[rlog] * p.out_stride + n0 + f] = (__half)(_Float16)v;
      }
    }
  }
}

template <int NIT, bool SILU>
__global__ __launch_bounds__(256)
void dmq_gemv_kernel(GemmParams p, int max_items) {
  __shared__ __attribute__((aligned(16))) uint8_t xs[DMQ_GEMV_MAX_ROWS * NIT * 4 * DMQ_GS * 2];
  __shared__ __attribute__((aligned(16))) uint8_t lut[256 * 16];
  const int wgs_per_item = p.n_out / 16;                 // four waves of four features
  const int item = blockIdx.x / wgs_per_item;
  if (item >= max_items || item >= p.n_items[0]) return;
  const int4_t* rec = (const int4_t*)(p.items + (long)DMQ_ITEM_WORDS * item);
  const int4_t r0 = rec[0];
  const int4_t r1 = rec[1];
  const int pool = r0[0];
  const int token_start = r0[3];
  const int cnt = min(r1[0], DMQ_GEMV_MAX_ROWS);
  if (cnt <= 0 || r0[2] != 0) return;                    // not the first record of its expert
  const int slice_start = p.slice_is_groups ? r1[2] : r1[1];
  const PoolW& pw = p.pool[pool];
  if (pw.mode != DMQ_MODE_A16 || pw.bit > 4) return;
  const int bit = pw.bit;
  // table entry e: the codebook values of the 8 / bit indices packed in byte value e
  {
    const uint32_t e = threadIdx.x;
    const uint16_t* cb = (const uint16_t*)pw.lut;
    const uint32_t mask = (1u << bit) - 1u;
    const int epb = 8 / bit;
    uint16_t* dst = (uint16_t*)(lut + e * (epb * 2));
    for (int i = 0; i < epb; ++i) dst[i] = cb[(e >> (i * bit)) & mask];
  }
  // the item's activation rows
  constexpr int kbytes = NIT * 4 * DMQ_GS * 2;
  for (int j = 0; j < cnt; ++j) {
    const int rlog = token_start + j;
    const long phys = pw.row_index ? pw.row_index[rlog] : rlog;
    const uint8_t* src = pw.act + phys * p.act_row_bytes;
    for (int o = threadIdx.x * 16; o < kbytes; o += 256 * 16)
      *(uint4_t*)(xs + j * kbytes + o) = *(const uint4_t*)(src + o);
  }
  __syncthreads();
  const int n0 = ((blockIdx.x - item * wgs_per_item) * 4 + (threadIdx.x >> 6)) * 4;
  if (bit == 2) gemv_body<2, NIT, SILU>(p, pw, xs, lut, token_start, cnt, slice_start, n0);
  else if (bit == 4) gemv_body<4, NIT, SILU>(p, pw, xs, lut, token_start, cnt, slice_start, n0);
  else gemv_body<1, NIT, SILU>(p, pw, xs, lut, token_start, cnt, slice_start, n0);
}

bool dmq_gemv_shape_ok(int groups, int n_out) {
  const int nit = groups / 4;
  return groups % 4 == 0 && (nit == 1 || nit == 2 || nit == 4 || nit == 6 || nit == 8) && n_out % 16 == 0;
}

template <int NIT>
static void gemv_launch_nit(const GemmParams& p, int silu, int max_items, int grid, hipStream_t stream) {
  if (silu) hipLaunchKernelGGL((dmq_gemv_kernel<NIT, true>), dim3(grid), dim3(256), 0, stream, p, max_items);
  else hipLaunchKernelGGL((dmq_gemv_kernel<NIT, false>), dim3(grid), dim3(256), 0, stream, p, max_items);
}

// p as for dmq_gemm_gf_kernel (pools, items, outputs); silu: gate_up with SiLU * up into p.out, else
// the down projection scattered into p.out_slots.  max_items: records the launch may look at.
int dmq_gemv_launch(const GemmParams& p, int silu, int max_items, hipStream_t stream) {
  if (!dmq_gemv_shape_ok(p.groups, p.n_out)) return DMQ_ERR_SHAPE;
  if (max_items <= 0) return DMQ_OK;
  const long grid = (long)max_items * (p.n_out / 16);
  if (grid > 0x7fffffffL) return DMQ_ERR_LIMIT;
  switch (p.groups / 4) {
    case 1: gemv_launch_nit<1>(p, silu, max_items, (int)grid, stream); break;
    case 2: gemv_launch_nit<2>(p, silu, max_items, (int)grid, stream); break;
    case 4: gemv_launch_nit<4>(p, silu, max_items, (int)grid, stream); break;
    case 6: gemv_launch_nit<6>(p, silu, max_items, (int)grid, stream); break;
    default: gemv_launch_nit<8>(p, silu, max_items, (int)grid, stream); break;
  }
  return dmq_check_launch();
}
