// Dequant GEMV for a handful of routed rows (fp16 activations, 1/2/4-bit pools): the gate_up and
// down projections of a decode step of a few tokens (work items of at most four rows) as dot
// products on the vector ALU.
//
// With one to four rows per expert an MFMA tile is 1/16 to 1/4 full and the 16-row GEMM spends
// about four instructions per weight and lane on a work item that lives a few microseconds; here a
// wave owns 4 * FR output features (and, for gate_up, their up features), its 64 lanes split the
// K range of every feature 16 ways (lane = load round x 4 groups, feature, quarter of a group: 32
// weights = 16 BIT / 4 bytes per lane and group; FR = 4 / 2 / 1 for K = 512 / 1024 / more, so
// that a lane has at least four loads in flight), every load of the wave is requested before the
// first is used, a packed byte is expanded through a small table (256 entries of 8 / BIT fp16
// values, several copies side by side: see GemvGeom) and multiplied with `v_dot2_f32_f16`, the norm
// is applied to the fp32 sum of a
// (group, quarter) and the sixteen partial sums of a feature meet in four cross-lane adds.  Same
// work list, pools and outputs as dmq_gemm_gf_kernel with the SiLU resp. scatter epilogue (results
// agree to fp32 summation order; the norm is not folded into an fp16 operand here).
//
// gate_up with the down rotation fused (p.split_partial set): the rotation of a block of 128
// SiLU*up features is a sum over those features, so every workgroup applies the columns of the
// expert's 128 x 128 matrix that belong to its own 16 * FR features (rounded to fp16 first, as the
// stand-alone rotation reads them) and stores the 128 fp32 partial sums of each row in its own plane
// (plane = the workgroup's place among the 8 / FR of its block).  The down launch adds the planes
// of a row in plane order while it stages the row and rounds the sum to fp16: no tickets, no
// waiting, the same bits from run to run.
#include "gemm_gf.h"
#include "gemm_dispatch.h"

#define DMQ_GEMV_MAX_ROWS 4           // rows of one work item (an expert's rows: one per token)

typedef _Float16 half2_v __attribute__((ext_vector_type(2)));
using u64 = unsigned long long;

template <int BIT> struct GemvGeom {
  static constexpr int PPG = 16 * BIT;       // packed bytes of one (group, weight row)
  static constexpr int QB = PPG / 4;         // bytes of a quarter group: a lane's share
  static constexpr int EPB = 8 / BIT;        // weights per packed byte
  static constexpr int ENTRY = EPB * 2;      // bytes of a table entry
  // copies of the table, entry-major (entry e of copy c at (e * COPIES + c) * ENTRY): a lane reads
  // copy lane % COPIES, so lanes with different copies never meet in a bank
  static constexpr int COPIES = 64 / ENTRY;
};
#define DMQ_GEMV_LUT_BYTES (256 * 64)

// 32 weights of one quarter group (packed in `wq`) against the 32 activations `xv`: fp32 sum.
// lut: the lane's copy of the table (entries 64 bytes apart)
template <int BIT>
__device__ __forceinline__ float gemv_quarter(const uint32_t (&wq)[GemvGeom<BIT>::QB / 4], const half8_t (&xv)[4],
                                              const uint8_t* lut) {
  using GG = GemvGeom<BIT>;
  float s = 0.f;
#pragma unroll
  for (int b = 0; b < GG::QB; ++b) {
    const uint32_t byte = (wq[b >> 2] >> ((b & 3) * 8)) & 0xffu;
    if constexpr (BIT == 2) {
      const half4_t c = *(const half4_t*)(lut + byte * 64);
      const half8_t x = xv[b >> 1];
      const int o = (b & 1) * 4;
      s = __builtin_amdgcn_fdot2((half2_v){c[0], c[1]}, (half2_v){x[o], x[o + 1]}, s, false);
      s = __builtin_amdgcn_fdot2((half2_v){c[2], c[3]}, (half2_v){x[o + 2], x[o + 3]}, s, false);
    } else if constexpr (BIT == 4) {
      const half2_v c = *(const half2_v*)(lut + byte * 64);
      const half8_t x = xv[b >> 2];
      const int o = (b & 3) * 2;
      s = __builtin_amdgcn_fdot2(c, (half2_v){x[o], x[o + 1]}, s, false);
    } else {
      const half8_t c = *(const half8_t*)(lut + byte * 64);
      const half8_t x = xv[b];
#pragma unroll
      for (int i = 0; i < 8; i += 2)
        s = __builtin_amdgcn_fdot2((half2_v){c[i], c[i + 1]}, (half2_v){x[i], x[i + 1]}, s, false);
    }
  }
  return s;
}

// One work item x (four output features x FR) per wave.  NIT = groups / 4 load rounds.  The packed
// weights are requested first; the table and the activation rows are staged while they travel.
// ROT: gate_up with the partial down rotation (see the top of the file).
template <int BIT, int NIT, int FR, bool SILU, bool ROT>
__device__ __forceinline__ void gemv_body(const GemmParams& p, const PoolW& pw, uint8_t* xs, uint8_t* lut,
                                          __half* act_s, float* red, int token_start, int cnt, int slice_start,
                                          int post_slice, int wg) {
  using GG = GemvGeom<BIT>;
  constexpr int WQ = GG::QB / 4;
  constexpr int NM = SILU ? 2 : 1;                       // weight rows per feature: gate and up
  constexpr int WF = 16 * FR;                            // features of the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int f = (lane >> 2) & 3, qtr = lane & 3, gq = lane >> 4;
  const int n0 = wg * WF + wave * (4 * FR);              // first feature of the wave
  const long n_total = pw.n_total;
  const long row0 = (p.slice_is_groups ? 0 : slice_start) + n0 + f;
  const int g_base = p.slice_is_groups ? slice_start : 0;
  uint32_t wq[FR][NIT][NM][WQ];
  float nrm[FR][NIT][NM];
#pragma unroll
  for (int fr = 0; fr < FR; ++fr)
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const long gg = (long)(g_base + it * 4 + gq) * n_total;
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        const long row = row0 + fr * 4 + (m ? p.half_width : 0);
        dmq_load_words<WQ>(pw.w + (gg + row) * GG::PPG + qtr * GG::QB, wq[fr][it][m]);
        nrm[fr][it][m] = __half2float(pw.norms[gg + row]);
      }
    }
  // ROT: thread (c, part) applies matrix row c (output c of the block) to half of the workgroup's
  // features: WF / 2 matrix values, requested now
  constexpr int RK = WF / 2;                             // 8 * FR fp16 values = FR 16-byte pieces
  uint4_t rmat[FR];
  const int rc = threadIdx.x & 127, rpart = threadIdx.x >> 7;
  if constexpr (ROT) {
    const int blk = wg * WF / DMQ_GS;
    const __half* rrow = pw.post_rot + (long)(post_slice + blk) * (DMQ_GS * DMQ_GS) + (long)rc * DMQ_GS +
                         (wg * WF - blk * DMQ_GS) + rpart * RK;
#pragma unroll
    for (int i = 0; i < FR; ++i) rmat[i] = *(const uint4_t*)(rrow + 8 * i);
  }
  // scatter epilogue: routing weight and slot row of the item's rows
  float rw[DMQ_GEMV_MAX_ROWS];
  int rs[DMQ_GEMV_MAX_ROWS];
  if constexpr (!SILU) {
#pragma unroll
    for (int j = 0; j < DMQ_GEMV_MAX_ROWS; ++j) {
      const int r = token_start + (j < cnt ? j : 0);
      rw[j] = p.row_weight[r];
      rs[j] = p.row_slot[r];
    }
  }
  // table entry e: the codebook values of the 8 / BIT indices packed in byte value e, every copy
  {
    const uint32_t e = threadIdx.x;
    const uint16_t* cb = (const uint16_t*)pw.lut;
    uint16_t ent[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) ent[i] = cb[(e >> ((i % GG::EPB) * BIT)) & ((1u << BIT) - 1u)];
    const uint4_t line = *(const uint4_t*)ent;             // 16 bytes = 16 / ENTRY copies of the entry
#pragma unroll
    for (int c = 0; c < 4; ++c) *(uint4_t*)(lut + e * 64 + c * 16) = line;
  }
  const uint8_t* lut_lane = lut + (lane % GG::COPIES) * GG::ENTRY;
  // the item's activation rows: fp16 rows, or (down after a ROT gate_up) the sum of the planes
  constexpr int kbytes = NIT * 4 * DMQ_GS * 2;           // bytes of one staged activation row
  if (!SILU && p.split_partial != nullptr) {
    constexpr int KF = NIT * 4 * DMQ_GS;                 // features of a row
    const long plane = (long)p.split_rows * KF;
    for (int j = 0; j < cnt; ++j) {
      const float* src = p.split_partial + (long)(token_start + j) * KF;
      for (int o = threadIdx.x * 4; o < KF; o += 256 * 4) {
        float4_t sum = *(const float4_t*)(src + o);
        for (int pl = 1; pl < p.wsplit; ++pl) sum += *(const float4_t*)(src + pl * plane + o);
        *(half4_t*)(xs + j * kbytes + o * 2) = (half4_t){(_Float16)sum[0], (_Float16)sum[1], (_Float16)sum[2],
                                                        (_Float16)sum[3]};
      }
    }
  } else {
    for (int j = 0; j < cnt; ++j) {
      const int rlog = token_start + j;
      const long phys = pw.row_index ? pw.row_index[rlog] : rlog;
      const uint8_t* src = pw.act + phys * p.act_row_bytes;
      for (int o = threadIdx.x * 16; o < kbytes; o += 256 * 16)
        *(uint4_t*)(xs + j * kbytes + o) = *(const uint4_t*)(src + o);
    }
  }
  __syncthreads();
  // one row after the other (at most four): the packed weights stay in registers
  for (int j = 0; j < cnt; ++j) {
    float acc[FR][NM];
#pragma unroll
    for (int fr = 0; fr < FR; ++fr)
#pragma unroll
      for (int m = 0; m < NM; ++m) acc[fr][m] = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int g = it * 4 + gq;
      const uint8_t* xp = xs + j * kbytes + (g * DMQ_GS + qtr * 32) * 2;
      half8_t xv[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) xv[c] = *(const half8_t*)(xp + c * 16);
#pragma unroll
      for (int fr = 0; fr < FR; ++fr) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
          acc[fr][m] += gemv_quarter<BIT>(wq[fr][it][m], xv, lut_lane) * nrm[fr][it][m];
        // keep the look-ups of one round together: hoisted across rounds they would hold
        // hundreds of registers
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // the sixteen lanes of a feature differ in bits 0, 1 (quarter) and 4, 5 (group of the round)
    const int rlog = token_start + j;
    half4_t hq[FR];
#pragma unroll
    for (int fr = 0; fr < FR; ++fr) {
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        float v = acc[fr][m];
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        acc[fr][m] = v;
      }
      float v = acc[fr][0];
      if constexpr (SILU) v = dmq_silu(v) * acc[fr][NM - 1];
      else v *= rw[j];
      // the four features of the round meet in one lane
      hq[fr] = (half4_t){(_Float16)__shfl(v, 0, 64), (_Float16)__shfl(v, 4, 64), (_Float16)__shfl(v, 8, 64),
                         (_Float16)__shfl(v, 12, 64)};
    }
    // lane fr holds round fr: 8 * FR contiguous bytes per wave
    half4_t mine = hq[0];
#pragma unroll
    for (int fr = 1; fr < FR; ++fr) if (lane == fr) mine = hq[fr];
    if constexpr (ROT) {
      if (lane < FR) *(half4_t*)(act_s + j * WF + wave * (4 * FR) + lane * 4) = mine;
    } else if constexpr (SILU) {
      if (lane < FR) *(half4_t*)(p.out + (long)rlog * p.out_stride + n0 + lane * 4) = mine;
    } else {
      if (lane < FR) *(half4_t*)(p.out_slots + (long)rs[j] * p.out_stride + n0 + lane * 4) = mine;
    }
  }
  if constexpr (ROT) {
    __syncthreads();
    const int blk = wg * WF / DMQ_GS;
    const int plane_idx = wg - blk * (DMQ_GS / WF);
    const long plane = (long)p.split_rows * p.n_out;
    float part[DMQ_GEMV_MAX_ROWS];
#pragma unroll
    for (int j = 0; j < DMQ_GEMV_MAX_ROWS; ++j) {
      part[j] = 0.f;
      if (j < cnt) {
        const __half* arow = act_s + j * WF + rpart * RK;
#pragma unroll
        for (int i = 0; i < FR; ++i) {
          const half8_t m = __builtin_bit_cast(half8_t, rmat[i]);
          const half8_t a = *(const half8_t*)(arow + 8 * i);
#pragma unroll
          for (int e = 0; e < 8; ++e) part[j] = fmaf((float)a[e], (float)m[e], part[j]);
        }
      }
    }
    if (rpart == 1)
#pragma unroll
      for (int j = 0; j < DMQ_GEMV_MAX_ROWS; ++j) red[j * DMQ_GS + rc] = part[j];
    __syncthreads();
    if (rpart == 0)
#pragma unroll
      for (int j = 0; j < DMQ_GEMV_MAX_ROWS; ++j)
        if (j < cnt)
          p.split_partial[plane_idx * plane + (long)(token_start + j) * p.n_out + blk * DMQ_GS + rc] =
              part[j] + red[j * DMQ_GS + rc];
  }
}

template <int NIT> constexpr int gemv_fr() { return NIT >= 4 ? 1 : 4 / NIT; }

template <int NIT, bool SILU>
__global__ __launch_bounds__(256)
void dmq_gemv_kernel(GemmParams p, int max_items) {
  constexpr int FR = gemv_fr<NIT>();
  constexpr int XS_BYTES = DMQ_GEMV_MAX_ROWS * NIT * 4 * DMQ_GS * 2;
  __shared__ __attribute__((aligned(16))) uint8_t xs[XS_BYTES];
  __shared__ __attribute__((aligned(16))) uint8_t lut[DMQ_GEMV_LUT_BYTES];
  // rotating gate_up: the workgroup's SiLU*up values [rows][16 * FR] and the partial sums of the
  // upper half of its threads [rows][128]
  __shared__ __attribute__((aligned(16))) __half act_s[SILU ? DMQ_GEMV_MAX_ROWS * 16 * FR : 8];
  __shared__ float red[SILU ? DMQ_GEMV_MAX_ROWS * DMQ_GS : 1];
  const int wgs_per_item = p.n_out / (16 * FR);          // four waves of 4 * FR features
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
  const int post_slice = r1[1] / (2 * DMQ_GS);           // first down group of the item's expert
  const PoolW& pw = p.pool[pool];
  if (pw.mode != DMQ_MODE_A16 || pw.bit > 4) return;
  const int bit = pw.bit;
  const int wg = blockIdx.x - item * wgs_per_item;
  auto run = [&](auto rot_tag) __attribute__((always_inline)) {
    constexpr bool ROT = decltype(rot_tag)::value;
    if (bit == 2) gemv_body<2, NIT, FR, SILU, ROT>(p, pw, xs, lut, act_s, red, token_start, cnt, slice_start, post_slice, wg);
    else if (bit == 4) gemv_body<4, NIT, FR, SILU, ROT>(p, pw, xs, lut, act_s, red, token_start, cnt, slice_start, post_slice, wg);
    else gemv_body<1, NIT, FR, SILU, ROT>(p, pw, xs, lut, act_s, red, token_start, cnt, slice_start, post_slice, wg);
  };
  if constexpr (SILU) {
    if (p.split_partial != nullptr) { run(std::true_type{}); return; }
  }
  run(std::false_type{});
}

// rotate: the gate_up launch also rotates its rows for the down projection (whole blocks of 128)
bool dmq_gemv_shape_ok(int groups, int n_out, int rotate) {
  const int nit = groups / 4;
  if (groups % 4 || !(nit == 1 || nit == 2 || nit == 4 || nit == 6 || nit == 8)) return false;
  const int fr = nit >= 4 ? 1 : 4 / nit;
  return n_out % (16 * fr) == 0 && (!rotate || n_out % DMQ_GS == 0);
}

// planes a rotating gate_up launch over `groups` groups writes per block of 128 features
int dmq_gemv_planes(int groups) {
  const int fr = groups >= 16 ? 1 : (groups >= 8 ? 2 : 4);
  return DMQ_GS / (16 * fr);
}

template <int NIT>
static void gemv_launch_nit(const GemmParams& p, int silu, int max_items, hipStream_t stream) {
  const int grid = max_items * (p.n_out / (16 * gemv_fr<NIT>()));
  if (silu) hipLaunchKernelGGL((dmq_gemv_kernel<NIT, true>), dim3(grid), dim3(256), 0, stream, p, max_items);
  else hipLaunchKernelGGL((dmq_gemv_kernel<NIT, false>), dim3(grid), dim3(256), 0, stream, p, max_items);
}

// p as for dmq_gemm_gf_kernel (pools, items, outputs).  silu: gate_up with SiLU * up into p.out, or,
// with p.split_partial set, rotated for the down projection into the dmq_gemv_planes(p.groups)
// fp32 planes [p.split_rows, p.n_out] of p.split_partial (p.out is not written).  Otherwise the down
// projection scattered into p.out_slots; with p.split_partial set its input rows are the sums of
// the first p.wsplit such planes ([p.split_rows, 128 * p.groups] each) instead of the pools' act rows.
// max_items: records the launch may look at.
int dmq_gemv_launch(const GemmParams& p, int silu, int max_items, hipStream_t stream) {
  if (!dmq_gemv_shape_ok(p.groups, p.n_out, silu && p.split_partial)) return DMQ_ERR_SHAPE;
  if (max_items <= 0) return DMQ_OK;
  if ((long)max_items * (p.n_out / 16) > 0x7fffffffL) return DMQ_ERR_LIMIT;
  switch (p.groups / 4) {
    case 1: gemv_launch_nit<1>(p, silu, max_items, stream); break;
    case 2: gemv_launch_nit<2>(p, silu, max_items, stream); break;
    case 4: gemv_launch_nit<4>(p, silu, max_items, stream); break;
    case 6: gemv_launch_nit<6>(p, silu, max_items, stream); break;
    default: gemv_launch_nit<8>(p, silu, max_items, stream); break;
  }
  return dmq_check_launch();
}
