// Codebook-dequant GEMM over group-first packed weights (gfx950 MFMA).
//
//   out[r, n] = sum_g  s_a[r, g] * norm[g, n] * sum_{k<128} a[r, g, k] * LUT[idx[g, n, k]]
//
// One launch covers every bit pool of a layer: a work item is (pool, expert, tile of 16*TT
// activation rows) and a workgroup of four waves handles one item for one block of output
// features.  Each wave owns NT tiles of 16 weight rows and TT tiles of 16 activation rows and
// walks K one quantization group (128 features) at a time:
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
//
// Two ways of feeding the waves, chosen by the K split KS:
//   KS > 1  (few activation rows, HBM-bound on the packed weights): the four waves share the
//           weight rows and split the groups; every wave issues the loads of its whole K
//           slice (up to PF groups) before computing, so one memory latency covers the
//           slice, and the partial sums meet in LDS at the end.
//   KS == 1 (many activation rows): the waves take different weight rows and share the
//           activation tile, which is staged once per group in LDS (double buffered,
//           16-byte chunks XOR-swizzled by row so the operand reads spread over the banks).
#pragma once
#include "common.h"
#include <type_traits>
#include "lut.h"


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
  // DMQ_EPI_SILU_ROT: rotation matrices [groups_total, 128, 128] fp16 applied to the SiLU*up rows
  // (matrix of block b of an item = post_rot[item's down slice + b]) and the scale factor folded
  // into the stored activation scale
  const __half* post_rot;
  float post_extra;
  // layers whose experts are cut into sub-experts living in several pools (width_filter != 0):
  // first activation column of the pool's share of each expert (act / post_out columns of the
  // gate_up launch, contracted columns of the down launch) and the expert's rank among the pools
  // that hold a share of it
  const int* col_start;        // [n_experts] or NULL (0)
  const int* home;             // [n_experts] or NULL (0)
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
  const int* items;            // [max_items, DMQ_ITEM_WORDS] work-item records, meaningful below n_items
  const int* n_items;          // device scalar
  int n_blocks;                // blocks of output features per item
  int nbl;                     // consecutive blocks one workgroup walks (1 unless KS == 1)
  int subs;                    // row tiles of this launch per work item (item rows / (16 * TT))
  int tail_slots;              // > 0: the last tail_slots blocks of every XCD's share go one per
                               // workgroup (nbl > 1, nbl divides n_blocks, wsplit == 1)
  // outputs
  __half* out;                 // STORE / SILU: fp16 [rows, out_stride]
  long out_stride;
  __half* out_slots;           // SCATTER: fp16 [slots, out_stride] addressed by row_slot[r]
  const float* row_weight;     // SCATTER: routing weight of logical row r
  const int* row_slot;         // SCATTER: destination row (token * top_k + slot) of logical row r
  int* dbg_acc;                // optional int32 [rows, groups, n_out] per-group accumulators (A8)
  // DMQ_EPI_SILU_ROT: rotated (+ quantized) rows: codes [rows, post_row_bytes], scales
  uint8_t* post_out;
  long post_row_bytes;
  void* post_scale;            // A8/FP8: fp16 [rows, post_scale_stride]; FP4: u8 [rows, post_scale_stride]
  int post_scale_stride;
  // K range of one (item, block) shared by wsplit workgroups (16-row tiles, SiLU and plain-store
  // epilogues): each parks its fp32 sums in its plane of split_partial and takes a ticket; the
  // last one adds the planes in plane order and runs the epilogue
  // Sub-expert layers: a launch serves the (pool, expert) shares of one width (and, for the down
  // projection, of one home rank); it skips work items whose slice count (expert_info[e][3]) differs
  // from width_filter (0 = take all) or whose rank differs from home_filter (< 0 = take all).
  // accumulate (SCATTER): add to the slot row instead of storing it (ranks above 0).
  int width_filter;
  int home_filter;
  int accumulate;
  int wsplit;                  // 1, 2, 4, 8 or 16
  int split_items;             // > 0: only the first min(n_items[1], split_items) items share K
  int spread;                  // work item i on XCD i % 8 instead of a contiguous share per XCD (nbl == 1)
  int split_rows;              // rows of one plane
  float* split_partial;        // fp32 [wsplit, split_rows, 2 * n_out (SiLU) or n_out (store)]
  int* split_counter;          // int32 [max_items * n_blocks], zero before the launch and after it
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

// Expand the packed bytes of MFMA step S into the lane's operand words.
// IDENT (int8 operands, 8-bit indices): the table is the identity w = idx - 128 of a uniform
// codebook, so the operand bytes are the index bytes with the top bit flipped and no table is read.
template <int MODE, int BIT, int S, bool IDENT = false, int ROW = DMQ_LUT_ROW>
__device__ __forceinline__ void dmq_dequant_step(const uint8_t* tbl, uint32_t lane_base,
                                                 const uint32_t* pk, uint32_t* w) {
  using T = ModeTraits<MODE>;
  using G = LutGeom<BIT, T::ES, ROW>;
  constexpr int BYTES = (4 * BIT) / T::STEPS;           // packed bytes per step
  if constexpr (IDENT) {
    static_assert(MODE == DMQ_MODE_A8 && BIT == 8, "identity table: int8 operands, 8-bit indices");
#pragma unroll
    for (int i = 0; i < BYTES / 4; ++i) w[i] = pk[S * (BYTES / 4) + i] ^ 0x80808080u;
    return;
  }
  auto one = [&](auto bc) {
    constexpr int b = decltype(bc)::value;
    constexpr int bi = S * BYTES + b;
    if constexpr (G::EB >= 4) {
      dmq_lut_read_word<BIT, T::ES, (bi & 3), ROW>(tbl, lane_base, pk[bi >> 2], w + b * (G::EB / 4));
    } else if constexpr (G::EB == 2) {                  // two two-byte entries per operand word
      uint32_t v;
      dmq_lut_read_word<BIT, T::ES, (bi & 3), ROW>(tbl, lane_base, pk[bi >> 2], &v);
      if (b & 1) w[b >> 1] |= v << 16; else w[b >> 1] = v;
    } else {                                            // four one-byte entries per operand word
      uint32_t v;
      dmq_lut_read_word<BIT, T::ES, (bi & 3), ROW>(tbl, lane_base, pk[bi >> 2], &v);
      if (b & 3) w[b >> 2] |= v << (8 * (b & 3)); else w[b >> 2] = v;
    }
  };
  one(std::integral_constant<int, 0>{});
  if constexpr (BYTES > 1) one(std::integral_constant<int, 1>{});
  if constexpr (BYTES > 2) { one(std::integral_constant<int, 2>{}); one(std::integral_constant<int, 3>{}); }
  if constexpr (BYTES > 4) {
    one(std::integral_constant<int, 4>{}); one(std::integral_constant<int, 5>{});
    one(std::integral_constant<int, 6>{}); one(std::integral_constant<int, 7>{});
  }
  if constexpr (BYTES > 8) {
    one(std::integral_constant<int, 8>{}); one(std::integral_constant<int, 9>{});
    one(std::integral_constant<int, 10>{}); one(std::integral_constant<int, 11>{});
    one(std::integral_constant<int, 12>{}); one(std::integral_constant<int, 13>{});
    one(std::integral_constant<int, 14>{}); one(std::integral_constant<int, 15>{});
  }
  static_assert(BYTES <= 16, "at most sixteen packed bytes per MFMA step");
}

// Groups in flight per wave on the staged path.  WW registers hold one (group, n-tile) of packed
// weights.  Rings of 8 words (16-row tiles) and 4 words (32-row tiles) keep three resp. two
// workgroups resident per CU; deeper rings cost a workgroup of occupancy and measured slower.
#define DMQ_XCDS 8          // accelerator dies of an MI355X; the grid is a multiple of it
#define DMQ_KOUT 1
#define DMQ_KOUT_MIN_TT 2
#define DMQ_FOLD_MIN_TT 2
#define DMQ_RING_TT1 8
#define DMQ_RING_TT2 4
#define DMQ_RING_TT4 4
template <int WW, int TT> constexpr int dmq_ring_depth() {
  constexpr int words = (TT == 1) ? DMQ_RING_TT1 : (TT == 2 ? DMQ_RING_TT2 : DMQ_RING_TT4);
  constexpr int d = words / WW;                     // words of packed weights per n-tile in flight
  return d < 2 ? 2 : (d > 8 ? 8 : d);
}

// Tiling facts shared by the kernel and its host launcher.
// Bytes of LDS the fused down-rotation epilogue needs beyond the staging slots: the fp16 SiLU*up
// tile of the block (16*TT rows x 256 B; fp16 layers reuse a staging slot of that very size) and
// the per-wave row maxima of the quantizers.
template <int MODE, int TT, int EPI> struct PostGeom {
  static constexpr bool ON = (EPI == DMQ_EPI_SILU_ROT);
  static constexpr int TILE = (ON && MODE != DMQ_MODE_A16) ? 16 * TT * 256 : 0;
  static constexpr int WMAX = (ON && MODE != DMQ_MODE_A16) ? 4 * 16 * TT * 4 : 0;
  static constexpr int BYTES = (TILE + WMAX) > 16 ? (TILE + WMAX) : 16;
};

template <int MODE, int NT, int TT, int KS> struct GemmGeom {
  static constexpr int AW = ModeTraits<MODE>::ACT_WORDS;          // activation words per lane and group
  static constexpr int AB = AW * 16;                              // activation bytes per row and group
  static constexpr bool STAGE = (KS == 1);                        // activations through LDS
  // direct path: groups in flight (a wave with a single n-tile keeps eight: its registers allow it
  // and a 4096-wide K split over four waves is then one round trip)
  static constexpr int PF = (NT == 1) ? 8 : 4;
  // staged path: one LDS slot = activation tile + norms of the 64*NT weight rows + tile scales
  static constexpr int SLOT = 16 * TT * AB + 128 * NT + 64 * TT;
  static constexpr int STAGE_BYTES = STAGE ? 2 * SLOT : 0;
  static constexpr int RED_BYTES = (KS > 1) ? 4 * NT * TT * 1024 : 0;
  static constexpr int SMEM2 = STAGE_BYTES > RED_BYTES ? (STAGE_BYTES > 16 ? STAGE_BYTES : 16)
                                                       : (RED_BYTES > 16 ? RED_BYTES : 16);
};

template <int MODE, int BIT, int NT, int TT, int EPI, int KS, bool DBG, bool IDENT = false,
          int ROW = DMQ_LUT_ROW, bool AHEAD = false>
__device__ __forceinline__ void dmq_gemm_body(const GemmParams& p, const PoolW& pw, uint8_t* tbl,
                                              uint8_t* smem2, uint8_t* smem_post, int token_start,
                                              int token_count, int slice_start, int post_slice,
                                              int ttile, int nb, int nbc, int split, int* ticket,
                                              int* wg_flag, int col0) {
  // split: index of this workgroup among those sharing the K range (low byte) and their number
  const int nsplit_in = split >> 8;
  split &= 0xff;
  using T = ModeTraits<MODE>;
  using acc_t = typename T::acc_t;
  using GG = GemmGeom<MODE, NT, TT, KS>;
  constexpr int WW = WeightWords<MODE, BIT>::N;
  constexpr int AW = GG::AW;
  constexpr int AB = GG::AB;
  constexpr bool STAGE = GG::STAGE;
  constexpr int PF = GG::PF;
  constexpr int ROWPARTS = 4 / KS;                                   // waves along the features
  constexpr bool SILU = (EPI == DMQ_EPI_SILU || EPI == DMQ_EPI_SILU_ROT);
  constexpr int UNIT = SILU ? 2 : 1;                                 // tiles finalized together
  constexpr int UNITS = NT / UNIT;
  constexpr int FEAT_TILES = NT / UNIT;                              // output tiles per wave
  constexpr int PPG = (MODE == DMQ_MODE_FP4) ? 64 : (DMQ_GS * BIT / 8);
  constexpr int FPB = ROWPARTS * FEAT_TILES * 16;                    // output features per n-block
  // K range shared across workgroups
  constexpr bool XSPLIT = STAGE && TT == 1 && (SILU || EPI == DMQ_EPI_STORE);
  static_assert(NT % UNIT == 0, "SiLU epilogue pairs gate/up tiles");

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const int kpart = wave % KS;
  const int rowpart = wave / KS;
  const uint32_t lane_base = (MODE == DMQ_MODE_FP4) ? 0u : dmq_lut_lane_base<BIT, T::ES, ROW>(lane);

  const int feat0 = (nb * ROWPARTS + rowpart) * (FEAT_TILES * 16);   // first output feature of the wave
  const bool wave_active = feat0 < p.n_out;                          // wave-uniform
  int feat_k = feat0;                                                // same, for the n-block in progress

  // weight row of each n-tile (inactive waves alias the first block; they never store)
  const int featw = wave_active ? feat0 : 0;
  int wrow[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (SILU) wrow[j] = slice_start + ((j & 1) ? p.half_width : 0) + featw + (j >> 1) * 16;
    else wrow[j] = (p.slice_is_groups ? 0 : slice_start) + featw + j * 16;
  }
  const int g_base = p.slice_is_groups ? slice_start : 0;
  // sub-expert layers: the down launch contracts the expert's columns from col0 on (whole groups),
  // the gate_up launch writes its SiLU*up columns from col0 on
  const int in_group0 = p.slice_is_groups ? col0 / DMQ_GS : 0;
  const int out_col0 = p.slice_is_groups ? 0 : col0;
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
    arow[t] = pw.act + (long)rphys[t] * p.act_row_bytes + q * (AW * 4) + in_group0 * AB;
  }

  // scatter epilogue: routing weight and destination row of the lane's rows, requested now so that
  // the epilogue does not end on a memory round trip (rows past the item take its last row's)
  float row_w[TT];
  int row_dst[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) { row_w[t] = 0.f; row_dst[t] = 0; }
  if constexpr (EPI == DMQ_EPI_SCATTER) {
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const int rr = min(rlog[t], r_end - 1);
      row_w[t] = p.row_weight[rr];
      row_dst[t] = p.row_slot[rr];
    }
  }

  float4_t total_acc[NT][TT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < TT; ++t) total_acc[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};

  // ---- loads of one group: packed weights, norms, activation scales (+ activations when direct)
  auto load_weights = [&](int g, uint32_t (&pk)[NT][WW], uint2_t (&nr)[NT]) {
    const long gg = (long)(g_base + g) * pw.n_total;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      dmq_load_words<WW>(pw.w + (gg + wrow[j] + l16) * PPG + q * (WW * 4), pk[j]);
      nr[j] = *(const uint2_t*)(pw.norms + gg + wrow[j] + 4 * q);
    }
  };
  auto load_scales = [&](int g, float (&xs)[TT], int (&xsb)[TT]) {
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      xs[t] = 1.0f; xsb[t] = 127;
      if (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
        xs[t] = avalid[t] ? (float)((const __half*)pw.act_scale)[(long)rphys[t] * p.act_scale_stride + in_group0 + g]
                          : 0.f;
      } else if (MODE == DMQ_MODE_FP4) {
        if (avalid[t])
          xsb[t] = ((const uint8_t*)pw.act_scale)[(long)rphys[t] * p.act_scale_stride + (in_group0 + g) * 4 + q];
      }
    }
  };
  auto load_acts = [&](int g, uint32_t (&xa)[TT][AW]) {
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      if (avalid[t]) {
        dmq_load_words<AW>(arow[t] + (long)g * (AW * 16), xa[t]);
      } else {
#pragma unroll
        for (int i = 0; i < AW; ++i) xa[t][i] = 0u;
      }
    }
  };

  // ---- MFMA work of one group
  // The look-ups of n-tile j + 1 are issued before the MFMAs of n-tile j, so their LDS latency
  // hides behind matrix work even when the wave has the SIMD to itself.
  constexpr int OPW = (MODE == DMQ_MODE_FP8) ? 2 : 4;                // operand words per MFMA step
  constexpr int WQ = (MODE == DMQ_MODE_FP4) ? 1 : T::STEPS * OPW;
  auto dequant_tile = [&](const uint32_t (&pkj)[WW], uint32_t (&w)[WQ]) {
    if constexpr (MODE != DMQ_MODE_FP4) {
      dmq_dequant_step<MODE, BIT, 0, IDENT, ROW>(tbl, lane_base, pkj, w);
      if constexpr (T::STEPS > 1) dmq_dequant_step<MODE, BIT, 1, IDENT, ROW>(tbl, lane_base, pkj, w + OPW);
      if constexpr (T::STEPS > 2) {
        dmq_dequant_step<MODE, BIT, 2, IDENT, ROW>(tbl, lane_base, pkj, w + 2 * OPW);
        dmq_dequant_step<MODE, BIT, 3, IDENT, ROW>(tbl, lane_base, pkj, w + 3 * OPW);
      }
    }
  };
  // FOLD (fp16 weights, tiles of 32 rows and more): the norm of the lane's weight row is
  // multiplied into the dequantized fp16 operand, so the MFMAs accumulate straight into the
  // running sums.  This drops the per-group accumulators (32 registers at TT = 2, which is
  // what lets a third workgroup fit a CU) at the price of one fp16 rounding per weight.
  constexpr bool FOLD = (MODE == DMQ_MODE_A16) && STAGE && (TT >= DMQ_FOLD_MIN_TT);
  // PREF (16-row tiles of the two-per-CU instances): the operands of n-tile 0 were looked up
  // while the previous group finished (wpre), so a group does not start on an LDS round trip
  // that nothing hides when the wave has its SIMD to itself.
  constexpr bool PREF = AHEAD && GG::STAGE && TT == 1 && MODE != DMQ_MODE_FP4 && NT > 1;
  uint32_t wpre[WQ];
  auto compute = [&](int g, const uint32_t (&pk)[NT][WW], const uint2_t (&nr)[NT],
                     const uint32_t (&xa)[TT][AW], const float (&xs)[TT], const int (&xsb)[TT]) {
    uint32_t wqb[2][WQ];
    if constexpr (!PREF) dequant_tile(pk[0], wqb[0]);
    if constexpr (FOLD) {
      // Explicit software pipeline, one fence per MFMA step: scale this step's operand, issue a
      // quarter of the next tile's look-ups, then the TT matrix instructions of the step.  The
      // vector ALU work of a step does not depend on its MFMAs, so the two pipes overlap.
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        uint32_t (&wn)[WQ] = wqb[(j + 1) & 1];
        const uint32_t (&wq)[WQ] = wqb[j & 1];
        const _Float16 n = __builtin_bit_cast(half2_t, nr[j].x)[0];
        const half8_t n8 = {n, n, n, n, n, n, n, n};
        auto step = [&](auto sc) {
          constexpr int s = decltype(sc)::value;
          if (j + 1 < NT) dmq_dequant_step<MODE, BIT, s, IDENT, ROW>(tbl, lane_base, pk[j + 1 < NT ? j + 1 : j], wn + s * OPW);
          const half8_t a = __builtin_bit_cast(half8_t, (uint4_t){wq[4 * s], wq[4 * s + 1],
                                                                    wq[4 * s + 2], wq[4 * s + 3]}) * n8;
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            const half8_t b = __builtin_bit_cast(half8_t, (uint4_t){xa[t][4 * s], xa[t][4 * s + 1],
                                                                    xa[t][4 * s + 2], xa[t][4 * s + 3]});
            total_acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, total_acc[j][t], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        };
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{});
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if (j + 1 < NT) dequant_tile(pk[j + 1], wqb[(j + 1) & 1]);
      const uint32_t (&wq)[WQ] = (PREF && j == 0) ? wpre : wqb[j & 1];
      acc_t acc[TT];
#pragma unroll
      for (int t = 0; t < TT; ++t) acc[t] = (acc_t){0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < T::STEPS; ++s) {
        if constexpr (MODE == DMQ_MODE_A16) {
          half8_t a = __builtin_bit_cast(half8_t, (uint4_t){wq[4 * s], wq[4 * s + 1], wq[4 * s + 2],
                                                            wq[4 * s + 3]});
          if constexpr (FOLD) {
            const _Float16 n = __builtin_bit_cast(half2_t, nr[j].x)[0];
            a = a * (half8_t){n, n, n, n, n, n, n, n};
          }
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            half8_t b = __builtin_bit_cast(half8_t, (uint4_t){xa[t][4 * s], xa[t][4 * s + 1],
                                                              xa[t][4 * s + 2], xa[t][4 * s + 3]});
            if constexpr (FOLD) total_acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, total_acc[j][t], 0, 0, 0);
            else acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[t], 0, 0, 0);
          }
        } else if constexpr (MODE == DMQ_MODE_A8) {
          int4_t a = {(int)wq[4 * s], (int)wq[4 * s + 1], (int)wq[4 * s + 2], (int)wq[4 * s + 3]};
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            int4_t b = {(int)xa[t][4 * s], (int)xa[t][4 * s + 1], (int)xa[t][4 * s + 2],
                        (int)xa[t][4 * s + 3]};
            acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[t], 0, 0, 0);
          }
        } else if constexpr (MODE == DMQ_MODE_FP8) {
          long a = (long)(((uint64_t)wq[2 * s + 1] << 32) | wq[2 * s]);
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            long b = (long)(((uint64_t)xa[t][2 * s + 1] << 32) | xa[t][2 * s]);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, acc[t], 0, 0, 0);
          }
        } else {
          int8_t8 a = {(int)pk[j][0], (int)pk[j][1], (int)pk[j][2], (int)pk[j][3], 0, 0, 0, 0};
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            int8_t8 b = {(int)xa[t][0], (int)xa[t][1], (int)xa[t][2], (int)xa[t][3], 0, 0, 0, 0};
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                a, b, acc[t], 4, 4, 0, pw.w_scale_byte, 0, xsb[t]);
          }
        }
      }
      const half4_t h = __builtin_bit_cast(half4_t, nr[j]);
      const float nrm[4] = {(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if constexpr (!FOLD) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = (float)acc[t][r];
            if (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) v = v * xs[t];
            total_acc[j][t][r] += v * nrm[r];
          }
        }
        if (DBG && MODE == DMQ_MODE_A8 && avalid[t] && wave_active) {
          int4_t* d = (int4_t*)(p.dbg_acc + ((long)rlog[t] * p.groups + g) * p.n_out +
                                feat_k + j * 16 + 4 * q);
          *d = __builtin_bit_cast(int4_t, acc[t]);
        }
      }
    }
  };

  // ---- store the finished sums of one n-block (features feat_k ...)
  auto epilogue = [&]() {
    if (!wave_active) return;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      if (!avalid[t]) continue;
#pragma unroll
      for (int j = 0; j < NT; j += UNIT) {
        if (KS > 1 && kpart != ((j / UNIT) * KS) / UNITS) continue;
        if (EPI == DMQ_EPI_STORE) {
          half4_t h = {(_Float16)total_acc[j][t][0], (_Float16)total_acc[j][t][1],
                       (_Float16)total_acc[j][t][2], (_Float16)total_acc[j][t][3]};
          *(half4_t*)(p.out + (long)rlog[t] * p.out_stride + feat_k + j * 16 + 4 * q) = h;
        } else if (SILU) {
          half4_t h;
#pragma unroll
          for (int r = 0; r < 4; ++r)
            h[r] = (_Float16)(dmq_silu(total_acc[j][t][r]) * total_acc[j + 1][t][r]);
          *(half4_t*)(p.out + (long)rlog[t] * p.out_stride + out_col0 + feat_k + (j >> 1) * 16 + 4 * q) = h;
        } else {
          float4_t v = total_acc[j][t] * row_w[t];
          half4_t* dst = (half4_t*)(p.out_slots + (long)row_dst[t] * p.out_stride + feat_k + j * 16 + 4 * q);
          if (p.accumulate) {                  // a further share of the expert: add to what is there
            const half4_t prev = *dst;
            v += (float4_t){(float)prev[0], (float)prev[1], (float)prev[2], (float)prev[3]};
          }
          const half4_t h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
          *dst = h;
        }
      }
    }
  };

  if constexpr (!STAGE) {
    // ------------------------------------------------------------------ direct path
    uint32_t pk[PF][NT][WW];
    uint2_t nr[PF][NT];
    uint32_t xa[PF][TT][AW];
    float xs[PF][TT];
    int xsb[PF][TT];
    auto load_chunk = [&](int g0) {
#pragma unroll
      for (int u = 0; u < PF; ++u) {
        if (g0 + u < g_hi) {
          load_weights(g0 + u, pk[u], nr[u]);
          load_acts(g0 + u, xa[u]);
          load_scales(g0 + u, xs[u], xsb[u]);
        }
      }
    };
    // the first chunk is in flight while the look-up table is built
    if (g_lo < g_hi) load_chunk(g_lo);
    if (MODE != DMQ_MODE_FP4 && !IDENT) dmq_lut_build<BIT, T::ES, ROW>(tbl, pw.lut);
    __syncthreads();
    for (int g0 = g_lo; g0 < g_hi; g0 += PF) {
      if (g0 != g_lo) load_chunk(g0);
#pragma unroll
      for (int u = 0; u < PF; ++u)
        if (g0 + u < g_hi) compute(g0 + u, pk[u], nr[u], xa[u], xs[u], xsb[u]);
    }
  } else {
    // ------------------------------------------------------------------ LDS-staged operands
    // Per group the workgroup shares one LDS slot: the 16*TT x AB activation tile (16-byte
    // chunks XOR-swizzled by row), the 64*NT norms of its weight rows and the activation
    // scales of the tile.  All of it and the packed weights travel D groups ahead of the MFMA
    // work in rings of registers; the slot of group g + 1 is written while group g computes.
    // Loads retire in order, so each iteration requests slot data before weights: the wait
    // for the slot of group g + 1 then never covers weights younger than group g + 1.
    constexpr int NC = AB / 16;                       // chunks per row
    constexpr int NCHUNK = 16 * TT * NC;              // chunks of the tile
    constexpr int CPT = (NCHUNK + 255) / 256;         // chunks per thread
    constexpr int ACT_BYTES = 16 * TT * AB;
    constexpr int NORM_OFF = ACT_BYTES;
    constexpr int SCALE_OFF = NORM_OFF + 128 * NT;
    constexpr int SLOT = GG::SLOT;
    constexpr bool SCALED = (MODE != DMQ_MODE_A16);
    static_assert(NT <= 4, "a wave stages the norms of at most four n-tiles");
    // Thread t stages chunks t, t + 256, ... of the tile (chunk L = row L / NC, position L % NC), so
    // the lanes of a load cover whole rows: 64 contiguous 16-byte pieces per row group, every
    // cache line it touches is used in full.  Rows past the item's last row stage a copy of that
    // last row: the loads stay unconditional (a predicated load is a branch and splits the loop
    // into blocks whose wait counters are taken conservatively), and nothing computed from such
    // a row is ever stored.
    bool s_active[CPT];
    uint32_t s_off[CPT], s_dst[CPT];
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      const int L0 = c * 256 + (int)threadIdx.x;
      s_active[c] = (NCHUNK % 256 == 0) || L0 < NCHUNK;     // threads past the tile reload its last chunk
      const int L = (NCHUNK % 256 == 0) ? L0 : min(L0, NCHUNK - 1);
      const int srow = L / NC, sc = L % NC;
      const int s_rlog = min(r_first + srow, r_end - 1);
      const int s_phys = pw.row_index ? pw.row_index[s_rlog] : s_rlog;
      s_off[c] = (uint32_t)s_phys * (uint32_t)p.act_row_bytes + sc * 16 + (uint32_t)in_group0 * AB;
      s_dst[c] = (uint32_t)(srow * AB + ((sc ^ (srow & (NC - 1))) * 16));
    }
    // lane (l16, q) stages the norm of row l16 of its wave's n-tile q
    const bool n_active = q < NT;
    const uint32_t n_off = 2u * (uint32_t)(SILU
        ? slice_start + ((q & 1) ? p.half_width : 0) + featw + (q >> 1) * 16 + l16
        : (p.slice_is_groups ? 0 : slice_start) + featw + q * 16 + l16);
    // thread t < 16*TT stages the scale word of tile row t
    // (threads past the tile and rows past the item's last row read a valid row's scale: the load
    // is unconditional, like the activation loads; only tile rows are stored)
    const int c_rlog = min(r_first + min((int)threadIdx.x, 16 * TT - 1), r_end - 1);
    const bool c_active = SCALED && threadIdx.x < 16 * TT;
    const int c_phys = SCALED ? (pw.row_index ? pw.row_index[c_rlog] : c_rlog) : 0;
    const uint32_t c_off = ((uint32_t)c_phys * (uint32_t)p.act_scale_stride) * (MODE == DMQ_MODE_FP4 ? 1u : 2u) +
                           (uint32_t)in_group0 * (MODE == DMQ_MODE_FP4 ? 4u : 2u);
    uint32_t w_off[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) w_off[j] = (uint32_t)(wrow[j] + l16) * PPG + q * (WW * 4);
    uint8_t* stage = smem2;

    struct Staged { uint4_t a[CPT]; uint32_t nrm; uint32_t sc; };
    // every address is a workgroup-uniform base (scalar registers) plus a 32-bit lane offset
    // fixed for the item; the empty asm keeps the zero-extension of the offset next to the
    // load, which is the form the scalar-base addressing mode of global loads needs
    const uint8_t* const act_p = pw.act;
    const uint8_t* const norms_p = (const uint8_t*)pw.norms;
    const uint8_t* const scale_p = (const uint8_t*)pw.act_scale;
    const uint8_t* const w_p = pw.w;
    const long group_rows = pw.n_total;
    auto lane_off = [](uint32_t o) { asm volatile("" : "+v"(o)); return o; };
    auto stage_load = [&](int k, int g, Staged& sr) {
      const uint8_t* abase = act_p + (long)g * AB;
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        sr.a[c] = *(const uint4_t*)(abase + lane_off(s_off[c]));
      }
      const uint8_t* nbase = norms_p + ((long)(g_base + g) * group_rows + (long)k * FPB) * 2;
      sr.nrm = n_active ? *(const uint16_t*)(nbase + lane_off(n_off)) : 0u;
      sr.sc = 0u;
      if constexpr (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
        const uint8_t* sbase = scale_p + (long)g * 2;
        sr.sc = *(const uint16_t*)(sbase + lane_off(c_off));
      } else if constexpr (MODE == DMQ_MODE_FP4) {
        const uint8_t* sbase = scale_p + (long)g * 4;
        sr.sc = *(const uint32_t*)(sbase + lane_off(c_off));
      }
    };
    auto stage_store = [&](int buf, const Staged& sr) {
      uint8_t* slot = stage + buf * SLOT;
#pragma unroll
      for (int c = 0; c < CPT; ++c)
        if (NCHUNK % 256 == 0 || s_active[c]) *(uint4_t*)(slot + s_dst[c]) = sr.a[c];
      if (n_active) *(uint16_t*)(slot + NORM_OFF + ((wave * NT + q) * 16 + l16) * 2) = (uint16_t)sr.nrm;
      if (c_active) *(uint32_t*)(slot + SCALE_OFF + threadIdx.x * 4) = sr.sc;
    };
    auto stage_read = [&](int buf, uint32_t (&xa)[TT][AW], uint2_t (&nr)[NT], float (&xs)[TT],
                          int (&xsb)[TT]) {
      const uint8_t* slot = stage + buf * SLOT;
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const int row = t * 16 + l16;
        const uint8_t* base = slot + row * AB;
#pragma unroll
        for (int i = 0; i < AW / 4; ++i) {
          const int c = q * (AW / 4) + i;
          uint4_t v = *(const uint4_t*)(base + ((c ^ (row & (NC - 1))) * 16));
          xa[t][4 * i] = v.x; xa[t][4 * i + 1] = v.y; xa[t][4 * i + 2] = v.z; xa[t][4 * i + 3] = v.w;
        }
        xs[t] = 1.0f; xsb[t] = 127;
        if constexpr (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
          xs[t] = (float)__builtin_bit_cast(_Float16, *(const uint16_t*)(slot + SCALE_OFF + row * 4));
        } else if constexpr (MODE == DMQ_MODE_FP4) {
          xsb[t] = *(const uint8_t*)(slot + SCALE_OFF + row * 4 + q);
        }
      }
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        if constexpr (FOLD) {     // the norm of the lane's own weight row, in both halves of a word
          const uint32_t n = *(const uint16_t*)(slot + NORM_OFF + ((wave * NT + j) * 16 + l16) * 2);
          nr[j] = (uint2_t){n | (n << 16), 0u};
        } else {
          nr[j] = *(const uint2_t*)(slot + NORM_OFF + ((wave * NT + j) * 16 + 4 * q) * 2);
        }
      }
    };
    auto load_packed = [&](int k, int g, uint32_t (&pk)[NT][WW]) {
      const uint8_t* wbase = w_p + ((long)(g_base + g) * group_rows + (long)k * FPB) * PPG;
#pragma unroll
      for (int j = 0; j < NT; ++j) dmq_load_words<WW>(wbase + lane_off(w_off[j]), pk[j]);
    };

    // ---- fused epilogue of the gate_up GEMM: SiLU*up rows of the block (one group of 128
    // features of the down projection) -> per-expert rotation -> (quantization) -> codes.
    // The fp16 tile of the block meets in LDS in the staged layout (fp16 layers reuse the slot
    // the finished step has consumed), every wave rotates it onto 32 of the 128 outputs with
    // its quarter of the rotation matrix, and the quantizers take the row maximum over the four
    // waves.  Same arithmetic, in the same order, as the stand-alone rotation kernel.
    auto epilogue_rot = [&](uint8_t* free_slot) {
      if constexpr (EPI == DMQ_EPI_SILU_ROT) {
        constexpr int PITCH = 256;                                 // fp16 row of one group
        const int blk = feat_k - 32 * wave;                        // first feature of the block (feat_k is the wave's)
        uint8_t* tile = (MODE == DMQ_MODE_A16) ? free_slot : smem_post;
        // quarter of the rotation matrix this wave applies: output tiles 2*wave, 2*wave + 1
        const __half* prot = pw.post_rot + (long)(post_slice + blk / DMQ_GS) * (DMQ_GS * DMQ_GS) +
                             (long)(32 * wave + l16) * DMQ_GS + 8 * q;
        uint4_t pa[2][4];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int s = 0; s < 4; ++s) pa[jt][s] = *(const uint4_t*)(prot + (long)jt * 16 * DMQ_GS + 32 * s);
        __syncthreads();                                           // every wave is done with the slot
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          const int row = t * 16 + l16;
#pragma unroll
          for (int j = 0; j < NT; j += 2) {
            half4_t h;
#pragma unroll
            for (int r = 0; r < 4; ++r)
              h[r] = (_Float16)(dmq_silu(total_acc[j][t][r]) * total_acc[j + 1][t][r]);
            // features 32*wave + (j/2)*16 + 4q .. +3 of the group: 8 bytes inside 16-byte chunk c
            const int f = 32 * wave + (j >> 1) * 16 + 4 * q;
            const int c = f >> 3;
            *(half4_t*)(tile + row * PITCH + ((c ^ (row & 15)) * 16) + (f & 7) * 2) = h;
          }
        }
        __syncthreads();
        float4_t racc[2][TT];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int t = 0; t < TT; ++t) racc[jt][t] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            const int row = t * 16 + l16;
            // features 32s + 8q .. +7 of the row, the assignment of the stand-alone rotation kernel
            const uint4_t braw = *(const uint4_t*)(tile + row * PITCH + (((4 * s + q) ^ (row & 15)) * 16));
            const half8_t b = __builtin_bit_cast(half8_t, braw);
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
              racc[jt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, pa[jt][s]), b,
                                                                   racc[jt][t], 0, 0, 0);
          }
        }
        const int col0 = out_col0 + blk + 32 * wave + 4 * q;       // + 16*jt: first of the lane's 4 outputs
        const int out_group = (out_col0 + blk) / DMQ_GS;           // group of the down projection's input
        if constexpr (MODE == DMQ_MODE_A16) {
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            if (!avalid[t]) continue;
            uint8_t* orow = p.post_out + (long)rlog[t] * p.post_row_bytes;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) {
              const half4_t h = {(_Float16)racc[jt][t][0], (_Float16)racc[jt][t][1],
                                 (_Float16)racc[jt][t][2], (_Float16)racc[jt][t][3]};
              *(half4_t*)(orow + (col0 + 16 * jt) * 2) = h;
            }
          }
        } else if constexpr (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
          float* wmax = (float*)(smem_post + 16 * TT * PITCH);     // [wave][row of the tile]
          float amax[TT];
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            float m = 0.f;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
              for (int r = 0; r < 4; ++r) m = fmaxf(m, fabsf(racc[jt][t][r]));
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            if (q == 0) wmax[wave * (16 * TT) + t * 16 + l16] = m;
          }
          __syncthreads();
          const float qmax = (MODE == DMQ_MODE_A8) ? 127.0f : 448.0f;
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            const int row = t * 16 + l16;
            amax[t] = fmaxf(fmaxf(wmax[row], wmax[16 * TT + row]),
                            fmaxf(wmax[2 * 16 * TT + row], wmax[3 * 16 * TT + row]));
            const float sc = fmaxf(__fdiv_rn(amax[t], qmax), 1e-8f);
            if (!avalid[t]) continue;
            uint8_t* orow = p.post_out + (long)rlog[t] * p.post_row_bytes;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) {
              uint32_t word = 0;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float y = __fdiv_rn(racc[jt][t][r], sc);
                uint32_t code;
                if (MODE == DMQ_MODE_A8) {
                  y = fminf(fmaxf(rintf(y), -127.f), 127.f);
                  code = (uint32_t)(int)y & 0xffu;
                } else {
                  y = fminf(fmaxf(y, -448.f), 448.f);
                  code = dmq_f32_to_e4m3(y);
                }
                word |= code << (8 * r);
              }
              *(uint32_t*)(orow + col0 + 16 * jt) = word;
            }
            if (wave == 0 && q == 0)
              ((__half*)p.post_scale)[(long)rlog[t] * p.post_scale_stride + out_group] =
                  __float2half_rn(sc * pw.post_extra);
          }
        } else {   // FP4: the wave's 32 outputs are one MX block
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            float m = 0.f;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt)
#pragma unroll
              for (int r = 0; r < 4; ++r) m = fmaxf(m, fabsf(racc[jt][t][r]));
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(fmaxf(m, __shfl_xor(m, 32, 64)), 1e-30f);
            const float z = __fdiv_rn(m, 6.0f);
            const float e = ceilf((float)log2((double)z));
            const float sblk = fmaxf(exp2f(e), 1e-30f);
            if (!avalid[t]) continue;
            uint8_t* orow = p.post_out + (long)rlog[t] * p.post_row_bytes;
#pragma unroll
            for (int jt = 0; jt < 2; ++jt) {
              uint32_t half_word = 0;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const float y = fminf(fmaxf(__fdiv_rn(racc[jt][t][r], sblk), -6.f), 6.f);
                const uint32_t nib = dmq_e2m1_mag(fabsf(y)) | ((y < 0.f) ? 8u : 0u);
                half_word |= nib << (4 * r);
              }
              *(uint16_t*)(orow + (col0 + 16 * jt) / 2) = (uint16_t)half_word;
            }
            if (q == 0)
              ((uint8_t*)p.post_scale)[(long)rlog[t] * p.post_scale_stride + out_group * 4 + wave] =
                  (uint8_t)fminf(fmaxf(e + 127.0f, 0.f), 254.f);
          }
        }
      }
    };

    // ---- 64-row tiles of fp16 layers: MFMA steps outermost.  The activation operands of one step
    // (16 registers) are read from the slot while the previous step computes instead of holding
    // the whole tile (64 registers), and the look-ups run two (step, n-tile) pairs ahead of their
    // MFMAs.  Every accumulator sees its operands in the same order as in the tile-outer loop.
    constexpr bool KOUT = DMQ_KOUT && MODE == DMQ_MODE_A16 && FOLD && TT >= DMQ_KOUT_MIN_TT;
    auto compute_kouter = [&](int buf, const uint32_t (&pk)[NT][WW]) {
      if constexpr (KOUT) {
        const uint8_t* slot = stage + buf * SLOT;
        half8_t n8[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const _Float16 n = __builtin_bit_cast(
              _Float16, *(const uint16_t*)(slot + NORM_OFF + ((wave * NT + j) * 16 + l16) * 2));
          n8[j] = (half8_t){n, n, n, n, n, n, n, n};
        }
        uint4_t braw[2][TT];
        auto read_b = [&](auto sc, uint4_t (&dst)[TT]) {
          constexpr int s_ = decltype(sc)::value;
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            const int row = t * 16 + l16;
            const int c = q * (AW / 4) + s_;
            dst[t] = *(const uint4_t*)(slot + row * AB + ((c ^ (row & (NC - 1))) * 16));
          }
        };
        uint32_t wq[3][4];
        auto look = [&](auto mc) {
          constexpr int m = decltype(mc)::value;
          if constexpr (m < 4 * NT)
            dmq_dequant_step<MODE, BIT, m / NT, IDENT, ROW>(tbl, lane_base, pk[m % NT], wq[m % 3]);
        };
        read_b(std::integral_constant<int, 0>{}, braw[0]);
        look(std::integral_constant<int, 0>{});
        look(std::integral_constant<int, 1>{});
        auto micro = [&](auto mc) {
          constexpr int m = decltype(mc)::value;
          constexpr int s_ = m / NT, j = m % NT;
          look(std::integral_constant<int, m + 2>{});
          if constexpr (j == 0 && s_ + 1 < 4) read_b(std::integral_constant<int, s_ + 1>{}, braw[(s_ + 1) & 1]);
          const half8_t a = __builtin_bit_cast(half8_t, (uint4_t){wq[m % 3][0], wq[m % 3][1],
                                                                    wq[m % 3][2], wq[m % 3][3]}) * n8[j];
#pragma unroll
          for (int t = 0; t < TT; ++t)
            total_acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                a, __builtin_bit_cast(half8_t, braw[s_ & 1][t]), total_acc[j][t], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        };
        micro(std::integral_constant<int, 0>{});  micro(std::integral_constant<int, 1>{});
        micro(std::integral_constant<int, 2>{});  micro(std::integral_constant<int, 3>{});
        micro(std::integral_constant<int, 4>{});  micro(std::integral_constant<int, 5>{});
        micro(std::integral_constant<int, 6>{});  micro(std::integral_constant<int, 7>{});
        micro(std::integral_constant<int, 8>{});  micro(std::integral_constant<int, 9>{});
        micro(std::integral_constant<int, 10>{}); micro(std::integral_constant<int, 11>{});
        micro(std::integral_constant<int, 12>{}); micro(std::integral_constant<int, 13>{});
        micro(std::integral_constant<int, 14>{}); micro(std::integral_constant<int, 15>{});
      }
    };

    // ---- K range shared by several workgroups: park the sums of the valid rows in this
    // workgroup's plane, take a ticket, and let the last arrival add the planes (always in plane
    // order, its own from registers, so the result does not depend on the order of arrival).
    // The planes are written and read with device-scope accesses, which go past the per-XCD L2
    // on their own: no cache-wide write-back or invalidate, only a wait for this wave's stores
    // to be acknowledged before the workgroup takes its ticket.
    // Ordering without a release / acquire pair on the ticket: (1) every plane store is a
    // device-scope store, performed at the memory side, and s_waitcnt vmcnt(0) returns only once
    // each of this wave's stores has been acknowledged from there (stores count in vmcnt on this
    // target); (2) the workgroup barrier orders all waves' waits before thread 0's ticket
    // increment; (3) the increment is performed at the same memory side, so the workgroup that
    // reads nsplit - 1 from it runs after all those acknowledgements; (4) its plane loads are
    // device-scope loads issued after the barrier that publishes the ticket value, and are
    // served from the memory side, never from a stale line of its own L2.  A release increment
    // and acquire read (an L2 write-back and invalidate per workgroup) measured 1-3 us slower
    // per layer at 1-16 tokens and changes no result.
    auto split_gather = [&](int nsplit_) -> bool {
      using u64 = unsigned long long;
      // one plane row holds the sums of a routed row: gate then up features (SiLU epilogues) or
      // the output features (plain store)
      const long row_floats = SILU ? 2L * p.n_out : (long)p.n_out;
      const long plane = (long)p.split_rows * row_floats;
      float* base = p.split_partial + (long)rlog[0] * row_floats + feat_k + 4 * q;
      auto col = [&](int j) -> long {
        return SILU ? (long)((j & 1) ? p.n_out : 0) + (j >> 1) * 16 : (long)j * 16;
      };
      const bool mine = avalid[0] && wave_active;
      if (mine) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          u64* dst = (u64*)(base + (long)split * plane + col(j));
          const float2_t lo = {total_acc[j][0][0], total_acc[j][0][1]};
          const float2_t hi = {total_acc[j][0][2], total_acc[j][0][3]};
          __hip_atomic_store(dst, __builtin_bit_cast(u64, lo), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(dst + 1, __builtin_bit_cast(u64, hi), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (threadIdx.x == 0) {
        const int t = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t == nsplit_ - 1)                           // ready for the next launch
          __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *wg_flag = t;
      }
      __syncthreads();
      if (*wg_flag != nsplit_ - 1) return false;
      if (mine) {
        // four planes are requested together; the sums are still taken in plane order
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          float4_t sum = (float4_t){0.f, 0.f, 0.f, 0.f};
          for (int s0 = 0; s0 < nsplit_; s0 += 4) {
            float4_t v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int s = s0 + i;
              v[i] = total_acc[j][0];
              if (s < nsplit_ && s != split) {
                const u64* src = (const u64*)(base + (long)s * plane + col(j));
                const float2_t lo = __builtin_bit_cast(
                    float2_t, __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                const float2_t hi = __builtin_bit_cast(
                    float2_t, __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                v[i] = (float4_t){lo[0], lo[1], hi[0], hi[1]};
              }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (s0 + i < nsplit_) sum += v[i];
          }
          total_acc[j][0] = sum;
        }
      }
      return true;
    };

    // A workgroup walks nbc consecutive n-blocks of its item as one stream of nbc * G steps
    // (step = one group of one n-block), so the loads of the next n-block are in flight while
    // the current one finishes; the sums are stored and cleared at each n-block boundary.
    // Every load is unconditional (positions past the last step repeat the last step) and ring
    // entry u is refilled only after its last use in program order: the loaded registers then
    // carry straight across the loop's back edge, with no copy that would have to wait for
    // loads still in flight.
    constexpr int D = dmq_ring_depth<WW, TT>();
    static_assert(D % 2 == 0, "the LDS slot of a ring entry is fixed by its parity");
    uint32_t pkb[D][NT][WW];
    Staged srb[D];
    const int nsplit = XSPLIT ? nsplit_in : 1;
    const int G = XSPLIT ? p.groups / nsplit : g_hi;   // groups this workgroup contracts
    const int g_first = XSPLIT ? split * G : 0;
    const int steps = nbc * G;
    int lk = 0, lg = 0;                                // load position: n-block, group
    auto next_load = [&]() {
      if (lk * G + lg < steps - 1) { if (++lg == G) { lg = 0; ++lk; } }
    };
    // the codebook entries of this thread's table row are requested first: they arrive while
    // the weights are still in flight and the table is ready one memory latency after launch
    uint32_t lutw[4];
    if constexpr (MODE != DMQ_MODE_FP4 && !IDENT) dmq_lut_fetch<BIT, T::ES>(pw.lut, threadIdx.x, lutw);
#pragma unroll
    for (int u = 0; u < D; ++u) {
      stage_load(lk, g_first + lg, srb[u]);
      load_packed(lk, g_first + lg, pkb[u]);
      next_load();
    }
    if constexpr (MODE != DMQ_MODE_FP4 && !IDENT) dmq_lut_store_wave<BIT, T::ES, ROW>(tbl, wave, lutw);
    stage_store(0, srb[0]);
    __syncthreads();
    if constexpr (PREF) dequant_tile(pkb[0][0], wpre);
    int cg = 0;                                        // group of the step being computed
    for (int sb = 0; sb < steps; sb += D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        const bool live = sb + u < steps;              // uniform over the workgroup
        stage_load(lk, g_first + lg, srb[u]);          // entry u went to LDS one step ago
        if (live) {
          if constexpr (KOUT) {
            compute_kouter(u & 1, pkb[u]);
          } else {
            uint32_t xa[TT][AW];
            uint2_t nr[NT];
            float xs[TT];
            int xsb[TT];
            stage_read(u & 1, xa, nr, xs, xsb);
            compute(cg, pkb[u], nr, xa, xs, xsb);
            // n-tile 0 of the next step (a step past the last one looks a stale entry up: unused)
            if constexpr (PREF) dequant_tile(pkb[(u + 1) % D][0], wpre);
          }
        }
        load_packed(lk, g_first + lg, pkb[u]);
        next_load();
        stage_store((u & 1) ^ 1, srb[(u + 1) % D]);
        if (live && ++cg == G) {                       // n-block finished
          bool whole = true;                           // uniform over the workgroup
          if constexpr (XSPLIT) { if (nsplit > 1) whole = split_gather(nsplit); }
          if (whole) {
            if constexpr (EPI == DMQ_EPI_SILU_ROT) epilogue_rot(stage + (u & 1) * SLOT);
            else epilogue();
          }
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int t = 0; t < TT; ++t) total_acc[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};
          cg = 0;
          feat_k += FPB;
        }
        __syncthreads();
      }
    }
  }

  // ------------------------------------------------------------------ K-split reduction
  // unit u (a tile, or a gate/up pair) is finalized by the wave with kpart == owner(u); the
  // other waves of the K group park their partial sums in LDS.
  if constexpr (KS > 1) {
    float4_t* red4 = (float4_t*)smem2;
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
  if constexpr (!STAGE) epilogue();
}

// Waves per SIMD the register allocation aims for: three for tiles up to 32 rows (the 32-row
// fp16 kernel sits a few registers above that limit otherwise), two for 64-row tiles.
// WIDE kernels serve the pools of 8-bit indices (one byte per weight: twice the packed words per
// lane of a 4-bit pool); they are separate instances so that their registers do not count against
// the kernels of the 1/2/4-bit pools.  A launch skips the work items of the other kind.
// WIDE == 2 serves both kinds in one launch (16-row tiles: the register budget is the wide one
// anyway, and a layer whose shared expert is 8-bit next to 2-bit routed pools then launches each
// GEMM once: the few workgroups of the shared expert run beside the routed ones).
// NT: n-tiles of 16 features per wave.  Four everywhere except the instances for a Linear with a
// handful of rows (NT = 1, K split over the four waves: a workgroup covers 16 features, so a
// 4096-feature matrix gives 256 workgroups instead of 64).
// ROOMY (16-row tiles, 1/2/4-bit pools): two waves per SIMD instead of three.  At three the body
// of the 4-bit weights keeps part of its weight ring in scratch memory inside the K loop; a
// launch that fills at most two workgroups per CU anyway, or one with 4-bit pools, runs the
// instance that has the registers.
//
// MODE2 >= 0: the launch also serves the pools of a second precision mode (a work item runs the
// body of its pool's mode).  For a layer whose shared expert keeps fp16 activations next to
// quantized routed pools: one launch per GEMM instead of one per mode, and the handful of
// workgroups of the smaller mode run beside the others instead of after them.  The launch
// parameters are those of MODE; the fp16 body ignores the ones that differ (activation scales).
template <int M, int NT, int TT, int KS> constexpr int dmq_smem2_bytes() {
  if constexpr (M < 0) return 16; else return GemmGeom<M, NT, TT, KS>::SMEM2;
}
template <int M, int TT, int EPI> constexpr int dmq_post_bytes() {
  if constexpr (M < 0) return 16; else return PostGeom<M, TT, EPI>::BYTES;
}
template <int MODE, int TT, int EPI, int KS, bool DBG, int WIDE = 0, int NT = 4, bool ROOMY = false,
          int MODE2 = -1>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((!WIDE && KS == 1 && TT <= 2 && !ROOMY) ? 3 : 2)))
void dmq_gemm_gf_kernel(GemmParams p) {
  constexpr int S2A = dmq_smem2_bytes<MODE, NT, TT, KS>(), S2B = dmq_smem2_bytes<MODE2, NT, TT, KS>();
  constexpr int PSA = dmq_post_bytes<MODE, TT, EPI>(), PSB = dmq_post_bytes<MODE2, TT, EPI>();
  // table rows of 256 bytes where two workgroups per CU leave the room (see LutGeom) and the K
  // range is long enough to pay for writing 64 KiB of table: the gate_up launches (K = hidden
  // size), not the down projection (four groups per block at I = 512: measured slower there)
  constexpr int ROW = (ROOMY && (EPI == DMQ_EPI_SILU || EPI == DMQ_EPI_SILU_ROT)) ? 256 : DMQ_LUT_ROW;
  __shared__ __attribute__((aligned(16))) uint8_t
      tbl[(MODE == DMQ_MODE_FP4 && (MODE2 < 0 || MODE2 == DMQ_MODE_FP4)) ? 16 : 256 * ROW];
  __shared__ __attribute__((aligned(16))) uint8_t smem2[S2A > S2B ? S2A : S2B];
  __shared__ __attribute__((aligned(16))) uint8_t smem_post[PSA > PSB ? PSA : PSB];
  static_assert(MODE2 < 0 || (!WIDE && !DBG && NT == 4), "two modes: 1/2/4-bit pools, four n-tiles per wave");
  static_assert(EPI != DMQ_EPI_SILU_ROT || KS == 1, "the fused rotation needs the whole block in one workgroup");
  // Workgroup b runs on XCD b % 8 (round-robin dispatch).  Each XCD gets a contiguous range of
  // the work list, so the workgroups that share an activation tile (the feature blocks of an
  // item) and those that share weights (the row tiles of an expert) meet in one L2.
  constexpr bool XSPLIT = KS == 1 && TT == 1 &&
                          (EPI == DMQ_EPI_SILU || EPI == DMQ_EPI_SILU_ROT || EPI == DMQ_EPI_STORE);
  __shared__ int wg_flag;
  const int wsplit = XSPLIT ? p.wsplit : 1;
  int item, nb, nbc, split = 0;
  int ns = wsplit;                                       // workgroups sharing this one's K range
  if (XSPLIT && p.split_items > 0) {
    // The list begins with a few long items (their number: n_items[1], at most split_items): those
    // share K between wsplit workgroups and take the first workgroups of the launch, every other
    // item gets one workgroup per block, each XCD a contiguous range of them as below.
    const int nsp = min(p.n_items[1], p.split_items);
    const int wpi = p.n_blocks * wsplit;                 // workgroups of a shared item
    const int head = (p.split_items * wpi + DMQ_XCDS - 1) / DMQ_XCDS * DMQ_XCDS;
    if ((int)blockIdx.x < head) {
      item = blockIdx.x / wpi;
      if (item >= nsp) return;
      const int sub = blockIdx.x - item * wpi;
      split = sub % wsplit;
      nb = sub / wsplit;
    } else {
      const int b = blockIdx.x - head;
      const int total = (p.n_items[0] - nsp) * p.n_blocks;
      const int per_xcd = (total + DMQ_XCDS - 1) / DMQ_XCDS;
      const int slot = b / DMQ_XCDS;
      const int unit = (b % DMQ_XCDS) * per_xcd + slot;
      if (slot >= per_xcd || unit >= total) return;
      item = nsp + unit / p.n_blocks;
      nb = unit % p.n_blocks;
      ns = 1;
    }
    nbc = 1;
  } else if (p.tail_slots > 0) {
    // Workgroups are dispatched in index order as slots free up, so the order of the list is the
    // schedule: the head of an XCD's share goes nbl blocks per workgroup (loads stay in flight
    // across blocks, one table build for several blocks), its last tail_slots blocks one per
    // workgroup, so that the last round of workgroups is short and full instead of long and
    // half empty.
    const int total_blocks = p.n_items[0] * p.subs * p.n_blocks;
    int per_xcd = (total_blocks + DMQ_XCDS - 1) / DMQ_XCDS;
    per_xcd = (per_xcd + p.nbl - 1) / p.nbl * p.nbl;
    const int xcd = blockIdx.x % DMQ_XCDS;
    const int slot = blockIdx.x / DMQ_XCDS;
    const int nblk = min(per_xcd, total_blocks - xcd * per_xcd);     // blocks of this XCD
    if (nblk <= 0) return;
    const int big = max(0, (nblk - p.tail_slots) / p.nbl);            // workgroups with nbl blocks
    const int first = slot < big ? slot * p.nbl : big * p.nbl + (slot - big);
    if (first >= nblk) return;
    const int blk = xcd * per_xcd + first;
    item = blk / p.n_blocks;
    nb = blk - item * p.n_blocks;
    nbc = min(slot < big ? p.nbl : 1, p.n_blocks - nb);
  } else {
    const int nbg = (p.n_blocks + p.nbl - 1) / p.nbl * wsplit;   // workgroups per item
    const int total = p.n_items[0] * p.subs * nbg;
    const int slot = blockIdx.x / DMQ_XCDS;
    int sub;
    if (p.spread) {
      // items dealt out one at a time: a run of items of this launch's pools anywhere in the
      // list still reaches every XCD
      item = (slot / nbg) * DMQ_XCDS + blockIdx.x % DMQ_XCDS;
      sub = slot % nbg;
      if (item >= p.n_items[0] * p.subs) return;
    } else {
      const int per_xcd = (total + DMQ_XCDS - 1) / DMQ_XCDS;
      const int unit = (blockIdx.x % DMQ_XCDS) * per_xcd + slot;
      if (slot >= per_xcd || unit >= total) return;
      item = unit / nbg;
      sub = unit - item * nbg;
    }
    split = sub % wsplit;                                  // workgroups sharing a block are neighbours
    nb = (sub / wsplit) * p.nbl;
    nbc = min(p.nbl, p.n_blocks - nb);
  }
  int* ticket = XSPLIT ? p.split_counter + (long)item * p.n_blocks + nb : nullptr;
  // a work item of 16 * TT * subs rows is `subs` row tiles of this launch
  const int vsub = item % p.subs;
  item /= p.subs;
  const int4_t* rec = (const int4_t*)(p.items + (long)DMQ_ITEM_WORDS * item);
  const int4_t r0 = rec[0];
  const int4_t r1 = rec[1];
  const int pool = r0[0];
  const int ttile = r0[2] * p.subs + vsub;
  const int token_start = r0[3];
  const int token_count = r1[0];
  if (ttile * (16 * TT) >= token_count) return;          // row tile past the item's last row
  const int slice_start = p.slice_is_groups ? r1[2] : r1[1];
  // first down group of the item's expert: its gate_up slice starts at weight row 2 * start, its
  // down slice at group start / 128 (holds for items of either origin)
  const int post_slice = r1[1] / (2 * DMQ_GS);
  const PoolW& pw = p.pool[pool];
  if (pw.mode != MODE && (MODE2 < 0 || pw.mode != MODE2)) return;
  if (WIDE != 2 && (WIDE == 1) != (pw.bit == 8)) return;
  int col0 = 0;
  if (p.width_filter != 0) {                             // sub-expert layers: one width (and rank) per launch
    const int e = r0[1];
    if (pw.expert_info[e * 4 + 3] != p.width_filter) return;
    if (p.home_filter >= 0 && (pw.home ? pw.home[e] : 0) != p.home_filter) return;
    col0 = pw.col_start ? pw.col_start[e] : 0;
  }
  auto run = [&](auto mode_tag) __attribute__((always_inline)) {
    constexpr int M = decltype(mode_tag)::value;
    if constexpr (M == DMQ_MODE_FP4) {
      dmq_gemm_body<M, 4, NT, TT, EPI, KS, DBG, false, ROW, ROOMY>(p, pw, tbl, smem2, smem_post, token_start, token_count, slice_start, post_slice, ttile, nb, nbc, split | (ns << 8), ticket, &wg_flag, col0);
      return;
    }
    if constexpr (M != DMQ_MODE_FP4 && WIDE != 0) {
      if (WIDE == 1 || pw.bit == 8) {                    // uniform over the workgroup
        if (M == DMQ_MODE_A8 && pw.lut == nullptr)       // uniform codebook: no table
          dmq_gemm_body<M, 8, NT, TT, EPI, KS, DBG, M == DMQ_MODE_A8, ROW, ROOMY>(p, pw, tbl, smem2, smem_post, token_start, token_count, slice_start, post_slice, ttile, nb, nbc, split | (ns << 8), ticket, &wg_flag, col0);
        else
          dmq_gemm_body<M, 8, NT, TT, EPI, KS, DBG, false, ROW, ROOMY>(p, pw, tbl, smem2, smem_post, token_start, token_count, slice_start, post_slice, ttile, nb, nbc, split | (ns << 8), ticket, &wg_flag, col0);
        return;
      }
    }
    if constexpr (M != DMQ_MODE_FP4 && WIDE != 1) {
      switch (pw.bit) {
        case 1: dmq_gemm_body<M, 1, NT, TT, EPI, KS, DBG, false, ROW, ROOMY>(p, pw, tbl, smem2, smem_post, token_start, token_count, slice_start, post_slice, ttile, nb, nbc, split | (ns << 8), ticket, &wg_flag, col0); break;
        case 2: dmq_gemm_body<M, 2, NT, TT, EPI, KS, DBG, false, ROW, ROOMY>(p, pw, tbl, smem2, smem_post, token_start, token_count, slice_start, post_slice, ttile, nb, nbc, split | (ns << 8), ticket, &wg_flag, col0); break;
        default: dmq_gemm_body<M, 4, NT, TT, EPI, KS, DBG, false, ROW, ROOMY>(p, pw, tbl, smem2, smem_post, token_start, token_count, slice_start, post_slice, ttile, nb, nbc, split | (ns << 8), ticket, &wg_flag, col0); break;
      }
    }
  };
  if constexpr (MODE2 >= 0) {
    if (pw.mode == MODE2) {                             // uniform over the workgroup
      run(std::integral_constant<int, MODE2>{});
      return;
    }
  }
  run(std::integral_constant<int, MODE>{});
}
