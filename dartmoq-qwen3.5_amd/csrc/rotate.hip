// Block-QR rotation of activations, optionally fused with per-token quantization.
//
//   y[r, g*128 + j] = sum_k x[r, g*128 + k] * P_g[j, k]          (fp32 accumulation on MFMA)
//
// followed, in registers, by one of
//   fp16 store                                    (WxA16)
//   per-(row, group) symmetric int8 + fp16 scale  (WxA8)
//   per-(row, group) e4m3 + fp16 scale            (WxFP8)
//   per-32 e2m1 + e8m0 scale byte                 (WxFP4)
// so the rotated activation never reaches HBM in fp32/fp16 form for the quantized modes.
//
// One wave handles one (tile of 16*TT rows, group): the rotation matrix rows are the MFMA
// "A" operand, activation rows the "B" operand, so lane (t = lane % 16, q = lane / 16) ends
// up with the 32 rotated values j = 16*jt + 4q + r (jt < 8, r < 4) of row t; the row maximum
// is a 32-value in-lane reduction plus two cross-lane steps.
//
// One launch serves every bit pool of a layer.  "Hoisted" pools rotate all input rows once
// (the rotation of gate_up does not depend on the expert); the others rotate only the rows
// routed to their experts, following the layer's work-item list, and may pick the matrix by
// expert (the down rotations).
#include "params.h"
#include "topk.h"
#include "router.h"
#include <type_traits>

__device__ __forceinline__ float wave_max16x4(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// One workgroup of the rotation launch (`block` = its index among the rotation workgroups, `mat` =
// 32 KiB of LDS for the staged matrix).
// PN: the rows are pre-norm (RotParams.pn): instances of their own, so that the others keep their
// registers (the row statistics hold a few dozen loads in flight).
template <int MODE, int TT, bool PN = false>
__device__ __forceinline__ void dmq_rotate_wg(const RotParams& p, const int block, uint8_t* mat) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  constexpr int ROWS_PER_ITEM = 16 * TT;

  // Workgroups [0, n_hoisted * hoisted_wgs_per_pool) rotate whole-batch pools: a workgroup owns
  // one group and four consecutive row tiles (one per wave) and stages the group's matrix in LDS
  // once.  The remaining workgroups take one work item per wave and read their matrices (one
  // per expert with rot_use_slice) straight from memory.
  int pool, g, r_first, r_end, rot_g;
  int cg = -1;                                          // column group of the rows; -1: the group g
  int stage_pool = -1;                                  // tiled workgroups: pool whose matrix is staged
  const int* row_index = nullptr;
  const long hoisted_wgs = (long)p.n_hoisted * p.hoisted_wgs_per_pool;
  const bool hoisted = (long)block < hoisted_wgs;                // uniform over the workgroup
  const bool staged = hoisted && p.hoisted_staged;
  if (hoisted) {
    pool = p.hoisted_pool[block / p.hoisted_wgs_per_pool];
    const int local = block % p.hoisted_wgs_per_pool;
    if (staged) {
      g = local % p.groups;
      r_first = ((local / p.groups) * 4 + wave) * ROWS_PER_ITEM;
    } else {                      // few rows: one (row tile, group) per wave, more workgroups
      const int idx = local * 4 + wave;
      g = idx % p.groups;
      r_first = (idx / p.groups) * ROWS_PER_ITEM;
    }
    r_end = p.rows;
    rot_g = g;
  } else if (p.tiled_staged) {
    // per-work-item pools whose matrices depend on the group only: a workgroup owns one group and
    // four consecutive row tiles of the item list and stages the matrix of its first item's
    // pool; a wave whose item belongs to another pool reads its matrix from memory instead
    if (!p.items) return;
    const long tb = (long)block - hoisted_wgs;
    g = (int)(tb % p.groups);
    const long rt0 = (tb / p.groups) * 4;
    const int sub = p.tile_rows / ROWS_PER_ITEM;          // waves per work item
    const int n_lim = p.n_items[p.items_prefix ? 1 : 0];
    if (rt0 / sub >= n_lim) return;                       // whole workgroup past the list
    const int pool0 = p.items[DMQ_ITEM_WORDS * (rt0 / sub)];
    stage_pool = (p.pool[pool0].mode == MODE && !p.pool[pool0].hoisted) ? pool0 : -1;
    const long rt = rt0 + wave;
    const long tile = rt / sub;
    pool = pool0;
    r_first = 0; r_end = 0; rot_g = g;
    if (tile < n_lim) {
      const int* it = p.items + DMQ_ITEM_WORDS * tile;
      pool = it[0];
      if (!p.pool[pool].hoisted && p.pool[pool].mode == MODE) {
        r_first = it[3] + it[2] * p.tile_rows + (int)(rt % sub) * ROWS_PER_ITEM;
        r_end = it[3] + it[4];
      }
    }
    row_index = p.row_index;
  } else {
    if (!p.items) return;
    long item = ((long)block - hoisted_wgs) * 4 + wave;
    g = (int)(item % p.groups);
    const long rt = item / p.groups;
    const int sub = p.tile_rows / ROWS_PER_ITEM;          // waves per work item
    const long tile = rt / sub;
    if (tile >= p.n_items[p.items_prefix ? 1 : 0]) return;
    const int* it = p.items + DMQ_ITEM_WORDS * tile;
    pool = it[0];
    if (p.pool[pool].hoisted) return;
    const int ttile = it[2];
    const int ts = it[3];
    const int tc = it[4];
    r_first = ts + ttile * p.tile_rows + (int)(rt % sub) * ROWS_PER_ITEM;
    r_end = ts + tc;
    rot_g = (p.pool[pool].rot_use_slice ? it[6] : 0) + g;
    row_index = p.row_index;
    if (p.pool[pool].col_start) {
      // sub-expert layers: the pool's share of the expert is expert_info[e][3] groups wide and
      // starts at column col_start[e] of the row
      const int e = it[1];
      if (g >= p.pool[pool].expert_info[e * 4 + 3]) return;
      cg = p.pool[pool].col_start[e] / DMQ_GS + g;
    }
  }
  if (cg < 0) cg = g;
  const RotPool& rp = p.pool[pool];
  const bool tiled_wg = !hoisted && p.tiled_staged;
  const bool f16_guest = MODE != DMQ_MODE_A16 && hoisted && p.also_f16 && rp.mode == DMQ_MODE_A16;
  if (!tiled_wg && rp.mode != MODE && !f16_guest) return;

  int rlog[TT];
  bool valid[TT];
  const __half* xrow[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    rlog[t] = r_first + t * 16 + l16;
    valid[t] = rlog[t] < r_end;
    int phys = valid[t] ? (row_index ? row_index[rlog[t]] : rlog[t]) : 0;
    xrow[t] = p.x + (long)phys * p.x_stride + cg * DMQ_GS + 8 * q;
  }
  // the rows of the tile are requested before the matrix is staged, so both are in flight together
  uint4_t xraw[4][TT];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int t = 0; t < TT; ++t)
      xraw[s][t] = valid[t] ? *(const uint4_t*)(xrow[t] + 32 * s) : (uint4_t){0u, 0u, 0u, 0u};
  if constexpr (PN && TT == 1) if (staged) {
    // pre-norm rows: the workgroup's four waves hold 64 consecutive rows; their rstd is computed
    // by all four waves together (also by those whose tile lies past the last row), then every
    // lane normalizes the pieces it holds
    __shared__ float s_rstd[64];
    const int row0 = r_first - wave * ROWS_PER_ITEM;
    dmq_wg_rstd(p.x, p.x_stride, row0, p.rows, p.groups * DMQ_GS, p.pn.eps, s_rstd);
    const float rstd = s_rstd[wave * 16 + l16];
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      float w8[8];
      dmq_norm_weights8(p.pn, cg * DMQ_GS + 8 * q + 32 * s4, w8);
      xraw[s4][0] = dmq_norm8(xraw[s4][0], rstd, w8);
    }
  }
  const bool stage_now = staged || (tiled_wg && stage_pool >= 0);   // uniform over the workgroup
  if (stage_now) {
    // 2048 chunks of 16 bytes, eight per thread; chunk c of row r sits at position c ^ (r % 16) so
    // that the sixteen rows a wave reads at once spread over all banks
    const __half* src_rot = staged ? rp.rot : p.pool[stage_pool].rot;
    const uint4_t* src = (const uint4_t*)(src_rot + (long)g * (DMQ_GS * DMQ_GS));
    uint4_t v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = src[threadIdx.x + 256 * i];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = threadIdx.x + 256 * i;
      const int row = c >> 4;
      *(uint4_t*)(mat + row * 256 + (((c & 15) ^ (row & 15)) * 16)) = v[i];
    }
    __syncthreads();
  }
  const bool from_lds = staged || (tiled_wg && pool == stage_pool);
  if (r_first >= r_end) return;
  const __half* prow = rp.rot + (long)rot_g * (DMQ_GS * DMQ_GS) + (long)l16 * DMQ_GS + 8 * q;

  float4_t acc[8][TT];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int t = 0; t < TT; ++t) acc[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};

  // same MFMA order on both paths (steps outer, output tiles inner): the results do not depend
  // on where the matrix comes from
  auto product = [&](auto load_a) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      half8_t b[TT];
#pragma unroll
      for (int t = 0; t < TT; ++t) b[t] = __builtin_bit_cast(half8_t, xraw[s][t]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const half8_t a = __builtin_bit_cast(half8_t, load_a(j, s));
#pragma unroll
        for (int t = 0; t < TT; ++t)
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[t], acc[j][t], 0, 0, 0);
      }
    }
  };
  if (from_lds) {
    // row j*16 + l16 of the matrix, chunk 4s + q
    const uint8_t* mrow = mat + l16 * 256;
    product([&](int j, int s) {
      return *(const uint4_t*)(mrow + j * (16 * 256) + (((4 * s + q) ^ l16) * 16));
    });
  } else {
    product([&](int j, int s) { return *(const uint4_t*)(prow + (long)j * 16 * DMQ_GS + 32 * s); });
  }

#pragma unroll
  for (int t = 0; t < TT; ++t) {
    uint8_t* orow = rp.out + (long)rlog[t] * rp.out_row_bytes;
    if (MODE == DMQ_MODE_A16 || f16_guest) {
      if (!valid[t]) continue;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        half4_t h = {(_Float16)acc[j][t][0], (_Float16)acc[j][t][1], (_Float16)acc[j][t][2],
                     (_Float16)acc[j][t][3]};
        *(half4_t*)(orow + (cg * DMQ_GS + j * 16 + 4 * q) * 2) = h;
      }
    } else if (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
      float amax = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) amax = fmaxf(amax, fabsf(acc[j][t][r]));
      amax = wave_max16x4(amax);
      const float qmax = (MODE == DMQ_MODE_A8) ? 127.0f : 448.0f;
      const float sc = fmaxf(__fdiv_rn(amax, qmax), 1e-8f);
      if (!valid[t]) continue;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        uint32_t word = 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float y = __fdiv_rn(acc[j][t][r], sc);
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
        *(uint32_t*)(orow + cg * DMQ_GS + j * 16 + 4 * q) = word;
      }
      if (q == 0) {
        const float stored = sc * rp.extra_scale;
        if (p.scale_fp32) ((float*)rp.scale)[(long)rlog[t] * rp.scale_stride + cg] = stored;
        else ((__half*)rp.scale)[(long)rlog[t] * rp.scale_stride + cg] = __float2half_rn(stored);
      }
    } else {   // FP4: four MX blocks of 32 per group
      uint32_t sbytes = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float amax = 0.f;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
          for (int r = 0; r < 4; ++r) amax = fmaxf(amax, fabsf(acc[2 * b + jj][t][r]));
        amax = fmaxf(wave_max16x4(amax), 1e-30f);
        const float z = __fdiv_rn(amax, 6.0f);
        float e = ceilf((float)log2((double)z));
        const float s = fmaxf(exp2f(e), 1e-30f);
        float eb = fminf(fmaxf(e + 127.0f, 0.f), 254.f);
        sbytes |= ((uint32_t)eb & 0xffu) << (8 * b);
        if (valid[t]) {
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            uint32_t half_word = 0;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float y = fminf(fmaxf(__fdiv_rn(acc[2 * b + jj][t][r], s), -6.f), 6.f);
              uint32_t nib = dmq_e2m1_mag(fabsf(y)) | ((y < 0.f) ? 8u : 0u);
              half_word |= nib << (4 * r);
            }
            *(uint16_t*)(orow + (cg * DMQ_GS + (2 * b + jj) * 16 + 4 * q) / 2) = (uint16_t)half_word;
          }
        }
      }
      if (valid[t] && q == 0)
        *(uint32_t*)((uint8_t*)rp.scale + (long)rlog[t] * rp.scale_stride + cg * 4) = sbytes;
    }
  }
}

// --------------------------------------------------------------------------------------------
template <int MODE, int TT, bool PN = false>
__global__ __launch_bounds__(256)
void dmq_rotate_kernel(RotParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t mat[DMQ_GS * DMQ_GS * 2];
  if (p.prep.info && blockIdx.x == 0) {
    // the records dmq_items_from_info_kernel would write for expert_info = [0, rows, 0, n_out]
    const LinearPrep& lp = p.prep;
    for (int i = threadIdx.x; i < lp.tiles; i += 256) {
      int4_t* it = (int4_t*)(lp.items + (long)DMQ_ITEM_WORDS * i);
      it[0] = (int4_t){0, 0, i, 0};
      it[1] = (int4_t){lp.rows, 0, 0, 0};
    }
    for (int i = threadIdx.x; i < lp.zero_count; i += 256) lp.zero[i] = 0;
    if (threadIdx.x == 0) {
      lp.n_items[0] = lp.tiles;
      *(int4_t*)lp.info = (int4_t){0, lp.rows, 0, lp.n_out};
    }
  }
  dmq_rotate_wg<MODE, TT, PN>(p, blockIdx.x, mat);
}

// The same launch with the router's top-k in front: workgroups [0, tp.blocks) take four tokens
// each (one per wave), the rest rotate.  Neither part depends on the other, so the launch costs
// the longer of the two instead of their sum.
template <int MODE, int TT, typename LT>
__global__ __launch_bounds__(256)
void dmq_rotate_topk_kernel(RotParams p, TopkParams tp) {
  __shared__ __attribute__((aligned(16))) uint8_t mat[DMQ_GS * DMQ_GS * 2];
  if ((int)blockIdx.x < tp.blocks) dmq_topk_wg<LT>(tp, blockIdx.x);
  else dmq_rotate_wg<MODE, TT>(p, (int)blockIdx.x - tp.blocks, mat);
}

// The launch of a decode step that starts from the block's pre-norm input: workgroups
// [0, rt.blocks) are the router (RMSNorm, projection, top-k; see router.h), the rest rotate the
// whole-batch pools and normalize their rows on the way in (RotParams.pn).
template <int MODE>
__global__ __launch_bounds__(256)
void dmq_rotate_router_kernel(RotParams p, RouterParams rt) {
  __shared__ __attribute__((aligned(16))) uint8_t mat[DMQ_GS * DMQ_GS * 2];
  if ((int)blockIdx.x < rt.blocks) dmq_router_wg(rt, blockIdx.x, mat);
  else dmq_rotate_wg<MODE, 1, true>(p, (int)blockIdx.x - rt.blocks, mat);
}

// Quantization of activations that are already rotated (no matrix product): one wave per
// (row, group), two consecutive features per lane.
template <int MODE>
__global__ __launch_bounds__(256)
void dmq_quantize_kernel(QuantParams p) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)p.rows * p.groups) return;
  const int g = (int)(item % p.groups);
  const long r = item / p.groups;
  const long col = (long)g * DMQ_GS + 2 * lane;
  float v0, v1;
  if (p.x_fp32) {
    const float* xr = (const float*)p.x + r * p.x_stride + col;
    v0 = xr[0]; v1 = xr[1];
  } else {
    const __half* xr = (const __half*)p.x + r * p.x_stride + col;
    v0 = __half2float(xr[0]); v1 = __half2float(xr[1]);
  }
  float amax = fmaxf(fabsf(v0), fabsf(v1));
  uint8_t* orow = p.out + r * p.out_row_bytes;
  if (MODE == DMQ_MODE_A8 || MODE == DMQ_MODE_FP8) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    const float qmax = (MODE == DMQ_MODE_A8) ? 127.0f : 448.0f;
    const float sc = fmaxf(__fdiv_rn(amax, qmax), 1e-8f);
    float y0 = __fdiv_rn(v0, sc), y1 = __fdiv_rn(v1, sc);
    uint32_t c0, c1;
    if (MODE == DMQ_MODE_A8) {
      c0 = (uint32_t)(int)fminf(fmaxf(rintf(y0), -127.f), 127.f) & 0xffu;
      c1 = (uint32_t)(int)fminf(fmaxf(rintf(y1), -127.f), 127.f) & 0xffu;
    } else {
      c0 = dmq_f32_to_e4m3(fminf(fmaxf(y0, -448.f), 448.f));
      c1 = dmq_f32_to_e4m3(fminf(fmaxf(y1, -448.f), 448.f));
    }
    *(uint16_t*)(orow + col) = (uint16_t)(c0 | (c1 << 8));
    if (lane == 0) {
      const float stored = sc * p.extra_scale;
      if (p.scale_fp32) ((float*)p.scale)[r * p.scale_stride + g] = stored;
      else ((__half*)p.scale)[r * p.scale_stride + g] = __float2half_rn(stored);
    }
  } else {   // FP4: a block of 32 features is 16 consecutive lanes
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    amax = fmaxf(amax, 1e-30f);
    const float z = __fdiv_rn(amax, 6.0f);
    const float e = ceilf((float)log2((double)z));
    const float s = fmaxf(exp2f(e), 1e-30f);
    float y0 = fminf(fmaxf(__fdiv_rn(v0, s), -6.f), 6.f);
    float y1 = fminf(fmaxf(__fdiv_rn(v1, s), -6.f), 6.f);
    uint32_t n0 = dmq_e2m1_mag(fabsf(y0)) | ((y0 < 0.f) ? 8u : 0u);
    uint32_t n1 = dmq_e2m1_mag(fabsf(y1)) | ((y1 < 0.f) ? 8u : 0u);
    orow[col / 2] = (uint8_t)(n0 | (n1 << 4));
    if ((lane & 15) == 0)
      ((uint8_t*)p.scale)[r * p.scale_stride + g * 4 + (lane >> 4)] =
          (uint8_t)fminf(fmaxf(e + 127.0f, 0.f), 254.f);
  }
}

// --------------------------------------------------------------------------------------------
#define DMQ_ROT_STAGE_MIN_TILES 1
// tiled_waves: waves of the per-work-item part (max_items * tile_rows / (16*tt) * groups); the
// whole-batch pools add n_hoisted * ceil(row tiles / 4) * groups workgroups in front
template <int MODE>
static int launch_rotate(const RotParams& p_in, long tiled_waves, int tt, hipStream_t stream,
                         const TopkParams* tp, int topk_fp16) {
  RotParams p = p_in;
  const long row_tiles = ((long)p.rows + 16 * tt - 1) / (16 * tt);
  // four row tiles share a staged matrix; measured faster than one matrix read per wave at
  // every batch size (a single row tile included: four waves fetch the matrix together)
  p.hoisted_staged = row_tiles >= DMQ_ROT_STAGE_MIN_TILES;
  p.hoisted_wgs_per_pool = p.hoisted_staged ? (int)(((row_tiles + 3) / 4) * p.groups)
                                            : (int)((row_tiles * p.groups + 3) / 4);
  if (p.hoisted_wgs_per_pool < 1) p.hoisted_wgs_per_pool = 1;
  // per-work-item part: matrices that depend on the group only are staged per workgroup (one
  // group, four row tiles); per-expert matrices (rot_use_slice) keep one task per wave
  bool sliced = false;
  for (int i = 0; i < DMQ_MAX_POOLS; ++i) sliced |= (p.pool[i].mode >= 0 && p.pool[i].rot_use_slice != 0);
  p.tiled_staged = !sliced;
  long tiled_wgs = (tiled_waves + 3) / 4;
  if (p.tiled_staged && tiled_waves > 0) {
    const long row_tasks = tiled_waves / p.groups;          // row tiles of the item list
    tiled_wgs = ((row_tasks + 3) / 4) * p.groups;
  }
  const long total = (long)p.n_hoisted * p.hoisted_wgs_per_pool + tiled_wgs + (tp ? tp->blocks : 0);
  if (total > 0x7fffffffL) return DMQ_ERR_LIMIT;
  const int grid = (int)total;
  if (grid <= 0) return DMQ_OK;
  if (p.pn.on) {                       // pre-norm rows: whole-batch pools, 16-row tiles, no top-k part
    if (tt != 1 || tp || tiled_wgs > 0) return DMQ_ERR_MODE;
    hipLaunchKernelGGL((dmq_rotate_kernel<MODE, 1, true>), dim3(grid), dim3(256), 0, stream, p);
    return dmq_check_launch();
  }
  if (tp) {
    auto go = [&](auto tt_tag) {
      constexpr int T_ = decltype(tt_tag)::value;
      if (topk_fp16)
        hipLaunchKernelGGL((dmq_rotate_topk_kernel<MODE, T_, __half>), dim3(grid), dim3(256), 0, stream, p, *tp);
      else
        hipLaunchKernelGGL((dmq_rotate_topk_kernel<MODE, T_, float>), dim3(grid), dim3(256), 0, stream, p, *tp);
    };
    if (tt == 4) go(std::integral_constant<int, 4>{});
    else if (tt == 2) go(std::integral_constant<int, 2>{});
    else go(std::integral_constant<int, 1>{});
    return dmq_check_launch();
  }
  if (tt == 4) hipLaunchKernelGGL((dmq_rotate_kernel<MODE, 4>), dim3(grid), dim3(256), 0, stream, p);
  else if (tt == 2) hipLaunchKernelGGL((dmq_rotate_kernel<MODE, 2>), dim3(grid), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((dmq_rotate_kernel<MODE, 1>), dim3(grid), dim3(256), 0, stream, p);
  return dmq_check_launch();
}

template <int MODE>
static int launch_rotate_router(const RotParams& p_in, const RouterParams& rt, hipStream_t stream) {
  RotParams p = p_in;
  const long row_tiles = ((long)p.rows + 15) / 16;
  p.hoisted_staged = 1;
  p.hoisted_wgs_per_pool = (int)(((row_tiles + 3) / 4) * p.groups);
  p.tiled_staged = 1;
  p.items = nullptr;
  const long total = (long)p.n_hoisted * p.hoisted_wgs_per_pool + rt.blocks;
  hipLaunchKernelGGL((dmq_rotate_router_kernel<MODE>), dim3((int)total), dim3(256), 0, stream, p, rt);
  return dmq_check_launch();
}

int dmq_rotate_router_dispatch(int mode, const RotParams& p, const RouterParams& rt, hipStream_t stream) {
  if (!p.pn.on || rt.tokens <= 0 || rt.tokens > DMQ_PRENORM_MAX_TOKENS || p.rows != rt.tokens)
    return DMQ_ERR_LIMIT;
  if (rt.hidden % DMQ_GS || rt.experts % 4 || rt.experts > 1024 || rt.h_stride % 8) return DMQ_ERR_ALIGN;
  switch (mode) {
    case DMQ_MODE_A16: return launch_rotate_router<DMQ_MODE_A16>(p, rt, stream);
    case DMQ_MODE_A8: return launch_rotate_router<DMQ_MODE_A8>(p, rt, stream);
    case DMQ_MODE_FP8: return launch_rotate_router<DMQ_MODE_FP8>(p, rt, stream);
    case DMQ_MODE_FP4: return launch_rotate_router<DMQ_MODE_FP4>(p, rt, stream);
  }
  return DMQ_ERR_MODE;
}

int dmq_rotate_dispatch(int mode, const RotParams& p, long tiled_waves, int tt, hipStream_t stream,
                        const TopkParams* tp, int topk_fp16) {
  switch (mode) {
    case DMQ_MODE_A16: return launch_rotate<DMQ_MODE_A16>(p, tiled_waves, tt, stream, tp, topk_fp16);
    case DMQ_MODE_A8: return launch_rotate<DMQ_MODE_A8>(p, tiled_waves, tt, stream, tp, topk_fp16);
    case DMQ_MODE_FP8: return launch_rotate<DMQ_MODE_FP8>(p, tiled_waves, tt, stream, tp, topk_fp16);
    case DMQ_MODE_FP4: return launch_rotate<DMQ_MODE_FP4>(p, tiled_waves, tt, stream, tp, topk_fp16);
  }
  return DMQ_ERR_MODE;
}

int dmq_quantize_dispatch(int mode, const QuantParams& p, hipStream_t stream) {
  const long items = (long)p.rows * p.groups;
  const int grid = (int)((items + 3) / 4);
  if (grid <= 0) return DMQ_OK;
  switch (mode) {
    case DMQ_MODE_A8:
      hipLaunchKernelGGL((dmq_quantize_kernel<DMQ_MODE_A8>), dim3(grid), dim3(256), 0, stream, p); break;
    case DMQ_MODE_FP8:
      hipLaunchKernelGGL((dmq_quantize_kernel<DMQ_MODE_FP8>), dim3(grid), dim3(256), 0, stream, p); break;
    case DMQ_MODE_FP4:
      hipLaunchKernelGGL((dmq_quantize_kernel<DMQ_MODE_FP4>), dim3(grid), dim3(256), 0, stream, p); break;
    default: return DMQ_ERR_MODE;
  }
  return dmq_check_launch();
}
