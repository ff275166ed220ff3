// Top-k routing device code shared by the routing kernels and the fused rotation + top-k launch.
#pragma once
#include "params.h"
#include "prenorm.h"

// ------------------------------------------------------------------------------ top-k
// Wave-wide max / min through data-parallel lane moves: xor 1, xor 2, mirror within 8 and within
// 16 lanes leave every lane with the result of its row of 16; the four rows are then combined
// through scalar registers.  The result is uniform over the wave.
template <typename F>
__device__ __forceinline__ int wave_reduce_i32(int v, F op) {
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, true));   // row_half_mirror
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, true));   // row_mirror
  const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
  const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
  return op(op(a, b), op(c, d));
}
__device__ __forceinline__ float wave_max_f32(float v) {
  // finite floats and -inf order like their bit patterns after this monotone map
  auto key = [](float f) { int b = __builtin_bit_cast(int, f); return b >= 0 ? b : (int)(0x80000000u - (unsigned)b); };
  const int k = wave_reduce_i32(key(v), [](int x, int y) { return x > y ? x : y; });
  return __builtin_bit_cast(float, k >= 0 ? k : (int)(0x80000000u - (unsigned)k));
}
__device__ __forceinline__ int wave_min_i32(int v) {
  return wave_reduce_i32(v, [](int x, int y) { return x < y ? x : y; });
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }

// Always-on shared experts ride the routed path as n_shared extra columns of the top-k arrays:
// column k + j names expert `experts + j` with weight sigmoid(x . gate_row), rounded to fp16 after
// the dot and after the sigmoid like an fp16 Linear followed by torch.sigmoid.  Wave-uniform result.
__device__ __forceinline__ float dmq_shared_gate_value(const SharedGate& sg, int tok, int lane) {
  const __half* xr = sg.x + (long)tok * sg.hidden;
  float dot = 0.f;
  const float rstd = sg.pn.on ? sg.row_rstd[tok] : 0.f;
  for (int h = lane * 8; h < sg.hidden; h += 512) {
    uint4_t raw = *(const uint4_t*)(xr + h);
    if (sg.pn.on) {                      // pre-norm rows: normalize the piece first
      float w[8];
      dmq_norm_weights8(sg.pn, h, w);
      raw = dmq_norm8(raw, rstd, w);
    }
    const half8_t a = __builtin_bit_cast(half8_t, raw);
    const half8_t b = *(const half8_t*)(sg.gate_row + h);
#pragma unroll
    for (int c = 0; c < 8; ++c) dot += (float)a[c] * (float)b[c];
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) dot += __shfl_xor(dot, m, 64);
  const float z = (float)(_Float16)dot;
  return (float)(_Float16)(1.f / (1.f + expf(-z)));
}

// The same value for four tokens tok0, tok0 + step, ... at once (their rows are requested together);
// every token sees the arithmetic of dmq_shared_gate_value in the same order.
__device__ __forceinline__ void dmq_shared_gate_values4(const SharedGate& sg, int tok0, int step, int tokens,
                                                        int lane, float (&g)[4]) {
  float dot[4] = {0.f, 0.f, 0.f, 0.f};
  for (int h = lane * 8; h < sg.hidden; h += 512) {
    const half8_t b = *(const half8_t*)(sg.gate_row + h);
    half8_t a[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = min(tok0 + i * step, tokens - 1);
      a[i] = *(const half8_t*)(sg.x + (long)tok * sg.hidden + h);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 8; ++c) dot[i] += (float)a[i][c] * (float)b[c];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float d = dot[i];
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) d += __shfl_xor(d, m, 64);
    const float z = (float)(_Float16)d;
    g[i] = (float)(_Float16)(1.f / (1.f + expf(-z)));
  }
}

__device__ __forceinline__ void dmq_shared_columns(const SharedGate& sg, int tok, int experts, int k,
                                                   int lane, float* out_w, int* out_idx) {
  if (sg.n_shared <= 0) return;
  const float g = dmq_shared_gate_value(sg, tok, lane);
  const int stride = k + sg.n_shared;
  if (lane < sg.n_shared) {
    out_w[(long)tok * stride + k + lane] = g;
    out_idx[(long)tok * stride + k + lane] = experts + lane;
  }
}

// softmax + top-k of one token by one wave: lane j < k returns the j-th largest probability and
// its expert (lowest expert index wins ties).  NV values per lane cover up to 64 * NV experts;
// the loads are a call of their own so that a caller can request the next token's row early.
template <typename T, int NV>
__device__ __forceinline__ void dmq_topk_load(const T* row, int experts, int lane, float (&v)[NV]) {
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    int e = lane + 64 * i;
    v[i] = (e < experts) ? to_f32<T>(row[e]) : -INFINITY;
  }
}

template <int NV>
__device__ __forceinline__ void dmq_topk_select(float (&v)[NV], int experts, int k, int renorm, int lane,
                                                float& my_w, int& my_e) {
  float vmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) vmax = fmaxf(vmax, v[i]);
  vmax = wave_max_f32(vmax);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) sum += (lane + 64 * i < experts) ? expf(v[i] - vmax) : 0.f;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) sum += __shfl_xor(sum, m, 64);

  float my_v = -INFINITY;
  my_e = 0;
  for (int round = 0; round < k; ++round) {
    float bv = -INFINITY;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int e = lane + 64 * i;
      if (v[i] > bv) { bv = v[i]; be = e; }
    }
    // wave arg-max in two reductions: the largest value, then the lowest expert index holding it
    const float top = wave_max_f32(bv);
    be = wave_min_i32(bv == top ? be : 0x7fffffff);
    if (lane == round) { my_v = top; my_e = be; }
    if ((be & 63) == lane) {
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (i == (be >> 6)) v[i] = -INFINITY;
    }
  }
  // lane j turns the j-th logit into its probability; the kept mass is summed in round order
  my_w = (lane < k) ? expf(my_v - vmax) / sum : 0.f;
  if (renorm) {
    float wsum = 0.f;
    for (int j = 0; j < k; ++j) wsum += __shfl(my_w, j, 64);
    my_w = my_w / wsum;
  }
}

// The sum of exponentials runs over the same values in the same order for every NV, so the
// weights do not depend on which instance serves a layer.
template <typename T>
__device__ __forceinline__ void dmq_topk_token(const T* row, int experts, int k, int renorm, int lane,
                                               float& my_w, int& my_e) {
  if (experts <= 256) {
    float v[4]; dmq_topk_load<T, 4>(row, experts, lane, v);
    dmq_topk_select<4>(v, experts, k, renorm, lane, my_w, my_e);
  } else if (experts <= 512) {
    float v[8]; dmq_topk_load<T, 8>(row, experts, lane, v);
    dmq_topk_select<8>(v, experts, k, renorm, lane, my_w, my_e);
  } else {
    float v[16]; dmq_topk_load<T, 16>(row, experts, lane, v);
    dmq_topk_select<16>(v, experts, k, renorm, lane, my_w, my_e);
  }
}

// A handful of tokens: the routing step inside one top-k workgroup.  With a few dozen routed rows the
// stable sort by expert is a brute-force ranking (every row counts the rows that come before it),
// and the work items (one per routed expert: at most four rows each) follow from the same scan:
// the record at the sorted position of an expert's first row carries the item, the positions of
// its other rows hold empty records.  Same permutation and counts as the chunked sort.  Measured
// with more tokens per wave (8 and 16 tokens): the serial top-k rounds cost more than the routing
// launch they replace, so four tokens (one per wave) is the limit.  It saves the routing
// launch (~9 us of a 37 us forward at one token).
#define DMQ_DIRECT_MAX_TOKENS 4
#define DMQ_DIRECT_MAX_ROWS 256
struct DirectPlan {
  int on;
  int pools, experts;            // experts including the shared slices
  const int* slice_start_rows;   // [pools, experts] first gate_up row of the expert's slice, -1: not a member
  const int* slice_count_rows;   // [pools, experts]
  int* items;                    // [rows, DMQ_ITEM_WORDS]
  int* n_items;                  // [2]: rows, 0 (no pool is rotated per work item)
  int* counts;                   // [experts]
  int* sorted_tokens;            // [rows] token of the row at each sorted position
  float* sorted_weights;         // [rows]
  int* sorted_rows;              // [rows] (token, slot) row at each sorted position
  int* clear_words;              // tickets of a K range shared between workgroups (or NULL)
  int clear_count;
};

// One workgroup of the top-k launch: four tokens, one per wave.
struct TopkParams {
  const void* logits;            // [tokens, experts] fp32 or fp16 (the kernel's template type)
  int tokens, experts, k, renorm;
  float* out_w;                  // [tokens, k + n_shared]
  int* out_idx;
  SharedGate sg;
  int blocks;                    // workgroups of the top-k part: ceil(tokens / 4)
  DirectPlan dp;
  const int* in_idx;             // direct plan without logits: the caller's top-k [tokens, k]
  const float* in_w;
};

template <typename T>
__device__ __forceinline__ void dmq_topk_wg(const TopkParams& tp, int block) {
  const int lane = threadIdx.x & 63;
  const int tok = block * 4 + (threadIdx.x >> 6);
  const int stride = tp.k + tp.sg.n_shared;
  if (!tp.dp.on) {
    if (tok >= tp.tokens) return;
    float my_w;
    int my_e;
    dmq_topk_token<T>((const T*)tp.logits + (long)tok * tp.experts, tp.experts, tp.k, tp.renorm, lane,
                      my_w, my_e);
    if (lane < tp.k) {
      tp.out_w[(long)tok * stride + lane] = my_w;
      tp.out_idx[(long)tok * stride + lane] = my_e;
    }
    dmq_shared_columns(tp.sg, tok, tp.experts, tp.k, lane, tp.out_w, tp.out_idx);
    return;
  }
  // direct plan: a single workgroup, wave v takes tokens v, v + 4, ...; every wave reaches the barrier
  __shared__ __attribute__((aligned(16))) int s_expert[DMQ_DIRECT_MAX_ROWS + 4];
  __shared__ float s_weight[DMQ_DIRECT_MAX_ROWS];
  const DirectPlan& dp = tp.dp;
  const int rows = tp.tokens * stride;
  const int wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < dp.clear_count; i += 256) dp.clear_words[i] = 0;
  for (int t = wave; t < tp.tokens; t += 4) {
    float my_w = 0.f;
    int my_e = 0;
    if (tp.logits) {
      dmq_topk_token<T>((const T*)tp.logits + (long)t * tp.experts, tp.experts, tp.k, tp.renorm, lane,
                        my_w, my_e);
    } else if (lane < tp.k) {
      my_w = tp.in_w[(long)t * tp.k + lane];
      my_e = tp.in_idx[(long)t * tp.k + lane];
    }
    if (tp.sg.n_shared > 0) {
      const float g = dmq_shared_gate_value(tp.sg, t, lane);
      if (lane >= tp.k && lane < stride) { my_w = g; my_e = tp.experts + (lane - tp.k); }
    }
    if (lane < stride) {
      const int r = t * stride + lane;
      tp.out_w[r] = my_w;
      tp.out_idx[r] = my_e;
      s_expert[r] = my_e;
      s_weight[r] = my_w;
    }
  }
  for (int i = rows + threadIdx.x; i < ((rows + 3) & ~3); i += 256) s_expert[i] = 0x7fffffff;   // pad to fours
  __syncthreads();
  // the scans read the list four experts at a time (one address for the whole wave: a broadcast)
  const int rows4 = (rows + 3) >> 2;
  for (int t = wave; t < tp.tokens; t += 4) {
    const bool mine = lane < stride;
    const int r = t * stride + lane;
    const int my_e = mine ? s_expert[r] : -1;
    // slices of the expert's pool (the first pool that holds a slice of it): requested before the scan
    int pool = 0, ss = -1;
    if (mine && my_e >= 0 && my_e < dp.experts) {      // a caller-made top-k may name no expert
      // all pools' table entries at once (one round trip), then the first pool wins
      int sc[DMQ_MAX_POOLS], st[DMQ_MAX_POOLS];
#pragma unroll
      for (int q = 0; q < DMQ_MAX_POOLS; ++q) {
        const int qq = q < dp.pools ? q : 0;
        sc[q] = dp.slice_count_rows[qq * dp.experts + my_e];
        st[q] = dp.slice_start_rows[qq * dp.experts + my_e];
      }
#pragma unroll
      for (int q = DMQ_MAX_POOLS - 1; q >= 0; --q)
        if (q < dp.pools && sc[q] > 0) { pool = q; ss = st[q]; }
    }
    int pos = 0, cnt = 0, before = 0;                 // before: rows of my expert ahead of mine
    for (int q = 0; q < rows4; ++q) {
      const int4_t e4 = *(const int4_t*)(s_expert + 4 * q);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int same = (e4[c] == my_e) ? 1 : 0;
        pos += (e4[c] < my_e) ? 1 : 0;
        cnt += same;
        before += (same && 4 * q + c < r) ? 1 : 0;
      }
    }
    pos += before;
    if (mine) {
      dp.sorted_tokens[pos] = t;
      dp.sorted_weights[pos] = s_weight[r];
      dp.sorted_rows[pos] = r;
      // the record at the row's own sorted position: the first row of an expert carries the item,
      // the others leave an empty record (no rows: its workgroups return at once)
      const bool item = before == 0 && ss >= 0;
      int4_t* it = (int4_t*)(dp.items + (long)DMQ_ITEM_WORDS * pos);
      it[0] = (int4_t){pool, my_e, 0, pos};
      it[1] = (int4_t){item ? cnt : 0, ss >= 0 ? ss : 0, ss >= 0 ? ss / (2 * DMQ_GS) : 0, 0};
    }
  }
  for (int e = threadIdx.x; e < dp.experts; e += 256) {
    int c = 0;
    for (int q = 0; q < rows4; ++q) {
      const int4_t e4 = *(const int4_t*)(s_expert + 4 * q);
      c += (e4[0] == e) + (e4[1] == e) + (e4[2] == e) + (e4[3] == e);
    }
    dp.counts[e] = c;
  }
  if (threadIdx.x == 0) { dp.n_items[0] = rows; dp.n_items[1] = 0; }
}
