// The router in front of the layer for a handful of tokens, as workgroups of the rotation launch:
// RMSNorm of the block input, router projection, softmax + top-k (and, for up to four tokens, the
// whole routing step).  Workgroup b < blocks computes the logits of experts [16 b, 16 b + 16) for
// all tokens (at most 16: one MFMA tile) and the last one to finish runs the top-k on all of them.
#pragma once
#include "params.h"
#include "prenorm.h"
#include "topk.h"

#define DMQ_PRENORM_MAX_TOKENS 16

struct RouterParams {
  const __half* h;               // [tokens, h_stride] pre-norm rows
  long h_stride;
  int tokens, hidden;            // tokens <= 16, hidden % 128 == 0
  PreNorm pn;
  const __half* gate_w;          // [experts, hidden] router projection
  int experts;                   // routed experts (<= 1024)
  __half* logits;                // [16, experts] scratch in device memory
  int* ticket;                   // one word, zero between launches
  __half* x_norm_out;            // optional [tokens, hidden]: the normalized rows
  __half* logits_out;            // optional [tokens, experts]: a copy of the logits for the caller
  int blocks;                    // ceil(experts / 16)
  TopkParams tp;                 // what the last workgroup runs (logits taken from LDS)
};

// The logits of 16 experts x 16 tokens: wave w contracts the w-th quarter of the hidden dimension
// in NS steps of 32 (NS = 0: any length, loads inside the loop).  With NS known every load of the
// wave for router rows and pre-norm rows is requested before the row statistics are
// computed, so the whole contraction waits on memory once.
template <int NS>
__device__ __forceinline__ float4_t dmq_router_logits(const RouterParams& rp, int block, float* s_rstd) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const int e0 = block * 16;
  const int erow = min(e0 + l16, rp.experts - 1);
  const int trow = min(l16, rp.tokens - 1);
  const int kq = rp.hidden / 4;
  const int col0 = wave * kq + 8 * q;
  const __half* wp = rp.gate_w + (long)erow * rp.hidden + col0;
  const __half* hp = rp.h + (long)trow * rp.h_stride + col0;
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  auto step = [&](int k, uint4_t a, uint4_t raw, const float (&w8)[8], float rstd) {
    const uint4_t xn = dmq_norm8(raw, rstd, w8);
    if (block == 0 && rp.x_norm_out && l16 < rp.tokens)
      *(uint4_t*)(rp.x_norm_out + (long)l16 * rp.hidden + col0 + k) = xn;
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                 __builtin_bit_cast(half8_t, xn), acc, 0, 0, 0);
  };
  if constexpr (NS > 0) {
    uint4_t a[NS], raw[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      a[s] = *(const uint4_t*)(wp + 32 * s);
      raw[s] = *(const uint4_t*)(hp + 32 * s);
    }
    dmq_wg_rstd(rp.h, rp.h_stride, 0, rp.tokens, rp.hidden, rp.pn.eps, s_rstd);
    const float rstd = s_rstd[trow];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      float w8[8];
      dmq_norm_weights8(rp.pn, col0 + 32 * s, w8);
      step(32 * s, a[s], raw[s], w8, rstd);
    }
  } else {
    dmq_wg_rstd(rp.h, rp.h_stride, 0, rp.tokens, rp.hidden, rp.pn.eps, s_rstd);
    const float rstd = s_rstd[trow];
#pragma unroll 4
    for (int k = 0; k < kq; k += 32) {
      const uint4_t a = *(const uint4_t*)(wp + k);
      const uint4_t raw = *(const uint4_t*)(hp + k);
      float w8[8];
      dmq_norm_weights8(rp.pn, col0 + k, w8);
      step(k, a, raw, w8, rstd);
    }
  }
  return acc;
}

// `lds`: 32 KiB of LDS the caller does not need while this runs.
__device__ __forceinline__ void dmq_router_wg(const RouterParams& rp, const int block, uint8_t* lds) {
  using u64 = unsigned long long;
  __shared__ float s_rstd[64];
  __shared__ int s_last;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const int e0 = block * 16;
  float4_t acc;
  if (rp.hidden == 2048) acc = dmq_router_logits<16>(rp, block, s_rstd);
  else if (rp.hidden == 3072) acc = dmq_router_logits<24>(rp, block, s_rstd);
  else acc = dmq_router_logits<0>(rp, block, s_rstd);
  float* part = (float*)lds;                           // [4 waves][64 lanes][4]
  *(float4_t*)(part + (wave * 64 + lane) * 4) = acc;
  __syncthreads();
  if (wave == 0) {
    float4_t sum = *(const float4_t*)(part + lane * 4);
#pragma unroll
    for (int w = 1; w < 4; ++w) sum += *(const float4_t*)(part + (w * 64 + lane) * 4);
    // lane (l16, q) holds experts e0 + 4q .. + 3 of token l16: one 8-byte store, visible to every XCD
    const half4_t hv = {(_Float16)sum[0], (_Float16)sum[1], (_Float16)sum[2], (_Float16)sum[3]};
    if (l16 < rp.tokens && e0 + 4 * q < rp.experts)
      __hip_atomic_store((u64*)(rp.logits + (long)l16 * rp.experts + e0 + 4 * q),
                         __builtin_bit_cast(u64, hv), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const int t = __hip_atomic_fetch_add(rp.ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t == rp.blocks - 1)                             // ready for the next launch
      __hip_atomic_store(rp.ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (t == rp.blocks - 1) ? 1 : 0;
  }
  __syncthreads();
  if (!s_last) return;

  // the last workgroup: all logits into LDS (they were written by other XCDs), then the top-k
  __half* s_logits = (__half*)lds;
  const int words = rp.tokens * rp.experts / 4;         // 8-byte pieces (experts % 4 == 0)
  for (int i = threadIdx.x; i < words; i += 256) {
    const u64 v = __hip_atomic_load((const u64*)rp.logits + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ((u64*)s_logits)[i] = v;
    if (rp.logits_out) ((u64*)rp.logits_out)[i] = v;
  }
  __syncthreads();
  TopkParams tp = rp.tp;
  tp.logits = s_logits;
  tp.sg.row_rstd = s_rstd;
  if (tp.dp.on) {
    dmq_topk_wg<__half>(tp, 0);
  } else {
    for (int b = 0; b < (rp.tokens + 3) / 4; ++b) dmq_topk_wg<__half>(tp, b);
  }
}
