// RMSNorm arithmetic shared by the stand-alone kernel and by the kernels that normalize the
// layer input on the fly: one definition, so both produce the same bits.
#pragma once
#include "params.h"

// acc + f * f as one fp32 FMA.  The value passes through an empty asm so that the compiler cannot
// merge neighbouring squares into a packed dot product in one caller and not in another: every
// user of these helpers adds the same squares with the same roundings.
__device__ __forceinline__ float dmq_sq_acc(float f, float acc) {
  asm volatile("" : "+v"(f));
  return __builtin_fmaf(f, f, acc);
}

// Sum of squares of a row of n values (n % 8 == 0) by one wave: lane l takes the 8-value pieces
// l, l + 64, ... in order, then the lanes are folded pairwise (xor 1, 2, ... 32).  Uniform result.
template <typename T, typename F>
__device__ __forceinline__ float dmq_row_sumsq(const T* xr, int n, int lane, F to_f32) {
  float sumsq = 0.f;
  for (int c = lane * 8; c < n; c += 512) {
    const uint4_t raw = *(const uint4_t*)(xr + c);
    const T* v = (const T*)&raw;
#pragma unroll
    for (int i = 0; i < 8; ++i) sumsq = dmq_sq_acc(to_f32(v[i]), sumsq);
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) sumsq += __shfl_xor(sumsq, m, 64);
  return sumsq;
}

__device__ __forceinline__ float dmq_rstd(float sumsq, int n, float eps) {
  return rsqrtf(sumsq / (float)n + eps);
}

// One normalized value: h * rstd * (1 + w), rounded once by the caller.
__device__ __forceinline__ float dmq_norm_value(float h, float rstd, float w) {
  float t = h * rstd;
  float u = 1.0f + w;
  asm volatile("" : "+v"(t), "+v"(u));               // two roundings, then the product: in every caller
  return t * u;
}

// The same sum for four fp16 rows at once (their pieces are requested together, NCH pieces per
// lane and row: n <= 512 * NCH); every row sees the additions of dmq_row_sumsq in the same order.
// A piece past the end of the row is read again from the row's last piece and enters as zeros.
template <int NCH>
__device__ __forceinline__ void dmq_rows_sumsq4(const __half* const (&xr)[4], int n, int lane, float (&out)[4]) {
  uint4_t raw[4][NCH];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      const int c = lane * 8 + 512 * ch;
      raw[r][ch] = *(const uint4_t*)(xr[r] + (c < n ? c : n - 8));
    }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float sumsq = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      const bool in = lane * 8 + 512 * ch < n;
      const __half* v = (const __half*)&raw[r][ch];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        sumsq = dmq_sq_acc(in ? __half2float(v[i]) : 0.f, sumsq);
      }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) sumsq += __shfl_xor(sumsq, m, 64);
    out[r] = sumsq;
  }
}

// rstd of up to 64 consecutive fp16 rows [row0, row0 + 64) and below `rows`, by the four waves
// of a workgroup (wave w takes rows w, w + 4, ...), into s_rstd[64] (LDS); rows past the end get 0.
// Ends on a barrier.  hidden <= 4096 takes the four-rows-at-once path.
__device__ __forceinline__ void dmq_wg_rstd(const __half* x, long x_stride, int row0, int rows, int hidden,
                                            float eps, float* s_rstd) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  for (int i0 = 0; i0 < 64; i0 += 16) {
    if (row0 + i0 >= rows) {                         // uniform over the workgroup
      if (threadIdx.x < 16) s_rstd[i0 + threadIdx.x] = 0.f;
      continue;
    }
    const __half* xr[4];
    bool live[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = row0 + i0 + wave + 4 * j;
      live[j] = r < rows;
      xr[j] = x + (long)(live[j] ? r : rows - 1) * x_stride;
    }
    float ss[4];
    if (hidden <= 2048) dmq_rows_sumsq4<4>(xr, hidden, lane, ss);
    else if (hidden <= 3072) dmq_rows_sumsq4<6>(xr, hidden, lane, ss);
    else if (hidden <= 4096) dmq_rows_sumsq4<8>(xr, hidden, lane, ss);
    else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        ss[j] = dmq_row_sumsq<__half>(xr[j], hidden, lane, [](__half v) { return __half2float(v); });
    }
    if (lane == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) s_rstd[i0 + wave + 4 * j] = live[j] ? dmq_rstd(ss[j], hidden, eps) : 0.f;
    }
  }
  __syncthreads();
}

// 1 + weight of eight consecutive columns
__device__ __forceinline__ void dmq_norm_weights8(const PreNorm& pn, int col, float (&w)[8]) {
  if (pn.weight_fp32) {
    const float4_t a = *(const float4_t*)((const float*)pn.weight + col);
    const float4_t b = *(const float4_t*)((const float*)pn.weight + col + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { w[i] = a[i]; w[4 + i] = b[i]; }
  } else {
    const uint4_t raw = *(const uint4_t*)((const __half*)pn.weight + col);
    const __half* v = (const __half*)&raw;
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = __half2float(v[i]);
  }
}

// Eight fp16 values of a pre-norm row -> the eight normalized fp16 values
__device__ __forceinline__ uint4_t dmq_norm8(const uint4_t raw, float rstd, const float (&w)[8]) {
  const __half* v = (const __half*)&raw;
  uint4_t packed;
  __half* o = (__half*)&packed;
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = __float2half_rn(dmq_norm_value(__half2float(v[i]), rstd, w[i]));
  return packed;
}
