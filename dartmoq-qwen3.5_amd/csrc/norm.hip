// RMSNorm of the layer input (the norm in front of the MoE block): out = x * rsqrt(mean(x^2) + eps)
// * (1 + weight), everything in fp32 with one final rounding to the activation type.  One wave per
// row; the row is read twice (the second time from cache) and written once.  HBM-bound byte mover.
#include "params.h"
#include "prenorm.h"
#include <hip/hip_bf16.h>

template <typename T> __device__ __forceinline__ float norm_to_f32(T v);
template <> __device__ __forceinline__ float norm_to_f32<__half>(__half v) { return __half2float(v); }
template <> __device__ __forceinline__ float norm_to_f32<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }
template <> __device__ __forceinline__ float norm_to_f32<float>(float v) { return v; }
template <typename T> __device__ __forceinline__ T norm_from_f32(float v);
template <> __device__ __forceinline__ __half norm_from_f32<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 norm_from_f32<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

template <typename T, typename W>
__global__ __launch_bounds__(256)
void dmq_rms_norm_kernel(const T* x, const W* weight, long rows, int n, long x_stride, long out_stride,
                         float eps, T* out) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * x_stride;
  T* orow = out + row * out_stride;
  const float sumsq = dmq_row_sumsq<T>(xr, n, lane, [](T v) { return norm_to_f32<T>(v); });
  const float rstd = dmq_rstd(sumsq, n, eps);
  for (int c = lane * 8; c < n; c += 512) {
    const uint4_t raw = *(const uint4_t*)(xr + c);
    const T* v = (const T*)&raw;
    uint4_t packed;
    T* o = (T*)&packed;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      o[i] = norm_from_f32<T>(dmq_norm_value(norm_to_f32<T>(v[i]), rstd, norm_to_f32<W>(weight[c + i])));
    *(uint4_t*)(orow + c) = packed;
  }
}

int dmq_rms_norm_launch(const void* x, int bf16, const void* weight, int weight_fp32, long rows, int n,
                        long x_stride, long out_stride, float eps, void* out, hipStream_t s) {
  if (rows <= 0) return DMQ_OK;
  const int grid = (int)((rows + 3) / 4);
#define DMQ_NORM_LAUNCH(T, W) \
  hipLaunchKernelGGL((dmq_rms_norm_kernel<T, W>), dim3(grid), dim3(256), 0, s, (const T*)x, \
                     (const W*)weight, rows, n, x_stride, out_stride, eps, (T*)out)
  if (bf16) {
    if (weight_fp32) DMQ_NORM_LAUNCH(__hip_bfloat16, float); else DMQ_NORM_LAUNCH(__hip_bfloat16, __hip_bfloat16);
  } else {
    if (weight_fp32) DMQ_NORM_LAUNCH(__half, float); else DMQ_NORM_LAUNCH(__half, __half);
  }
#undef DMQ_NORM_LAUNCH
  return dmq_check_launch();
}
