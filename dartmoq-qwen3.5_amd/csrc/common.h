// Shared definitions for the gfx950 quantized-MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define DMQ_GS 128            // quantization group: 128 consecutive input features
#define DMQ_WAVE 64
// The persistent GEMM for big batches of fp16 layers (gemm_rows.h), selected by tt == DMQ_ROWS_TT:
#define DMQ_ROWS_TT 8
#define DMQ_ROWS_TILE 128                 // rows of a work item
#define DMQ_ROWS_MAX_ITEMS 2048           // work items a launch can order (it sorts them in LDS)
#define DMQ_ROWS_MIN_STEPS 8              // group steps per unit its descriptor pipeline needs
// queue words in device memory: [0, 8) next position of every XCD's queue, [8] workgroups that left
#define DMQ_ROWS_QUEUE_WORDS 16

// status codes, precision modes and epilogue kinds come from the public C header
#include "dartmoq_hip.h"

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef int int8_t8 __attribute__((ext_vector_type(8)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

static inline int dmq_check_launch() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DMQ_OK : DMQ_ERR_HIP;
}

static inline bool dmq_valid_bit(int bit) { return bit == 1 || bit == 2 || bit == 4; }
// 8-bit indices (256-entry codebooks of the Linear path) are served by the GEMM, the dequantized
// tile and the layout kernels, not by the e2m1 fold
static inline bool dmq_valid_bit_wide(int bit) { return dmq_valid_bit(bit) || bit == 8; }

// ---------------------------------------------------------------- device helpers
// silu(x) = x * sigmoid(x); the hardware reciprocal (1 ulp) replaces the IEEE division, the
// result is rounded to fp16 by every caller
__device__ __forceinline__ float dmq_silu(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// OCP e4m3fn encode of a finite fp32 already clamped to [-448, 448]; round to nearest even.
__device__ __forceinline__ uint32_t dmq_f32_to_e4m3(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t sign = (u >> 24) & 0x80u;
  uint32_t a = u & 0x7fffffffu;
  float af = __uint_as_float(a);
  uint32_t r;
  if (af >= 0.015625f) {                       // normal e4m3 range: 2^-6 ..
    // keep 3 mantissa bits: add half-ulp with tie-to-even on bit 20
    uint32_t lsb = (a >> 20) & 1u;
    a += 0x7ffffu + lsb;
    uint32_t e = (a >> 23) - 127u + 7u;        // rebias 127 -> 7
    r = (e << 3) | ((a >> 20) & 7u);
    if (r > 0x7eu) r = 0x7eu;                  // 448 is the largest finite code
  } else {
    // subnormals: multiples of 2^-9; rintf rounds half to even
    r = (uint32_t)rintf(af * 512.0f);          // 0..8 (8 == smallest normal 0x08)
  }
  return sign | r;
}

// e2m1 magnitude index of |y| (y already clamped to [0, 6]); ties go to the smaller magnitude.
__device__ __forceinline__ uint32_t dmq_e2m1_mag(float ay) {
  return (uint32_t)(ay > 0.25f) + (uint32_t)(ay > 0.75f) + (uint32_t)(ay > 1.25f) +
         (uint32_t)(ay > 1.75f) + (uint32_t)(ay > 2.5f) + (uint32_t)(ay > 3.5f) +
         (uint32_t)(ay > 5.0f);
}
