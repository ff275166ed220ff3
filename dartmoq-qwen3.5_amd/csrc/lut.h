// Byte-indexed codebook look-up table held in LDS.
//
// A packed weight byte carries 8/BIT codebook indices.  The table maps a byte
// value straight to its 8/BIT dequantized elements (fp16 for WxA16, one byte
// each for the int8 / e4m3 look-ups), so dequantizing costs one LDS read per
// packed byte.  Every entry is replicated across a 128-byte row; lane L reads
// the copy at (L % copies) so that the lanes of a wave hit distinct LDS banks
// whatever byte values they look up.  The table always occupies 32 KiB.
#pragma once
#include "common.h"

#define DMQ_LUT_BYTES (256 * 128)

template <int BIT, int ES>   // ES = bytes per dequantized element (2: fp16, 1: int8 / e4m3)
struct LutGeom {
  static constexpr int ELEMS = 8 / BIT;                 // elements per packed byte
  static constexpr int EB = ELEMS * ES;                 // payload bytes per entry
  static constexpr int STRIDE = EB < 4 ? 4 : EB;        // bytes between copies
  static constexpr int COPIES = 128 / STRIDE;
};

// Build the table with the whole workgroup (blockDim.x threads); caller syncs afterwards.
template <int BIT, int ES>
__device__ __forceinline__ void dmq_lut_build(uint8_t* tbl, const void* codebook) {
  using G = LutGeom<BIT, ES>;
  constexpr uint32_t mask = (1u << BIT) - 1u;
  for (int e = threadIdx.x; e < 256; e += blockDim.x) {
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < G::ELEMS; ++j) {
      uint32_t idx = ((uint32_t)e >> (j * BIT)) & mask;
      if (ES == 2) {
        uint32_t v = ((const uint16_t*)codebook)[idx];
        w[j >> 1] |= v << ((j & 1) * 16);
      } else {
        uint32_t v = ((const uint8_t*)codebook)[idx];
        w[j >> 2] |= v << ((j & 3) * 8);
      }
    }
    uint8_t* row = tbl + e * 128;
#pragma unroll
    for (int c = 0; c < G::COPIES; ++c) {
      uint32_t* dst = (uint32_t*)(row + c * G::STRIDE);
#pragma unroll
      for (int i = 0; i < (G::STRIDE / 4); ++i) dst[i] = w[i];
    }
  }
}

template <int BIT, int ES>
__device__ __forceinline__ uint32_t dmq_lut_lane_base(int lane) {
  using G = LutGeom<BIT, ES>;
  return (uint32_t)(lane % G::COPIES) * G::STRIDE;
}

// Look one packed byte up.  out receives EB bytes (rounded up to whole words).
template <int BIT, int ES>
__device__ __forceinline__ void dmq_lut_read(const uint8_t* tbl, uint32_t lane_base,
                                             uint32_t byte, uint32_t* out) {
  using G = LutGeom<BIT, ES>;
  const uint8_t* p = tbl + (byte << 7) + lane_base;
  if (G::EB == 2) {
    out[0] = *(const uint16_t*)p;
  } else if (G::EB == 4) {
    out[0] = *(const uint32_t*)p;
  } else if (G::EB == 8) {
    uint2_t v = *(const uint2_t*)p;
    out[0] = v.x; out[1] = v.y;
  } else {
    uint4_t v = *(const uint4_t*)p;
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  }
}
