// Byte-indexed codebook look-up table held in LDS.
//
// A packed weight byte carries 8/BIT codebook indices (one for the 8-bit codebooks of the Linear
// path).  The table maps a byte
// value straight to its 8/BIT dequantized elements (fp16 for WxA16, one byte
// each for the int8 / e4m3 look-ups), so dequantizing costs one LDS read per
// packed byte.  Every entry is replicated across a row of DMQ_LUT_ROW bytes; lane L
// reads the copy at (L % copies) so that the lanes of a wave hit distinct LDS banks
// whatever byte values they look up.  128-byte rows (a 32 KiB table) let three workgroups share a
// CU; the kernel instances that keep two per CU anyway take 256-byte rows (64 KiB), where the
// address of a look-up, (byte << 8) | lane offset, is one byte permute (see LutGeom).
#pragma once
#include "common.h"

#define DMQ_LUT_ROW 128
#define DMQ_LUT_BYTES (256 * DMQ_LUT_ROW)

// ROW = bytes of a table row (all copies of one entry): 128, or 256 for the kernel instances that
// keep two workgroups per CU anyway (a 64 KiB table; the address of a look-up is then one byte
// permute instead of a bit-field extract and a shift-or)
template <int BIT, int ES, int ROW = DMQ_LUT_ROW>   // ES = bytes per dequantized element (2: fp16, 1: int8 / e4m3)
struct LutGeom {
  static constexpr int ELEMS = 8 / BIT;                 // elements per packed byte
  static constexpr int EB = ELEMS * ES;                 // payload bytes per entry
  static constexpr int STRIDE = EB < 4 ? 4 : EB;        // bytes between copies
  static constexpr int COPIES = ROW / STRIDE;
  // 2-bit codebooks (4 values: 8 bytes of fp16, 4 bytes of int8 / e4m3) fit the source operands
  // of one byte permute, so every lane composes table entries itself instead of receiving them
  // from the lane that fetched them
  static constexpr bool PERM_BUILD = (BIT == 2);
};

// Entry `e` of the table: the codebook values of the 8/BIT indices packed in byte value e.
template <int BIT, int ES>
__device__ __forceinline__ void dmq_lut_fetch(const void* codebook, int e, uint32_t (&w)[4]) {
  using G = LutGeom<BIT, ES>;
  constexpr uint32_t mask = (1u << BIT) - 1u;
  w[0] = w[1] = w[2] = w[3] = 0u;
  if constexpr (G::PERM_BUILD) {        // the whole codebook, same for every thread
    if (ES == 2) {
      const uint16_t* cb = (const uint16_t*)codebook;
      w[0] = (uint32_t)cb[0] | ((uint32_t)cb[1] << 16);
      w[1] = (uint32_t)cb[2] | ((uint32_t)cb[3] << 16);
    } else {
      const uint8_t* cb = (const uint8_t*)codebook;
      w[0] = (uint32_t)cb[0] | ((uint32_t)cb[1] << 8) | ((uint32_t)cb[2] << 16) | ((uint32_t)cb[3] << 24);
    }
    return;
  }
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
}

// Write the 64 entries a wave fetched (lane i holds entry 64*wave + i) with all their copies.
// Each store covers 256 contiguous bytes, one dword per lane, so it touches every LDS bank once;
// the entry words are broadcast from the lane that fetched them.
template <int BIT, int ES, int ROW = DMQ_LUT_ROW>
__device__ __forceinline__ void dmq_lut_store_wave(uint8_t* tbl, int wave, const uint32_t (&w)[4]) {
  using G = LutGeom<BIT, ES, ROW>;
  constexpr int DW = G::STRIDE / 4;                     // dwords per copy
  constexpr int RPW = 256 / ROW;                        // table rows per 256-byte store
  const int lane = threadIdx.x & 63;
  if constexpr (G::PERM_BUILD) {
    // A store covers 64 * 16 / ROW whole rows: lane l writes 16 bytes (two or four copies) of entry
    // e = 64 v + EPS t + l / LPR.  The four indices of e are its 2-bit digits; the top one is the wave.
    constexpr int LPR = ROW / 16;                       // lanes per row
    constexpr int EPS = 64 / LPR;                       // entries per store
    const uint32_t sub = (uint32_t)lane / LPR;
    uint8_t* dst = tbl + ((long)wave * 64 + sub) * ROW + (lane % LPR) * 16;
#pragma unroll
    for (int t = 0; t < 64 / EPS; ++t) {
      const uint32_t el = (uint32_t)t * EPS + sub;      // entry of this wave
      const uint32_t i0 = el & 3u, i1 = (el >> 2) & 3u, i2 = (el >> 4) & 3u, i3 = (uint32_t)wave;
      uint4_t v;
      if (ES == 2) {
        const uint32_t s0 = 0x01000100u + i0 * 0x0202u + i1 * 0x02020000u;
        const uint32_t s1 = 0x01000100u + i2 * 0x0202u + i3 * 0x02020000u;
        const uint32_t e0 = __builtin_amdgcn_perm(w[1], w[0], s0);
        const uint32_t e1 = __builtin_amdgcn_perm(w[1], w[0], s1);
        v = (uint4_t){e0, e1, e0, e1};
      } else {
        const uint32_t sel = i0 | (i1 << 8) | (i2 << 16) | (i3 << 24);
        const uint32_t e0 = __builtin_amdgcn_perm(0u, w[0], sel);
        v = (uint4_t){e0, e0, e0, e0};
      }
      *(uint4_t*)(dst + t * EPS * ROW) = v;
    }
    return;
  }
  const int d = lane % DW;
  uint32_t* dst = (uint32_t*)(tbl + (long)wave * 64 * ROW) + lane;
#pragma unroll
  for (int t = 0; t < 64 / RPW; ++t) {
    uint32_t v = 0u;
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const int i = t * RPW + r;                        // entry of this wave, compile-time
      uint32_t e = __builtin_amdgcn_readlane(w[0], i);
      if (DW > 1) { const uint32_t e1 = __builtin_amdgcn_readlane(w[1], i); e = (d == 1) ? e1 : e; }
      if (DW > 2) {
        const uint32_t e2 = __builtin_amdgcn_readlane(w[2], i);
        const uint32_t e3 = __builtin_amdgcn_readlane(w[3], i);
        e = (d == 2) ? e2 : ((d == 3) ? e3 : e);
      }
      v = (RPW == 1 || (lane * 4) / ROW == r) ? e : v;
    }
    dst[t * 64] = v;
  }
}

// Build the table with a workgroup of 256 threads; caller syncs afterwards.
template <int BIT, int ES, int ROW = DMQ_LUT_ROW>
__device__ __forceinline__ void dmq_lut_build(uint8_t* tbl, const void* codebook) {
  uint32_t w[4];
  dmq_lut_fetch<BIT, ES>(codebook, threadIdx.x, w);
  dmq_lut_store_wave<BIT, ES, ROW>(tbl, threadIdx.x >> 6, w);
}

template <int BIT, int ES, int ROW = DMQ_LUT_ROW>
__device__ __forceinline__ uint32_t dmq_lut_lane_base(int lane) {
  using G = LutGeom<BIT, ES, ROW>;
  return (uint32_t)(lane % G::COPIES) * G::STRIDE;
}

// Look up byte K (0..3) of a packed word.  out receives EB bytes (rounded up to whole words).
template <int BIT, int ES, int K, int ROW = DMQ_LUT_ROW>
__device__ __forceinline__ void dmq_lut_read_word(const uint8_t* tbl, uint32_t lane_base,
                                                  uint32_t word, uint32_t* out) {
  using G = LutGeom<BIT, ES, ROW>;
  uint32_t off;
  if (ROW == 256) {
    // result bytes: [0] lane offset, [1] byte K of the word, [2] = [3] = 0
    off = __builtin_amdgcn_perm(word, lane_base, 0x0c0c0400u + ((uint32_t)K << 8));
  } else {
    off = (((word >> (8 * K)) & 0xffu) * ROW) + lane_base;
  }
  const uint8_t* p = tbl + off;
  if (G::EB == 1) {
    out[0] = *p;
  } else if (G::EB == 2) {
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

// Look one packed byte value up.
template <int BIT, int ES>
__device__ __forceinline__ void dmq_lut_read(const uint8_t* tbl, uint32_t lane_base,
                                             uint32_t byte, uint32_t* out) {
  dmq_lut_read_word<BIT, ES, 0>(tbl, lane_base, byte & 0xffu, out);
}
