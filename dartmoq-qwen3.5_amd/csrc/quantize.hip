// TurboQuant weight quantizer: W[N, K] fp16 -> packed codebook indices + fp16 group norms.
//
// Per row n and group g of 128 input features
//   norm = max(||W[n, g]||_2, 1e-8)
//   Y    = (W[n, g] / norm) . P_g^T . sqrt(128)          P_g: fp32 rotation matrix of the group
//   idx  = clamp(#boundaries < Y, 0, 2^bit - 1)          boundaries of the scalar quantizer
// and the indices are packed little-endian inside each byte, row-major [N, K * bit / 8].
//
// One wave handles 16 rows of one group.  The rotation runs on the fp32 matrix cores
// (v_mfma_f32_16x16x4_f32; operand A = rows of P_g, operand B = the normalised weight rows, lane
// group q contracting the contiguous features 32q .. 32q+31), so lane (t = lane % 16, q = lane / 16)
// ends with Y[t, 16*jt + 4q + r], jt < 8, r < 4 -- four consecutive features per tile, which is
// a whole number of packed bytes for 2, 4 and 8 bits and half a byte for 1 bit (paired over q).
#include "params.h"

template <int BIT>
__global__ __launch_bounds__(256)
void dmq_quantize_weights_kernel(const __half* w, long w_stride, const float* rot, const float* bounds,
                                 int n_rows, int groups, uint8_t* idx_out, __half* norms_out) {
  const int lane = threadIdx.x & 63;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const long row_tiles = (n_rows + 15) / 16;
  if (item >= row_tiles * groups) return;
  const int g = (int)(item % groups);
  const int row = (int)(item / groups) * 16 + l16;
  const bool valid = row < n_rows;
  constexpr int LEVELS = 1 << BIT;

  // this lane's 32 features of its row: 32q .. 32q + 31
  float x[32];
  const __half* wr = w + (long)(valid ? row : 0) * w_stride + g * DMQ_GS + 32 * q;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint4_t raw = valid ? *(const uint4_t*)(wr + 8 * c) : (uint4_t){0u, 0u, 0u, 0u};
    const half8_t h = __builtin_bit_cast(half8_t, raw);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[8 * c + i] = (float)h[i];
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 32; ++i) ss += x[i] * x[i];
  ss += __shfl_xor(ss, 16, 64);
  ss += __shfl_xor(ss, 32, 64);
  const float nrm = fmaxf(sqrtf(ss), 1e-8f);
#pragma unroll
  for (int i = 0; i < 32; ++i) x[i] = __fdiv_rn(x[i], nrm);

  float4_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = (float4_t){0.f, 0.f, 0.f, 0.f};
  const float* pg = rot + (long)g * (DMQ_GS * DMQ_GS) + (long)l16 * DMQ_GS + 32 * q;
#pragma unroll
  for (int s4 = 0; s4 < 8; ++s4) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float4_t a = *(const float4_t*)(pg + (long)j * 16 * DMQ_GS + 4 * s4);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], x[4 * s4 + u], acc[j], 0, 0, 0);
    }
  }

  const float scale = 11.3137084989847603904f;           // sqrt(128)
  uint8_t* orow = idx_out + (long)(valid ? row : 0) * ((long)groups * (DMQ_GS * BIT / 8)) +
                  (long)g * (DMQ_GS * BIT / 8);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t code[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float y = acc[j][r] * scale;
      uint32_t c = 0;
      if (BIT <= 4) {
#pragma unroll
        for (int b = 0; b < LEVELS - 1; ++b) c += (bounds[b] < y) ? 1u : 0u;
      } else {
        // lower bound by bisection: the number of boundaries strictly below y
        int lo = 0, hi = LEVELS - 1;
#pragma unroll
        for (int it = 0; it < BIT; ++it) {
          const int mid = (lo + hi) >> 1;
          if (lo < hi) { if (bounds[mid] < y) lo = mid + 1; else hi = mid; }
        }
        c = (uint32_t)lo;
      }
      code[r] = c > (uint32_t)(LEVELS - 1) ? (uint32_t)(LEVELS - 1) : c;
    }
    const int feat = j * 16 + 4 * q;                      // first of the lane's four features
    if (BIT == 8) {
      const uint32_t word = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
      if (valid) *(uint32_t*)(orow + feat) = word;
    } else if (BIT == 4) {
      const uint32_t word = code[0] | (code[1] << 4) | (code[2] << 8) | (code[3] << 12);
      if (valid) *(uint16_t*)(orow + feat / 2) = (uint16_t)word;
    } else if (BIT == 2) {
      const uint32_t word = code[0] | (code[1] << 2) | (code[2] << 4) | (code[3] << 6);
      if (valid) orow[feat / 4] = (uint8_t)word;
    } else {
      const uint32_t nib = code[0] | (code[1] << 1) | (code[2] << 2) | (code[3] << 3);
      const uint32_t other = __shfl_xor(nib, 16, 64);     // the neighbouring lane group's nibble
      if (valid && !(q & 1)) orow[feat / 8] = (uint8_t)(nib | (other << 4));
    }
  }
  if (valid && q == 0) norms_out[(long)row * groups + g] = __float2half_rn(nrm);
}

int dmq_quantize_weights_launch(const __half* w, long w_stride, const float* rot, const float* bounds,
                                int n_rows, int groups, int bit, uint8_t* idx_out, __half* norms_out,
                                hipStream_t s) {
  const long items = (long)((n_rows + 15) / 16) * groups;
  if (items <= 0) return DMQ_OK;
  const long grid = (items + 3) / 4;
  if (grid > 0x7fffffffL) return DMQ_ERR_LIMIT;
#define DMQ_QW(B) hipLaunchKernelGGL(dmq_quantize_weights_kernel<B>, dim3((int)grid), dim3(256), 0, s, \
                                     w, w_stride, rot, bounds, n_rows, groups, idx_out, norms_out)
  switch (bit) {
    case 1: DMQ_QW(1); break;
    case 2: DMQ_QW(2); break;
    case 4: DMQ_QW(4); break;
    case 8: DMQ_QW(8); break;
    default: return DMQ_ERR_BIT;
  }
#undef DMQ_QW
  return dmq_check_launch();
}
