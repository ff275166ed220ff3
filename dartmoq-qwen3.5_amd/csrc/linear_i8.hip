// int8 GEMM for a Linear whose 8-bit weights sit on a uniform grid (w = idx - 128, the reference's
// IDENTITY_CB, triton_kernels_a8.py:769-799) and whose batch is large:
//
//   out[r, n] = sum_g  s_a[r, g] * norm[g, n] * sum_k a[r, g, k] * (idx[g, n, k] - 128)
//
// The look-up kernels re-read the weights once per 32-row tile; with nothing to look up the
// weights are an ordinary MFMA operand, so this kernel takes 128 x 128 output tiles with both
// operands staged through LDS (one quantization group = 128 bytes of K per step), which cuts the
// weight traffic by four.  A workgroup is four waves in a 2 x 2 arrangement, each owning 64 rows x
// 64 features = 4 x 4 MFMA tiles (i32 16x16x64, weights as the A operand like the look-up
// kernels, so a lane ends up with four consecutive features of one row).  The group's integer
// sums are exact; they are scaled and added in fp32 group by group in the order of the look-up
// kernels: total += (float(acc) * s_a) * norm.
#include "params.h"

namespace {

constexpr int TILE = 128;                  // rows and features per workgroup
constexpr int GROUP_BYTES = DMQ_GS;        // int8: one byte per element
constexpr int SLOT = TILE * GROUP_BYTES;   // 16 KiB per operand and group

// 16-byte chunk c (0..7) of row r sits at chunk position c ^ (r & 7): the sixteen rows a wave
// reads at once then spread over all banks
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * GROUP_BYTES + ((chunk ^ (row & 7)) << 4);
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void dmq_linear_i8_kernel(LinearI8Params p) {
  __shared__ __attribute__((aligned(16))) uint8_t wbuf[2][SLOT];
  __shared__ __attribute__((aligned(16))) uint8_t xbuf[2][SLOT];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l16 = lane & 15;
  const int q = lane >> 4;
  const int n0 = blockIdx.x * TILE;          // first feature of the workgroup
  const int r0 = blockIdx.y * TILE;          // first row
  const int wn = n0 + (wave & 1) * 64;       // first feature of the wave
  const int wr = r0 + (wave >> 1) * 64;      // first row of the wave

  // staging: chunk c = threadIdx.x + 256 i of the 1024 chunks of a slot; rows and features past the
  // end repeat the last one (their sums are never stored)
  int s_row[4], s_chunk[4];
  long w_off[4], x_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = threadIdx.x + 256 * i;
    s_row[i] = c >> 3;
    s_chunk[i] = c & 7;
    const int n = min(n0 + s_row[i], p.n_out - 1);
    const int r = min(r0 + s_row[i], p.rows - 1);
    w_off[i] = (long)n * GROUP_BYTES + s_chunk[i] * 16;
    x_off[i] = (long)r * p.x_row_bytes + s_chunk[i] * 16;
  }
  const long w_group = (long)p.n_out * GROUP_BYTES;       // bytes of one group of the weights
  uint4_t wreg[4], xreg[4];
  auto load = [&](int g) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      wreg[i] = *(const uint4_t*)(p.w + g * w_group + w_off[i]);
      xreg[i] = *(const uint4_t*)(p.x + x_off[i] + (long)g * GROUP_BYTES);
    }
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint4_t w = wreg[i] ^ (uint4_t){0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
      *(uint4_t*)(wbuf[buf] + lds_off(s_row[i], s_chunk[i])) = w;          // idx - 128 as int8
      *(uint4_t*)(xbuf[buf] + lds_off(s_row[i], s_chunk[i])) = xreg[i];
    }
  };

  // scales of the wave's tiles: norms of features wn + 16 j + 4 q .. + 3, activation scale of row
  // wr + 16 t + l16 (clamped like the operands)
  int nidx[4], ridx[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    nidx[j] = min(wn + 16 * j + 4 * q, p.n_out - 4);
    ridx[j] = min(wr + 16 * j + l16, p.rows - 1);
  }

  float4_t total[4][4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int t = 0; t < 4; ++t) total[j][t] = (float4_t){0.f, 0.f, 0.f, 0.f};

  load(0);
  store(0);
  __syncthreads();
  for (int g = 0; g < p.groups; ++g) {
    const int buf = g & 1;
    if (g + 1 < p.groups) load(g + 1);                  // in flight during the MFMA work
    half4_t nrm[4];
    float xs[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      nrm[j] = *(const half4_t*)(p.norms + (long)g * p.n_out + nidx[j]);
      xs[j] = (float)p.x_scale[(long)ridx[j] * p.scale_stride + g];
    }
    const int wl = (wave & 1) * 64, xl = (wave >> 1) * 64;   // the wave's rows inside the slots
    // the activation operands of both MFMA steps stay in registers; the feature tiles go one
    // after the other, so the scaling of tile row j overlaps the matrix work of tile row j + 1
    int4_t b[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        b[s][t] = *(const int4_t*)(xbuf[buf] + lds_off(xl + 16 * t + l16, 4 * s + q));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int4_t acc[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[t] = (int4_t){0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int4_t a = *(const int4_t*)(wbuf[buf] + lds_off(wl + 16 * j + l16, 4 * s + q));
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[s][t], acc[t], 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float v = (float)acc[t][r] * xs[t];
          total[j][t][r] += v * (float)nrm[j][r];
        }
    }
    if (g + 1 < p.groups) store(buf ^ 1);               // the other slot: last read one step ago
    __syncthreads();
  }

#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int r = wr + 16 * t + l16;
    if (r >= p.rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = wn + 16 * j + 4 * q;
      if (n >= p.n_out) continue;
      const half4_t h = {(_Float16)total[j][t][0], (_Float16)total[j][t][1], (_Float16)total[j][t][2],
                         (_Float16)total[j][t][3]};
      *(half4_t*)(p.out + (long)r * p.out_stride + n) = h;
    }
  }
}

}  // namespace

int dmq_linear_i8_launch(const LinearI8Params& p, hipStream_t stream) {
  if (p.rows <= 0) return DMQ_OK;
  const dim3 grid((p.n_out + TILE - 1) / TILE, (p.rows + TILE - 1) / TILE);
  hipLaunchKernelGGL(dmq_linear_i8_kernel, grid, dim3(256), 0, stream, p);
  return dmq_check_launch();
}
