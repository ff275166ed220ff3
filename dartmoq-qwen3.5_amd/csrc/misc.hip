// Format kernels around the GEMMs: index unpacking, weight-tile dequantization through the
// same LDS byte table the GEMM uses, the group-first relayout, the load-time e2m1 fold and
// the fp32 -> fp16 output conversion.  All of them are plain HBM-bound byte movers.
#include "params.h"
#include "lut.h"

// packed bytes -> one index per byte (element i of a byte at bit offset i*bit)
template <int BIT>
__global__ __launch_bounds__(256)
void dmq_unpack_kernel(const uint8_t* packed, long n_bytes, uint8_t* out) {
  constexpr int EPB = 8 / BIT;
  constexpr uint32_t mask = (1u << BIT) - 1u;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_bytes;
       i += (long)gridDim.x * blockDim.x) {
    const uint32_t b = packed[i];
#pragma unroll
    for (int j = 0; j < EPB; ++j) out[i * EPB + j] = (uint8_t)((b >> (j * BIT)) & mask);
  }
}

// Dequantize rows [n0, n0+n_cnt) of groups [g0, g0+g_cnt) to fp16 [g_cnt, n_cnt, 128]:
// value = codebook[idx] (optionally times norms_gf[g, n], rounded once to fp16).
template <int BIT>
__global__ __launch_bounds__(256)
void dmq_dequant_tile_kernel(const uint8_t* idx_gf, const __half* codebook, const __half* norms_gf,
                             int n_total, int g0, int g_cnt, int n0, int n_cnt, __half* out) {
  __shared__ __attribute__((aligned(16))) uint8_t tbl[DMQ_LUT_BYTES];
  dmq_lut_build<BIT, 2>(tbl, codebook);
  __syncthreads();
  using G = LutGeom<BIT, 2>;
  constexpr int PPG = DMQ_GS * BIT / 8;
  const uint32_t lane_base = dmq_lut_lane_base<BIT, 2>(threadIdx.x & 63);
  const long total = (long)g_cnt * n_cnt * PPG;          // one packed byte per iteration
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const int byte_in_row = (int)(i % PPG);
    const long gn = i / PPG;
    const int n = (int)(gn % n_cnt);
    const int g = (int)(gn / n_cnt);
    const long src = ((long)(g0 + g) * n_total + (n0 + n)) * PPG + byte_in_row;
    uint32_t w[4];
    dmq_lut_read<BIT, 2>(tbl, lane_base, idx_gf[src], w);
    __half* dst = out + ((long)g * n_cnt + n) * DMQ_GS + byte_in_row * G::ELEMS;
    const float nv = norms_gf ? __half2float(norms_gf[(long)(g0 + g) * n_total + n0 + n]) : 1.0f;
#pragma unroll
    for (int j = 0; j < G::ELEMS; ++j) {
      const uint16_t bits = (uint16_t)(w[j >> 1] >> ((j & 1) * 16));
      __half hv = __ushort_as_half(bits);
      dst[j] = norms_gf ? __float2half_rn(__half2float(hv) * nv) : hv;
    }
  }
}

// [N, G*ppg] -> [G, N, ppg] and [N, G] -> [G, N] (optionally scaled by 1/sqrt(128) in fp16).
__global__ __launch_bounds__(256)
void dmq_group_first_idx_kernel(const uint8_t* src, int n_rows, int groups, int ppg, uint8_t* dst) {
  // 4-byte granules; ppg is 16, 32, 64 or 128
  const int wpg = ppg / 4;
  const long total = (long)n_rows * groups * wpg;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const int w = (int)(i % wpg);
    const long gn = i / wpg;
    const int n = (int)(gn % n_rows);
    const int g = (int)(gn / n_rows);
    ((uint32_t*)dst)[i] = ((const uint32_t*)src)[((long)n * groups + g) * wpg + w];
  }
}

__global__ __launch_bounds__(256)
void dmq_group_first_norms_kernel(const __half* src, int n_rows, int groups, int prescale,
                                  __half* dst) {
  const long total = (long)n_rows * groups;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const int n = (int)(i % n_rows);
    const int g = (int)(i / n_rows);
    __half v = src[(long)n * groups + g];
    // fp16 tensor divided by sqrt(128): quotient formed in fp32, rounded once to fp16
    if (prescale) v = __float2half_rn(__fdiv_rn(__half2float(v), 11.313708498984761f));
    dst[i] = v;
  }
}

// packed codebook indices -> packed e2m1 (low nibble = even feature), [*, ppg] -> [*, 64]
template <int BIT>
__global__ __launch_bounds__(256)
void dmq_fold_e2m1_kernel(const uint8_t* idx_gf, const uint8_t* nib, long rows, uint8_t* out) {
  constexpr int PPG = DMQ_GS * BIT / 8;
  constexpr uint32_t mask = (1u << BIT) - 1u;
  __shared__ uint8_t lut[16];
  if (threadIdx.x < (1 << BIT)) lut[threadIdx.x] = nib[threadIdx.x];
  __syncthreads();
  const long total = rows * 64;                           // one output byte per iteration
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const long row = i / 64;
    const int k = (int)(i % 64) * 2;                      // first of the two features
    const uint8_t* src = idx_gf + row * PPG;
    const uint32_t i0 = (src[(k * BIT) >> 3] >> ((k * BIT) & 7)) & mask;
    const uint32_t i1 = (src[((k + 1) * BIT) >> 3] >> (((k + 1) * BIT) & 7)) & mask;
    out[i] = (uint8_t)(lut[i0] | (lut[i1] << 4));
  }
}

// out16[t, h] = fp16(acc32[t, h] (+ add16[t, h]))
__global__ __launch_bounds__(256)
void dmq_finalize_kernel(const float* acc, const __half* add, long n, __half* out) {
  for (long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < n;
       i += (long)gridDim.x * blockDim.x * 4) {
    float4_t v = *(const float4_t*)(acc + i);
    if (add) {
      half4_t a = *(const half4_t*)(add + i);
      v[0] += (float)a[0]; v[1] += (float)a[1]; v[2] += (float)a[2]; v[3] += (float)a[3];
    }
    half4_t h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
    *(half4_t*)(out + i) = h;
  }
}

static inline int grid_for(long items, int per_block = 256, int cap = 8192) {
  long g = (items + per_block - 1) / per_block;
  if (g < 1) g = 1;
  return (int)(g > cap ? cap : g);
}

int dmq_unpack_launch(const uint8_t* packed, long n_bytes, int bit, uint8_t* out, hipStream_t s) {
  if (n_bytes <= 0) return DMQ_OK;
  const int grid = grid_for(n_bytes);
  switch (bit) {
    case 1: hipLaunchKernelGGL(dmq_unpack_kernel<1>, dim3(grid), dim3(256), 0, s, packed, n_bytes, out); break;
    case 2: hipLaunchKernelGGL(dmq_unpack_kernel<2>, dim3(grid), dim3(256), 0, s, packed, n_bytes, out); break;
    case 4: hipLaunchKernelGGL(dmq_unpack_kernel<4>, dim3(grid), dim3(256), 0, s, packed, n_bytes, out); break;
    case 8: hipLaunchKernelGGL(dmq_unpack_kernel<8>, dim3(grid), dim3(256), 0, s, packed, n_bytes, out); break;
    default: return DMQ_ERR_BIT;
  }
  return dmq_check_launch();
}

int dmq_dequant_tile_launch(const uint8_t* idx_gf, const __half* cb, const __half* norms, int n_total,
                            int g0, int g_cnt, int n0, int n_cnt, int bit, __half* out, hipStream_t s) {
  const long items = (long)g_cnt * n_cnt * (DMQ_GS * bit / 8);
  if (items <= 0) return DMQ_OK;
  const int grid = grid_for(items, 256, 1024);
  switch (bit) {
    case 1: hipLaunchKernelGGL(dmq_dequant_tile_kernel<1>, dim3(grid), dim3(256), 0, s, idx_gf, cb, norms, n_total, g0, g_cnt, n0, n_cnt, out); break;
    case 2: hipLaunchKernelGGL(dmq_dequant_tile_kernel<2>, dim3(grid), dim3(256), 0, s, idx_gf, cb, norms, n_total, g0, g_cnt, n0, n_cnt, out); break;
    case 4: hipLaunchKernelGGL(dmq_dequant_tile_kernel<4>, dim3(grid), dim3(256), 0, s, idx_gf, cb, norms, n_total, g0, g_cnt, n0, n_cnt, out); break;
    case 8: hipLaunchKernelGGL(dmq_dequant_tile_kernel<8>, dim3(grid), dim3(256), 0, s, idx_gf, cb, norms, n_total, g0, g_cnt, n0, n_cnt, out); break;
    default: return DMQ_ERR_BIT;
  }
  return dmq_check_launch();
}

int dmq_group_first_launch(const uint8_t* idx, const __half* norms, int n_rows, int groups, int ppg,
                           int prescale, uint8_t* idx_gf, __half* norms_gf, hipStream_t s) {
  const long words = (long)n_rows * groups * (ppg / 4);
  if (words > 0)
    hipLaunchKernelGGL(dmq_group_first_idx_kernel, dim3(grid_for(words)), dim3(256), 0, s, idx,
                       n_rows, groups, ppg, idx_gf);
  const long nn = (long)n_rows * groups;
  if (nn > 0)
    hipLaunchKernelGGL(dmq_group_first_norms_kernel, dim3(grid_for(nn)), dim3(256), 0, s, norms,
                       n_rows, groups, prescale, norms_gf);
  return dmq_check_launch();
}

int dmq_fold_e2m1_launch(const uint8_t* idx_gf, const uint8_t* nib, long rows, int bit, uint8_t* out,
                         hipStream_t s) {
  if (rows <= 0) return DMQ_OK;
  const int grid = grid_for(rows * 64);
  switch (bit) {
    case 1: hipLaunchKernelGGL(dmq_fold_e2m1_kernel<1>, dim3(grid), dim3(256), 0, s, idx_gf, nib, rows, out); break;
    case 2: hipLaunchKernelGGL(dmq_fold_e2m1_kernel<2>, dim3(grid), dim3(256), 0, s, idx_gf, nib, rows, out); break;
    case 4: hipLaunchKernelGGL(dmq_fold_e2m1_kernel<4>, dim3(grid), dim3(256), 0, s, idx_gf, nib, rows, out); break;
    default: return DMQ_ERR_BIT;
  }
  return dmq_check_launch();
}

int dmq_finalize_launch(const float* acc, const __half* add, long n, __half* out, hipStream_t s) {
  if (n <= 0) return DMQ_OK;
  hipLaunchKernelGGL(dmq_finalize_kernel, dim3(grid_for((n + 3) / 4)), dim3(256), 0, s, acc, add, n, out);
  return dmq_check_launch();
}
