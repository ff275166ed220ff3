// Top-k routing and token permutation: sort the T*k routed rows by expert (stable) and
// partition the experts of every bit pool into tiles of activation rows, all on the device
// (no host synchronisation, no atomics, deterministic output order).
//
//   1. dmq_topk_kernel         one wave per token: softmax statistics + k arg-max rounds
//   2. dmq_expert_count_kernel one wave per expert: count rows routed to it
//   3. dmq_plan_kernel         one workgroup: exclusive scan -> offsets, per-pool expert_info
//                              and the work-item list (pool, expert, row tile) of the layer
//   4. dmq_expert_fill_kernel  one wave per expert: write its rows in (token, slot) order
//   5. dmq_combine_kernel      out[t] = sum over the k slot rows of token t (fixed order)
#include "params.h"

// ------------------------------------------------------------------------------ top-k
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }

template <typename T>
__global__ __launch_bounds__(256)
void dmq_topk_kernel(const T* logits, int tokens, int experts, int k, int renorm,
                     float* out_w, int* out_idx) {
  const int lane = threadIdx.x & 63;
  const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= tokens) return;
  const T* row = logits + (long)tok * experts;
  // up to 16 experts per lane (experts <= 1024), strided so lane l owns l, l+64, ...
  float v[16];
  float vmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    int e = lane + 64 * i;
    v[i] = (e < experts) ? to_f32<T>(row[e]) : -INFINITY;
    vmax = fmaxf(vmax, v[i]);
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, m, 64));
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) sum += (lane + 64 * i < experts) ? expf(v[i] - vmax) : 0.f;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) sum += __shfl_xor(sum, m, 64);

  float wsum = 0.f;
  float my_w = 0.f;
  int my_e = 0;
  for (int round = 0; round < k; ++round) {
    // lane-local best (lowest expert index wins ties), then wave arg-max
    float bv = -INFINITY;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      int e = lane + 64 * i;
      if (v[i] > bv) { bv = v[i]; be = e; }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
      float ov = __shfl_xor(bv, m, 64);
      int oe = __shfl_xor(be, m, 64);
      if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; }
    }
    const float w = expf(bv - vmax) / sum;
    wsum += w;
    if (lane == round) { my_w = w; my_e = be; }
    if ((be & 63) == lane) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (i == (be >> 6)) v[i] = -INFINITY;
    }
  }
  if (lane < k) {
    out_w[(long)tok * k + lane] = renorm ? my_w / wsum : my_w;
    out_idx[(long)tok * k + lane] = my_e;
  }
}

// ------------------------------------------------------------------------------ counting
// Each lane inspects 8 consecutive rows per step (two 16-byte loads), a wave 512 rows.
__device__ __forceinline__ void load8(const int* p, int base, int rows, int* v) {
  if (base + 8 <= rows) {
    int4_t a = *(const int4_t*)(p + base);
    int4_t b = *(const int4_t*)(p + base + 4);
    v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
    v[4] = b[0]; v[5] = b[1]; v[6] = b[2]; v[7] = b[3];
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (base + i < rows) ? p[base + i] : -1;
  }
}

__global__ __launch_bounds__(256)
void dmq_expert_count_kernel(const int* topk_idx, int rows, int experts, int* counts) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= experts) return;
  int c = 0;
  for (int base = lane * 8; base < rows; base += 512) {
    int v[8];
    load8(topk_idx, base, rows, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) c += (v[i] == e) ? 1 : 0;
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) c += __shfl_xor(c, m, 64);
  if (lane == 0) counts[e] = c;
}

// inclusive scan over the 1024 threads of the workgroup (16 waves)
__device__ __forceinline__ int block_scan_incl(int v, int* wave_tot) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int o = __shfl_up(v, d, 64);
    if (lane >= d) v += o;
  }
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  int add = 0;
  for (int w = 0; w < wave; ++w) add += wave_tot[w];
  __syncthreads();
  return v + add;
}

__global__ __launch_bounds__(1024)
void dmq_plan_kernel(PlanParams p) {
  __shared__ int wave_tot[16];
  __shared__ int carry;
  const int tid = threadIdx.x;
  if (tid == 0) carry = 0;
  __syncthreads();
  // expert offsets: exclusive scan of counts, 1024 experts per pass
  for (int base = 0; base < p.experts; base += 1024) {
    const int e = base + tid;
    const int c = (e < p.experts) ? p.counts[e] : 0;
    const int incl = block_scan_incl(c, wave_tot) + carry;
    if (e < p.experts) p.offsets[e + 1] = incl;
    __syncthreads();
    if (tid == 1023) carry = incl;
    __syncthreads();
  }
  if (tid == 0) p.offsets[0] = 0;
  __syncthreads();

  // per-pool expert_info and the work-item list, pools in caller order, experts ascending
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int pool = 0; pool < p.pools; ++pool) {
    for (int base = 0; base < p.experts; base += 1024) {
      const int e = base + tid;
      int ntile = 0;
      if (e < p.experts) {
        const int ss = p.slice_start_rows[pool * p.experts + e];
        const int sc = p.slice_count_rows[pool * p.experts + e];
        const int tc = (ss >= 0) ? p.counts[e] : 0;
        const int ts = p.offsets[e + 1] - p.counts[e];
        ntile = (tc + p.tile_rows - 1) / p.tile_rows;
        int* gi = p.gu_info + ((long)pool * p.experts + e) * 4;
        gi[0] = ts; gi[1] = tc; gi[2] = ss >= 0 ? ss : 0; gi[3] = sc;
        int* di = p.dn_info + ((long)pool * p.experts + e) * 4;
        di[0] = ts; di[1] = tc; di[2] = ss >= 0 ? ss / (2 * DMQ_GS) : 0; di[3] = sc / (2 * DMQ_GS);
      }
      const int incl = block_scan_incl(ntile, wave_tot);
      const int first = incl - ntile + carry;
      for (int i = 0; i < ntile; ++i) {
        if (first + i < p.max_items) {
          int* it = p.items + 4L * (first + i);
          it[0] = pool; it[1] = e; it[2] = i; it[3] = 0;
        }
      }
      __syncthreads();
      if (tid == 1023) carry = incl + carry;
      __syncthreads();
    }
  }
  if (tid == 0) p.n_items[0] = min(carry, p.max_items);
}

__global__ __launch_bounds__(256)
void dmq_expert_fill_kernel(const int* topk_idx, const float* topk_w, int rows, int k, int experts,
                            const int* offsets, int* sorted_tokens, float* sorted_weights,
                            int* sorted_rows) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= experts) return;
  int pos = offsets[e];
  const int end = offsets[e + 1];
  if (pos == end) return;
  for (int base0 = 0; base0 < rows; base0 += 512) {
    const int base = base0 + lane * 8;
    int v[8];
    load8(topk_idx, base, rows, v);
    int hits = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) hits += (v[i] == e) ? 1 : 0;
    int incl = hits;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(incl, d, 64);
      if (lane >= d) incl += o;
    }
    int at = pos + incl - hits;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (v[i] == e) {
        const int r = base + i;
        sorted_tokens[at] = r / k;
        sorted_weights[at] = topk_w[r];
        sorted_rows[at] = r;
        ++at;
      }
    }
    pos += __shfl(incl, 63, 64);
  }
}

// Work items for a caller-supplied expert_info (merged-GEMM entry points): one workgroup.
__global__ __launch_bounds__(1024)
void dmq_items_from_info_kernel(const int* expert_info, int experts, int tile_rows, int max_items,
                                int pool, int* n_items, int* items) {
  __shared__ int wave_tot[16];
  __shared__ int carry;
  const int tid = threadIdx.x;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < experts; base += 1024) {
    const int e = base + tid;
    int ntile = 0;
    if (e < experts) {
      const int tc = expert_info[4 * e + 1];
      const int sc = expert_info[4 * e + 3];
      ntile = (tc > 0 && sc > 0) ? (tc + tile_rows - 1) / tile_rows : 0;
    }
    const int incl = block_scan_incl(ntile, wave_tot);
    const int first = incl - ntile + carry;
    for (int i = 0; i < ntile; ++i)
      if (first + i < max_items) {
        int* it = items + 4L * (first + i);
        it[0] = pool; it[1] = e; it[2] = i; it[3] = 0;
      }
    __syncthreads();
    if (tid == 1023) carry = incl + carry;
    __syncthreads();
  }
  if (tid == 0) n_items[0] = min(carry, max_items);
}

// out[t, h] = fp16( sum_{j<k} slots[t*k + j, h]  (+ add[t, h]) ), slots summed in slot order
__global__ __launch_bounds__(256)
void dmq_combine_kernel(const float* slots, int k, const __half* add, long tokens, int hidden,
                        __half* out) {
  const int hv = hidden / 4;
  const long total = tokens * hv;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const long t = i / hv;
    const int h = (int)(i % hv) * 4;
    float4_t s = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) s += *(const float4_t*)(slots + (t * k + j) * hidden + h);
    if (add) {
      half4_t a = *(const half4_t*)(add + t * hidden + h);
      s[0] += (float)a[0]; s[1] += (float)a[1]; s[2] += (float)a[2]; s[3] += (float)a[3];
    }
    half4_t o = {(_Float16)s[0], (_Float16)s[1], (_Float16)s[2], (_Float16)s[3]};
    *(half4_t*)(out + t * hidden + h) = o;
  }
}

// ------------------------------------------------------------------------------ host
int dmq_route_topk_launch(const void* logits, int logits_fp16, int tokens, int experts, int k,
                          int renorm, float* out_w, int* out_idx, hipStream_t stream) {
  if (tokens <= 0) return DMQ_OK;
  if (experts > 1024 || k > 64 || k > experts || k <= 0) return DMQ_ERR_LIMIT;
  const int grid = (tokens + 3) / 4;
  if (logits_fp16)
    hipLaunchKernelGGL(dmq_topk_kernel<__half>, dim3(grid), dim3(256), 0, stream,
                       (const __half*)logits, tokens, experts, k, renorm, out_w, out_idx);
  else
    hipLaunchKernelGGL(dmq_topk_kernel<float>, dim3(grid), dim3(256), 0, stream,
                       (const float*)logits, tokens, experts, k, renorm, out_w, out_idx);
  return dmq_check_launch();
}

int dmq_route_permute_launch(const int* topk_idx, const float* topk_w, int tokens, int k,
                             int* counts, const PlanParams& plan, int* sorted_tokens,
                             float* sorted_weights, int* sorted_rows, hipStream_t stream) {
  const int rows = tokens * k;
  const int experts = plan.experts;
  const int grid_e = (experts + 3) / 4;
  hipLaunchKernelGGL(dmq_expert_count_kernel, dim3(grid_e), dim3(256), 0, stream, topk_idx, rows,
                     experts, counts);
  hipLaunchKernelGGL(dmq_plan_kernel, dim3(1), dim3(1024), 0, stream, plan);
  hipLaunchKernelGGL(dmq_expert_fill_kernel, dim3(grid_e), dim3(256), 0, stream, topk_idx, topk_w,
                     rows, k, experts, plan.offsets, sorted_tokens, sorted_weights, sorted_rows);
  return dmq_check_launch();
}

int dmq_items_from_info_launch(const int* expert_info, int experts, int tile_rows, int max_items,
                               int pool, int* n_items, int* items, hipStream_t stream) {
  hipLaunchKernelGGL(dmq_items_from_info_kernel, dim3(1), dim3(1024), 0, stream, expert_info,
                     experts, tile_rows, max_items, pool, n_items, items);
  return dmq_check_launch();
}

int dmq_combine_launch(const float* slots, int k, const __half* add, long tokens, int hidden,
                       __half* out, hipStream_t stream) {
  const long total = tokens * (hidden / 4);
  if (total <= 0) return DMQ_OK;
  long g = (total + 255) / 256;
  if (g > 16384) g = 16384;
  hipLaunchKernelGGL(dmq_combine_kernel, dim3((int)g), dim3(256), 0, stream, slots, k, add, tokens,
                     hidden, out);
  return dmq_check_launch();
}
