// Top-k routing and token permutation: sort the T*k routed rows by expert (stable) and
// partition the experts of every bit pool into tiles of activation rows, all on the device
// (no host synchronisation, no atomics, deterministic output order).
//
//   1. dmq_topk_kernel        one wave per token: softmax statistics + k arg-max rounds
//   2. dmq_expert_count_kernel one wave per expert: count rows routed to it
//   3. dmq_plan_kernel        one workgroup: exclusive scan -> offsets, per-pool expert_info
//                             and tile lists
//   4. dmq_expert_fill_kernel one wave per expert: write its rows in (token, slot) order
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
__global__ __launch_bounds__(256)
void dmq_expert_count_kernel(const int* topk_idx, int rows, int experts, int* counts) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= experts) return;
  int c = 0;
  for (int r = lane; r < rows; r += 64) c += (topk_idx[r] == e) ? 1 : 0;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) c += __shfl_xor(c, m, 64);
  if (lane == 0) counts[e] = c;
}

// Layout of the plan buffer (int32):
//   offsets[experts + 1]
//   per pool p (pools in caller order):
//     expert_info[experts][4]   token_start, token_count, slice_start, slice_count
//     n_tiles[1] (+3 padding)
//     tiles[max_tiles][2]       expert slot, token tile
// Every expert gets an expert_info row in every pool; non-members have token_count 0.

__global__ __launch_bounds__(1024)
void dmq_plan_kernel(PlanParams p) {
  __shared__ int scan[1024];
  __shared__ int carry;
  const int tid = threadIdx.x;
  if (tid == 0) carry = 0;
  __syncthreads();
  // exclusive scan of counts, 1024 experts per pass
  for (int base = 0; base < p.experts; base += 1024) {
    const int e = base + tid;
    const int c = (e < p.experts) ? p.counts[e] : 0;
    scan[tid] = c;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
      int add = (tid >= d) ? scan[tid - d] : 0;
      __syncthreads();
      scan[tid] += add;
      __syncthreads();
    }
    const int incl = scan[tid] + carry;
    if (e < p.experts) p.offsets[e + 1] = incl;
    __syncthreads();
    if (tid == 1023) carry = incl;
    __syncthreads();
  }
  if (tid == 0) p.offsets[0] = 0;
  __syncthreads();
  __threadfence_block();

  for (int pool = 0; pool < p.pools; ++pool) {
    if (tid == 0) carry = 0;
    __syncthreads();
    for (int base = 0; base < p.experts; base += 1024) {
      const int e = base + tid;
      int ntile = 0, ts = 0, tc = 0, ss = 0, sc = 0;
      if (e < p.experts) {
        ss = p.slice_start_rows[pool * p.experts + e];
        sc = p.slice_count_rows[pool * p.experts + e];
        ts = (e == 0) ? 0 : p.offsets[e];
        tc = (ss >= 0) ? p.counts[e] : 0;
        ntile = (tc + p.tile_rows - 1) / p.tile_rows;
        int* gi = p.gu_info + ((long)pool * p.experts + e) * 4;
        gi[0] = ts; gi[1] = tc; gi[2] = ss >= 0 ? ss : 0; gi[3] = sc;
        int* di = p.dn_info + ((long)pool * p.experts + e) * 4;
        di[0] = ts; di[1] = tc; di[2] = ss >= 0 ? ss / (2 * DMQ_GS) : 0; di[3] = sc / (2 * DMQ_GS);
      }
      scan[tid] = ntile;
      __syncthreads();
      for (int d = 1; d < 1024; d <<= 1) {
        int add = (tid >= d) ? scan[tid - d] : 0;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
      }
      const int first = scan[tid] - ntile + carry;
      int* tl = p.tiles + (long)pool * p.max_tiles * 2;
      for (int i = 0; i < ntile; ++i) {
        if (first + i < p.max_tiles) { tl[2 * (first + i)] = e; tl[2 * (first + i) + 1] = i; }
      }
      __syncthreads();
      if (tid == 1023) carry = scan[1023] + carry;
      __syncthreads();
    }
    if (tid == 0) p.n_tiles[pool * 4] = min(carry, p.max_tiles);
    __syncthreads();
  }
}

__global__ __launch_bounds__(256)
void dmq_expert_fill_kernel(const int* topk_idx, const float* topk_w, int rows, int k, int experts,
                            const int* offsets, int* sorted_tokens, float* sorted_weights,
                            int* sorted_slots) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= experts) return;
  int pos = offsets[e];
  for (int base = 0; base < rows; base += 64) {
    const int r = base + lane;
    const bool hit = (r < rows) && (topk_idx[r] == e);
    const unsigned long long mask = __ballot(hit);
    if (hit) {
      const int rank = __popcll(mask & ((1ull << lane) - 1ull));
      sorted_tokens[pos + rank] = r / k;
      sorted_weights[pos + rank] = topk_w[r];
      if (sorted_slots) sorted_slots[pos + rank] = r % k;
    }
    pos += __popcll(mask);
  }
}

// Tile list for a caller-supplied expert_info (merged-GEMM entry points): one workgroup.
__global__ __launch_bounds__(1024)
void dmq_tiles_from_info_kernel(const int* expert_info, int experts, int tile_rows, int max_tiles,
                                int* n_tiles, int* tiles) {
  __shared__ int scan[1024];
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
    scan[tid] = ntile;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
      int add = (tid >= d) ? scan[tid - d] : 0;
      __syncthreads();
      scan[tid] += add;
      __syncthreads();
    }
    const int first = scan[tid] - ntile + carry;
    for (int i = 0; i < ntile; ++i)
      if (first + i < max_tiles) { tiles[2 * (first + i)] = e; tiles[2 * (first + i) + 1] = i; }
    __syncthreads();
    if (tid == 1023) carry = scan[1023] + carry;
    __syncthreads();
  }
  if (tid == 0) n_tiles[0] = min(carry, max_tiles);
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
                             float* sorted_weights, int* sorted_slots, hipStream_t stream) {
  const int rows = tokens * k;
  const int experts = plan.experts;
  const int grid_e = (experts + 3) / 4;
  hipLaunchKernelGGL(dmq_expert_count_kernel, dim3(grid_e), dim3(256), 0, stream, topk_idx, rows,
                     experts, counts);
  hipLaunchKernelGGL(dmq_plan_kernel, dim3(1), dim3(1024), 0, stream, plan);
  hipLaunchKernelGGL(dmq_expert_fill_kernel, dim3(grid_e), dim3(256), 0, stream, topk_idx, topk_w,
                     rows, k, experts, plan.offsets, sorted_tokens, sorted_weights, sorted_slots);
  return dmq_check_launch();
}

int dmq_tiles_from_info_launch(const int* expert_info, int experts, int tile_rows, int max_tiles,
                               int* n_tiles, int* tiles, hipStream_t stream) {
  hipLaunchKernelGGL(dmq_tiles_from_info_kernel, dim3(1), dim3(1024), 0, stream, expert_info,
                     experts, tile_rows, max_tiles, n_tiles, tiles);
  return dmq_check_launch();
}
