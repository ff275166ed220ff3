// Top-k routing and token permutation: sort the T*k routed rows by expert (stable) and
// partition the experts of every bit pool into tiles of activation rows, all on the device
// (no host synchronisation, no global atomics, deterministic output order).
//
//   1. dmq_topk_kernel        one wave per token: softmax statistics + k arg-max rounds
//   2. dmq_chunk_count_kernel one wave per chunk of rows: per-chunk expert histogram (LDS)
//   3. dmq_plan_kernel        one workgroup: counts, exclusive scan -> offsets, start position
//                             of every (chunk, expert), per-pool expert_info and the work-item
//                             list (pool, expert, row tile) of the layer
//   4. dmq_chunk_fill_kernel  one wave per chunk: write its rows to their sorted positions
//   5. dmq_combine_kernel     out[t] = sum over the k slot rows of token t (fixed order)
#include "params.h"

// ------------------------------------------------------------------------------ top-k
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }

// Always-on shared experts ride the routed path as n_shared extra columns of the top-k arrays:
// column k + j names expert `experts + j` with weight sigmoid(x . gate_row), rounded to fp16 after
// the dot and after the sigmoid like an fp16 Linear followed by torch.sigmoid.
__device__ __forceinline__ void dmq_shared_columns(const SharedGate& sg, int tok, int experts, int k,
                                                   int lane, float* out_w, int* out_idx) {
  if (sg.n_shared <= 0) return;
  const __half* xr = sg.x + (long)tok * sg.hidden;
  float dot = 0.f;
  for (int h = lane * 8; h < sg.hidden; h += 512) {
    const half8_t a = *(const half8_t*)(xr + h);
    const half8_t b = *(const half8_t*)(sg.gate_row + h);
#pragma unroll
    for (int c = 0; c < 8; ++c) dot += (float)a[c] * (float)b[c];
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) dot += __shfl_xor(dot, m, 64);
  const float z = (float)(_Float16)dot;
  const float g = (float)(_Float16)(1.f / (1.f + expf(-z)));
  const int stride = k + sg.n_shared;
  if (lane < sg.n_shared) {
    out_w[(long)tok * stride + k + lane] = g;
    out_idx[(long)tok * stride + k + lane] = experts + lane;
  }
}

// Widen caller-made top-k arrays [tokens, k] by the shared columns.
__global__ __launch_bounds__(256)
void dmq_topk_widen_kernel(const int* in_idx, const float* in_w, int tokens, int experts, int k,
                           float* out_w, int* out_idx, SharedGate sg) {
  const int lane = threadIdx.x & 63;
  const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= tokens) return;
  const int stride = k + sg.n_shared;
  for (int j = lane; j < k; j += 64) {
    out_w[(long)tok * stride + j] = in_w[(long)tok * k + j];
    out_idx[(long)tok * stride + j] = in_idx[(long)tok * k + j];
  }
  dmq_shared_columns(sg, tok, experts, k, lane, out_w, out_idx);
}

template <typename T>
__global__ __launch_bounds__(256)
void dmq_topk_kernel(const T* logits, int tokens, int experts, int k, int renorm,
                     float* out_w, int* out_idx, SharedGate sg) {
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
  const int stride = k + sg.n_shared;
  if (lane < k) {
    out_w[(long)tok * stride + lane] = renorm ? my_w / wsum : my_w;
    out_idx[(long)tok * stride + lane] = my_e;
  }
  dmq_shared_columns(sg, tok, experts, k, lane, out_w, out_idx);
}

// ------------------------------------------------------------------------------ counting
// The routed rows (token-major, k per token) are cut into chunks of chunk_rows; one wave owns a
// chunk and walks it 64 rows at a time.  hist[c, e] first holds the number of rows of chunk c
// routed to expert e; the plan kernel turns it into the position of the first such row in the
// expert-sorted order, which makes the permutation a stable counting sort.
__global__ __launch_bounds__(256)
void dmq_chunk_count_kernel(const int* topk_idx, int rows, int experts, int chunk_rows, int n_chunks,
                            int* hist) {
  __shared__ int cnt_all[4 * DMQ_SORT_MAX_EXPERTS];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 4 + wave;
  if (c >= n_chunks) return;
  int* cnt = cnt_all + wave * DMQ_SORT_MAX_EXPERTS;
  for (int e = lane; e < experts; e += 64) cnt[e] = 0;
  __builtin_amdgcn_wave_barrier();
  const int r0 = c * chunk_rows;
  const int r1 = min(rows, r0 + chunk_rows);
  for (int r = r0 + lane; r < r1; r += 64) {
    const int e = topk_idx[r];
    if (e >= 0 && e < experts) atomicAdd(&cnt[e], 1);
  }
  __builtin_amdgcn_wave_barrier();
  for (int e = lane; e < experts; e += 64) hist[(long)c * experts + e] = cnt[e];
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
  // counts and offsets live in LDS between the phases; global memory is only written, so the
  // kernel pays one round trip for the histogram and one for the slice tables
  __shared__ int wave_tot[16];
  __shared__ int carry;
  __shared__ int partial[1024];
  __shared__ int s_cnt[DMQ_SORT_MAX_EXPERTS];
  __shared__ int s_off[DMQ_SORT_MAX_EXPERTS + 1];
  const int tid = threadIdx.x;
  if (tid == 0) carry = 0;
  // The chunk axis of the histogram is split over `parts` threads per expert so that all 1024
  // threads load; a thread keeps at most 16 loads in flight and its values stay in registers
  // when its share of the chunks fits (16 per thread: up to 64 chunks at <= 256 experts).
  int epad = 64;
  while (epad < p.experts && epad < 1024) epad <<= 1;
  const int parts = 1024 / epad;
  const int part = tid / epad;
  const int el = tid % epad;
  const int cpp = (p.n_chunks + parts - 1) / parts;
  const int c_lo = part * cpp;
  const int c_hi = min(p.n_chunks, c_lo + cpp);
  const bool one_pass = p.experts <= epad && cpp <= 16;
  int h[16];
  auto load16 = [&](int e, int c0) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      h[i] = (e < p.experts && c0 + i < c_hi) ? p.hist[(long)(c0 + i) * p.experts + e] : 0;
  };
  auto chunk_sum = [&](int e) {
    int sum = 0;
    for (int c0 = c_lo; c0 < c_hi; c0 += 16) {
      load16(e, c0);
#pragma unroll
      for (int i = 0; i < 16; ++i) sum += h[i];
    }
    return sum;
  };
  // rows per expert: column sums of the chunk histogram
  for (int ebase = 0; ebase < p.experts; ebase += epad) {
    const int e = ebase + el;
    partial[tid] = chunk_sum(e);
    __syncthreads();
    if (part == 0 && e < p.experts) {
      int total = 0;
      for (int q = 0; q < parts; ++q) total += partial[q * epad + el];
      s_cnt[e] = total;
      p.counts[e] = total;
    }
    if (!one_pass) __syncthreads();                    // partial[] is reused by the next pass
  }
  __syncthreads();
  // expert offsets: exclusive scan of counts, 1024 experts per pass
  for (int base = 0; base < p.experts; base += 1024) {
    const int e = base + tid;
    const int c = (e < p.experts) ? s_cnt[e] : 0;
    const int incl = block_scan_incl(c, wave_tot) + carry;
    if (e < p.experts) { s_off[e + 1] = incl; p.offsets[e + 1] = incl; }
    __syncthreads();
    if (tid == 1023) carry = incl;
    __syncthreads();
  }
  if (tid == 0) { s_off[0] = 0; p.offsets[0] = 0; }
  __syncthreads();
  // hist[c, e] <- position of the first row of chunk c routed to expert e
  for (int ebase = 0; ebase < p.experts; ebase += epad) {
    const int e = ebase + el;
    if (!one_pass) {
      partial[tid] = chunk_sum(e);
      __syncthreads();
    }
    if (e < p.experts) {
      int at = s_off[e];
      for (int q = 0; q < part; ++q) at += partial[q * epad + el];
      for (int c0 = c_lo; c0 < c_hi; c0 += 16) {
        if (!one_pass) load16(e, c0);                  // one_pass: h[] still holds this thread's chunks
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (c0 + i < c_hi) p.hist[(long)(c0 + i) * p.experts + e] = at;
          at += h[i];
        }
      }
    }
    if (!one_pass) __syncthreads();
  }

  // per-pool expert_info and the work-item list, pools in caller order, experts ascending
  if (tid == 0) carry = 0;
  // the slice tables of all pools are requested at once when one pass covers the experts
  int ss_pre[DMQ_MAX_POOLS], sc_pre[DMQ_MAX_POOLS];
  const bool pre = p.experts <= 1024;
#pragma unroll
  for (int pool = 0; pool < DMQ_MAX_POOLS; ++pool) {
    const bool ok = pre && pool < p.pools && tid < p.experts;
    ss_pre[pool] = ok ? p.slice_start_rows[pool * p.experts + tid] : -1;
    sc_pre[pool] = ok ? p.slice_count_rows[pool * p.experts + tid] : 0;
  }
  __syncthreads();
#pragma unroll
  for (int pool = 0; pool < DMQ_MAX_POOLS; ++pool) {
    if (pool >= p.pools) break;
    for (int base = 0; base < p.experts; base += 1024) {
      const int e = base + tid;
      int ntile = 0, ts = 0, tc = 0, gu_ss = 0, dn_ss = 0;
      if (e < p.experts) {
        const int ss = pre ? ss_pre[pool] : p.slice_start_rows[pool * p.experts + e];
        const int sc = pre ? sc_pre[pool] : p.slice_count_rows[pool * p.experts + e];
        tc = (ss >= 0) ? s_cnt[e] : 0;
        ts = s_off[e];
        gu_ss = ss >= 0 ? ss : 0;
        dn_ss = ss >= 0 ? ss / (2 * DMQ_GS) : 0;
        ntile = (tc + p.tile_rows - 1) / p.tile_rows;
        int* gi = p.gu_info + ((long)pool * p.experts + e) * 4;
        gi[0] = ts; gi[1] = tc; gi[2] = gu_ss; gi[3] = sc;
        int* di = p.dn_info + ((long)pool * p.experts + e) * 4;
        di[0] = ts; di[1] = tc; di[2] = dn_ss; di[3] = sc / (2 * DMQ_GS);
      }
      const int incl = block_scan_incl(ntile, wave_tot);
      const int first = incl - ntile + carry;
      for (int i = 0; i < ntile; ++i) {
        if (first + i < p.max_items) {
          int4_t* it = (int4_t*)(p.items + (long)DMQ_ITEM_WORDS * (first + i));
          it[0] = (int4_t){pool, e, i, ts};
          it[1] = (int4_t){tc, gu_ss, dn_ss, 0};
        }
      }
      __syncthreads();
      if (tid == 1023) carry = incl + carry;
      __syncthreads();
    }
  }
  if (tid == 0) p.n_items[0] = min(carry, p.max_items);
}

// Stable scatter of one chunk.  The rows of one token name distinct experts, so the lanes of a
// token bump distinct counters; tokens are taken one after the other and LDS executes a wave's
// operations in order, hence rows of an expert keep their original order.
__global__ __launch_bounds__(256)
void dmq_chunk_fill_kernel(const int* topk_idx, const float* topk_w, int rows, int k, int experts,
                           int chunk_rows, int n_chunks, const int* hist, int* sorted_tokens,
                           float* sorted_weights, int* sorted_rows) {
  __shared__ int pos_all[4 * DMQ_SORT_MAX_EXPERTS];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 4 + wave;
  if (c >= n_chunks) return;
  int* pos = pos_all + wave * DMQ_SORT_MAX_EXPERTS;
  for (int e = lane; e < experts; e += 64) pos[e] = hist[(long)c * experts + e];
  __builtin_amdgcn_wave_barrier();
  const int r0 = c * chunk_rows;
  const int r1 = min(rows, r0 + chunk_rows);
  for (int base = r0; base < r1; base += 64) {
    const int r = base + lane;
    const bool in = r < r1;
    const int e = in ? topk_idx[r] : -1;
    const float w = in ? topk_w[r] : 0.f;
    const bool hit = e >= 0 && e < experts;
    const int tok = r / k;
    const int tok_first = base / k;
    const int tok_last = (min(base + 64, r1) - 1) / k;
    int at = -1;
    for (int t = tok_first; t <= tok_last; ++t) {
      if (hit && tok == t) at = atomicAdd(&pos[e], 1);
    }
    if (at >= 0) {
      sorted_tokens[at] = tok;
      sorted_weights[at] = w;
      sorted_rows[at] = r;
    }
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
    int ntile = 0, ts = 0, tc = 0, ss = 0;
    if (e < experts) {
      ts = expert_info[4 * e + 0];
      tc = expert_info[4 * e + 1];
      ss = expert_info[4 * e + 2];
      const int sc = expert_info[4 * e + 3];
      ntile = (tc > 0 && sc > 0) ? (tc + tile_rows - 1) / tile_rows : 0;
    }
    const int incl = block_scan_incl(ntile, wave_tot);
    const int first = incl - ntile + carry;
    for (int i = 0; i < ntile; ++i)
      if (first + i < max_items) {
        int4_t* it = (int4_t*)(items + (long)DMQ_ITEM_WORDS * (first + i));
        it[0] = (int4_t){pool, e, i, ts};
        it[1] = (int4_t){tc, ss, ss, 0};
      }
    __syncthreads();
    if (tid == 1023) carry = incl + carry;
    __syncthreads();
  }
  if (tid == 0) n_items[0] = min(carry, max_items);
}

// out[t, h] = fp16( sum_{j<k} slots[t*k + j, h]  (+ add[t, h]) ): fp16 slots summed in fp32 in
// slot order (the reference accumulates the same fp16 expert rows with index_add_ in fp16)
__global__ __launch_bounds__(256)
void dmq_combine_kernel(const __half* slots, int k, const __half* add, long tokens, int hidden,
                        __half* out) {
  const int hv = hidden / 8;
  const long total = tokens * hv;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const long t = i / hv;
    const int h = (int)(i % hv) * 8;
    float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const half8_t v = *(const half8_t*)(slots + (t * k + j) * hidden + h);
#pragma unroll
      for (int c = 0; c < 8; ++c) s[c] += (float)v[c];
    }
    if (add) {
      const half8_t a = *(const half8_t*)(add + t * hidden + h);
#pragma unroll
      for (int c = 0; c < 8; ++c) s[c] += (float)a[c];
    }
    half8_t o;
#pragma unroll
    for (int c = 0; c < 8; ++c) o[c] = (_Float16)s[c];
    *(half8_t*)(out + t * hidden + h) = o;
  }
}

// ------------------------------------------------------------------------------ host
int dmq_route_topk_launch(const void* logits, int logits_fp16, const int* in_idx, const float* in_w,
                          int tokens, int experts, int k, int renorm, float* out_w, int* out_idx,
                          const SharedGate& sg, hipStream_t stream) {
  if (tokens <= 0) return DMQ_OK;
  if (experts > 1024 || k > 64 || k > experts || k <= 0 || sg.n_shared > 64) return DMQ_ERR_LIMIT;
  if (sg.n_shared > 0 && sg.hidden % 8) return DMQ_ERR_ALIGN;
  const int grid = (tokens + 3) / 4;
  if (!logits)
    hipLaunchKernelGGL(dmq_topk_widen_kernel, dim3(grid), dim3(256), 0, stream, in_idx, in_w, tokens,
                       experts, k, out_w, out_idx, sg);
  else if (logits_fp16)
    hipLaunchKernelGGL(dmq_topk_kernel<__half>, dim3(grid), dim3(256), 0, stream,
                       (const __half*)logits, tokens, experts, k, renorm, out_w, out_idx, sg);
  else
    hipLaunchKernelGGL(dmq_topk_kernel<float>, dim3(grid), dim3(256), 0, stream,
                       (const float*)logits, tokens, experts, k, renorm, out_w, out_idx, sg);
  return dmq_check_launch();
}

int dmq_route_permute_launch(const int* topk_idx, const float* topk_w, int tokens, int k,
                             const PlanParams& plan, int* sorted_tokens,
                             float* sorted_weights, int* sorted_rows, hipStream_t stream) {
  const int rows = tokens * k;
  const int experts = plan.experts;
  if (experts > DMQ_SORT_MAX_EXPERTS) return DMQ_ERR_LIMIT;
  const int grid_c = (plan.n_chunks + 3) / 4;
  hipLaunchKernelGGL(dmq_chunk_count_kernel, dim3(grid_c), dim3(256), 0, stream, topk_idx, rows,
                     experts, plan.chunk_rows, plan.n_chunks, plan.hist);
  hipLaunchKernelGGL(dmq_plan_kernel, dim3(1), dim3(1024), 0, stream, plan);
  hipLaunchKernelGGL(dmq_chunk_fill_kernel, dim3(grid_c), dim3(256), 0, stream, topk_idx, topk_w,
                     rows, k, experts, plan.chunk_rows, plan.n_chunks, plan.hist, sorted_tokens,
                     sorted_weights, sorted_rows);
  return dmq_check_launch();
}

int dmq_items_from_info_launch(const int* expert_info, int experts, int tile_rows, int max_items,
                               int pool, int* n_items, int* items, hipStream_t stream) {
  hipLaunchKernelGGL(dmq_items_from_info_kernel, dim3(1), dim3(1024), 0, stream, expert_info,
                     experts, tile_rows, max_items, pool, n_items, items);
  return dmq_check_launch();
}

int dmq_combine_launch(const __half* slots, int k, const __half* add, long tokens, int hidden,
                       __half* out, hipStream_t stream) {
  const long total = tokens * (hidden / 8);
  if (total <= 0) return DMQ_OK;
  long g = (total + 255) / 256;
  if (g > 16384) g = 16384;
  hipLaunchKernelGGL(dmq_combine_kernel, dim3((int)g), dim3(256), 0, stream, slots, k, add, tokens,
                     hidden, out);
  return dmq_check_launch();
}
