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
//      (up to DMQ_FUSED_FILL_EXPERTS experts steps 3 and 4 are one launch, dmq_plan_fill_kernel,
//      which up to DMQ_FILL_COUNT_ROWS routed rows also counts and so replaces step 2)
//   5. dmq_combine_kernel     out[t] = sum over the k slot rows of token t (fixed order)
#include "params.h"
#include "topk.h"
#include <type_traits>

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
void dmq_topk_kernel(TopkParams tp) {
  dmq_topk_wg<T>(tp, blockIdx.x);
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
  for (int base = r0; base < r1; base += 64 * 8) {      // eight steps of 64 rows per round trip
    int ev[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = base + 64 * i + lane;
      ev[i] = (r < r1) ? topk_idx[r] : -1;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (ev[i] >= 0 && ev[i] < experts) atomicAdd(&cnt[ev[i]], 1);
  }
  __builtin_amdgcn_wave_barrier();
  for (int e = lane; e < experts; e += 64) hist[(long)c * experts + e] = cnt[e];
}

// Inclusive scan over the 64 lanes of a wave with data-parallel lane moves: shifts by 1, 2, 4 and
// 8 inside the rows of 16 lanes, then lane 15 of rows 0 and 2 added to rows 1 and 3 and lane 31 to
// the upper half (a lane with no source adds zero).
__device__ __forceinline__ int wave_scan_incl(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);        // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);        // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);        // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);        // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);        // row_bcast:15 into rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);        // row_bcast:31 into rows 2, 3
  return v;
}

// inclusive scan over the 1024 threads of the workgroup (16 waves)
__device__ __forceinline__ int block_scan_incl(int v, int* wave_tot) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  v = wave_scan_incl(v);
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  int add = 0;                                          // all 16 totals requested at once
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int t = wave_tot[w];
    add += (w < wave) ? t : 0;
  }
  __syncthreads();
  return v + add;
}

// 64-bit variant of the scan: four 16-bit fields scanned at once (no field overflows, so the two
// halves of the word are scanned on their own)
__device__ __forceinline__ unsigned long long block_scan_incl_u64(unsigned long long v,
                                                                  unsigned long long* wave_tot,
                                                                  unsigned long long* total) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  v = (unsigned long long)(unsigned)wave_scan_incl((int)(unsigned)v) |
      ((unsigned long long)(unsigned)wave_scan_incl((int)(unsigned)(v >> 32)) << 32);
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  unsigned long long add = 0, all = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const unsigned long long t = wave_tot[w];
    add += (w < wave) ? t : 0ull;
    all += t;
  }
  *total = all;
  return v + add;
}

// Element `i` (run-time) of a four-entry register array, without indexing it through memory.
__device__ __forceinline__ int pick4(const int (&v)[DMQ_MAX_POOLS], int i) {
  return i == 0 ? v[0] : (i == 1 ? v[1] : (i == 2 ? v[2] : v[3]));
}

// Slice tables of thread tid's expert in every pool, requested early by the callers so that the
// memory latency hides behind the counting phases (one pass: experts <= 1024).
struct PlanSlices { int ss[DMQ_MAX_POOLS], sc[DMQ_MAX_POOLS]; };
__device__ __forceinline__ PlanSlices plan_load_slices(const PlanParams& p) {
  PlanSlices s;
  const int tid = threadIdx.x;
  const bool pre = p.experts <= 1024;
#pragma unroll
  for (int pool = 0; pool < DMQ_MAX_POOLS; ++pool) {
    const bool ok = pre && pool < p.pools && tid < p.experts;
    s.ss[pool] = ok ? p.slice_start_rows[pool * p.experts + tid] : -1;
    s.sc[pool] = ok ? p.slice_count_rows[pool * p.experts + tid] : 0;
  }
  return s;
}

// Per-pool expert_info and the work-item list from the per-expert counts and offsets in LDS
// (pools in caller order, experts ascending).  Called by all 1024 threads of the workgroup.
// With one expert per thread and fewer than 65536 items the tile counts of the (up to four)
// pools are scanned together, 16 bits each: one scan and two barriers for the whole list.
__device__ __forceinline__ void plan_emit_items(const PlanParams& p, const int* s_cnt, const int* s_off,
                                                int* wave_tot, unsigned long long* wave_tot64,
                                                int* carry_p, const PlanSlices& pre_s,
                                                int* item_first = nullptr, int* item_ss = nullptr) {
  const int tid = threadIdx.x;
  if (tid < p.zero_count) p.zero_words[tid] = 0;           // words later launches want cleared
  const bool pre = p.experts <= 1024;
  if (pre && p.max_items < 65536) {
    const bool tile_pow2 = (p.tile_rows & (p.tile_rows - 1)) == 0;
    const int tile_shift = __builtin_ctz((unsigned)p.tile_rows);
    const int e = tid;
    const bool live = e < p.experts;
    const int ts = live ? s_off[e] : 0;
    int ntile[DMQ_MAX_POOLS], tcs[DMQ_MAX_POOLS];
    unsigned long long packed = 0;
#pragma unroll
    for (int pool = 0; pool < DMQ_MAX_POOLS; ++pool) {
      ntile[pool] = 0; tcs[pool] = 0;
      if (pool < p.pools && live) {
        const int ss = pre_s.ss[pool], sc = pre_s.sc[pool];
        const int tc = (ss >= 0) ? s_cnt[e] : 0;
        tcs[pool] = tc;
        ntile[pool] = tile_pow2 ? (tc + p.tile_rows - 1) >> tile_shift : (tc + p.tile_rows - 1) / p.tile_rows;
        packed |= (unsigned long long)ntile[pool] << (16 * pool);
        int4_t* gi = (int4_t*)(p.gu_info + ((long)pool * p.experts + e) * 4);
        *gi = (int4_t){ts, tc, ss >= 0 ? ss : 0, sc};
        int4_t* di = (int4_t*)(p.dn_info + ((long)pool * p.experts + e) * 4);
        *di = (int4_t){ts, tc, ss >= 0 ? ss / (2 * DMQ_GS) : 0, sc / (2 * DMQ_GS)};
      }
    }
    unsigned long long totals;                         // per-pool totals
    const unsigned long long incl = block_scan_incl_u64(packed, wave_tot64, &totals);
    int base = 0, lead = 0;
    if (item_first) {
      // Long batches: an expert with many rows has many tiles, so the records are written one
      // per thread: item_first[o * experts + e] is the first record of (o-th pool of the order,
      // e), and record i belongs to the last entry that starts at or before i.
#pragma unroll
      for (int o = 0; o < DMQ_MAX_POOLS; ++o) {
        if (o < p.pools) {
          const int pool = p.pool_order[o];
          if (live) {
            item_first[o * p.experts + e] = base + (int)((incl >> (16 * pool)) & 0xffffu) - pick4(ntile, pool);
            item_ss[o * p.experts + e] = pick4(pre_s.ss, pool);
          }
          base += (int)((totals >> (16 * pool)) & 0xffffu);
          if (o + 1 == p.lead_pools) lead = base;
        }
      }
      __syncthreads();
      const int n = min(base, p.max_items);
      const int entries = p.pools * p.experts;
      for (int i = tid; i < n; i += 1024) {
        int lo = 0, hi = entries;                        // first entry that starts after i
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if (item_first[mid] <= i) lo = mid + 1; else hi = mid;
        }
        const int idx = lo - 1;
        const int o = idx / p.experts;
        const int ex = idx - o * p.experts;
        const int pool = p.pool_order[o];
        const int ss = item_ss[idx];
        int4_t* it = (int4_t*)(p.items + (long)DMQ_ITEM_WORDS * i);
        it[0] = (int4_t){pool, ex, i - item_first[idx], s_off[ex]};
        it[1] = (int4_t){s_cnt[ex], ss >= 0 ? ss : 0, ss >= 0 ? ss / (2 * DMQ_GS) : 0, 0};
      }
      if (tid == 0) {
        p.n_items[0] = n;
        if (p.lead_pools >= 0) p.n_items[1] = min(lead, p.max_items);
      }
      return;
    }
#pragma unroll
    for (int o = 0; o < DMQ_MAX_POOLS; ++o) {
      if (o < p.pools) {
        const int pool = p.pool_order[o];
        const int nt = pick4(ntile, pool);
        const int first = base + (int)((incl >> (16 * pool)) & 0xffffu) - nt;
        const int ss = pick4(pre_s.ss, pool);
        const int tc = pick4(tcs, pool);
        for (int i = 0; i < nt; ++i) {
          if (first + i < p.max_items) {
            int4_t* it = (int4_t*)(p.items + (long)DMQ_ITEM_WORDS * (first + i));
            it[0] = (int4_t){pool, e, i, ts};
            it[1] = (int4_t){tc, ss >= 0 ? ss : 0, ss >= 0 ? ss / (2 * DMQ_GS) : 0, 0};
          }
        }
        base += (int)((totals >> (16 * pool)) & 0xffffu);
        if (o + 1 == p.lead_pools) lead = base;
      }
    }
    if (tid == 0) {
      p.n_items[0] = min(base, p.max_items);
      if (p.lead_pools >= 0) p.n_items[1] = min(lead, p.max_items);
    }
    return;
  }
  if (tid == 0) *carry_p = 0;
  __syncthreads();
  int lead = 0;
  for (int o = 0; o < p.pools; ++o) {
    const int pool = p.pool_order[o];
    for (int base = 0; base < p.experts; base += 1024) {
      const int e = base + tid;
      int ntile = 0, ts = 0, tc = 0, gu_ss = 0, dn_ss = 0;
      if (e < p.experts) {
        const int ss = pre ? pick4(pre_s.ss, pool) : p.slice_start_rows[pool * p.experts + e];
        const int sc = pre ? pick4(pre_s.sc, pool) : p.slice_count_rows[pool * p.experts + e];
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
      const int first = incl - ntile + *carry_p;
      for (int i = 0; i < ntile; ++i) {
        if (first + i < p.max_items) {
          int4_t* it = (int4_t*)(p.items + (long)DMQ_ITEM_WORDS * (first + i));
          it[0] = (int4_t){pool, e, i, ts};
          it[1] = (int4_t){tc, gu_ss, dn_ss, 0};
        }
      }
      __syncthreads();
      if (tid == 1023) *carry_p = incl + *carry_p;
      __syncthreads();
    }
    if (o + 1 == p.lead_pools) lead = *carry_p;
  }
  if (tid == 0) {
    p.n_items[0] = min(*carry_p, p.max_items);
    if (p.lead_pools >= 0) p.n_items[1] = min(lead, p.max_items);
  }
}

// POSITIONS: also turn hist[c, e] into the position of the first row of chunk c routed to expert e
// (for dmq_chunk_fill_kernel); without it the histogram is only read.
// count_idx != NULL: the rows per expert are counted from the routed rows themselves (no chunk
// histogram is read; at most 16 rows per thread: count_rows <= 16384).
template <bool POSITIONS>
__device__ __forceinline__ void plan_body(const PlanParams& p, const int* count_idx = nullptr,
                                          int count_rows = 0) {
  // counts and offsets live in LDS between the phases; global memory is only written, so the
  // kernel pays one round trip for the histogram and one for the slice tables
  __shared__ int wave_tot[16];
  __shared__ int carry;
  __shared__ int partial[1024];
  __shared__ int s_cnt[DMQ_SORT_MAX_EXPERTS];
  __shared__ int s_off[DMQ_SORT_MAX_EXPERTS + 1];
  __shared__ unsigned long long wave_tot64[17];
  __shared__ int item_first[DMQ_MAX_POOLS * 1024];
  __shared__ int item_ss[DMQ_MAX_POOLS * 1024];
  const int tid = threadIdx.x;
  if (tid == 0) carry = 0;
  const PlanSlices slices = plan_load_slices(p);       // in flight during the counting phases
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
  if (count_idx) {
    // sixteen rows per thread and round trip, each into a counter array of its own: the rows of a
    // popular expert then meet at sixteen addresses instead of one (experts <= DMQ_FUSED_FILL_EXPERTS)
    __shared__ int cnt16[16 * DMQ_FUSED_FILL_EXPERTS];
    for (int i = tid; i < 16 * DMQ_FUSED_FILL_EXPERTS; i += 1024) cnt16[i] = 0;
    int ev[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = 1024 * i + tid;
      ev[i] = (r < count_rows) ? count_idx[r] : -1;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (ev[i] >= 0 && ev[i] < p.experts) atomicAdd(&cnt16[i * DMQ_FUSED_FILL_EXPERTS + ev[i]], 1);
    __syncthreads();
    if (tid < p.experts) {
      int total = 0;
#pragma unroll
      for (int i = 0; i < 16; ++i) total += cnt16[i * DMQ_FUSED_FILL_EXPERTS + tid];
      s_cnt[tid] = total;
      p.counts[tid] = total;
    }
  }
  // rows per expert: column sums of the chunk histogram
  for (int ebase = 0; !count_idx && ebase < p.experts; ebase += epad) {
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
  for (int ebase = 0; POSITIONS && ebase < p.experts; ebase += epad) {
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
  plan_emit_items(p, s_cnt, s_off, wave_tot, wave_tot64, &carry, slices, item_first, item_ss);
}

__global__ __launch_bounds__(1024)
void dmq_plan_kernel(PlanParams p) { plan_body<true>(p); }

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

// Planning and scatter in one launch (layers of at most DMQ_FUSED_FILL_EXPERTS experts).  The last
// workgroup writes counts, offsets, expert_info and the work-item list; the others scatter
// DMQ_FILL_CHUNKS chunks each (one per wave: the scattered stores of more waves would queue up in
// one CU's memory pipeline) and derive the start positions of their chunks themselves, all 16
// waves helping: rows of the experts below e, rows of e in earlier chunks.  Nothing waits for
// another workgroup.
//   COUNT (at most DMQ_FILL_COUNT_ROWS routed rows): straight from the top-k arrays, no histogram
//     launch in front and nothing in global memory between the two: every workgroup counts all
//     routed rows itself (16 per thread, one round trip), per expert and group of DMQ_FILL_CHUNKS
//     chunks.  One CU's LDS takes ~1 us per 16384 atomic adds, so beyond that size
//   !COUNT reads the chunk histogram of dmq_chunk_count_kernel, which 16 CUs build together.
#define DMQ_FILL_CHUNKS 4
#define DMQ_FILL_COUNT_ROWS (1024 * 16)
struct FillParams {
  const int* topk_idx;
  const float* topk_w;
  int rows, k;
  int* sorted_tokens;
  float* sorted_weights;
  int* sorted_rows;
};

template <bool COUNT>
__global__ __launch_bounds__(1024)
void dmq_plan_fill_kernel(PlanParams p, FillParams f) {
  const int fill_blocks = (p.n_chunks + DMQ_FILL_CHUNKS - 1) / DMQ_FILL_CHUNKS;
  if ((int)blockIdx.x >= fill_blocks) {
    if constexpr (COUNT) plan_body<false>(p, f.topk_idx, f.rows);
    else plan_body<false>(p);
    return;
  }
  constexpr int EMAX = DMQ_FUSED_FILL_EXPERTS;
  constexpr int CPB = DMQ_FILL_CHUNKS;
  constexpr int GMAX = DMQ_SORT_MAX_CHUNKS / CPB;
  __shared__ int own[CPB * EMAX];          // rows per (chunk of the block, expert), then their positions
  __shared__ int idle_all[CPB * 64];
  __shared__ int wave_tot[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int experts = p.experts;
  const int c0 = blockIdx.x * CPB;
  const int c = c0 + wave;
  // the first PRE steps of 64 rows of the wave's chunk are requested at once
  constexpr int PRE = 8;
  const int r0 = c * p.chunk_rows;
  const int r1 = (wave < CPB && c < p.n_chunks) ? min(f.rows, r0 + p.chunk_rows) : r0;
  int pre_e[PRE];
  float pre_w[PRE];
  auto prefetch = [&]() {
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
      const int r = r0 + 64 * i + lane;
      pre_e[i] = (r < r1) ? f.topk_idx[r] : -1;
      pre_w[i] = (r < r1) ? f.topk_w[r] : 0.f;
    }
  };
  int tot = 0, bef = 0;
  if constexpr (COUNT) {
    __shared__ int cnt[GMAX * EMAX];       // rows per (group of CPB chunks, expert)
    for (int i = tid; i < GMAX * EMAX; i += 1024) cnt[i] = 0;
    for (int i = tid; i < CPB * EMAX; i += 1024) own[i] = 0;
    prefetch();
    // all rows, sixteen per thread; the group of row r = tid + 1024 i follows without dividing per row
    const int grows = CPB * p.chunk_rows;
    const int gq = 1024 / grows, gm = 1024 % grows;
    int g = tid / grows, rem = tid % grows;
    int ev[16], gv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = 1024 * i + tid;
      ev[i] = (r < f.rows) ? f.topk_idx[r] : -1;
      gv[i] = g;
      g += gq; rem += gm;
      if (rem >= grows) { rem -= grows; ++g; }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (ev[i] >= 0 && ev[i] < experts) atomicAdd(&cnt[gv[i] * EMAX + ev[i]], 1);
    if (wave < CPB) {
      int* mine = own + wave * EMAX;
#pragma unroll
      for (int i = 0; i < PRE; ++i)
        if (pre_e[i] >= 0 && pre_e[i] < experts) atomicAdd(&mine[pre_e[i]], 1);
      for (int r = r0 + 64 * PRE + lane; r < r1; r += 64) {
        const int e = f.topk_idx[r];
        if (e >= 0 && e < experts) atomicAdd(&mine[e], 1);
      }
    }
    __syncthreads();
    if (tid < experts) {
#pragma unroll
      for (int gi = 0; gi < GMAX; ++gi) {
        const int v = cnt[gi * EMAX + tid];
        tot += v;
        bef += (gi < (int)blockIdx.x) ? v : 0;
      }
    }
  } else {
    __shared__ int part_all[1024], part_before[1024];
    if (wave < CPB) {
      for (int e = lane; e < experts; e += 64)
        own[wave * EMAX + e] = (c < p.n_chunks) ? p.hist[(long)c * experts + e] : 0;
    }
    // column sums of the histogram: all chunks, and the chunks in front of this block
    int epad = 64;
    while (epad < experts) epad <<= 1;
    const int parts = 1024 / epad;
    const int part = tid / epad, el = tid % epad;
    const int cpp = (p.n_chunks + parts - 1) / parts;
    const int c_lo = part * cpp;
    const int c_hi = min(p.n_chunks, c_lo + cpp);
    int all = 0, before = 0;
    for (int cc = c_lo; cc < c_hi; cc += 16) {
      int h[16];
#pragma unroll
      for (int i = 0; i < 16; ++i)
        h[i] = (el < experts && cc + i < c_hi) ? p.hist[(long)(cc + i) * experts + el] : 0;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        all += h[i];
        before += (cc + i < c0) ? h[i] : 0;
      }
    }
    prefetch();
    part_all[tid] = all;
    part_before[tid] = before;
    __syncthreads();
    if (tid < experts) {
      for (int q = 0; q < parts; ++q) {
        tot += part_all[q * epad + tid];
        bef += part_before[q * epad + tid];
      }
    }
  }
  const int incl = block_scan_incl(tot, wave_tot);
  // thread e walks the block's chunks of expert e: own[j][e] <- position of the first row of
  // chunk c0 + j routed to e (rows of the experts below e, rows of e in earlier chunks)
  if (tid < experts) {
    int at = incl - tot + bef;
    int h[CPB];
#pragma unroll
    for (int j = 0; j < CPB; ++j) h[j] = own[j * EMAX + tid];
#pragma unroll
    for (int j = 0; j < CPB; ++j) {
      own[j * EMAX + tid] = at;
      at += h[j];
    }
  }
  __syncthreads();
  if (wave >= CPB || c >= p.n_chunks) return;
  int* pos = own + wave * EMAX;
  // Rows of one token name distinct experts, rows of different tokens may share one: the lanes of
  // token j of the step bump the counters in the j-th of a fixed number of operations (LDS executes
  // a wave's operations in order; the other lanes add zero to a word of their own, so the code has
  // no branches and nothing waits for a result before all operations of a step are requested).
  const int k = f.k;
  constexpr int TOKS = 9;                                // tokens a step of 64 rows touches when k >= 8
  int* idle = idle_all + wave * 64 + lane;
  auto rank_fast = [&](int e, int tj) {
    const bool hit = e >= 0 && e < experts;
    int* mine = hit ? pos + e : idle;
    int res[TOKS];
#pragma unroll
    for (int j = 0; j < TOKS; ++j) {
      const bool on = hit && tj == j;
      res[j] = atomicAdd(on ? mine : idle, on ? 1 : 0);
    }
    int at = -1;
#pragma unroll
    for (int j = 0; j < TOKS; ++j) at = (hit && tj == j) ? res[j] : at;
    return at;
  };
  auto rank_any = [&](int base, int e, int tok) {
    const bool hit = e >= 0 && e < experts;
    const int tok_first = base / k;
    const int tok_last = (min(base + 64, r1) - 1) / k;
    int at = -1;
    for (int t = tok_first; t <= tok_last; ++t)
      if (hit && tok == t) at = atomicAdd(&pos[e], 1);
    return at;
  };
  auto put = [&](int r, int tok, int at, float w) {
    if (at >= 0) {
      f.sorted_tokens[at] = tok;
      f.sorted_weights[at] = w;
      f.sorted_rows[at] = r;
    }
  };
  // token of the lane's row, advanced by 64 rows per step without dividing again
  const int q64 = 64 / k, m64 = 64 % k;
  int tok = (r0 + lane) / k, rem = (r0 + lane) % k;
  auto advance = [&]() {
    tok += q64; rem += m64;
    if (rem >= k) { rem -= k; ++tok; }
  };
  if (k >= 8) {
    int at[PRE], tk[PRE];
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
      tk[i] = tok;
      at[i] = (r0 + 64 * i < r1) ? rank_fast(pre_e[i], tok - __builtin_amdgcn_readfirstlane(tok)) : -1;
      advance();
    }
#pragma unroll
    for (int i = 0; i < PRE; ++i) put(r0 + 64 * i + lane, tk[i], at[i], pre_w[i]);
    for (int base = r0 + 64 * PRE; base < r1; base += 64) {
      const int r = base + lane;
      const bool in = r < r1;
      const int at1 = rank_fast(in ? f.topk_idx[r] : -1, tok - __builtin_amdgcn_readfirstlane(tok));
      put(r, tok, at1, in ? f.topk_w[r] : 0.f);
      advance();
    }
  } else {
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
      if (r0 + 64 * i < r1) put(r0 + 64 * i + lane, tok, rank_any(r0 + 64 * i, pre_e[i], tok), pre_w[i]);
      advance();
    }
    for (int base = r0 + 64 * PRE; base < r1; base += 64) {
      const int r = base + lane;
      const bool in = r < r1;
      put(r, tok, rank_any(base, in ? f.topk_idx[r] : -1, tok), in ? f.topk_w[r] : 0.f);
      advance();
    }
  }
}

// Small batches: the whole routing step in one workgroup of 16 waves.  Wave w computes the top-k
// of tokens w, w + 16, ... (or copies the caller's), appends the shared columns and keeps the
// rows in LDS; the sort is the chunked counting sort above with one chunk of 64 rows per wave and
// every table in LDS.
template <typename T>
__global__ __launch_bounds__(1024)
void dmq_route_small_kernel(RouteSmallParams p) {
  __shared__ int wave_tot[16];
  __shared__ int carry;
  __shared__ int s_cnt[DMQ_ROUTE_SMALL_EXPERTS];
  __shared__ int s_off[DMQ_ROUTE_SMALL_EXPERTS + 1];
  __shared__ int s_hist[16 * DMQ_ROUTE_SMALL_EXPERTS];
  __shared__ int s_idx[DMQ_ROUTE_SMALL_ROWS];
  __shared__ float s_w[DMQ_ROUTE_SMALL_ROWS];
  __shared__ int s_idle[1024];
  __shared__ unsigned long long wave_tot64[17];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int k = p.k;
  const int kt = k + p.sg.n_shared;
  const int rows = p.tokens * kt;
  const int experts = p.plan.experts;
  const PlanSlices slices = plan_load_slices(p.plan);  // in flight during the top-k
  for (int i = tid; i < 16 * experts; i += 1024) s_hist[i] = 0;
  for (int i = tid; i < p.clear_count; i += 1024) p.clear_words[i] = 0;
  // top-k (or the caller's), shared columns: the rows of the next token of the wave are requested
  // before the current token is worked on
  auto tokens_of_wave = [&](auto nv_tag) {
    constexpr int NV = decltype(nv_tag)::value;
    float v_next[NV];
    if (p.logits && wave < p.tokens)
      dmq_topk_load<T, NV>((const T*)p.logits + (long)wave * p.router_experts, p.router_experts, lane, v_next);
    for (int tok = wave; tok < p.tokens; tok += 16) {
      float w = 0.f;
      int e = -1;
      float g = 0.f;
      if (p.sg.n_shared > 0) g = dmq_shared_gate_value(p.sg, tok, lane);
      if (p.logits) {
        float v[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = v_next[i];
        if (tok + 16 < p.tokens)
          dmq_topk_load<T, NV>((const T*)p.logits + (long)(tok + 16) * p.router_experts,
                               p.router_experts, lane, v_next);
        dmq_topk_select<NV>(v, p.router_experts, k, p.renorm, lane, w, e);
      } else if (lane < k) {
        w = p.in_w[(long)tok * k + lane];
        e = p.in_idx[(long)tok * k + lane];
      }
      if (lane >= k && lane < kt) { w = g; e = p.router_experts + (lane - k); }
      if (lane < kt) {
        s_idx[tok * kt + lane] = e;
        s_w[tok * kt + lane] = w;
        if (p.out_w) { p.out_w[(long)tok * kt + lane] = w; p.out_idx[(long)tok * kt + lane] = e; }
      }
    }
  };
  if (!p.logits) {
    // a caller-made top-k: one routed row per thread (rows <= 1024), one round trip for all of them;
    // the shared columns four tokens at a time per wave
    if (tid < rows) {
      const int tok = tid / kt, j = tid - tok * kt;
      if (j < k) {
        const float w = p.in_w[(long)tok * k + j];
        const int e = p.in_idx[(long)tok * k + j];
        s_idx[tid] = e;
        s_w[tid] = w;
        if (p.out_w) { p.out_w[tid] = w; p.out_idx[tid] = e; }
      }
    }
    if (p.sg.n_shared > 0) {
      for (int tok0 = wave; tok0 < p.tokens; tok0 += 64) {
        float g[4];
        dmq_shared_gate_values4(p.sg, tok0, 16, p.tokens, lane, g);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int tok = tok0 + 16 * i;
          if (tok < p.tokens && lane >= k && lane < kt) {
            const int e = p.router_experts + (lane - k);
            s_idx[tok * kt + lane] = e;
            s_w[tok * kt + lane] = g[i];
            if (p.out_w) { p.out_w[(long)tok * kt + lane] = g[i]; p.out_idx[(long)tok * kt + lane] = e; }
          }
        }
      }
    }
  } else if (p.router_experts <= 256) tokens_of_wave(std::integral_constant<int, 4>{});
  else if (p.router_experts <= 512) tokens_of_wave(std::integral_constant<int, 8>{});
  else tokens_of_wave(std::integral_constant<int, 16>{});
  __syncthreads();
  // rows per (wave chunk, expert)
  const int r = tid;
  const int e_r = (r < rows) ? s_idx[r] : -1;
  const bool hit = e_r >= 0 && e_r < experts;
  int* my_hist = s_hist + wave * experts;
  if (hit) atomicAdd(&my_hist[e_r], 1);
  __syncthreads();
  if (tid < experts) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) total += s_hist[w * experts + tid];
    s_cnt[tid] = total;
    p.plan.counts[tid] = total;
  }
  __syncthreads();
  {
    const int c = (tid < experts) ? s_cnt[tid] : 0;
    const int incl = block_scan_incl(c, wave_tot);
    if (tid < experts) { s_off[tid + 1] = incl; p.plan.offsets[tid + 1] = incl; }
    if (tid == 0) { s_off[0] = 0; p.plan.offsets[0] = 0; }
  }
  __syncthreads();
  // s_hist[w, e] <- sorted position of the first row of wave chunk w routed to expert e
  if (tid < experts) {
    int at = s_off[tid];
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int n = s_hist[w * experts + tid];
      s_hist[w * experts + tid] = at;
      at += n;
    }
  }
  __syncthreads();
  plan_emit_items(p.plan, s_cnt, s_off, wave_tot, wave_tot64, &carry, slices);
  // stable scatter of the wave's chunk: tokens one after the other, the rows of a token name
  // distinct experts
  const int base = wave * 64;
  if (base < rows) {
    const int tok = r / kt;
    const int tok_first = base / kt;
    const int tok_last = (min(base + 64, rows) - 1) / kt;
    int at = -1;
    if (kt >= 8) {
      // at most nine tokens in the wave's 64 rows: one operation per token, issued back to back
      // (lanes of other tokens add zero to a word of their own)
      int* idle = s_idle + tid;
      int res[9];
#pragma unroll
      for (int j = 0; j < 9; ++j) {
        const bool on = hit && tok - tok_first == j;
        res[j] = atomicAdd(on ? &my_hist[e_r] : idle, on ? 1 : 0);
      }
#pragma unroll
      for (int j = 0; j < 9; ++j) at = (hit && tok - tok_first == j) ? res[j] : at;
    } else {
      for (int t = tok_first; t <= tok_last; ++t) {
        if (hit && tok == t) at = atomicAdd(&my_hist[e_r], 1);
      }
    }
    if (at >= 0) {
      p.sorted_tokens[at] = tok;
      p.sorted_weights[at] = s_w[r];
      p.sorted_rows[at] = r;
    }
  }
}

// See RouteRankParams.  Rows with an expert id outside the layer rank behind all others and get no
// entry anywhere (like the counting sort, which skips them).
#define DMQ_ROUTE_RANK_THREADS 256
__global__ __launch_bounds__(DMQ_ROUTE_RANK_THREADS)
void dmq_route_rank_kernel(RouteRankParams p) {
  __shared__ __attribute__((aligned(16))) int s_expert[DMQ_ROUTE_RANK_ROWS + 4];
  __shared__ __attribute__((aligned(16))) int s_tiles[DMQ_ROUTE_RANK_ROWS + 4];
  const int r = threadIdx.x;
  const bool mine = r < p.rows;
  int e = mine ? p.in_idx[r] : 0x7fffffff;
  const float w = mine ? p.in_w[r] : 0.f;
  const bool valid = mine && e >= 0 && e < p.experts;
  if (!valid) e = 0x7fffffff;
  // the workgroup has more threads than the list has entries (the extra ones only help with the
  // clearing and the per-expert counts): they own no list entry
  static_assert(DMQ_ROUTE_RANK_ROWS <= DMQ_ROUTE_RANK_THREADS && DMQ_ROUTE_RANK_ROWS % 4 == 0,
                "one list entry per thread, read four at a time");
  if (r < DMQ_ROUTE_RANK_ROWS) { s_expert[r] = e; s_tiles[r] = 0; }
  if (r < 4) { s_expert[DMQ_ROUTE_RANK_ROWS + r] = 0x7fffffff; s_tiles[DMQ_ROUTE_RANK_ROWS + r] = 0; }
  for (int i = r; i < p.clear_count; i += DMQ_ROUTE_RANK_THREADS) p.clear_words[i] = 0;
  // slice of the expert in the first pool that holds one: in flight during the scan
  int pool = 0, ss = -1;
  if (valid) {
    // all pools' table entries are requested at once (one round trip), then the first pool wins
    int sc[DMQ_MAX_POOLS], st[DMQ_MAX_POOLS];
#pragma unroll
    for (int q = 0; q < DMQ_MAX_POOLS; ++q) {
      const int qq = q < p.pools ? q : 0;
      sc[q] = p.slice_count_rows[qq * p.experts + e];
      st[q] = p.slice_start_rows[qq * p.experts + e];
    }
#pragma unroll
    for (int q = DMQ_MAX_POOLS - 1; q >= 0; --q)
      if (q < p.pools && sc[q] > 0) { pool = q; ss = st[q]; }
  }
  __syncthreads();
  // the list is read four experts at a time (one address for the whole wave: a broadcast)
  const int rows4 = (p.rows + 3) >> 2;
  int pos = 0, cnt = 0, before = 0;                   // before: rows of my expert ahead of mine
  for (int q = 0; q < rows4; ++q) {
    const int4_t e4 = *(const int4_t*)(s_expert + 4 * q);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int same = (e4[c] == e) ? 1 : 0;
      pos += (e4[c] < e) ? 1 : 0;
      cnt += same;
      before += (same && 4 * q + c < r) ? 1 : 0;
    }
  }
  if (valid) {
    p.sorted_tokens[pos + before] = r / p.k;
    p.sorted_weights[pos + before] = w;
    p.sorted_rows[pos + before] = r;
    if (before == 0 && ss >= 0) s_tiles[r] = (cnt + p.tile_rows - 1) / p.tile_rows;
  }
  __syncthreads();
  // work items: expert order, the tiles of an expert one after the other; the row that opens a
  // tile writes its record
  if (valid && ss >= 0 && before % p.tile_rows == 0) {
    int base = 0;
    for (int q = 0; q < rows4; ++q) {
      const int4_t e4 = *(const int4_t*)(s_expert + 4 * q);
      const int4_t t4 = *(const int4_t*)(s_tiles + 4 * q);
#pragma unroll
      for (int c = 0; c < 4; ++c) base += (e4[c] < e) ? t4[c] : 0;
    }
    const int idx = base + before / p.tile_rows;
    if (idx < p.max_items) {
      int4_t* it = (int4_t*)(p.items + (long)DMQ_ITEM_WORDS * idx);
      it[0] = (int4_t){pool, e, before / p.tile_rows, pos};
      it[1] = (int4_t){cnt, ss, ss / (2 * DMQ_GS), 0};
    }
  }
  for (int x = r; x < p.experts; x += DMQ_ROUTE_RANK_THREADS) {
    int c = 0;
    for (int q = 0; q < rows4; ++q) {
      const int4_t e4 = *(const int4_t*)(s_expert + 4 * q);
      c += (e4[0] == x) + (e4[1] == x) + (e4[2] == x) + (e4[3] == x);
    }
    p.counts[x] = c;
  }
  if (r == 0) {
    int n = 0;
    for (int q = 0; q < rows4; ++q) {
      const int4_t t4 = *(const int4_t*)(s_tiles + 4 * q);
      n += t4[0] + t4[1] + t4[2] + t4[3];
    }
    p.n_items[0] = min(n, p.max_items);
    p.n_items[1] = 0;
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
  else {
    const TopkParams tp{logits, tokens, experts, k, renorm, out_w, out_idx, sg, grid};
    if (logits_fp16) hipLaunchKernelGGL(dmq_topk_kernel<__half>, dim3(grid), dim3(256), 0, stream, tp);
    else hipLaunchKernelGGL(dmq_topk_kernel<float>, dim3(grid), dim3(256), 0, stream, tp);
  }
  return dmq_check_launch();
}

int dmq_route_permute_launch(const int* topk_idx, const float* topk_w, int tokens, int k,
                             const PlanParams& plan, int* sorted_tokens,
                             float* sorted_weights, int* sorted_rows, hipStream_t stream) {
  const int rows = tokens * k;
  const int experts = plan.experts;
  if (experts > DMQ_SORT_MAX_EXPERTS) return DMQ_ERR_LIMIT;
  const FillParams f{topk_idx, topk_w, rows, k, sorted_tokens, sorted_weights, sorted_rows};
  const dim3 grid_pf((plan.n_chunks + DMQ_FILL_CHUNKS - 1) / DMQ_FILL_CHUNKS + 1);
  if (experts <= DMQ_FUSED_FILL_EXPERTS && rows <= DMQ_FILL_COUNT_ROWS) {
    hipLaunchKernelGGL(dmq_plan_fill_kernel<true>, grid_pf, dim3(1024), 0, stream, plan, f);
    return dmq_check_launch();
  }
  const int grid_c = (plan.n_chunks + 3) / 4;
  hipLaunchKernelGGL(dmq_chunk_count_kernel, dim3(grid_c), dim3(256), 0, stream, topk_idx, rows,
                     experts, plan.chunk_rows, plan.n_chunks, plan.hist);
  if (experts <= DMQ_FUSED_FILL_EXPERTS) {
    hipLaunchKernelGGL(dmq_plan_fill_kernel<false>, grid_pf, dim3(1024), 0, stream, plan, f);
    return dmq_check_launch();
  }
  hipLaunchKernelGGL(dmq_plan_kernel, dim3(1), dim3(1024), 0, stream, plan);
  hipLaunchKernelGGL(dmq_chunk_fill_kernel, dim3(grid_c), dim3(256), 0, stream, topk_idx, topk_w,
                     rows, k, experts, plan.chunk_rows, plan.n_chunks, plan.hist, sorted_tokens,
                     sorted_weights, sorted_rows);
  return dmq_check_launch();
}

int dmq_route_small_launch(const RouteSmallParams& p, hipStream_t stream) {
  const int kt = p.k + p.sg.n_shared;
  if ((long)p.tokens * kt > DMQ_ROUTE_SMALL_ROWS || p.plan.experts > DMQ_ROUTE_SMALL_EXPERTS || kt > 64)
    return DMQ_ERR_LIMIT;
  if (p.logits && (p.router_experts > 1024 || p.k > p.router_experts)) return DMQ_ERR_LIMIT;
  if (p.sg.n_shared > 0 && p.sg.hidden % 8) return DMQ_ERR_ALIGN;
  if (p.logits && p.logits_fp16)
    hipLaunchKernelGGL(dmq_route_small_kernel<__half>, dim3(1), dim3(1024), 0, stream, p);
  else
    hipLaunchKernelGGL(dmq_route_small_kernel<float>, dim3(1), dim3(1024), 0, stream, p);
  return dmq_check_launch();
}

int dmq_route_rank_launch(const RouteRankParams& p, hipStream_t stream) {
  if (p.rows <= 0 || p.rows > DMQ_ROUTE_RANK_ROWS || p.k <= 0 || p.tile_rows <= 0) return DMQ_ERR_LIMIT;
  if (p.pools <= 0 || p.pools > DMQ_MAX_POOLS || p.experts <= 0) return DMQ_ERR_LIMIT;
  hipLaunchKernelGGL(dmq_route_rank_kernel, dim3(1), dim3(DMQ_ROUTE_RANK_THREADS), 0, stream, p);
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
