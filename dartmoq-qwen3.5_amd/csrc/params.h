// Kernel parameter blocks and host launchers shared between the kernel translation units
// and the extern "C" layer.
#pragma once
#include "common.h"

#define DMQ_MAX_POOLS 4

struct RotPool {
  const __half* rot;       // [*, 128, 128] fp16
  uint8_t* out;            // codes by logical row
  long out_row_bytes;
  void* scale;             // fp16 / fp32 [rows, scale_stride] or u8 [rows, scale_stride] (FP4)
  int scale_stride;
  const int* expert_info;  // tiled pools: [n_experts, 4]
  float extra_scale;
  int mode;                // pools whose mode differs from the kernel's are skipped
  int hoisted;             // 1: every input row is rotated once; 0: rows follow the work items
  int rot_use_slice;       // tiled: 1 = matrices start at the expert's slice_start (down), 0 = at 0
  const int* col_start;    // sub-expert layers (per-work-item pools whose matrix depends on the slice):
                           // first column of the pool's share of each expert [n_experts]; NULL = 0 and
                           // every item spans all `groups`
};

// Side job of a rotation launch in front of a stand-alone Linear GEMM: workgroup 0 also writes the
// work-item list of the GEMM (row tiles of one matrix) and clears its arrival counters.
struct LinearPrep {
  int* info;               // [4] expert_info of the one matrix; NULL = no side job
  int* n_items;            // [1]
  int* items;              // [tiles, DMQ_ITEM_WORDS]
  int tiles, rows, n_out;
  int* zero;               // optional int32 words to clear
  int zero_count;
};

// RMSNorm folded into a consumer of the layer input: the rows handed over are the block's
// pre-norm input h, and every consumer forms x = fp16(h * rstd(row) * (1 + weight)) itself, with
// the arithmetic of dmq_rms_norm_kernel (same bits as the stand-alone kernel's output).
struct PreNorm {
  const void* weight;      // [hidden] fp16 or fp32
  int weight_fp32;
  float eps;
  int on;
};

struct RotParams {
  RotPool pool[DMQ_MAX_POOLS];
  const __half* x;         // [*, x_stride] fp16
  long x_stride;
  const int* row_index;    // tiled pools: physical input row of logical row r (optional)
  int rows;                // hoisted pools: number of input rows
  int groups;              // groups per row
  int n_hoisted;
  int hoisted_pool[DMQ_MAX_POOLS];
  int hoisted_wgs_per_pool;     // set by the launcher
  int hoisted_staged;           // 1: workgroup = one group x four row tiles, matrix staged in LDS
  int tiled_staged;             // same for the per-work-item part (set by the launcher)
  const int* items;        // [*, DMQ_ITEM_WORDS] work-item records
  const int* n_items;
  int tile_rows;           // rows per work item (multiple of 16*TT)
  int scale_fp32;
  int items_prefix;        // 1: only the first n_items[1] items belong to tiled pools
  int also_f16;            // 1: whole-batch pools of mode DMQ_MODE_A16 are served too (rows stored as fp16)
  LinearPrep prep;
  PreNorm pn;              // on: x holds pre-norm rows (whole-batch pools, 16-row tiles only)
};

struct QuantParams {
  const void* x;          // fp16 or fp32 [rows, K]
  int x_fp32;
  long x_stride;
  int rows, groups;
  uint8_t* out;
  long out_row_bytes;
  void* scale;
  int scale_stride;
  int scale_fp32;
  float extra_scale;
};

// Chunking of the routed rows for the counting sort: at most DMQ_SORT_MAX_CHUNKS chunks of a
// multiple of 64 rows.
#define DMQ_SORT_MAX_EXPERTS 2048
#define DMQ_SORT_MAX_CHUNKS 64
#define DMQ_FUSED_FILL_EXPERTS 512      // planning and scatter share a launch up to this many experts
static inline void dmq_sort_chunks(long rows, int* chunk_rows, int* n_chunks) {
  long cr = (rows + DMQ_SORT_MAX_CHUNKS - 1) / DMQ_SORT_MAX_CHUNKS;
  cr = (cr + 63) / 64 * 64;
  if (cr < 64) cr = 64;
  *chunk_rows = (int)cr;
  *n_chunks = (int)((rows + cr - 1) / cr);
}

// Sigmoid gate of the always-on shared experts (n_shared == 0: none).
struct SharedGate {
  const __half* x;               // [tokens, hidden]
  const __half* gate_row;        // [hidden]
  int hidden;
  int n_shared;
  PreNorm pn;                    // on: x holds pre-norm rows, row_rstd their rsqrt(mean square + eps)
  const float* row_rstd;         // [tokens]
};

struct PlanParams {
  int* counts;                   // [experts] rows per expert (written by the plan kernel)
  int* hist;                     // [n_chunks, experts] chunk histogram, then chunk start positions
  int chunk_rows;
  int n_chunks;
  int experts;
  int pools;
  int tile_rows;                 // rows per work item
  int max_items;                 // capacity of the work-item list
  const int* slice_start_rows;   // [pools, experts] gate_up slice start (2*start) or -1 if not a member
  const int* slice_count_rows;   // [pools, experts] gate_up slice count (2*I)
  int* offsets;                  // [experts + 1]
  int* gu_info;                  // [pools, experts, 4]
  int* dn_info;                  // [pools, experts, 4]  slice in groups: start/128, I/128
  int* n_items;                  // [1]; [2] when lead_pools >= 0
  int* items;                    // [max_items, DMQ_ITEM_WORDS]
  // Order in which the pools' items are listed (a permutation of 0 .. pools-1).  With
  // lead_pools >= 0, n_items[1] receives the number of items of the first lead_pools pools of
  // that order (the layer forward lists the pools whose rows are rotated per work item first, so
  // their items are a prefix of the list); lead_pools < 0 leaves n_items[1] alone.
  int pool_order[DMQ_MAX_POOLS];
  int lead_pools;
  // up to 1024 int32 words the planning step sets to zero (the queue words of the persistent GEMM
  // launches that follow); zero_count == 0: none
  int* zero_words;
  int zero_count;
};

// One-workgroup routing for small batches: top-k (or a copy of the caller's top-k), the shared
// columns, the stable sort by expert and the work-item list in a single launch.
#define DMQ_ROUTE_SMALL_ROWS 1024       // routed rows (tokens * (k + n_shared)) it handles
#define DMQ_ROUTE_SMALL_EXPERTS 512     // experts including the shared slices
#define DMQ_ROUTE_SMALL_TOKENS 4        // tokens when the top-k is computed inside (one per wave;
                                        // from 8 tokens on it rides the rotation launch instead)
struct RouteSmallParams {
  const void* logits;            // [tokens, router_experts] fp32 / fp16, or NULL
  int logits_fp16;
  const int* in_idx;             // logits == NULL: top-k of the router [tokens, k]
  const float* in_w;
  int tokens, router_experts, k, renorm;
  SharedGate sg;
  float* out_w;                  // optional [tokens, k + n_shared]: the widened top-k
  int* out_idx;
  PlanParams plan;               // experts = router_experts + n_shared; hist / chunk fields unused
  int* sorted_tokens;
  float* sorted_weights;
  int* sorted_rows;
  int* clear_words;              // optional: clear_count int32 words set to zero by the launch
  int clear_count;
};
int dmq_route_small_launch(const RouteSmallParams& p, hipStream_t stream);

// Routing of at most DMQ_ROUTE_RANK_ROWS routed rows from a finished top-k, for the layer forward:
// one workgroup, one row per thread, every row ranks itself against the whole list (stable sort by
// expert without histograms or scans over experts).  Writes the permutation, the per-expert counts
// and the work items (expert order, dense); no per-pool expert_info, no offsets: the layer's
// launches read neither.  Needs every pool rotated by token (no per-work-item prefix).
#define DMQ_ROUTE_RANK_ROWS 128
struct RouteRankParams {
  const int* in_idx;             // [rows] expert per routed row (token-major, k per token)
  const float* in_w;             // [rows]
  int rows, k, experts, pools, tile_rows, max_items;
  const int* slice_start_rows;   // [pools, experts]
  const int* slice_count_rows;
  int* counts;                   // [experts]
  int* n_items;                  // [2]
  int* items;                    // [max_items, DMQ_ITEM_WORDS]
  int* sorted_tokens;
  float* sorted_weights;
  int* sorted_rows;
  int* clear_words;              // optional: clear_count int32 words set to zero by the launch
  int clear_count;
};
int dmq_route_rank_launch(const RouteRankParams& p, hipStream_t stream);

struct TopkParams;
// tp != NULL: the launch also runs the router's top-k (workgroups in front; logits fp16 or fp32)
int dmq_rotate_dispatch(int mode, const RotParams& p, long tiled_waves, int tt, hipStream_t stream,
                        const TopkParams* tp = nullptr, int topk_fp16 = 0);
struct RouterParams;
int dmq_rotate_router_dispatch(int mode, const RotParams& p, const RouterParams& rt, hipStream_t stream);
int dmq_quantize_dispatch(int mode, const QuantParams& p, hipStream_t stream);

// int8 GEMM of a Linear with 8-bit weights on a uniform grid (w = idx - 128), 128 x 128 tiles
struct LinearI8Params {
  const uint8_t* x;          // int8 codes [rows, x_row_bytes]
  long x_row_bytes;
  const _Float16* x_scale;   // fp16 [rows, scale_stride]
  int scale_stride;
  const uint8_t* w;          // u8 [groups, n_out, 128] group-first indices
  const _Float16* norms;     // fp16 [groups, n_out]
  int rows, groups, n_out;   // n_out % 4 == 0
  _Float16* out;             // fp16 [rows, out_stride]
  long out_stride;
};
int dmq_linear_i8_launch(const LinearI8Params& p, hipStream_t stream);
int dmq_route_topk_launch(const void* logits, int logits_fp16, const int* in_idx, const float* in_w,
                          int tokens, int experts, int k, int renorm, float* out_w, int* out_idx,
                          const SharedGate& sg, hipStream_t stream);
int dmq_route_permute_launch(const int* topk_idx, const float* topk_w, int tokens, int k,
                             const PlanParams& plan, int* sorted_tokens,
                             float* sorted_weights, int* sorted_rows, hipStream_t stream);
int dmq_items_from_info_launch(const int* expert_info, int experts, int tile_rows, int max_items,
                               int pool, int* n_items, int* items, hipStream_t stream);
int dmq_combine_launch(const __half* slots, int k, const __half* add, long tokens, int hidden,
                       __half* out, hipStream_t stream);
int dmq_unpack_launch(const uint8_t* packed, long n_bytes, int bit, uint8_t* out, hipStream_t s);
int dmq_dequant_tile_launch(const uint8_t* idx_gf, const __half* cb, const __half* norms, int n_total,
                            int g0, int g_cnt, int n0, int n_cnt, int bit, __half* out, hipStream_t s);
int dmq_group_first_launch(const uint8_t* idx, const __half* norms, int n_rows, int groups, int ppg,
                           int prescale, uint8_t* idx_gf, __half* norms_gf, hipStream_t s);
int dmq_fold_e2m1_launch(const uint8_t* idx_gf, const uint8_t* nib, long rows, int bit, uint8_t* out,
                         hipStream_t s);
int dmq_quantize_weights_launch(const __half* w, long w_stride, const float* rot, const float* bounds,
                                int n_rows, int groups, int bit, uint8_t* idx_out, __half* norms_out,
                                hipStream_t s);
int dmq_rms_norm_launch(const void* x, int bf16, const void* weight, int weight_fp32, long rows, int n,
                        long x_stride, long out_stride, float eps, void* out, hipStream_t s);
int dmq_finalize_launch(const float* acc, const __half* add, long n, __half* out, hipStream_t s);
