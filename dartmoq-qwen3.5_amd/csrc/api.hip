// extern "C" surface of libdartmoq_hip.so: argument checks, workspace carving and launches.
#include "params.h"
#include "topk.h"
#include "gemm_dispatch.h"
#include "router.h"

__global__ __launch_bounds__(256) void dmq_fill_zero_kernel(uint32_t* p, long n_words) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_words;
       i += (long)gridDim.x * blockDim.x)
    p[i] = 0u;
}

static inline int act_bytes_per_group(int mode) {
  return mode == DMQ_MODE_A16 ? 256 : (mode == DMQ_MODE_FP4 ? 64 : 128);
}

// Inside the layer workspace every code row spans K*2 bytes and every scale row 4 bytes per
// group whatever the precision mode, so pools of different modes can share one buffer
// without their rows overlapping.  The stride is counted in scale elements (fp16 or byte).
static inline int scale_stride_for(int mode, int k) {
  return mode == DMQ_MODE_FP4 ? k / 32 : k / 64;
}

static inline bool valid_mode(int m) { return m >= DMQ_MODE_A16 && m <= DMQ_MODE_FP4; }

// K split of the 16-row tile kernels for short work lists.  Up to 128 routed rows leave most CUs
// with at most one workgroup: two workgroups then share the K range of every gate_up block, four
// with at most 16 rows (negative value; the group count must divide).  Measured at H=2048 / 3072:
// four-way wins up to 16 rows (1 token: 30.6 -> 28.7 us), two-way up to 128, none beyond.
// Splitting K over the four waves of a workgroup instead only pays when the groups do not divide.
static inline int pick_ks(int tt, long rows, int groups, int weights = 0) {
  if (tt != 1) return 1;
  if (rows <= 16 && groups % 4 == 0) return -4;
  // (launch-shape tuner, weights from HBM: H = 2048 top-8, 32 / 64 / 128 rows 35.8 / 39.4 / 44.5 us
  // per forward against 36.8 / 40.4 / 45.0 unshared; H = 3072 wxa8, 72 rows 57.2 against 56.8, 144
  // rows 61.8 against 59.7, 288 rows 80.1 against 68.2)
  // layers of mostly 4-bit weights (weights != 0: twice the bytes per work item) up to 32 rows only:
  // 64 rows 49.1 against 47.3 (fp16), 50.9 against 45.7 (FP4), 128 rows 76.4 against 66.3 and 73.6
  // against 65.6
  // (the same search after the routing of 65-1024 rows went to the one-workgroup counting sort:
  // H = 2048, 96 / 128 rows 41.2 / 41.5 against 40.7 / 40.9 unshared; H = 3072 wxa8, 72 / 108 rows
  // 57.8 / 60.6 against 55.6 / 58.9: two ways up to 64 rows)
  if (rows <= (weights == 0 ? 64 : 32) && groups % 2 == 0) return -2;
  return rows <= 16 ? 4 : 1;
}

// rows up to which the gate_up GEMM may share the K range of a block between workgroups (bounds
// the fp32 scratch of the partial sums)
#define DMQ_SPLIT_MAX_ROWS 1024
#define DMQ_ROUTE_RANK_AUTO_ROWS 64
// routed rows x feature blocks of the gate_up launch up to which 16-row tiles run the two-per-CU instance
#define DMQ_TWO_PER_CU_MAX 4096
// single-block workgroups at the end of every XCD's share of a GEMM launch that otherwise walks
// several blocks per workgroup: one round of resident workgroups (32 CUs x 3)
#define DMQ_DOWN_TT4_MIN_AVG 256
#define DMQ_TT4_MIN_AVG 112
#define DMQ_HOIST_ALL_TOKENS 1024
#define DMQ_TAIL_SLOTS 96
// routed rows from which an fp16 layer is cut into work items of 128 rows (the persistent GEMM).
// Not chosen automatically at present: at 16384 routed rows (H = 2048, I = 512, Zipf routing) the
// launch pair measures slower than the 32-row launches; tt = 8 asks for it explicitly.
#define DMQ_ROWS_MIN_ROUTED (1L << 40)

// Feature blocks one workgroup walks back to back.  With few row tiles every block gets its own
// workgroup (parallelism); with many, a workgroup amortizes its start-up over several blocks.
static inline int pick_nbl(long rows, int tt) {
  const long tiles = rows / (16 * tt);
  return tiles >= 1024 ? 4 : (tiles >= 384 ? 2 : 1);
}

extern "C" {

int dmq_abi_version(void) { return 21; }

const char* dmq_status_string(int status) {
  switch (status) {
    case DMQ_OK: return "ok";
    case DMQ_ERR_BIT: return "unsupported bit width";
    case DMQ_ERR_ALIGN: return "size not aligned to the quantization group or tile";
    case DMQ_ERR_SHAPE: return "inconsistent shapes";
    case DMQ_ERR_EMPTY: return "empty work list";
    case DMQ_ERR_MODE: return "unknown mode or flag";
    case DMQ_ERR_NULL: return "required pointer is null";
    case DMQ_ERR_HIP: return "HIP runtime error";
    case DMQ_ERR_LIMIT: return "size exceeds a documented limit";
  }
  return "unknown status";
}

int dmq_unpack_nbit(const void* packed, long n_bytes, int bit, void* out_u8, void* stream) {
  if (!packed || !out_u8) return n_bytes ? DMQ_ERR_NULL : DMQ_OK;
  return dmq_unpack_launch((const uint8_t*)packed, n_bytes, bit, (uint8_t*)out_u8, (hipStream_t)stream);
}

int dmq_convert_to_group_first(const void* indices_packed, const void* norms, int n_rows, int groups,
                               int bit, int prescale, void* idx_gf, void* norms_gf, void* stream) {
  if (bit != 1 && bit != 2 && bit != 4 && bit != 8) return DMQ_ERR_BIT;
  if (n_rows < 0 || groups < 0) return DMQ_ERR_SHAPE;
  if (!indices_packed || !norms || !idx_gf || !norms_gf) return DMQ_ERR_NULL;
  return dmq_group_first_launch((const uint8_t*)indices_packed, (const __half*)norms, n_rows, groups,
                                DMQ_GS * bit / 8, prescale, (uint8_t*)idx_gf, (__half*)norms_gf,
                                (hipStream_t)stream);
}

int dmq_dequant_tile(const void* idx_gf, const void* codebook_f16, const void* norms_gf, int n_total,
                     int g0, int g_cnt, int n0, int n_cnt, int bit, void* out_f16, void* stream) {
  if (!dmq_valid_bit_wide(bit)) return DMQ_ERR_BIT;
  if (!idx_gf || !codebook_f16 || !out_f16) return DMQ_ERR_NULL;
  if (g0 < 0 || n0 < 0 || g_cnt < 0 || n_cnt < 0 || n0 + n_cnt > n_total) return DMQ_ERR_SHAPE;
  return dmq_dequant_tile_launch((const uint8_t*)idx_gf, (const __half*)codebook_f16,
                                 (const __half*)norms_gf, n_total, g0, g_cnt, n0, n_cnt, bit,
                                 (__half*)out_f16, (hipStream_t)stream);
}

int dmq_fold_indices_to_e2m1(const void* idx_gf, const void* nib_lut, long rows, int bit, void* out,
                             void* stream) {
  if (!dmq_valid_bit(bit)) return DMQ_ERR_BIT;
  if (!idx_gf || !nib_lut || !out) return DMQ_ERR_NULL;
  return dmq_fold_e2m1_launch((const uint8_t*)idx_gf, (const uint8_t*)nib_lut, rows, bit,
                              (uint8_t*)out, (hipStream_t)stream);
}

int dmq_route_topk(const void* logits, int logits_fp16, int tokens, int experts, int k, int renorm,
                   void* out_w, void* out_idx, void* stream) {
  if (!logits || !out_w || !out_idx) return DMQ_ERR_NULL;
  return dmq_route_topk_launch(logits, logits_fp16, nullptr, nullptr, tokens, experts, k, renorm,
                               (float*)out_w, (int*)out_idx, SharedGate{nullptr, nullptr, 0, 0},
                               (hipStream_t)stream);
}

int dmq_route_topk_shared(const void* logits, int logits_fp16, const void* topk_idx_in,
                          const void* topk_w_in, int tokens, int experts, int k, int renorm,
                          const void* x_f16, const void* gate_row_f16, int hidden, int n_shared,
                          void* out_w, void* out_idx, void* stream) {
  if (!out_w || !out_idx) return DMQ_ERR_NULL;
  if (!logits && (!topk_idx_in || !topk_w_in)) return DMQ_ERR_NULL;
  if (n_shared < 0) return DMQ_ERR_SHAPE;
  if (n_shared > 0 && (!x_f16 || !gate_row_f16 || hidden <= 0)) return DMQ_ERR_NULL;
  return dmq_route_topk_launch(logits, logits_fp16, (const int*)topk_idx_in, (const float*)topk_w_in,
                               tokens, experts, k, renorm, (float*)out_w, (int*)out_idx,
                               SharedGate{(const __half*)x_f16, (const __half*)gate_row_f16, hidden,
                                          n_shared},
                               (hipStream_t)stream);
}

size_t dmq_route_scratch_bytes(int tokens, int k, int experts) {
  if (tokens <= 0 || k <= 0 || experts <= 0) return 0;
  int chunk_rows, n_chunks;
  dmq_sort_chunks((long)tokens * k, &chunk_rows, &n_chunks);
  return (size_t)n_chunks * experts * sizeof(int);
}

// pool_order / lead_pools: see PlanParams (NULL = pools in index order, n_items[1] not written)
static int route_permute_ordered(const void* topk_idx, const void* topk_w, int tokens, int k, int experts,
                      int pools, const void* slice_start, const void* slice_count, int tile_rows,
                      int max_items, void* counts, void* offsets, void* sorted_tokens,
                      void* sorted_weights, void* sorted_rows, void* gu_info, void* dn_info,
                      void* n_items, void* items, void* scratch, size_t scratch_bytes,
                      const int* pool_order, int lead_pools, void* stream, int* zero_words = nullptr,
                      int zero_count = 0) {
  if (!topk_idx || !topk_w || !slice_start || !slice_count || !counts || !offsets ||
      !sorted_tokens || !sorted_weights || !sorted_rows || !gu_info || !dn_info || !n_items ||
      !items || !scratch)
    return DMQ_ERR_NULL;
  if (tokens <= 0 || k <= 0 || experts <= 0 || pools <= 0) return DMQ_ERR_SHAPE;
  if (pools > DMQ_MAX_POOLS || experts > DMQ_SORT_MAX_EXPERTS) return DMQ_ERR_LIMIT;
  if (tile_rows <= 0 || tile_rows % 16) return DMQ_ERR_ALIGN;
  if (scratch_bytes < dmq_route_scratch_bytes(tokens, k, experts)) return DMQ_ERR_LIMIT;
  PlanParams plan{};
  plan.counts = (int*)counts; plan.hist = (int*)scratch;
  dmq_sort_chunks((long)tokens * k, &plan.chunk_rows, &plan.n_chunks);
  plan.experts = experts; plan.pools = pools; plan.tile_rows = tile_rows; plan.max_items = max_items;
  plan.slice_start_rows = (const int*)slice_start; plan.slice_count_rows = (const int*)slice_count;
  plan.offsets = (int*)offsets; plan.gu_info = (int*)gu_info; plan.dn_info = (int*)dn_info;
  plan.n_items = (int*)n_items; plan.items = (int*)items;
  for (int i = 0; i < DMQ_MAX_POOLS; ++i) plan.pool_order[i] = pool_order ? pool_order[i] : i;
  plan.lead_pools = pool_order ? lead_pools : -1;
  plan.zero_words = zero_words; plan.zero_count = zero_words ? zero_count : 0;
  if ((long)tokens * k <= DMQ_ROUTE_SMALL_ROWS && experts <= DMQ_ROUTE_SMALL_EXPERTS && k <= 64) {
    RouteSmallParams sp{};                   // one launch instead of three
    sp.in_idx = (const int*)topk_idx; sp.in_w = (const float*)topk_w;
    sp.tokens = tokens; sp.router_experts = experts; sp.k = k;
    sp.plan = plan;
    sp.sorted_tokens = (int*)sorted_tokens; sp.sorted_weights = (float*)sorted_weights;
    sp.sorted_rows = (int*)sorted_rows;
    return dmq_route_small_launch(sp, (hipStream_t)stream);
  }
  return dmq_route_permute_launch((const int*)topk_idx, (const float*)topk_w, tokens, k, plan,
                                  (int*)sorted_tokens, (float*)sorted_weights, (int*)sorted_rows,
                                  (hipStream_t)stream);
}

int dmq_route_permute(const void* topk_idx, const void* topk_w, int tokens, int k, int experts,
                      int pools, const void* slice_start, const void* slice_count, int tile_rows,
                      int max_items, void* counts, void* offsets, void* sorted_tokens,
                      void* sorted_weights, void* sorted_rows, void* gu_info, void* dn_info,
                      void* n_items, void* items, void* scratch, size_t scratch_bytes,
                      void* stream) {
  return route_permute_ordered(topk_idx, topk_w, tokens, k, experts, pools, slice_start, slice_count,
                               tile_rows, max_items, counts, offsets, sorted_tokens, sorted_weights,
                               sorted_rows, gu_info, dn_info, n_items, items, scratch, scratch_bytes,
                               nullptr, -1, stream);
}

// Scratch of dmq_route_permute_static: the per-chunk expert histograms of the counting sort at their
// largest (DMQ_SORT_MAX_CHUNKS chunks x DMQ_SORT_MAX_EXPERTS experts), one copy per GPU, held until the
// process ends.  Host code never uses the array's name as an address: the device address is looked
// up once per device (with that device current) and cached.  Two host threads making the first
// call on a device at once both look it up and store the same value.
#define DMQ_STATIC_SCRATCH_BYTES (DMQ_SORT_MAX_CHUNKS * DMQ_SORT_MAX_EXPERTS * 4)
#define DMQ_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char dmq_static_scratch[DMQ_STATIC_SCRATCH_BYTES];
static void* dmq_static_scratch_ptr[DMQ_STATIC_MAX_DEVICES];

static int static_scratch_address(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return DMQ_ERR_HIP;
  if (dev < 0 || dev >= DMQ_STATIC_MAX_DEVICES) return DMQ_ERR_LIMIT;
  if (!dmq_static_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(dmq_static_scratch)) != hipSuccess || !ptr) return DMQ_ERR_HIP;
    dmq_static_scratch_ptr[dev] = ptr;
  }
  *out = dmq_static_scratch_ptr[dev];
  return DMQ_OK;
}

int dmq_route_permute_static(const void* topk_idx, const void* topk_w, int tokens, int k, int experts,
                             int pools, const void* slice_start, const void* slice_count,
                             int tile_rows, int max_items, void* counts, void* offsets,
                             void* sorted_tokens, void* sorted_weights, void* sorted_rows,
                             void* gu_info, void* dn_info, void* n_items, void* items, void* stream) {
  if (tokens <= 0 || k <= 0 || experts <= 0) return DMQ_ERR_SHAPE;
  if (experts > DMQ_SORT_MAX_EXPERTS) return DMQ_ERR_LIMIT;          // histograms would not fit
  if (dmq_route_scratch_bytes(tokens, k, experts) > (size_t)DMQ_STATIC_SCRATCH_BYTES) return DMQ_ERR_LIMIT;
  void* scratch = nullptr;
  const int rc = static_scratch_address(&scratch);
  if (rc) return rc;
  // every (chunk, expert) cell the launch reads is written by its counting pass first: nothing
  // has to start at zero
  return route_permute_ordered(topk_idx, topk_w, tokens, k, experts, pools, slice_start, slice_count,
                               tile_rows, max_items, counts, offsets, sorted_tokens, sorted_weights,
                               sorted_rows, gu_info, dn_info, n_items, items, scratch,
                               DMQ_STATIC_SCRATCH_BYTES, nullptr, -1, stream);
}

int dmq_build_tiles(const void* expert_info, int n_experts, int tile_rows, int max_items, int pool,
                    void* n_items, void* items, void* stream) {
  if (!expert_info || !n_items || !items) return DMQ_ERR_NULL;
  if (n_experts <= 0 || max_items <= 0) return DMQ_ERR_EMPTY;
  if (tile_rows <= 0 || tile_rows % 16) return DMQ_ERR_ALIGN;
  if (pool < 0 || pool >= DMQ_MAX_POOLS) return DMQ_ERR_LIMIT;
  return dmq_items_from_info_launch((const int*)expert_info, n_experts, tile_rows, max_items, pool,
                                    (int*)n_items, (int*)items, (hipStream_t)stream);
}

int dmq_rotate(int mode, const void* x, long x_stride, const void* row_index, const void* rot,
               int rows, int groups, void* out, long out_row_bytes, void* scale, int scale_stride,
               int scale_fp32, float extra_scale, int tt, void* stream) {
  if (rows <= 0) return DMQ_OK;
  if (!valid_mode(mode)) return DMQ_ERR_MODE;
  if (tt != 1 && tt != 2 && tt != 4) return DMQ_ERR_MODE;
  if (row_index) return DMQ_ERR_MODE;    // gathered rows go through dmq_rotate_tiled
  if (!x || !rot || !out) return DMQ_ERR_NULL;
  if (mode != DMQ_MODE_A16 && !scale) return DMQ_ERR_NULL;
  if (groups <= 0) return DMQ_ERR_SHAPE;
  RotParams p{};
  p.pool[0] = RotPool{(const __half*)rot, (uint8_t*)out, out_row_bytes, scale, scale_stride, nullptr,
                      extra_scale, mode, 1, 0};
  p.x = (const __half*)x; p.x_stride = x_stride; p.row_index = nullptr;
  p.rows = rows; p.groups = groups;
  p.n_hoisted = 1; p.hoisted_pool[0] = 0;
  p.items = nullptr; p.n_items = nullptr; p.tile_rows = 16 * tt; p.scale_fp32 = scale_fp32;
  return dmq_rotate_dispatch(mode, p, 0, tt, (hipStream_t)stream);
}

int dmq_rotate_tiled(int mode, const void* x, long x_stride, const void* row_index, const void* rot,
                     int rot_per_expert, int groups, const void* expert_info, const void* items,
                     const void* n_items, int tile_rows, int max_items, void* out,
                     long out_row_bytes, void* scale, int scale_stride, int scale_fp32,
                     float extra_scale, int tt, void* stream) {
  if (!expert_info || !items || !n_items) return DMQ_ERR_NULL;
  if (max_items <= 0) return DMQ_OK;
  if (!valid_mode(mode)) return DMQ_ERR_MODE;
  if (tt != 1 && tt != 2 && tt != 4) return DMQ_ERR_MODE;
  if (tile_rows <= 0 || tile_rows % (16 * tt)) return DMQ_ERR_ALIGN;
  if (!x || !rot || !out) return DMQ_ERR_NULL;
  if (mode != DMQ_MODE_A16 && !scale) return DMQ_ERR_NULL;
  if (groups <= 0) return DMQ_ERR_SHAPE;
  RotParams p{};
  const RotPool rp{(const __half*)rot, (uint8_t*)out, out_row_bytes, scale, scale_stride,
                   (const int*)expert_info, extra_scale, mode, 0, rot_per_expert ? 1 : 0};
  for (int i = 0; i < DMQ_MAX_POOLS; ++i) p.pool[i] = rp;     // items may carry any pool id
  p.x = (const __half*)x; p.x_stride = x_stride; p.row_index = (const int*)row_index;
  p.rows = 0; p.groups = groups; p.n_hoisted = 0;
  p.items = (const int*)items; p.n_items = (const int*)n_items; p.tile_rows = tile_rows;
  p.scale_fp32 = scale_fp32;
  const long n = (long)max_items * (tile_rows / (16 * tt)) * groups;
  return dmq_rotate_dispatch(mode, p, n, tt, (hipStream_t)stream);
}

int dmq_quantize_act(int mode, const void* x, int x_fp32, long x_stride, int rows, int groups,
                     void* out, long out_row_bytes, void* scale, int scale_stride, int scale_fp32,
                     float extra_scale, void* stream) {
  if (rows <= 0) return DMQ_OK;
  if (!x || !out || !scale) return DMQ_ERR_NULL;
  if (groups <= 0) return DMQ_ERR_SHAPE;
  QuantParams p{x, x_fp32, x_stride, rows, groups, (uint8_t*)out, out_row_bytes, scale, scale_stride,
                scale_fp32, extra_scale};
  return dmq_quantize_dispatch(mode, p, (hipStream_t)stream);
}

int dmq_matmul_merged_gf(const dmq_gemm_args* a, void* stream) {
  if (!a) return DMQ_ERR_NULL;
  if (a->n_pools <= 0 || a->n_pools > DMQ_MAX_POOLS) return DMQ_ERR_LIMIT;
  bool any_wide = false, any_narrow = false;
  const int mode2 = a->mode2_on ? a->mode2 : -1;
  for (int i = 0; i < a->n_pools; ++i) {
    const int b = a->pool[i].bit;
    if (!dmq_valid_bit_wide(b)) return DMQ_ERR_BIT;
    if (a->pool[i].mode != a->mode && a->pool[i].mode != mode2) continue;
    if (b == 8 && a->mode == DMQ_MODE_FP4) return DMQ_ERR_BIT;
    (b == 8 ? any_wide : any_narrow) = true;
  }
  if (mode2 >= 0) {
    const int ks2 = a->ks > 0 ? a->ks : 1;
    if (mode2 != DMQ_MODE_A16 || a->mode == DMQ_MODE_A16 || !valid_mode(a->mode)) return DMQ_ERR_MODE;
    if (a->tt > 2 || ks2 != 1 || any_wide || a->epi == DMQ_EPI_STORE || a->dbg_acc || a->nt == 1)
      return DMQ_ERR_MODE;
  }
  if (!valid_mode(a->mode)) return DMQ_ERR_MODE;
  if (a->epi < DMQ_EPI_STORE || a->epi > DMQ_EPI_SILU_ROT) return DMQ_ERR_MODE;
  const int ks = a->ks > 0 ? a->ks : 1;
  const bool rows_kernel = a->tt == DMQ_ROWS_TT;          // work items of 128 rows (fp16 pools)
  if (!rows_kernel && !dmq_gemm_config_ok(a->tt, ks)) return DMQ_ERR_MODE;
  if (rows_kernel) {
    if (a->mode != DMQ_MODE_A16 || mode2 >= 0 || ks != 1 || a->k_split > 1 || a->dbg_acc || any_wide ||
        (a->nt != 0 && a->nt != 4) || (a->item_tile_rows != 0 && a->item_tile_rows != DMQ_ROWS_TILE) ||
        a->width_filter != 0 || a->accumulate)
      return DMQ_ERR_MODE;
    if (a->groups % 4) return DMQ_ERR_ALIGN;
    if (!a->rows_queue) return DMQ_ERR_NULL;
    if (a->max_items > DMQ_ROWS_MAX_ITEMS) return DMQ_ERR_LIMIT;
    // lane offsets into the activation rows are 32 bits wide
    if ((long)a->max_items * DMQ_ROWS_TILE * a->act_row_bytes > 0xffffffffL) return DMQ_ERR_LIMIT;
  }
  if (!a->items || !a->n_items || (!a->out && a->epi != DMQ_EPI_SILU_ROT)) return DMQ_ERR_NULL;
  for (int i = 0; i < a->n_pools; ++i) {
    const dmq_gemm_pool& q = a->pool[i];
    if (!q.act || !q.w || !q.norms || !q.expert_info) return DMQ_ERR_NULL;
    if (q.mode == a->mode && a->mode != DMQ_MODE_FP4 && !q.lut &&
        !(a->mode == DMQ_MODE_A8 && q.bit == 8))          // 8-bit int8: NULL = identity table
      return DMQ_ERR_NULL;
    if (mode2 >= 0 && q.mode == mode2 && !q.lut) return DMQ_ERR_NULL;
    if (q.mode == a->mode && a->mode != DMQ_MODE_A16 && !q.act_scale) return DMQ_ERR_NULL;
    if (q.n_total <= 0 || q.n_total % 16) return DMQ_ERR_ALIGN;
  }
  if (a->epi == DMQ_EPI_SCATTER && (!a->row_weight || !a->row_slot)) return DMQ_ERR_NULL;
  if (a->max_items <= 0) return DMQ_ERR_EMPTY;
  if (a->groups <= 0 || a->n_out <= 0) return DMQ_ERR_SHAPE;
  const bool silu = a->epi == DMQ_EPI_SILU || a->epi == DMQ_EPI_SILU_ROT;
  // one n-tile per wave: the launch of a Linear with a handful of rows (any bit width)
  const bool one_tile = a->nt == 1;
  if (a->nt != 0 && a->nt != 4 && !one_tile) return DMQ_ERR_MODE;
  if (one_tile && (a->epi != DMQ_EPI_STORE || a->tt != 1 || ks != 4 || a->mode == DMQ_MODE_FP4 ||
                 a->dbg_acc || a->k_split > 1))
    return DMQ_ERR_MODE;
  const int feat_per_wave = silu ? 32 : (one_tile ? 16 : 64);
  if (a->n_out % (rows_kernel ? 4 * feat_per_wave : feat_per_wave)) return DMQ_ERR_ALIGN;
  if (silu && (a->half_width != a->n_out)) return DMQ_ERR_SHAPE;
  // 16-row tiles, no K sharing: the 8-bit pools and the others ride one launch (and the fused down
  // rotation is then open to 8-bit pools as well)
  const bool both_widths = any_wide && !a->widths_apart && a->tt == 1 && ks == 1 && !a->dbg_acc &&
                           mode2 < 0 && a->nt != 1 && a->epi != DMQ_EPI_STORE && a->mode != DMQ_MODE_FP4;
  if (a->epi == DMQ_EPI_SILU_ROT) {
    if (ks != 1) return DMQ_ERR_MODE;
    if (a->n_out % DMQ_GS) return DMQ_ERR_ALIGN;
    if (!a->post_out || (a->mode != DMQ_MODE_A16 && !a->post_scale)) return DMQ_ERR_NULL;
    for (int i = 0; i < a->n_pools; ++i)
      if ((a->pool[i].mode == a->mode || a->pool[i].mode == mode2) && !a->post_rot[i]) return DMQ_ERR_NULL;
  }
  if (a->act_row_bytes < (long)a->groups * act_bytes_per_group(a->mode)) return DMQ_ERR_SHAPE;
  const int wsplit = a->k_split > 1 ? a->k_split : 1;
  int subs = 1;
  if (a->item_tile_rows > 0 && !rows_kernel) {
    if (a->item_tile_rows % (16 * a->tt)) return DMQ_ERR_ALIGN;
    subs = a->item_tile_rows / (16 * a->tt);
    if (subs > 1 && wsplit > 1) return DMQ_ERR_MODE;
  }
  if (wsplit > 1) {
    // SiLU epilogues: 2 or 4 workgroups; plain store (a Linear with a handful of rows): up to 16
    const bool store = a->epi == DMQ_EPI_STORE;
    if (!silu && !store) return DMQ_ERR_MODE;
    if (wsplit != 2 && wsplit != 4 && !(store && (wsplit == 8 || wsplit == 16))) return DMQ_ERR_MODE;
    if (ks != 1 || a->tt != 1) return DMQ_ERR_MODE;
    if (a->groups % wsplit || (silu && a->n_out % DMQ_GS)) return DMQ_ERR_ALIGN;
    if (!a->split_partial || !a->split_counter) return DMQ_ERR_NULL;
    if (a->split_rows <= 0) return DMQ_ERR_SHAPE;
  }

  GemmLaunch L;
  GemmParams& p = L.p;
  for (int i = 0; i < DMQ_MAX_POOLS; ++i) {
    const dmq_gemm_pool& q = a->pool[i < a->n_pools ? i : 0];
    const int qi = i < a->n_pools ? i : 0;
    p.pool[i] = PoolW{(const uint8_t*)q.w, (const __half*)q.norms, q.lut, (const int*)q.expert_info,
                      (const uint8_t*)q.act, q.act_scale, (const int*)q.row_index, q.n_total, q.bit,
                      q.mode, q.w_scale_byte, (const __half*)a->post_rot[qi], a->post_extra_scale[qi],
                      (const int*)q.col_start, (const int*)q.home};
  }
  p.act_row_bytes = a->act_row_bytes;
  p.act_scale_stride = a->act_scale_stride;
  p.groups = a->groups;
  p.n_out = a->n_out;
  p.half_width = a->half_width;
  p.slice_is_groups = a->slice_is_groups;
  p.items = (const int*)a->items;
  p.n_items = (const int*)a->n_items;
  p.out = (__half*)a->out;
  p.out_stride = a->out_stride;
  p.out_slots = (__half*)a->out;
  p.row_weight = (const float*)a->row_weight;
  p.row_slot = (const int*)a->row_slot;
  p.dbg_acc = (int*)a->dbg_acc;
  p.post_out = (uint8_t*)a->post_out;
  p.post_row_bytes = a->post_row_bytes;
  p.post_scale = a->post_scale;
  p.post_scale_stride = a->post_scale_stride;
  if (a->width_filter != 0 && wsplit > 1) return DMQ_ERR_MODE;
  p.width_filter = a->width_filter;
  p.home_filter = a->width_filter != 0 ? a->home_filter : -1;
  p.accumulate = (a->epi == DMQ_EPI_SCATTER && a->accumulate) ? 1 : 0;
  p.wsplit = wsplit;
  p.split_items = 0;
  if (wsplit > 1 && a->k_split_items > 0) {
    if (a->spread || subs > 1 || rows_kernel) return DMQ_ERR_MODE;
    p.split_items = a->k_split_items < a->max_items ? a->k_split_items : a->max_items;
  }
  p.spread = a->spread != 0;
  p.subs = subs;
  p.split_rows = a->split_rows;
  p.split_partial = (float*)a->split_partial;
  p.split_counter = (int*)a->split_counter;
  if (a->gemv) {
    if (a->mode != DMQ_MODE_A16 || a->tt != 1 || ks != 1 || wsplit > 1 || mode2 >= 0 || a->dbg_acc ||
        a->width_filter != 0 || a->accumulate || rows_kernel)
      return DMQ_ERR_MODE;
    const bool rot = a->epi == DMQ_EPI_SILU_ROT, scatter = a->epi == DMQ_EPI_SCATTER;
    if (!rot && !scatter && a->epi != DMQ_EPI_SILU) return DMQ_ERR_MODE;
    for (int i = 0; i < a->n_pools; ++i)
      if (a->pool[i].mode == DMQ_MODE_A16 && a->pool[i].bit > 4) return DMQ_ERR_BIT;
    if (!dmq_gemv_shape_ok(a->groups, a->n_out, rot)) return DMQ_ERR_SHAPE;
    const bool planes = rot || (scatter && a->gemv_planes > 0);
    if (planes && (!a->split_partial || a->split_rows <= 0)) return DMQ_ERR_NULL;
    if (scatter && a->gemv_planes > 8) return DMQ_ERR_LIMIT;
    p.split_partial = planes ? (float*)a->split_partial : nullptr;
    p.split_rows = a->split_rows;
    p.wsplit = scatter ? a->gemv_planes : dmq_gemv_planes(a->groups);
    return dmq_gemv_launch(p, !scatter, a->max_items, (hipStream_t)stream);
  }
  L.epi = a->epi;
  L.tt = a->tt;
  L.nt = one_tile ? 1 : 4;
  L.dbg = a->dbg_acc != nullptr;
  L.roomy = (a->roomy != 0 && a->tt == 1 && ks == 1 && !L.dbg) ? 1 : 0;
  L.mode2 = mode2;
  L.stream = (hipStream_t)stream;
  if (rows_kernel) {
    // a unit is a run of feature blocks of one work item: the smallest run that gives 16 group steps
    // (8 at least, or the unit after it cannot be looked up while it runs)
    p.n_blocks = a->n_out / (4 * feat_per_wave);
    int run = 0;
    for (int want = 16; want >= DMQ_ROWS_MIN_STEPS && !run; want -= 8)
      for (int d = 1; d <= p.n_blocks && !run; ++d)
        if (p.n_blocks % d == 0 && d * a->groups >= want) run = d;
    if (!run) run = p.n_blocks;                          // short units: drawn one after the other
    p.nbl = run; p.tail_slots = 0; p.spread = 0;
    return dmq_gemm_rows_launch(p, a->epi, (int*)a->rows_queue, run, (hipStream_t)stream);
  }
  // the 1/2/4-bit pools and the 8-bit pools of the mode are separate launches over the same work
  // list (each skips the items of the other kind); 8-bit pools never split K over the waves
  for (int wide = 0; wide < 2; ++wide) {
    if (both_widths && wide == 0) continue;           // one launch, issued as the "wide" pass
    if (!(wide ? any_wide : any_narrow)) continue;
    const int lks = (wide && !one_tile) ? 1 : ks;
    const int feat_per_block = (4 / lks) * feat_per_wave;
    p.n_blocks = (a->n_out + feat_per_block - 1) / feat_per_block;
    // several n-blocks per workgroup need every block complete and the waves on distinct features
    // 8-bit pools next to 1/2/4-bit pools are the few wide Linears of a layer (a shared expert):
    // their items sit together in the list, so their launch deals the items out (see spread)
    const bool spread_l = a->spread != 0 || (wide && any_narrow && !both_widths);
    p.spread = spread_l;
    int nbl = a->nbl > 0 ? a->nbl : 1;
    if (lks > 1 || wsplit > 1 || a->n_out % feat_per_block || spread_l) nbl = 1;
    if (nbl > p.n_blocks) nbl = p.n_blocks;
    p.nbl = nbl;
    // several blocks per workgroup: the tail of every XCD's share is cut into single blocks
    p.tail_slots = (nbl > 1 && wsplit == 1 && p.n_blocks % nbl == 0) ? DMQ_TAIL_SLOTS : 0;
    L.p = p;
    if (spread_l) L.p.split_items = 0;                 // items dealt out: every item shares K
    L.ks = lks;
    L.wide = both_widths ? 2 : wide;
    long work;
    if (p.tail_slots > 0) {
      long per_xcd = ((long)a->max_items * subs * p.n_blocks + DMQ_XCDS - 1) / DMQ_XCDS;
      per_xcd = (per_xcd + nbl - 1) / nbl * nbl;
      work = (per_xcd / nbl + p.tail_slots) * DMQ_XCDS;
    } else {
      const long units = spread_l ? ((long)a->max_items * subs + DMQ_XCDS - 1) / DMQ_XCDS * DMQ_XCDS
                                  : (long)a->max_items * subs;
      work = units * ((p.n_blocks + nbl - 1) / nbl) * wsplit;
      work = (work + DMQ_XCDS - 1) / DMQ_XCDS * DMQ_XCDS;    // every XCD gets the same number of slots
      if (L.p.split_items > 0) {
        // the shared items in front (their bound), then one workgroup per block for the rest
        const long head = ((long)L.p.split_items * p.n_blocks * wsplit + DMQ_XCDS - 1) / DMQ_XCDS * DMQ_XCDS;
        const long bulk = ((long)a->max_items * p.n_blocks + DMQ_XCDS - 1) / DMQ_XCDS * DMQ_XCDS;
        work = head + bulk;
      }
    }
    if (work > 0x7fffffffL) return DMQ_ERR_LIMIT;
    L.grid = (int)work;
    int rc = DMQ_ERR_MODE;
    switch (a->mode) {
      case DMQ_MODE_A16: rc = dmq_gemm_launch_a16(L); break;
      case DMQ_MODE_A8: rc = dmq_gemm_launch_a8(L); break;
      case DMQ_MODE_FP8: rc = dmq_gemm_launch_fp8(L); break;
      case DMQ_MODE_FP4: rc = dmq_gemm_launch_fp4(L); break;
    }
    if (rc) return rc;
  }
  return DMQ_OK;
}

int dmq_combine_slots(const void* slots_f16, int k, const void* add_f16, long tokens, int hidden,
                      void* out_f16, void* stream) {
  if (!slots_f16 || !out_f16) return DMQ_ERR_NULL;
  if (k <= 0 || hidden <= 0) return DMQ_ERR_SHAPE;
  if (hidden % 8) return DMQ_ERR_ALIGN;
  return dmq_combine_launch((const __half*)slots_f16, k, (const __half*)add_f16, tokens, hidden,
                            (__half*)out_f16, (hipStream_t)stream);
}

int dmq_finalize_f16(const void* acc_f32, const void* add_f16, long n, void* out_f16, void* stream) {
  if (!acc_f32 || !out_f16) return DMQ_ERR_NULL;
  if (n % 4) return DMQ_ERR_ALIGN;
  return dmq_finalize_launch((const float*)acc_f32, (const __half*)add_f16, n, (__half*)out_f16,
                             (hipStream_t)stream);
}

int dmq_quantize_weights(const void* w_f16, long w_row_stride, const void* rot_f32,
                         const void* boundaries_f32, int n_rows, int groups, int bit,
                         void* indices_packed, void* norms_f16, void* stream) {
  if (!dmq_valid_bit_wide(bit)) return DMQ_ERR_BIT;
  if (n_rows <= 0 || groups <= 0) return DMQ_ERR_SHAPE;
  if (!w_f16 || !rot_f32 || !boundaries_f32 || !indices_packed || !norms_f16) return DMQ_ERR_NULL;
  if (w_row_stride % 8 || w_row_stride < (long)groups * DMQ_GS) return DMQ_ERR_ALIGN;
  return dmq_quantize_weights_launch((const __half*)w_f16, w_row_stride, (const float*)rot_f32,
                                     (const float*)boundaries_f32, n_rows, groups, bit,
                                     (uint8_t*)indices_packed, (__half*)norms_f16, (hipStream_t)stream);
}

// ------------------------------------------------------------------------------ Linear forward
static inline size_t align_up(size_t v);

struct LinearWs {
  int *counter, *info, *n_items, *items;
  uint8_t *codes, *scale;
  float* partial;
  int tiles, counters, k_split;
  long code_row_bytes;
  int scale_stride;
  size_t bytes;
};

// Launch shape of a stand-alone Linear by batch size: up to 16 rows one n-tile per wave with K split
// over the waves; up to 64 rows K split over the waves of four n-tiles (8-bit weights: K shared by
// workgroups instead); beyond, the largest row tile that still gives every CU a workgroup (8-bit
// weights: at most 32 rows, their 64-row instances spill), and with 16-row tiles on less than half
// the CUs two workgroups share K.  Measured on 4096 x 4096: 256 rows 59 -> 36 us (4 bit) and
// 112 -> 41 us (8 bit), 512 rows 59 -> 47 and 112 -> 42 us, 1024 rows of 8-bit weights 119 -> 81 us.
struct LinearShape { int tt, ks, nt, k_split, rot_tt; };
static LinearShape linear_shape(const dmq_linear_desc* L, int rows) {
  const int groups = L->in_features / DMQ_GS;
  const long blocks = (L->out_features + 255) / 256;
  LinearShape s{1, 0, 0, 0, rows >= 1024 ? 4 : 1};
  if (rows <= 16) { s.ks = 4; s.nt = 1; }
  else if (rows <= 64) {
    if (L->bit != 8) s.ks = 4;
    else s.k_split = groups % 4 == 0 ? 4 : (groups % 2 == 0 ? 2 : 0);
  } else {
    auto wgs = [&](int tt) { return ((rows + 16 * tt - 1) / (16 * tt)) * blocks; };
    for (int tt = (L->bit == 8 ? 2 : 4); tt > 1; tt >>= 1)
      if (wgs(tt) >= 256) { s.tt = tt; break; }
    if (s.tt == 1 && wgs(1) <= 128 && groups % 2 == 0) s.k_split = 2;
  }
  return s;
}

static LinearWs carve_linear(const dmq_linear_desc* L, int rows, uint8_t* base) {
  LinearWs w{};
  const LinearShape sh = linear_shape(L, rows);
  const int groups = L->in_features / DMQ_GS;
  w.tiles = (rows + 16 * sh.tt - 1) / (16 * sh.tt);
  w.k_split = sh.k_split;
  w.counters = (w.tiles + 1) * ((L->out_features + 127) / 128);
  w.code_row_bytes = (long)groups * act_bytes_per_group(L->mode);
  w.scale_stride = groups;
  size_t off = 0;
  auto take = [&](size_t n) { uint8_t* p = base ? base + off : nullptr; off += align_up(n); return p; };
  w.counter = (int*)take((size_t)w.counters * 4);
  w.info = (int*)take(16);
  w.n_items = (int*)take(16);
  w.items = (int*)take((size_t)(w.tiles + 1) * DMQ_ITEM_WORDS * 4);
  w.codes = take((size_t)rows * w.code_row_bytes);
  w.scale = take(L->mode == DMQ_MODE_A16 ? 0 : (size_t)rows * groups * 2);
  w.partial = (float*)take(sh.k_split > 1 ? (size_t)sh.k_split * rows * L->out_features * 4 : 0);
  w.bytes = off;
  return w;
}

static int linear_desc_ok(const dmq_linear_desc* L) {
  if (!L) return DMQ_ERR_NULL;
  if (L->mode != DMQ_MODE_A16 && L->mode != DMQ_MODE_A8 && L->mode != DMQ_MODE_FP8) return DMQ_ERR_MODE;
  if (!dmq_valid_bit_wide(L->bit)) return DMQ_ERR_BIT;
  if (L->in_features <= 0 || L->out_features <= 0) return DMQ_ERR_SHAPE;
  if (L->in_features % DMQ_GS || L->out_features % 64) return DMQ_ERR_ALIGN;
  return DMQ_OK;
}

int dmq_linear_gemm_i8(const void* x_i8, long x_row_bytes, const void* x_scale_f16, int scale_stride,
                       const void* indices_gf, const void* norms_gf, int rows, int in_features,
                       int out_features, void* out_f16, long out_stride, void* stream) {
  if (rows <= 0) return DMQ_OK;
  if (!x_i8 || !x_scale_f16 || !indices_gf || !norms_gf || !out_f16) return DMQ_ERR_NULL;
  if (in_features <= 0 || out_features <= 0) return DMQ_ERR_SHAPE;
  if (in_features % DMQ_GS || out_features % 4 || x_row_bytes % 16 || out_stride % 4) return DMQ_ERR_ALIGN;
  const int groups = in_features / DMQ_GS;
  if (x_row_bytes < in_features || scale_stride < groups || out_stride < out_features) return DMQ_ERR_SHAPE;
  const LinearI8Params p{(const uint8_t*)x_i8, x_row_bytes, (const _Float16*)x_scale_f16, scale_stride,
                         (const uint8_t*)indices_gf, (const _Float16*)norms_gf, rows, groups,
                         out_features, (_Float16*)out_f16, out_stride};
  return dmq_linear_i8_launch(p, (hipStream_t)stream);
}

// 8-bit weights on a uniform grid, int8 path, enough rows to fill the chip with 128 x 128 tiles:
// the plain int8 GEMM instead of the look-up kernels.  4096 x 4096, forward time: 2048 rows
// 146 -> 80 us, 4096 rows 290 -> 150 us, 768 rows 79 -> 61 us; with fewer tiles (640 rows: 160)
// the 32-row look-up tiles win.
#define DMQ_LINEAR_I8_MIN_WGS 192
static bool linear_uses_i8_gemm(const dmq_linear_desc* L, int rows) {
  if (L->mode != DMQ_MODE_A8 || L->bit != 8 || L->lut) return false;
  const long wgs = (long)((L->out_features + 127) / 128) * ((rows + 127) / 128);
  return wgs >= DMQ_LINEAR_I8_MIN_WGS;
}

int dmq_linear_uses_i8_gemm(const dmq_linear_desc* L, int rows) {
  return (linear_desc_ok(L) == DMQ_OK && rows > 0 && linear_uses_i8_gemm(L, rows)) ? 1 : 0;
}

size_t dmq_linear_workspace_bytes(const dmq_linear_desc* L, int max_rows) {
  if (linear_desc_ok(L) != DMQ_OK || max_rows <= 0) return 0;
  // the carve of any batch up to max_rows fits the largest of the shapes
  size_t best = 0;
  // (the fp32 planes of a shared K range exist only for some batch sizes: up to 64 rows of 8-bit
  // weights, and 16-row tiles on at most 128 workgroups)
  const long blocks = (L->out_features + 255) / 256;
  const long split_rows = 16 * (128 / blocks > 4 ? 128 / blocks : 4);
  const int probes[] = {max_rows, max_rows < 64 ? max_rows : 64, max_rows < 16 ? max_rows : 16,
                        max_rows < split_rows ? max_rows : (int)split_rows};
  for (int r : probes) {
    const size_t b = carve_linear(L, r, nullptr).bytes;
    if (b > best) best = b;
  }
  return best;
}

int dmq_linear_forward(const dmq_linear_desc* L, const void* x_f16, long x_stride, int rows,
                       void* out_f16, long out_stride, void* workspace, size_t workspace_bytes,
                       void* stream) {
  int rc = linear_desc_ok(L);
  if (rc) return rc;
  if (rows <= 0) return DMQ_OK;
  if (!x_f16 || !out_f16 || !workspace) return DMQ_ERR_NULL;
  if (!L->indices_gf || !L->norms_gf || !L->rot) return DMQ_ERR_NULL;
  if (!L->lut && !(L->mode == DMQ_MODE_A8 && L->bit == 8)) return DMQ_ERR_NULL;
  if (x_stride < L->in_features || out_stride < L->out_features) return DMQ_ERR_SHAPE;
  if (x_stride % 8 || out_stride % 4) return DMQ_ERR_ALIGN;
  if ((uintptr_t)workspace % 256) return DMQ_ERR_ALIGN;
  const LinearWs w = carve_linear(L, rows, (uint8_t*)workspace);
  if (w.bytes > workspace_bytes) return DMQ_ERR_LIMIT;
  const LinearShape sh = linear_shape(L, rows);
  const int groups = L->in_features / DMQ_GS;

  // launch 1: rotation (+ quantization) of the rows; its first workgroup also writes the work
  // items of launch 2 and clears the arrival counters
  RotParams p{};
  p.pool[0] = RotPool{(const __half*)L->rot, w.codes, w.code_row_bytes, w.scale, w.scale_stride, nullptr,
                      L->extra_scale, L->mode, 1, 0};
  p.x = (const __half*)x_f16; p.x_stride = x_stride; p.row_index = nullptr;
  p.rows = rows; p.groups = groups;
  p.n_hoisted = 1; p.hoisted_pool[0] = 0;
  p.items = nullptr; p.n_items = nullptr; p.tile_rows = 16 * sh.rot_tt; p.scale_fp32 = 0;
  p.prep = LinearPrep{w.info, w.n_items, w.items, w.tiles, rows, L->out_features, w.counter,
                      sh.k_split > 1 ? w.counters : 0};
  const bool i8_gemm = linear_uses_i8_gemm(L, rows);
  if (i8_gemm) p.prep = LinearPrep{};
  rc = dmq_rotate_dispatch(L->mode, p, 0, sh.rot_tt, (hipStream_t)stream);
  if (rc) return rc;
  if (i8_gemm)
    return dmq_linear_gemm_i8(w.codes, w.code_row_bytes, w.scale, w.scale_stride, L->indices_gf,
                              L->norms_gf, rows, L->in_features, L->out_features, out_f16, out_stride,
                              stream);

  // launch 2: dequant GEMM, plain store
  dmq_gemm_args a{};
  a.mode = L->mode; a.epi = DMQ_EPI_STORE; a.tt = sh.tt; a.ks = sh.ks; a.nt = sh.nt; a.n_pools = 1;
  dmq_gemm_pool& q = a.pool[0];
  q.w = L->indices_gf; q.norms = L->norms_gf; q.lut = L->lut; q.expert_info = w.info;
  q.act = w.codes; q.act_scale = L->mode == DMQ_MODE_A16 ? nullptr : w.scale; q.row_index = nullptr;
  q.n_total = L->out_features; q.bit = L->bit; q.mode = L->mode; q.w_scale_byte = 127;
  a.act_row_bytes = w.code_row_bytes; a.act_scale_stride = w.scale_stride;
  a.groups = groups; a.n_out = L->out_features; a.half_width = 0; a.slice_is_groups = 0;
  a.items = w.items; a.n_items = w.n_items; a.max_items = w.tiles;
  a.out = out_f16; a.out_stride = out_stride;
  if (sh.k_split > 1) {
    a.k_split = sh.k_split; a.split_rows = rows;
    a.split_partial = w.partial; a.split_counter = w.counter;
  }
  return dmq_matmul_merged_gf(&a, stream);
}

int dmq_rms_norm(const void* x, int x_bf16, const void* weight, int weight_fp32, long rows, int n,
                 long x_row_stride, long out_row_stride, float eps, void* out, void* stream) {
  if (rows <= 0) return DMQ_OK;
  if (!x || !weight || !out) return DMQ_ERR_NULL;
  if (n <= 0) return DMQ_ERR_SHAPE;
  if (n % 8 || x_row_stride % 8 || out_row_stride % 8) return DMQ_ERR_ALIGN;
  if (x_row_stride < n || out_row_stride < n) return DMQ_ERR_SHAPE;
  return dmq_rms_norm_launch(x, x_bf16, weight, weight_fp32, rows, n, x_row_stride, out_row_stride,
                             eps, out, (hipStream_t)stream);
}

int dmq_fill_zero(void* ptr, long n_bytes, void* stream) {
  if (n_bytes <= 0) return DMQ_OK;
  if (!ptr) return DMQ_ERR_NULL;
  if (n_bytes % 4) return DMQ_ERR_ALIGN;
  const long words = n_bytes / 4;
  long g = (words + 255) / 256;
  if (g > 4096) g = 4096;
  hipLaunchKernelGGL(dmq_fill_zero_kernel, dim3((int)g), dim3(256), 0, (hipStream_t)stream,
                     (uint32_t*)ptr, words);
  return dmq_check_launch();
}

// ------------------------------------------------------------------------------- whole layer
struct MoeWorkspace {
  int *counts, *offsets, *sorted_tokens, *sorted_rows, *gu_info, *dn_info, *n_items, *items;
  int* topk_idx;                     // [tokens, top_k] incl. the shared columns (routed entry point)
  float* topk_w;
  float* sorted_weights;
  uint8_t* slots;                    // fp16 [tokens * top_k, hidden]
  uint8_t* xq[DMQ_MAX_POOLS];        // hoisted pools: codes by token; others share xq_rows
  uint8_t* xq_scale[DMQ_MAX_POOLS];
  uint8_t *xq_rows, *xq_rows_scale, *act, *actq, *actq_scale;
  float* split_partial;              // gate_up K range shared between workgroups: fp32 sums
  int* split_counter;
  int* rows_queue;                   // queue words of the persistent gate_up and down launches
  __half* router_logits;             // [16, experts] logits of the router workgroups (pre-norm entry)
  int split_rows, split_counters;
  void* sort_scratch;
  size_t sort_scratch_bytes;
  int max_items, tile_rows;
  size_t bytes;
};

static inline size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// weights: 0 = mostly 1- and 2-bit pools, 1 = mostly 4-bit pools behind the look-up table,
// 2 = mostly FP4 (e2m1 weights, no table)
static int pick_tt(int tokens, int top_k, int experts, int weights, bool two_per_cu = false) {
  const long avg = (long)tokens * top_k / (experts > 0 ? experts : 1);
  // 64-row work items halve the gate_up GEMM's look-ups per row (two workgroups per CU instead of
  // three) and, where an expert's rows fit one 64-row tile but not one 32-row tile, its tiles.
  // 2-bit layers (Zipf routing: most experts stay small): equal at 96 rows per expert, -1 % at 128,
  // -4 % at 256.  4-bit layers pay twice the look-ups per weight (uniform routing, 256 experts:
  // +3 % at 32 rows per expert, -10 % at 48, -2 % at 64); FP4 streams its weights and gains from
  // 12 rows per expert on (-5 % at 24, -6 % at 32, -3 % at 64).  The down GEMM keeps 32-row tiles
  // on those items (down_tt below).
  const long min4 = weights == 2 ? 10 : (weights == 1 ? 40 : DMQ_TT4_MIN_AVG);
  // 16-row tiles: 4-bit look-up layers (uniform routing) keep them up to 12 rows per expert (3 %
  // ahead there), FP4 up to 8.  Layers of narrow pools are measured under Zipf routing, where the
  // hot experts fill several 16-row tiles long before the average does, each of them streaming
  // the expert's weights again: 32-row tiles from 2 rows per expert on (H = 2048, I = 512, 256
  // experts, top-8, whole forward: 64 tokens 73.2 -> 69.3 us, 128 tokens equal, 256 tokens
  // 92.8 -> 86.2; H = 3072, I = 1024 with a shared expert, wxa8: 64 tokens 108 -> 102, 128 tokens
  // 133 -> 128, 256 tokens 183 -> 164; at 1 row per expert 16-row tiles are 2-7 % ahead).
  if (weights == 0 ? avg < 2 : avg <= (weights == 1 ? 12 : 8)) return 1;
  // Narrow pools, 3 rows per expert and more, while the launch is still small enough for the
  // two-per-CU instance of the 16-row kernel: 32-row items then number a little more than the CUs,
  // and the CUs that get two of them set the time of the launch.  H = 2048, I = 512, top-8, weights
  // from HBM, 96 / 112 / 128 tokens: Zipf routing 57.0 / 57.5 / 58.2 us with 32-row items against
  // 52.7 / 55.9 / 56.8; uniform routing 97.2 / 98.5 / 98.2 against 89.8 / 89.6 / 90.6 (at 64 and 80
  // tokens Zipf has 32-row items 6 % ahead, uniform 16-row items 6 %: left with 32).
  if (weights == 0 && two_per_cu && avg >= 3) return 1;
  return avg <= min4 ? 2 : 4;
}

static MoeWorkspace carve(const dmq_layer_desc* L, int tokens, int tt, uint8_t* base) {
  MoeWorkspace w;
  const size_t R = (size_t)tokens * L->top_k;
  const size_t E = L->experts, P = L->pools, H = L->hidden, I = L->inter;
  w.tile_rows = tt == DMQ_ROWS_TT ? DMQ_ROWS_TILE : 16 * tt;
  // an expert of a sub-expert layer has work items in every pool that holds a share of it
  const size_t homes = L->n_widths > 0 && L->max_homes > 1 ? (size_t)L->max_homes : 1;
  w.max_items = (int)((R / w.tile_rows + E) * homes);
  size_t off = 0;
  auto take = [&](size_t n) { uint8_t* p = base + off; off += align_up(n); return p; };
  w.counts = (int*)take(E * 4);
  w.offsets = (int*)take((E + 1) * 4);
  w.sorted_tokens = (int*)take(R * 4);
  w.sorted_rows = (int*)take(R * 4);
  w.sorted_weights = (float*)take(R * 4);
  w.topk_idx = (int*)take(R * 4);
  w.topk_w = (float*)take(R * 4);
  w.gu_info = (int*)take(P * E * 16);
  w.dn_info = (int*)take(P * E * 16);
  w.n_items = (int*)take(16);
  w.rows_queue = (int*)take(2 * DMQ_ROWS_QUEUE_WORDS * 4);
  w.router_logits = (__half*)take((size_t)DMQ_PRENORM_MAX_TOKENS * E * 2);
  w.sort_scratch_bytes = dmq_route_scratch_bytes(tokens, L->top_k, L->experts);
  w.sort_scratch = take(w.sort_scratch_bytes);
  w.items = (int*)take((size_t)w.max_items * DMQ_ITEM_WORDS * sizeof(int));
  w.slots = take(R * H * 2);
  for (size_t i = 0; i < DMQ_MAX_POOLS; ++i) {
    // every pool gets a by-token buffer so the size does not depend on which pools are hoisted
    w.xq[i] = i < P ? take((size_t)tokens * H * 2) : nullptr;
    w.xq_scale[i] = i < P ? take((size_t)tokens * (H / DMQ_GS) * 4) : nullptr;
  }
  w.xq_rows = take(R * H * 2);
  w.xq_rows_scale = take(R * (H / DMQ_GS) * 4);
  w.act = take(R * I * 2);
  w.actq = take(R * I * 2);
  // two areas: the second holds the block scales of the FP4 pools of a sub-expert layer, whose
  // rows may also carry the int8 share of another pool
  w.actq_scale = take(2 * R * (I / DMQ_GS) * 4);
  w.split_rows = (int)(R < DMQ_SPLIT_MAX_ROWS ? R : DMQ_SPLIT_MAX_ROWS);
  w.split_partial = (float*)take((size_t)4 * w.split_rows * 2 * I * 4);
  w.split_counters = (int)((R / 16 + E) * (I / DMQ_GS));
  w.split_counter = (int*)take((size_t)w.split_counters * 4);
  w.bytes = off;
  return w;
}

size_t dmq_moe_workspace_bytes(const dmq_layer_desc* layer, int tokens) {
  if (!layer || tokens <= 0) return 0;
  // tile size 16 gives the largest item list; everything else is independent of tt
  return carve(layer, tokens, 1, nullptr).bytes;
}

int dmq_moe_ffn_forward(const dmq_layer_desc* layer, const void* x, const void* topk_idx,
                        const void* topk_w, int tokens, const void* add_f16, void* out,
                        void* workspace, size_t workspace_bytes, int tt, int ks, int nbl,
                        void* stream) {
  return dmq_moe_ffn_forward_staged(layer, x, topk_idx, topk_w, tokens, add_f16, out, workspace,
                                    workspace_bytes, tt, ks, nbl, nullptr, nullptr, stream);
}

int dmq_moe_ffn_forward_staged(const dmq_layer_desc* layer, const void* x, const void* topk_idx,
                               const void* topk_w, int tokens, const void* add_f16, void* out,
                               void* workspace, size_t workspace_bytes, int tt, int ks, int nbl,
                               void* const* stage_events, void* aux_out, void* stream) {
  if (!topk_idx || !topk_w) return DMQ_ERR_NULL;
  dmq_router_args r{};
  r.topk_idx = topk_idx; r.topk_w = topk_w;
  return dmq_moe_ffn_forward_routed(layer, &r, x, tokens, add_f16, out, workspace, workspace_bytes,
                                    tt, ks, nbl, stage_events, aux_out, stream);
}

// pre != NULL: x holds the block's pre-norm input; the first launch normalizes it, projects it onto
// the router and runs the top-k (dmq_moe_ffn_forward_prenorm)
static int forward_routed_impl(const dmq_layer_desc* layer, const dmq_router_args* router,
                               const dmq_prenorm_args* pre, const void* x, int tokens,
                               const void* add_f16, void* out, void* workspace,
                               size_t workspace_bytes, int tt, int ks, int nbl,
                               void* const* stage_events, void* aux_out, void* stream);

int dmq_moe_ffn_forward_routed(const dmq_layer_desc* layer, const dmq_router_args* router,
                               const void* x, int tokens, const void* add_f16, void* out,
                               void* workspace, size_t workspace_bytes, int tt, int ks, int nbl,
                               void* const* stage_events, void* aux_out, void* stream) {
  if (!router) return DMQ_ERR_NULL;
  if (!router->logits && (!router->topk_idx || !router->topk_w)) return DMQ_ERR_NULL;
  return forward_routed_impl(layer, router, nullptr, x, tokens, add_f16, out, workspace, workspace_bytes,
                             tt, ks, nbl, stage_events, aux_out, stream);
}

int dmq_moe_ffn_forward_prenorm(const dmq_layer_desc* layer, const dmq_router_args* router,
                                const dmq_prenorm_args* pre, const void* h, int tokens,
                                const void* add_f16, void* out, void* workspace,
                                size_t workspace_bytes, int tt, int ks, int nbl,
                                void* const* stage_events, void* aux_out, void* stream) {
  if (!router || !pre || !pre->norm_weight || !pre->gate_weight || !pre->state) return DMQ_ERR_NULL;
  if (router->logits || router->topk_idx || router->topk_w) return DMQ_ERR_MODE;   // the launch makes them
  if (tokens > DMQ_PRENORM_MAX_TOKENS) return DMQ_ERR_LIMIT;
  return forward_routed_impl(layer, router, pre, h, tokens, add_f16, out, workspace, workspace_bytes,
                             tt, ks, nbl, stage_events, aux_out, stream);
}

static int forward_routed_impl(const dmq_layer_desc* layer, const dmq_router_args* router,
                               const dmq_prenorm_args* pre, const void* x, int tokens,
                               const void* add_f16, void* out, void* workspace,
                               size_t workspace_bytes, int tt, int ks, int nbl,
                               void* const* stage_events, void* aux_out, void* stream) {
  if (!layer || !router || !x || !out || !workspace || !layer->pool) return DMQ_ERR_NULL;
  const int n_shared = router->n_shared;
  if (n_shared < 0 || n_shared >= layer->top_k || n_shared >= layer->experts) return DMQ_ERR_SHAPE;
  if (n_shared > 0 && !router->shared_gate_row) return DMQ_ERR_NULL;
  auto mark = [&](int i) {
    if (stage_events && stage_events[i]) (void)hipEventRecord((hipEvent_t)stage_events[i], (hipStream_t)stream);
  };
  if (tokens <= 0) return DMQ_ERR_EMPTY;
  const int H = layer->hidden, I = layer->inter, E = layer->experts, K = layer->top_k;
  const int P = layer->pools;
  if (H % DMQ_GS || I % DMQ_GS || H / DMQ_GS < 1 || I / DMQ_GS < 1) return DMQ_ERR_ALIGN;
  if (P <= 0 || E <= 0 || K <= 0) return DMQ_ERR_SHAPE;
  if (P > DMQ_MAX_POOLS) return DMQ_ERR_LIMIT;
  long w4 = 0, wf4 = 0, w_all = 0;         // gate_up rows held by 4-bit look-up pools / FP4 pools / all pools
  for (int i = 0; i < P; ++i) {
    w_all += layer->pool[i].n_gate_up;
    if (layer->pool[i].mode == DMQ_MODE_FP4) wf4 += layer->pool[i].n_gate_up;
    else if (layer->pool[i].bit == 4) w4 += layer->pool[i].n_gate_up;
  }
  // Big batches of fp16 layers (1/2/4-bit pools, group counts multiples of four, single-home
  // experts): work items of 128 rows for the persistent GEMM launches (tt = 8).  A caller's tt = 8
  // on another layer falls back to 64-row items.
  bool rows_ok = (H / DMQ_GS) % 4 == 0 && (I / DMQ_GS) % 4 == 0 && H % 256 == 0 &&
                 layer->n_widths == 0 &&
                 (long)tokens * K / DMQ_ROWS_TILE + E <= DMQ_ROWS_MAX_ITEMS &&
                 ((long)tokens * K + (long)E * DMQ_ROWS_TILE) * 2 * (H > I ? H : I) <= 0xffffffffL;
  for (int i = 0; i < P; ++i)
    rows_ok = rows_ok && layer->pool[i].mode == DMQ_MODE_A16 && layer->pool[i].bit != 8;
  // A decode step of one or two tokens on an fp16 layer of 1/2/4-bit pools: both GEMMs as dot
  // products on the vector ALU (csrc/gemv.hip) unless the caller names a tiling -- while the gate_up
  // launch (one workgroup per routed row and 16 features) is at most two workgroups per CU and its
  // body keeps two workgroups' registers per CU (H <= 2048).  Measured: H=2048 I=512 top-8 one token
  // 32.0 -> 25.7 us, two tokens 33.1 -> 32.1, three 35.4 -> 40.5; H=3072 I=1024 with a shared
  // expert, one token 43.6 -> 52.0 (576 workgroups of 256 registers), so not there.
  bool gemv = tt <= 0 && ks == 0 && tokens <= DMQ_GEMV_MAX_TOKENS && layer->n_widths == 0 &&
              dmq_gemv_shape_ok(H / DMQ_GS, I, 1) && dmq_gemv_shape_ok(I / DMQ_GS, H, 0) &&
              H <= 2048 && (long)tokens * K * (I / 16) <= 2 * DMQ_GEMV_CUS;
  for (int i = 0; i < P; ++i)
    gemv = gemv && layer->pool[i].mode == DMQ_MODE_A16 && layer->pool[i].bit <= 4;
  if (gemv) { tt = 1; ks = 1; }
  if (tt <= 0) {
    tt = pick_tt(tokens, K, E, 2 * wf4 > w_all ? 2 : (2 * w4 > w_all ? 1 : 0),
                 (long)tokens * K * (I / DMQ_GS) <= DMQ_TWO_PER_CU_MAX);
    if (rows_ok && (long)tokens * K >= DMQ_ROWS_MIN_ROUTED) tt = DMQ_ROWS_TT;
  }
  if (tt == DMQ_ROWS_TT && !rows_ok) tt = 4;
  if (tt != 1 && tt != 2 && tt != 4 && tt != DMQ_ROWS_TT) return DMQ_ERR_MODE;
  const bool ks_auto = ks == 0;            // (not for the dot-product launches: no K sharing)
  if (ks == 0) {
    ks = pick_ks(tt, (long)tokens * K, H / DMQ_GS, 2 * wf4 > w_all ? 2 : (2 * w4 > w_all ? 1 : 0));
    // an 8-bit pool on the fp16 path (a shared expert with a 256-entry table) makes few, long work
    // items: two workgroups per block pay up to 256 routed rows (configs[3] with such a shared
    // expert, wxa16, 16 tokens: 88 -> 75 us; the int8 identity path gains nothing there)
    if (ks == 1 && tt == 1 && (long)tokens * K <= 256 && (H / DMQ_GS) % 2 == 0)
      for (int i = 0; i < P; ++i)
        if (layer->pool[i].bit == 8 && layer->pool[i].mode == DMQ_MODE_A16) ks = -2;
  }
  // ks < 0: -ks workgroups share the K range of a gate_up block; the other launches do not split
  const int wsplit = ks < 0 ? -ks : 1;
  if (ks < 0) {
    if ((wsplit != 2 && wsplit != 4) || tt != 1 || (H / DMQ_GS) % wsplit) return DMQ_ERR_MODE;
    if ((long)tokens * K > DMQ_SPLIT_MAX_ROWS) return DMQ_ERR_LIMIT;
    ks = 1;
  }
  // Sub-expert layers (experts spread over several pools, shares of several widths): one gate_up
  // launch per width and one down launch per (rank, width); no K sharing between workgroups or
  // waves, every pool rotated by token (a routed row may feed several pools)
  const bool sub = layer->n_widths > 0;
  if (sub) {
    if (layer->n_widths > 8 || layer->max_homes <= 0 || layer->max_homes > P) return DMQ_ERR_LIMIT;
    if (!layer->col_start || !layer->home) return DMQ_ERR_NULL;
    for (int i = 0; i < layer->n_widths; ++i)
      if (layer->widths[i] <= 0 || layer->widths[i] % DMQ_GS || layer->widths[i] > I) return DMQ_ERR_ALIGN;
    ks = 1;
  }
  const int wsplit_eff = sub ? 1 : wsplit;
  // (dmq_gemm_args.k_split_items could share only the leading items of the list, say those of the
  // pools with few, long items; with weights that come from HBM every such rule measured slower than
  // one workgroup per block: configs[1] 32 tokens 45.9 against 43.5 us, configs[3] wxa8 48 tokens
  // 82.6 against 72.0.)
  const int wsplit_launch = wsplit_eff;
  if (tt == DMQ_ROWS_TT ? ks != 1 : !dmq_gemm_config_ok(tt, ks)) return DMQ_ERR_MODE;
  const bool nbl_auto = nbl <= 0;
  if (nbl_auto) {
    nbl = pick_nbl((long)tokens * K, tt > 4 ? 4 : tt);
    // layers of mostly 4-bit look-up weights: two blocks per workgroup from 512 routed rows on
    // (launch-shape search, 64 / 256 / 1024 tokens of top-8: int8 106.2 / 115.4 / 174.5 us with one
    // block against 103.6 / 113.1 / 168.9; fp16 64 / 512 tokens 100.6 / 134.6 against 99.3 / 130.0)
    if (nbl < 2 && 2 * w4 > w_all && (long)tokens * K >= 512) nbl = 2;
  }
  // a rotation wave covers 16 or 32 rows: 64-row work items are rotated by two waves each
  const int rot_tt = tt > 2 ? 2 : tt;
  MoeWorkspace w = carve(layer, tokens, tt, (uint8_t*)workspace);
  if (w.bytes > workspace_bytes) return DMQ_ERR_LIMIT;
  // Rotated down-projection input.  In a sub-expert layer one routed row may hold the shares of
  // pools of two precision modes (wxfp4: 4-bit pools run FP4, 2-bit pools int8), whose codes and
  // scales are laid out by column at different densities: the FP4 codes go to the upper half of the
  // row (bytes [I, 1.5 I); int8 / fp8 codes fill [0, I)) and the FP4 scales to an area of their own.
  auto actq_of = [&](int m) { return (sub && m == DMQ_MODE_FP4) ? w.actq + I : w.actq; };
  auto actq_scale_of = [&](int m) {
    return (sub && m == DMQ_MODE_FP4) ? w.actq_scale + (size_t)tokens * K * (I / DMQ_GS) * 4 : w.actq_scale;
  };
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (aux_out) {
    long* aux = (long*)aux_out;
    aux[0] = gemv ? 0 : tt; aux[1] = wsplit_eff > 1 ? -wsplit_eff : ks; aux[2] = (long)((uint8_t*)w.counts - (uint8_t*)workspace);
    aux[3] = w.max_items; aux[4] = (long)((uint8_t*)w.n_items - (uint8_t*)workspace);
    aux[5] = nbl;
  }
  mark(0);

  // distinct precision modes of the pools (one launch per mode and stage)
  int modes[DMQ_MAX_POOLS], n_modes = 0;
  for (int i = 0; i < P; ++i) {
    const int m = layer->pool[i].mode;
    if (!valid_mode(m)) return DMQ_ERR_MODE;
    if (!dmq_valid_bit_wide(layer->pool[i].bit)) return DMQ_ERR_BIT;
    if (layer->pool[i].bit == 8 && m == DMQ_MODE_FP4) return DMQ_ERR_BIT;
    bool seen = false;
    for (int j = 0; j < n_modes; ++j) seen |= (modes[j] == m);
    if (!seen) modes[n_modes++] = m;
  }

  // A layer with pools of several precision modes launches each GEMM once per mode over the whole
  // work list.  The mode with the most weights keeps the contiguous XCD shares; the items of a
  // smaller mode sit together somewhere in the list (a shared expert's slices: the last items), so
  // its launches deal the items out one per XCD (dmq_gemm_args.spread) instead of leaving them to
  // the one XCD whose share they fall into (configs[3] wxa8, 256 tokens: the fp16 launch of the
  // 4-bit shared expert 67 -> 28 us).
  int main_mode = modes[0];
  {
    long best = -1;
    for (int mi = 0; mi < n_modes; ++mi) {
      long rows_m = 0;
      for (int i = 0; i < P; ++i) if (layer->pool[i].mode == modes[mi]) rows_m += layer->pool[i].n_gate_up;
      if (rows_m > best) { best = rows_m; main_mode = modes[mi]; }
    }
  }

  // Several modes, a smaller one fp16 (a shared expert that keeps fp16 activations), no 8-bit pools:
  // the fp16 mode rides the main mode's launch of each GEMM (dmq_gemm_args.mode2).  With 16-row
  // tiles always; with 32-row tiles up to 1024 tokens, the items dealt out one per XCD (the shared
  // expert's items are neighbours in the list): configs[3] wxa8 512 tokens 227 -> 198 us, 1024
  // tokens 340 -> 323, 2048 tokens 545 -> 551; the 64-row kernel with both bodies spills.
  bool dual = false;
  if (n_modes >= 2 && (tt == 1 || (tt == 2 && tokens <= 1024)) && ks == 1 && !sub && main_mode != DMQ_MODE_A16) {
    for (int mi = 0; mi < n_modes; ++mi) dual |= modes[mi] == DMQ_MODE_A16;
    for (int i = 0; i < P; ++i)
      if (layer->pool[i].mode == main_mode || layer->pool[i].mode == DMQ_MODE_A16) dual &= layer->pool[i].bit != 8;
  }

  // 16-row tiles: which kernel instance (see dmq_gemm_args.roomy).  The two-per-CU instance wins
  // while the gate_up launch has few workgroups (routed rows x feature blocks; measured: H=2048
  // I=512 up to 128 tokens, H=3072 I=1024 up to 32) and whenever most rows go to 4-bit weights.
  bool roomy = false;
  if (tt == 1) {
    roomy = (long)tokens * K * (I / DMQ_GS) <= DMQ_TWO_PER_CU_MAX;
    if (2 * w4 > w_all) roomy = true;
  }

  // The gate_up GEMM rotates (and quantizes) its SiLU*up rows for the down projection itself when
  // a workgroup owns whole blocks of 128 features: no K split over the waves.
  // 8-bit pools next to narrower ones: up to about a hundred work items one 16-row launch serves
  // both index widths and fuses as well (dmq_gemm_args.widths_apart; configs[3] with the reference's
  // default 8-bit shared expert, wxa8: 64 tokens 133 -> 107 us, 128 tokens 153 -> 146, 256 tokens
  // 196 -> 240, so beyond 1280 routed rows the widths keep their own launches).
  const bool widths_apart = tt != 1 || (long)tokens * K > 1280;
  bool fuse_rot[DMQ_MAX_POOLS];
  // (dot-product launches: the rotated rows travel as fp32 planes of partial sums)
  const bool gemv_rot = gemv && (long)tokens * K <= w.split_rows;
  for (int mi = 0; mi < n_modes; ++mi) fuse_rot[mi] = (ks == 1) && (!gemv || gemv_rot);
  if (aux_out) {
    // which pools get their SiLU*up rows rotated inside the gate_up launch (bit i: pool i)
    long mask = 0;
    for (int mi = 0; mi < n_modes; ++mi)
      for (int i = 0; i < P; ++i)
        if (fuse_rot[mi] && layer->pool[i].mode == modes[mi]) mask |= 1L << i;
    ((long*)aux_out)[6] = mask;
  }

  // Which pools rotate every token once instead of their routed rows: the caller's choice (pools
  // expected to see more routed rows than tokens) and, for small batches, all of them: rotating a
  // few dozen tokens for a pool that ends up using a handful is cheaper than the dependent
  // per-work-item pass (same values either way).
  bool whole_batch[DMQ_MAX_POOLS] = {false, false, false, false};
  for (int i = 0; i < P; ++i)
    whole_batch[i] = sub || layer->pool[i].major != 0 || tokens <= DMQ_HOIST_ALL_TOKENS;

  // The pools whose rows are rotated per work item come first in the item list, so that the
  // rotation launch knows their items as a prefix (n_items[1]) and touches no other record.
  int pool_order[DMQ_MAX_POOLS] = {0, 1, 2, 3}, lead_pools = 0;
  {
    int n = 0;
    for (int i = 0; i < P; ++i) if (!whole_batch[i]) pool_order[n++] = i;
    lead_pools = n;
    for (int i = 0; i < P; ++i) if (whole_batch[i]) pool_order[n++] = i;
    // Among the whole-batch pools the ones with the longest work items go first (the order of the
    // list is the order in which workgroups get their slots): 4-bit weights cost twice the look-ups
    // of 2-bit ones, fp16 activations more than quantized ones.  A 4-bit fp16 shared expert at the
    // end of the list would start when the first routed items finish and end long after them.
    auto item_cost = [&](int i) { return layer->pool[i].bit * (layer->pool[i].mode == DMQ_MODE_A16 ? 2 : 1); };
    for (int a = lead_pools; a < n; ++a)
      for (int b = a + 1; b < n; ++b)
        if (item_cost(pool_order[b]) > item_cost(pool_order[a])) {
          const int t = pool_order[a]; pool_order[a] = pool_order[b]; pool_order[b] = t;
        }
  }

  // Rotation (+ quantization) of the gate_up input of one precision mode.  whole: the pools that
  // rotate every token once (no dependence on the routing step); tiled: the pools rotated per
  // work item; tp: the router's top-k rides the same launch.
  bool whole_done[DMQ_MAX_POOLS] = {false, false, false, false};   // per mode
  int a16_mi = -1;
  for (int mi = 0; mi < n_modes; ++mi) if (modes[mi] == DMQ_MODE_A16) a16_mi = mi;
  PreNorm pn{};
  if (pre) pn = PreNorm{pre->norm_weight, pre->norm_weight_fp32, pre->eps, 1};
  auto rotate_gate_up_input = [&](int mode, bool whole, bool tiled, const TopkParams* tp,
                                  int tp_fp16, const RouterParams* rt = nullptr) -> int {
    // the whole-batch pools of the fp16 mode ride the main mode's launch (see `dual`): same
    // rotation, their rows are stored as fp16 instead of going through the quantizer
    const bool with_f16 = dual && mode == main_mode && whole && !whole_done[a16_mi];
    RotParams rp{};
    rp.x = (const __half*)x; rp.x_stride = H; rp.row_index = w.sorted_tokens;
    rp.pn = pn;
    rp.rows = tokens; rp.groups = H / DMQ_GS;
    rp.items = w.items; rp.n_items = w.n_items; rp.tile_rows = w.tile_rows; rp.scale_fp32 = 0;
    rp.items_prefix = 1;
    bool any_tiled = false;
    for (int i = 0; i < DMQ_MAX_POOLS; ++i) {
      const int pi = i < P ? i : 0;
      const dmq_pool_desc& pd = layer->pool[pi];
      const bool hoisted = whole_batch[pi];
      const bool live = i < P && (pd.mode == mode || (with_f16 && pd.mode == DMQ_MODE_A16 && hoisted));
      const long row_bytes = (long)H * 2;
      rp.pool[i] = RotPool{(const __half*)pd.gu_rot, hoisted ? w.xq[pi] : w.xq_rows, row_bytes,
                           hoisted ? (void*)w.xq_scale[pi] : (void*)w.xq_rows_scale,
                           scale_stride_for(pd.mode, H), w.gu_info + (size_t)pi * E * 4,
                           pd.gu_extra_scale, live ? pd.mode : -1, hoisted ? 1 : 0, 0};
      if (live && hoisted && whole) rp.hoisted_pool[rp.n_hoisted++] = i;
      if (live && !hoisted && tiled) any_tiled = true;
    }
    // 16 rows per wave wherever the launch does not fill the chip several times over: a wave's
    // chain (matrix, rows, 32 MFMAs per tile, quantization) is serial, so more and shorter waves
    // finish earlier (FP4, whose quantization is the longest: -6 us at 512 tokens, -8 at 4096);
    // the per-work-item pass of big batches keeps the tile of the work items
    const int rtt = (!any_tiled || tokens <= 2048) ? 1 : rot_tt;
    long n = 0;                                    // waves of the per-work-item part
    if (any_tiled) n = (long)w.max_items * (w.tile_rows / (16 * rtt)) * rp.groups;
    else rp.items = nullptr;
    if (rp.n_hoisted == 0 && !any_tiled && !tp) return DMQ_OK;
    rp.also_f16 = with_f16 ? 1 : 0;
    if (pn.on && (any_tiled || (!rt && rp.n_hoisted == 0))) return any_tiled ? DMQ_ERR_MODE : DMQ_OK;
    const int rc_rot = rt ? dmq_rotate_router_dispatch(mode, rp, *rt, st)
                          : dmq_rotate_dispatch(mode, rp, n, rtt, st, tp, tp_fp16);
    if (!rc_rot && with_f16) whole_done[a16_mi] = true;   // fp16 pools rotated per work item keep their own pass
    return rc_rot;
  };
  const bool route_small = !pre && (long)tokens * K <= DMQ_ROUTE_SMALL_ROWS && E <= DMQ_ROUTE_SMALL_EXPERTS &&
                           K <= 64 && (!router->logits || tokens <= DMQ_ROUTE_SMALL_TOKENS);
  // When the top-k is a launch of its own (logits, more than 16 tokens) it shares the launch of the
  // whole-batch rotation of the first mode: neither needs the other, both are short.
  bool topk_done = false;
  // Up to four tokens (logits or a caller-made top-k): no sort launch.  The top-k workgroup of the
  // rotation launch ranks the routed rows itself and writes the work items (see DirectPlan); the
  // routing launch below is skipped.
  const long R = (long)tokens * K;
  bool direct = !sub && tokens <= DMQ_DIRECT_MAX_TOKENS && R <= DMQ_DIRECT_MAX_ROWS &&
                R <= w.max_items && K <= 64 &&
                (wsplit_eff == 1 || R * (I / DMQ_GS) <= w.split_counters);
  bool direct_done = false;
  if (direct || (!route_small && router->logits) || pre) {
    bool any_whole = false;
    for (int i = 0; i < P; ++i) any_whole |= (whole_batch[i] && layer->pool[i].mode == modes[0]);
    const int rk = K - n_shared, re = E - n_shared;
    const bool topk_fits = any_whole && re <= 1024 && rk <= 64 && rk <= re && rk > 0 && n_shared <= 64;
    if (pre && (!topk_fits || sub || re % 4)) return DMQ_ERR_LIMIT;
    if (topk_fits) {
      const SharedGate sg{(const __half*)x, (const __half*)router->shared_gate_row, H, n_shared, pn, nullptr};
      TopkParams tp{router->logits, tokens, re, rk, router->renorm, w.topk_w, w.topk_idx, sg,
                    (tokens + 3) / 4, DirectPlan{}, (const int*)router->topk_idx,
                    (const float*)router->topk_w};
      if (direct) {
        tp.blocks = 1;
        DirectPlan& dp = tp.dp;
        dp.on = 1; dp.pools = P; dp.experts = E;
        dp.slice_start_rows = (const int*)layer->slice_start;
        dp.slice_count_rows = (const int*)layer->slice_count;
        dp.items = w.items; dp.n_items = w.n_items; dp.counts = w.counts;
        dp.sorted_tokens = w.sorted_tokens; dp.sorted_weights = w.sorted_weights;
        dp.sorted_rows = w.sorted_rows;
        if (wsplit_launch > 1) { dp.clear_words = w.split_counter; dp.clear_count = w.split_counters; }
        direct_done = true;
      }
      if (pre) {
        RouterParams rt{};
        rt.h = (const __half*)x; rt.h_stride = H; rt.tokens = tokens; rt.hidden = H; rt.pn = pn;
        rt.gate_w = (const __half*)pre->gate_weight; rt.experts = re;
        rt.logits = w.router_logits; rt.ticket = (int*)pre->state;
        rt.x_norm_out = (__half*)pre->x_norm_out; rt.logits_out = (__half*)pre->logits_out;
        rt.blocks = (re + 15) / 16;
        rt.tp = tp;
        rc = rotate_gate_up_input(modes[0], true, false, nullptr, 0, &rt);
      } else {
        rc = rotate_gate_up_input(modes[0], true, false, &tp, router->logits_fp16);
      }
      if (rc) return rc;
      whole_done[0] = true;
      topk_done = true;
    }
  }

  // 1. top-k (when the router hands over logits), shared columns, sort by expert, per-pool
  //    expert_info, work items: one launch for small batches
  {
    const int rk = K - n_shared, re = E - n_shared;          // the router's own k and experts
    const SharedGate sg{(const __half*)x, (const __half*)router->shared_gate_row, H, n_shared, pn, nullptr};
    // a few routed rows with the top-k at hand: the one-row-per-thread ranking kernel.  Its scans
    // grow with the square of the rows (kernel trace: 64 rows 5.7 us, 128 rows 9.1 us; the
    // one-workgroup counting sort below takes 5.7 us at 256 rows), so it serves up to 64.
    const int* rank_idx = topk_done ? w.topk_idx
                                    : ((!router->logits && n_shared == 0) ? (const int*)router->topk_idx : nullptr);
    const float* rank_w = topk_done ? w.topk_w
                                    : ((!router->logits && n_shared == 0) ? (const float*)router->topk_w : nullptr);
    if (direct_done) {
      rc = DMQ_OK;
    } else if (!sub && rank_idx && rank_w && R <= DMQ_ROUTE_RANK_AUTO_ROWS && lead_pools == 0) {
      RouteRankParams rr{};
      rr.in_idx = rank_idx; rr.in_w = rank_w;
      rr.rows = (int)R; rr.k = K; rr.experts = E; rr.pools = P; rr.tile_rows = w.tile_rows;
      rr.max_items = w.max_items;
      rr.slice_start_rows = (const int*)layer->slice_start;
      rr.slice_count_rows = (const int*)layer->slice_count;
      rr.counts = w.counts; rr.n_items = w.n_items; rr.items = w.items;
      rr.sorted_tokens = w.sorted_tokens; rr.sorted_weights = w.sorted_weights;
      rr.sorted_rows = w.sorted_rows;
      if (wsplit_launch > 1) { rr.clear_words = w.split_counter; rr.clear_count = w.split_counters; }
      rc = dmq_route_rank_launch(rr, st);
    } else if (route_small) {
      RouteSmallParams sp{};
      sp.logits = router->logits; sp.logits_fp16 = router->logits_fp16;
      sp.in_idx = (const int*)router->topk_idx; sp.in_w = (const float*)router->topk_w;
      sp.tokens = tokens; sp.router_experts = re; sp.k = rk; sp.renorm = router->renorm;
      sp.sg = sg;
      sp.out_w = w.topk_w; sp.out_idx = w.topk_idx;
      PlanParams& plan = sp.plan;
      plan.counts = w.counts; plan.experts = E; plan.pools = P; plan.tile_rows = w.tile_rows;
      plan.max_items = w.max_items;
      plan.slice_start_rows = (const int*)layer->slice_start;
      plan.slice_count_rows = (const int*)layer->slice_count;
      plan.offsets = w.offsets; plan.gu_info = w.gu_info; plan.dn_info = w.dn_info;
      plan.n_items = w.n_items; plan.items = w.items;
      for (int i = 0; i < DMQ_MAX_POOLS; ++i) plan.pool_order[i] = pool_order[i];
      plan.lead_pools = lead_pools;
      sp.sorted_tokens = w.sorted_tokens; sp.sorted_weights = w.sorted_weights;
      sp.sorted_rows = w.sorted_rows;
      if (wsplit_launch > 1) { sp.clear_words = w.split_counter; sp.clear_count = w.split_counters; }
      rc = dmq_route_small_launch(sp, st);
    } else {
      const void* tk_idx = router->topk_idx;
      const void* tk_w = router->topk_w;
      if (topk_done) {
        tk_idx = w.topk_idx; tk_w = w.topk_w;
      } else if (router->logits || n_shared > 0) {
        rc = dmq_route_topk_launch(router->logits, router->logits_fp16, (const int*)router->topk_idx,
                                   (const float*)router->topk_w, tokens, re, rk, router->renorm,
                                   w.topk_w, w.topk_idx, sg, st);
        if (rc) return rc;
        tk_idx = w.topk_idx; tk_w = w.topk_w;
      }
      rc = route_permute_ordered(tk_idx, tk_w, tokens, K, E, P, layer->slice_start, layer->slice_count,
                                 w.tile_rows, w.max_items, w.counts, w.offsets, w.sorted_tokens,
                                 w.sorted_weights, w.sorted_rows, w.gu_info, w.dn_info, w.n_items,
                                 w.items, w.sort_scratch, w.sort_scratch_bytes, pool_order,
                                 lead_pools, stream, tt == DMQ_ROWS_TT ? w.rows_queue : nullptr,
                                 2 * DMQ_ROWS_QUEUE_WORDS);
      if (!rc && wsplit_launch > 1) rc = dmq_fill_zero(w.split_counter, (long)w.split_counters * 4, stream);
    }
  }
  if (rc) return rc;
  mark(1);

  // 2. gate_up input: rotate (+quantize) once per token (whole-batch pools not yet done) and per
  //    routed row (the other pools)
  for (int mi = 0; mi < n_modes; ++mi) {
    rc = rotate_gate_up_input(modes[mi], !whole_done[mi], true, nullptr, 0);
    if (rc) return rc;
  }

  mark(2);

  // 3. gate_up GEMM with fused SiLU * up -> act[R, I]
  for (int mi = 0; mi < n_modes; ++mi) {
    const int mode = modes[mi];
    if (dual && mode == DMQ_MODE_A16) continue;        // rides the main mode's launch
    dmq_gemm_args g{};
    g.mode = mode; g.epi = fuse_rot[mi] ? DMQ_EPI_SILU_ROT : DMQ_EPI_SILU;
    g.gemv = gemv;
    if (gemv_rot) { g.split_partial = w.split_partial; g.split_rows = w.split_rows; }
    // (every record of such a step holds at least one routed row: no more than R of them)
    if (gemv && R < g.max_items) g.max_items = (int)R;
    if (dual && mode == main_mode) { g.mode2_on = 1; g.mode2 = DMQ_MODE_A16; }
    // the gate_up blocks are four times as long as the down blocks (K = H against K = I) and end in
    // the rotation epilogue: more than two per workgroup costs more in balance than it saves
    g.tt = tt; g.ks = ks; g.nbl = nbl > 2 ? 2 : nbl; g.n_pools = P; g.roomy = roomy;
    g.spread = ((n_modes > 1 && mode != main_mode) || (dual && tt > 1)) ? 1 : 0;
    g.widths_apart = widths_apart;
    for (int i = 0; i < P; ++i) {
      const dmq_pool_desc& pd = layer->pool[i];
      const bool hoisted = whole_batch[i];
      g.post_rot[i] = pd.dn_rot;
      g.post_extra_scale[i] = pd.dn_extra_scale;
      g.pool[i] = dmq_gemm_pool{pd.gu_w, pd.gu_norms, pd.gu_lut, w.gu_info + (size_t)i * E * 4,
                                hoisted ? w.xq[i] : w.xq_rows,
                                hoisted ? w.xq_scale[i] : w.xq_rows_scale,
                                hoisted ? w.sorted_tokens : nullptr, pd.n_gate_up, pd.bit, pd.mode,
                                pd.gu_w_scale_byte};
    }
    if (sub)
      for (int i = 0; i < P; ++i) {
        g.pool[i].col_start = (const int*)layer->col_start + (size_t)i * E;
        g.pool[i].home = (const int*)layer->home + (size_t)i * E;
      }
    g.act_row_bytes = (long)H * 2;
    g.act_scale_stride = scale_stride_for(mode, H);
    g.groups = H / DMQ_GS; g.n_out = I; g.half_width = I; g.slice_is_groups = 0;
    g.items = w.items; g.n_items = w.n_items; g.max_items = w.max_items;
    g.out = w.act; g.out_stride = I;
    g.post_out = actq_of(mode); g.post_row_bytes = (long)I * 2;
    g.post_scale = actq_scale_of(mode); g.post_scale_stride = scale_stride_for(mode, I);
    g.rows_queue = w.rows_queue;
    if (wsplit_launch > 1) {
      g.k_split = wsplit_launch; g.split_rows = w.split_rows;
      g.split_partial = w.split_partial; g.split_counter = w.split_counter;
    }
    if (!sub) {
      rc = dmq_matmul_merged_gf(&g, stream);
      if (rc) return rc;
    } else {
      for (int wi = 0; wi < layer->n_widths; ++wi) {     // one launch per share width
        const int W = layer->widths[wi];
        g.n_out = W; g.half_width = W; g.width_filter = 2 * W; g.home_filter = -1;
        rc = dmq_matmul_merged_gf(&g, stream);
        if (rc) return rc;
      }
    }
  }

  mark(3);

  // 4. down input: per-expert rotation (+quantize) of act, unless the gate_up launch did it
  for (int mi = 0; mi < n_modes; ++mi) {
    const int mode = modes[mi];
    if (fuse_rot[mi]) continue;
    RotParams rp{};
    rp.x = (const __half*)w.act; rp.x_stride = I; rp.row_index = nullptr;
    rp.rows = 0; rp.groups = I / DMQ_GS; rp.n_hoisted = 0;
    rp.items = w.items; rp.n_items = w.n_items; rp.tile_rows = w.tile_rows; rp.scale_fp32 = 0;
    for (int i = 0; i < DMQ_MAX_POOLS; ++i) {
      const int pi = i < P ? i : 0;
      const dmq_pool_desc& pd = layer->pool[pi];
      const bool live = i < P && pd.mode == mode;
      rp.pool[i] = RotPool{(const __half*)pd.dn_rot, actq_of(pd.mode),
                           (long)I * 2, actq_scale_of(pd.mode),
                           scale_stride_for(pd.mode, I), w.dn_info + (size_t)pi * E * 4,
                           pd.dn_extra_scale, live ? pd.mode : -1, 0, 1,
                           sub ? (const int*)layer->col_start + (size_t)pi * E : nullptr};
    }
    const long n = (long)w.max_items * (w.tile_rows / (16 * rot_tt)) * rp.groups;
    rc = dmq_rotate_dispatch(mode, rp, n, rot_tt, st);
    if (rc) return rc;
  }

  mark(4);

  // 5. down GEMM with fused routing weight, rows scattered to their (token, slot) rows
  for (int mi = 0; mi < n_modes; ++mi) {
    const int mode = modes[mi];
    if (dual && mode == DMQ_MODE_A16) continue;
    dmq_gemm_args d{};
    if (dual && mode == main_mode) { d.mode2_on = 1; d.mode2 = DMQ_MODE_A16; }
    // 64-row work items: the down GEMM (K = I, four steps per block) runs them as two 32-row tiles
    // until the experts are big enough for its 64-row kernel to pay
    const long avg_rows = (long)tokens * K / E;
    // (re-measured on weights from HBM, 64-row against 2 x 32-row: FP4 1024 / 2048 / 4096 tokens of
    // the all-4-bit layer 135.9 / 189.5 / 287.4 against 137.9 / 192.7 / 293.1 us; int8 4096 tokens
    // 409.9 against 414.9; fp16 2 bpw layer 4096 tokens 358.1 against 356.9, 8192 633.0 against 641.2)
    const long down_min = 2 * wf4 > w_all ? 0 : DMQ_DOWN_TT4_MIN_AVG;
    const int down_tt = (tt == 4 && avg_rows < down_min) ? 2 : tt;
    d.mode = mode; d.epi = DMQ_EPI_SCATTER; d.tt = down_tt; d.item_tile_rows = w.tile_rows; d.roomy = roomy;
    if (aux_out && mi == 0) ((long*)aux_out)[7] = down_tt;
    d.spread = ((n_modes > 1 && mode != main_mode) || (dual && tt > 1)) ? 1 : 0;
    d.widths_apart = widths_apart;
    d.ks = ks; d.n_pools = P; d.gemv = gemv;
    d.nbl = (nbl_auto && down_tt != tt) ? pick_nbl((long)tokens * K, down_tt) : nbl;   // by its own tile count
    for (int i = 0; i < P; ++i) {
      const dmq_pool_desc& pd = layer->pool[i];
      d.pool[i] = dmq_gemm_pool{pd.dn_w, pd.dn_norms, pd.dn_lut, w.dn_info + (size_t)i * E * 4,
                                w.actq, w.actq_scale, nullptr, H, pd.bit, pd.mode,
                                pd.dn_w_scale_byte};
    }
    d.act_row_bytes = (long)I * 2;
    d.act_scale_stride = scale_stride_for(mode, I);
    d.groups = I / DMQ_GS; d.n_out = H; d.half_width = 0; d.slice_is_groups = 1;
    d.items = w.items; d.n_items = w.n_items; d.max_items = w.max_items;
    d.out = w.slots; d.out_stride = H;
    d.row_weight = w.sorted_weights; d.row_slot = w.sorted_rows;
    d.rows_queue = w.rows_queue + DMQ_ROWS_QUEUE_WORDS;
    if (gemv && R < d.max_items) d.max_items = (int)R;
    if (gemv_rot) {
      d.gemv_planes = dmq_gemv_planes(H / DMQ_GS);
      d.split_partial = w.split_partial; d.split_rows = w.split_rows;
    }
    if (!sub) {
      rc = dmq_matmul_merged_gf(&d, stream);
      if (rc) return rc;
    }
  }
  if (sub) {
    // rank 0 stores every slot row (every routed expert has a first share), the following ranks
    // add theirs in rank order: the sum over the pools of bit_partitioned_moe.py:818-822
    for (int h = 0; h < layer->max_homes; ++h)
      for (int mi = 0; mi < n_modes; ++mi)
        for (int wi = 0; wi < layer->n_widths; ++wi) {
          const int mode = modes[mi], W = layer->widths[wi];
          dmq_gemm_args d{};
          d.mode = mode; d.epi = DMQ_EPI_SCATTER; d.tt = tt == 4 ? 2 : tt; d.item_tile_rows = 16 * tt; d.roomy = roomy;
          d.ks = 1; d.nbl = nbl; d.n_pools = P;
          for (int i = 0; i < P; ++i) {
            const dmq_pool_desc& pd = layer->pool[i];
            d.pool[i] = dmq_gemm_pool{pd.dn_w, pd.dn_norms, pd.dn_lut, w.dn_info + (size_t)i * E * 4,
                                      actq_of(pd.mode), actq_scale_of(pd.mode), nullptr, H, pd.bit,
                                      pd.mode, pd.dn_w_scale_byte,
                                      (const int*)layer->col_start + (size_t)i * E,
                                      (const int*)layer->home + (size_t)i * E};
          }
          d.act_row_bytes = (long)I * 2;
          d.act_scale_stride = scale_stride_for(mode, I);
          d.groups = W / DMQ_GS; d.n_out = H; d.half_width = 0; d.slice_is_groups = 1;
          d.items = w.items; d.n_items = w.n_items; d.max_items = w.max_items;
          d.out = w.slots; d.out_stride = H;
          d.row_weight = w.sorted_weights; d.row_slot = w.sorted_rows;
          d.width_filter = W / DMQ_GS; d.home_filter = h; d.accumulate = h > 0;
          rc = dmq_matmul_merged_gf(&d, stream);
          if (rc) return rc;
        }
  }

  mark(5);

  // 6. out[t] = sum of the k slot rows of token t
  rc = dmq_combine_slots(w.slots, K, add_f16, tokens, H, out, stream);
  mark(6);
  return rc;
}

}  // extern "C"
