/*
 * dartmoq_hip -- C ABI of the MI355X (gfx950) quantized MoE FFN kernels.
 *
 * Every entry point takes raw device pointers, explicit sizes and a HIP stream
 * (passed as void*; NULL = the default stream), launches asynchronously on that
 * stream, never allocates or synchronizes, and returns a DMQ_* status code.
 * Inputs are never modified; outputs and workspaces are caller-owned.
 *
 * The reference (zzningxp/DartMoQ-Qwen3.5) has no FFI for this path: its
 * boundary is the set of Python callables in turboquant_utils/triton_kernels*.py
 * that quantization/{wxa16,wxa8,wxfp8,wxfp4}/bit_partitioned_moe.py import.  Each
 * declaration below names the callable(s) it stands in for (paths relative to
 * the reference checkout).
 *
 * Conventions shared by all entry points
 *   group size            128 input features per quantization group
 *   bit                   1, 2 or 4 bits per codebook index; 8 (the 256-entry codebooks of the
 *                         quantized Linears) everywhere except the e2m1 fold and DMQ_MODE_FP4
 *   idx_gf                uint8 [G, N, 128*bit/8]  group-first packed indices
 *   norms_gf              fp16  [G, N]             per-(group,row) norms / sqrt(128)
 *   mode                  DMQ_MODE_A16 / A8 / FP8 / FP4
 *   expert_info           int32 [n_experts, 4] = token_start, token_count,
 *                         slice_start, slice_count   (device memory)
 *   work items            int32 [n, DMQ_ITEM_WORDS] = pool, expert index, row tile inside the
 *                         expert, token_start, token_count, slice_start in weight rows
 *                         (gate_up), slice_start in groups (down), 0; a row tile covers
 *                         tile_rows = 16*tt activation rows.  Items made by dmq_build_tiles
 *                         carry the slice_start of their expert_info in both slice fields.
 */
#ifndef DARTMOQ_HIP_H
#define DARTMOQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  DMQ_OK = 0, DMQ_ERR_BIT = 1, DMQ_ERR_ALIGN = 2, DMQ_ERR_SHAPE = 3, DMQ_ERR_EMPTY = 4,
  DMQ_ERR_MODE = 5, DMQ_ERR_NULL = 6, DMQ_ERR_HIP = 7, DMQ_ERR_LIMIT = 8
};
enum { DMQ_MODE_A16 = 0, DMQ_MODE_A8 = 1, DMQ_MODE_FP8 = 2, DMQ_MODE_FP4 = 3 };
/* STORE: fp16 [rows, n_out].  SILU: fp16 silu(gate)*up [rows, I].  SCATTER: fp16 routing-weighted
 * rows stored at out[row_slot[r]] (one slot per (token, top-k slot)); dmq_combine_slots adds
 * the k slots of each token in fp32, in slot order.  SILU_ROT: SILU followed in the same kernel
 * by the per-expert rotation (+ quantization) of the down projection's input, i.e. the output is
 * what dmq_rotate_tiled would make of the SILU rows (post_* fields of dmq_gemm_args). */
enum { DMQ_EPI_STORE = 0, DMQ_EPI_SILU = 1, DMQ_EPI_SCATTER = 2, DMQ_EPI_SILU_ROT = 3 };
#define DMQ_MAX_POOLS 4
#define DMQ_ITEM_WORDS 8

/* Library / build identification: returns the ABI version (currently 21). */
int dmq_abi_version(void);
/* Human-readable text for a status code (static storage). */
const char* dmq_status_string(int status);

/* ------------------------------------------------------------------ packed format */

/* unpack_nbit, turboquant_utils/quantize.py:74-100.  out holds one index per byte,
 * n_bytes * 8/bit entries. */
int dmq_unpack_nbit(const void* packed, long n_bytes, int bit, void* out_u8, void* stream);

/* convert_to_group_first, turboquant_utils/triton_kernels.py:1042-1069, plus the optional
 * pre-division of the norms by sqrt(128) that WxA16Weights._build_group_first performs
 * (quantization/wxa16/bit_partitioned_moe.py:193-204).
 * indices_packed [n_rows, groups*ppg] -> idx_gf [groups, n_rows, ppg];
 * norms [n_rows, groups] -> norms_gf [groups, n_rows]. */
int dmq_convert_to_group_first(const void* indices_packed, const void* norms, int n_rows,
                               int groups, int bit, int prescale, void* idx_gf, void* norms_gf,
                               void* stream);

/* The dequantized weight tile the GEMM kernels consume: out fp16 [g_cnt, n_cnt, 128] =
 * codebook[idx] (times norms_gf when given), produced through the same LDS byte table.
 * Stands in for the in-kernel "w_quant" tile of
 * turboquant_utils/triton_kernels.py:893-991. */
int dmq_dequant_tile(const void* idx_gf, const void* codebook_f16, const void* norms_gf,
                     int n_total, int g0, int g_cnt, int n0, int n_cnt, int bit, void* out_f16,
                     void* stream);

/* fold_indices_to_e2m1, turboquant_utils/triton_kernels_fp4.py:80-122.
 * idx_gf [rows, 128*bit/8] -> out [rows, 64], rows = G*N. */
int dmq_fold_indices_to_e2m1(const void* idx_gf, const void* nib_lut, long rows, int bit,
                             void* out, void* stream);

/* turboquant_quantize_packed_full, turboquant_utils/quantize.py:350-474 (rotation "qr"): per row
 * and group of 128 features norm = max(||w||, 1e-8), Y = (w / norm) . P_g^T . sqrt(128),
 * index = clamp(number of boundaries < Y, 0, 2^bit - 1), packed low bits first.
 *   w fp16 [n_rows, w_row_stride >= groups*128]; rot fp32 [groups, 128, 128] (the matrices of
 *   seeds seed + g*128); boundaries fp32 [2^bit - 1] ascending (codebook.py:77-100, or the uniform
 *   grid of quantize.py:394-402); indices_packed u8 [n_rows, groups*128*bit/8]; norms fp16
 *   [n_rows, groups].  bit 1, 2, 4 or 8.  The product runs on the fp32 matrix cores: indices equal
 *   the torch quantizer's except where Y sits within fp32 rounding of a boundary. */
int dmq_quantize_weights(const void* w_f16, long w_row_stride, const void* rot_f32,
                         const void* boundaries_f32, int n_rows, int groups, int bit,
                         void* indices_packed, void* norms_f16, void* stream);

/* ------------------------------------------------------------------ routing */

/* softmax + top-k of quantization/wxa16/bit_partitioned_moe.py:1112-1120 (lowest expert
 * index wins ties; renorm != 0 divides by the kept mass like the HF TopKRouter).
 * logits [tokens, experts] fp32 (logits_fp16 == 0) or fp16; out_w fp32 [tokens, k],
 * out_idx int32 [tokens, k].  experts <= 1024, k <= 64. */
int dmq_route_topk(const void* logits, int logits_fp16, int tokens, int experts, int k,
                   int renorm, void* out_w, void* out_idx, void* stream);

/* The same top-k widened by the always-on shared expert of
 * quantization/wxa16/bit_partitioned_moe.py:1101-1106: the shared expert is handed to the routed
 * path as n_shared extra experts that every token selects (its intermediate neurons cut into
 * n_shared slices of the routed experts' width), so out_w / out_idx are [tokens, k + n_shared]
 * with out_idx[t, k + j] = experts + j and out_w[t, k + j] = sigmoid(x[t] . gate_row) -- the
 * torch.sigmoid(self.shared_expert_gate(x)) factor, rounded to fp16 after the dot product and
 * after the sigmoid.  With logits == NULL the first k columns are copied from topk_idx_in int32 /
 * topk_w_in fp32 [tokens, k] (a router that already returned its top-k).  x fp16 [tokens, hidden],
 * gate_row fp16 [hidden], hidden % 8 == 0, n_shared <= 64. */
int dmq_route_topk_shared(const void* logits, int logits_fp16, const void* topk_idx_in,
                          const void* topk_w_in, int tokens, int experts, int k, int renorm,
                          const void* x_f16, const void* gate_row_f16, int hidden, int n_shared,
                          void* out_w, void* out_idx, void* stream);

/* Sort / bincount / pool partition of bit_partitioned_moe.py:1125-1138 and
 * _merged_pools / _merged_expert_info_rows / _merged_expert_info_groups (:1014-1057) and
 * _build_merged_block_info (turboquant_utils/triton_kernels_a8.py:938-956), without the
 * host round trip.
 *   slice_start [pools, experts] int32: 2*start of the expert in that pool, -1 = not a member
 *   slice_count [pools, experts] int32: 2*I
 * Outputs (device, int32 unless noted):
 *   counts [experts], offsets [experts+1], sorted_tokens [tokens*k],
 *   sorted_weights fp32 [tokens*k], sorted_rows [tokens*k] (token*k + slot of each sorted row),
 *   gu_info / dn_info [pools, experts, 4], n_items [1], items [max_items, DMQ_ITEM_WORDS] (all pools,
 *   pool-major, experts ascending).
 * scratch: device memory of at least dmq_route_scratch_bytes(tokens, k, experts) bytes
 * (per-chunk expert histograms of the counting sort).  experts <= 2048. */
size_t dmq_route_scratch_bytes(int tokens, int k, int experts);
int dmq_route_permute(const void* topk_idx, const void* topk_w, int tokens, int k, int experts,
                      int pools, const void* slice_start, const void* slice_count, int tile_rows,
                      int max_items, void* counts, void* offsets, void* sorted_tokens,
                      void* sorted_weights, void* sorted_rows, void* gu_info, void* dn_info,
                      void* n_items, void* items, void* scratch, size_t scratch_bytes,
                      void* stream);

/* dmq_route_permute for callers that cannot allocate or bring a scratch buffer (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The scratch (per-chunk expert histograms) lives in a static device array of 512 KiB inside the
 * library, one copy per GPU, held until the process ends; its size covers every accepted call
 * (any number of tokens, experts <= 2048; larger problems return DMQ_ERR_LIMIT).  The call
 * allocates nothing.  All calls on one GPU share that array: calls that overlap on a GPU (two
 * streams, two threads) race; calls ordered on one stream do not.  The first call on a GPU looks
 * the array's address up (hipGetSymbolAddress, which may load the code object): make that call
 * outside any stream capture; later calls on that GPU only launch kernels.  Arguments and outputs
 * as dmq_route_permute. */
int dmq_route_permute_static(const void* topk_idx, const void* topk_w, int tokens, int k,
                             int experts, int pools, const void* slice_start,
                             const void* slice_count, int tile_rows, int max_items, void* counts,
                             void* offsets, void* sorted_tokens, void* sorted_weights,
                             void* sorted_rows, void* gu_info, void* dn_info, void* n_items,
                             void* items, void* stream);

/* Work items for a caller-built expert_info: n_items int32[1], items int32 [max_items, 4]
 * with the given pool id. */
int dmq_build_tiles(const void* expert_info, int n_experts, int tile_rows, int max_items,
                    int pool, void* n_items, void* items, void* stream);

/* ------------------------------------------------------------------ activations */

/* batch_rotate_input (turboquant_utils/rotation.py:176-212) for mode A16 and the fused
 * rotate+quantize kernels rotate_quantize_fused (triton_kernels_a8.py:486-523),
 * rotate_quantize_fused_fp8 (triton_kernels_fp8.py:188-226) and rotate_quantize_fused_fp4
 * (triton_kernels_fp4.py:1111-1135) for A8 / FP8 / FP4.
 *   x fp16 [*, x_stride]; row_index (optional) gathers input rows; rot fp16 [groups,128,128]
 *   out: fp16 [rows, K] | int8 / e4m3 [rows, K] | packed e2m1 [rows, K/2] (row-major)
 *   scale: fp16 (scale_fp32 == 0) or fp32 [rows, scale_stride] | FP4: u8 [rows, scale_stride]
 * tt = 1 or 4 activation tiles of 16 rows per wave. */
int dmq_rotate(int mode, const void* x, long x_stride, const void* row_index, const void* rot,
               int rows, int groups, void* out, long out_row_bytes, void* scale,
               int scale_stride, int scale_fp32, float extra_scale, int tt, void* stream);

/* Same, for rows grouped by expert: work item (pool, e, i) covers rows
 * token_start_e + i*tile_rows .. of expert_info.  With rot_per_expert != 0 group g of expert e
 * uses rot[slice_start_e + g] (the per-expert down rotations, seed + original_start of
 * triton_kernels.py:1310), otherwise rot[g].  The slice is read from the work items, which must
 * therefore be built from this expert_info (dmq_build_tiles) or come from dmq_route_permute; the
 * caller guarantees slice_start_e + groups <= number of matrices.  max_items bounds the list. */
int dmq_rotate_tiled(int mode, const void* x, long x_stride, const void* row_index,
                     const void* rot, int rot_per_expert, int groups, const void* expert_info,
                     const void* items, const void* n_items, int tile_rows, int max_items,
                     void* out, long out_row_bytes, void* scale, int scale_stride, int scale_fp32,
                     float extra_scale, int tt, void* stream);

/* quantize_act_per_token_group (triton_kernels_a8.py:384-421), ..._fp8
 * (triton_kernels_fp8.py:94-124) and quantize_act_e2m1_per32 (triton_kernels_fp4.py:125-150):
 * quantization of already rotated activations (fp16 or fp32 input). */
int dmq_quantize_act(int mode, const void* x, int x_fp32, long x_stride, int rows, int groups,
                     void* out, long out_row_bytes, void* scale, int scale_stride, int scale_fp32,
                     float extra_scale, void* stream);

/* ------------------------------------------------------------------ dequant GEMMs */

typedef struct {
  const void* w;            /* idx_gf, or folded e2m1 [G, N, 64] for FP4 */
  const void* norms;        /* norms_gf */
  const void* lut;          /* fp16 / int8 / e4m3 codebook; unused for FP4.  DMQ_MODE_A8 with bit 8:
                               NULL = the identity w = idx - 128 of a uniform codebook (the
                               reference's IDENTITY_CB, triton_kernels_a8.py:769-799), no table read */
  const void* expert_info;
  const void* act;          /* activation codes of this pool, row-major */
  const void* act_scale;    /* fp16 [rows, act_scale_stride] (A8/FP8), u8 (FP4), NULL (A16) */
  const void* row_index;    /* optional gather of activation rows (int32) */
  int n_total;              /* N of the pool's weight */
  int bit;                  /* index width of idx_gf (FP4 reads folded e2m1: pass the pool bit) */
  int mode;                 /* must equal the launch mode; other pools are skipped */
  int w_scale_byte;         /* FP4: 127 + E0 */
  /* Layers whose experts are cut into sub-experts that live in several pools (width_filter of
   * dmq_gemm_args != 0), both int32 [n_experts] in device memory, NULL = all zero:
   * col_start: first column of this pool's share inside the expert's SiLU*up row (gate_up: where
   * the launch writes; down: where it starts contracting); home: rank of this pool among the pools
   * that hold a share of the expert. */
  const void* col_start;
  const void* home;
} dmq_gemm_pool;

typedef struct {
  int mode;                 /* DMQ_MODE_* */
  int epi;                  /* DMQ_EPI_* */
  int tt;                   /* activation tiles of 16 rows per wave: 1, 2 or 4; 8: see rows_queue */
  int ks;                   /* waves of a workgroup splitting K: 0 = 1; 4 or 1 for tt == 1, else 1 */
  int nbl;                  /* blocks of output features one workgroup walks back to back (its
                               loads stay in flight across blocks): 0 = 1; used when ks == 1 */
  int n_pools;
  dmq_gemm_pool pool[DMQ_MAX_POOLS];
  long act_row_bytes;
  int act_scale_stride;
  int groups;               /* groups contracted per expert */
  int n_out;                /* output features per row (SILU: I) */
  int half_width;           /* SILU: I */
  int slice_is_groups;      /* 0 gate_up (slice offsets rows), 1 down (slice offsets groups) */
  const void* items;        /* from dmq_build_tiles / dmq_route_permute, tile_rows == 16*tt, or
                               item_tile_rows when that is set */
  const void* n_items;
  int max_items;
  void* out;                /* STORE/SILU: fp16 [rows, out_stride]; SCATTER: fp16 [slots, out_stride] */
  long out_stride;
  const void* row_weight;   /* SCATTER: fp32 routing weight per row */
  const void* row_slot;     /* SCATTER: int32 destination slot row per row */
  void* dbg_acc;            /* A8, ks == 1, STORE only: int32 [rows, groups, n_out] or NULL */
  /* DMQ_EPI_SILU_ROT (ks == 1, n_out % 128 == 0): per pool the rotation matrices fp16
   * [groups_total, 128, 128] (the matrix of group g of an expert is post_rot[slice_g + g], slice_g
   * the expert's first down group = gate_up slice_start / 256) and the factor folded into the
   * stored scales; rotated codes go to post_out [rows, post_row_bytes] (fp16 / int8 / e4m3 /
   * packed e2m1 by mode), scales to post_scale (fp16 [rows, post_scale_stride] for A8 / FP8, u8
   * for FP4, unused for A16).  `out` is not written. */
  const void* post_rot[DMQ_MAX_POOLS];
  float post_extra_scale[DMQ_MAX_POOLS];
  void* post_out;
  long post_row_bytes;
  void* post_scale;
  int post_scale_stride;
  /* k_split = 2 or 4 (0 / 1 = off): the groups of one (work item, feature block) are shared by
   * that many workgroups, for short work lists that leave most of the chip idle.  tt == 1,
   * ks <= 1, groups % k_split == 0, any bit width; nbl is ignored.  With a SILU epilogue:
   * n_out a multiple of 128, split_partial fp32 [k_split, split_rows, 2 * n_out].  With
   * DMQ_EPI_STORE (a Linear with a handful of rows): k_split may also be 8 or 16,
   * split_partial fp32 [k_split, split_rows, n_out].  split_rows >= every routed row index + 1.
   * Each workgroup parks its fp32 sums in its plane of split_partial and the last to arrive adds
   * the planes in a fixed order and runs the epilogue, so the result does not depend on the order
   * of arrival.  split_counter: int32 [max_items * ceil(n_out / 128)], zero before the launch;
   * the launch leaves it zero. */
  int k_split;
  int split_rows;
  void* split_partial;
  void* split_counter;
  /* Rows per work item of `items` when it differs from 16*tt (0 = 16*tt): a multiple of 16*tt;
   * the launch walks every item as item_tile_rows / (16*tt) row tiles.  Lets one work-item list
   * serve launches of different tile sizes.  Not with k_split. */
  int item_tile_rows;
  /* n-tiles of 16 output features per wave: 0 or 4 = the normal launch; 1 = the launch of a Linear
   * with a handful of rows: DMQ_EPI_STORE, tt == 1, ks == 4 (the four waves of a workgroup split K
   * and the workgroup covers 16 features, so a 4096-feature matrix gives 256 workgroups), any bit
   * width, not WxFP4, not with k_split or dbg_acc; n_out a multiple of 16. */
  int nt;
  /* Sub-expert layers (the reference's --slices checkpoints: an expert's neurons are spread over
   * several bit pools, quantization/wxa16/bit_partitioned_moe.py:499-521; its output is the sum
   * over its pools, :818-822).  A launch serves the shares of one width: work items whose
   * expert_info slice_count differs from width_filter are skipped (0 = no filter); n_out /
   * half_width / groups describe that width.  home_filter >= 0 further restricts the launch to the
   * shares of that rank (the down projection runs rank after rank); accumulate != 0 makes
   * DMQ_EPI_SCATTER add to the slot row instead of storing it (ranks above 0).  Not with k_split. */
  int width_filter;
  int home_filter;
  int accumulate;
  /* tt == 1, ks == 1, 1/2/4-bit pools (not WxFP4): != 0 selects the kernel instance that keeps two
   * workgroups per CU instead of three and in exchange holds the weight ring of 4-bit pools in
   * registers (the three-per-CU instance keeps part of it in scratch memory).  Pays for launches
   * of at most two workgroups per CU and for layers with 4-bit pools; same results either way. */
  int roomy;
  /* != 0: work item i goes to XCD i % 8 (with all its feature blocks) instead of every XCD taking a
   * contiguous eighth of the list.  For launches that serve a small part of the list sitting in
   * one place (the mode of a shared expert: its items are the last ones), which the contiguous
   * split would leave to one XCD; nbl is then 1.  Same results either way. */
  int spread;
  /* mode2_on != 0: the launch also serves the pools whose mode is mode2 (a work item runs the body of
   * its pool's mode).  Only mode2 == DMQ_MODE_A16 next to a quantized `mode`, tt <= 2, ks == 1, no
   * 8-bit pool in either mode, epilogues other than the plain store, no dbg_acc: the shared
   * expert that keeps fp16 activations rides the routed pools' launch.  Scalar fields
   * (act_scale_stride, post_scale ...) are those of `mode`.  Same results as one launch per mode. */
  int mode2_on;
  int mode2;
  /* A launch with 8-bit pools next to narrower ones, tt == 1, ks <= 1, not WxFP4, not the plain
   * store: one kernel instance serves both index widths in ONE launch (two
   * workgroups per CU).  widths_apart != 0 keeps the two launches (the narrower pools then run
   * three workgroups per CU, which wins once the list holds more than about a hundred work
   * items).  Same results. */
  int widths_apart;
  /* tt == 8: the launch for big batches of fp16 layers (DMQ_MODE_A16, 1/2/4-bit pools only): work
   * items of 128 rows (items built with tile_rows == 128; item_tile_rows 0 or 128), one persistent
   * workgroup per CU that dequantizes a weight tile once per stretch of up to 128 rows and draws its
   * units from per-XCD queues, longest first.  groups % 4 == 0; n_out a multiple of 128 (SiLU
   * epilogues) or 256; max_items <= 2048; not with ks > 1, k_split, nt == 1, dbg_acc, mode2,
   * width_filter or accumulate; other pools' items are skipped.  rows_queue: 16 int32 words of
   * device memory, zero before the launch; the launch leaves them zero.  Same results, bit for bit,
   * as tt == 2 and tt == 4. */
  void* rows_queue;
  /* With k_split > 1 and k_split_items > 0: only the first min(n_items[1], k_split_items) work
   * items of the list share their K range between k_split workgroups; the rest run one workgroup
   * per feature block.  For lists that begin with a few long items (pools with a wider index or a
   * table that takes longer to build, ordered first by dmq_route_permute's pool order, their
   * number written to n_items[1]): the launch then ends with the bulk instead of with them.
   * k_split_items bounds that number from the host; not with spread or item_tile_rows. */
  int k_split_items;
  /* gemv != 0: work items of at most 4 rows each (a decode step of at most 4 tokens: one row per
   * token and expert) run as dot products on the vector ALU instead of MFMA tiles: DMQ_MODE_A16,
   * 1/2/4-bit pools, tt == 1, groups a multiple of 4 with groups / 4 in {1, 2, 4, 6, 8},
   * n_out % 64 == 0 (16 from 16 groups on); no ks, k_split, mode2, dbg_acc, width_filter or
   * accumulate.  Rows of an item beyond the fourth are not computed.  Same outputs as the MFMA
   * launch up to the order of the fp32 sums (the norm multiplies the fp32 sum of a quarter group
   * instead of the fp16 operand).  Epilogues:
   *  DMQ_EPI_SILU      SiLU * up rows into out;
   *  DMQ_EPI_SILU_ROT  (n_out % 128 == 0) the rotated SiLU * up rows as partial sums: fp32 planes
   *                    [split_rows, n_out] in split_partial, 8 planes for groups >= 16, 4 for 8
   *                    groups, 2 for 4 (out, post_out and split_counter are not used); the rotated
   *                    row is the sum of the planes in plane order, rounded to fp16;
   *  DMQ_EPI_SCATTER   as the MFMA launch; with gemv_planes > 0 the input rows are those sums of
   *                    the first gemv_planes planes [split_rows, 128 * groups] of split_partial
   *                    instead of the pools' act rows. */
  int gemv;
  int gemv_planes;
} dmq_gemm_args;

/* Merged dequant GEMM: one launch for all 1/2/4-bit pools of a layer that share `mode`, one more
 * for its 8-bit pools (never split over K; see widths_apart for the single launch at tt == 1).  Stands in for
 *   triton_fused_matmul_merged_rows_gf / _merged_in_features_gf   (triton_kernels.py:1482-1615)
 *   wxa8_matmul_merged_rows_gf / _merged_in_features_gf           (triton_kernels_a8.py:959-1068)
 *   wxfp8_matmul_merged_rows_gf / _merged_in_features_gf          (triton_kernels_fp8.py:641-750)
 *   wxfp4_matmul_merged_rows_gf / _merged_in_features_gf          (triton_kernels_fp4.py:740-874)
 * and, with a one-row expert_info, for the per-expert *_grouped_slice_rows_gf /
 * *_grouped_slice_in_features_gf / *_grouped_gf wrappers.  DMQ_EPI_SILU fuses
 * F.silu(gate) * up (bit_partitioned_moe.py:925-930); DMQ_EPI_SCATTER fuses the routing
 * weight and the scatter of :965-967 (the add is dmq_combine_slots). */
int dmq_matmul_merged_gf(const dmq_gemm_args* args, void* stream);

/* out[t, h] = fp16( sum_{j<k} slots[t*k + j, h] (+ add[t, h]) ): the index_add_ of
 * bit_partitioned_moe.py:967 with a fixed summation order and an fp32 sum.  hidden % 8 == 0. */
int dmq_combine_slots(const void* slots_f16, int k, const void* add_f16, long tokens, int hidden,
                      void* out_f16, void* stream);

/* A quantized Linear (the shared-expert and attention Linears of a checkpoint): out = x @ W^T with W
 * in the packed format.  Replaces WxA16Linear.forward (quantization/wxa16/linear.py:224-260, which
 * calls triton_fused_matmul_grouped, triton_kernels.py:600-684), WxA8Linear.forward
 * (quantization/wxa8/linear.py:130-159: rotate_quantize_fused + wxa8_matmul_grouped_gf) and
 * WxFP8Linear.forward (quantization/wxfp8/linear.py): two launches, the rotation (+ quantization)
 * of the rows and the dequant GEMM with its launch shape chosen by batch size.  The bias, if any,
 * is the caller's add. */
typedef struct {
  int mode;                 /* DMQ_MODE_A16 / _A8 / _FP8 */
  int bit;                  /* 1 / 2 / 4 / 8 */
  int in_features;          /* multiple of 128 */
  int out_features;         /* multiple of 64 */
  const void* indices_gf;   /* u8 [G, out_features, 128*bit/8]: group-first packed indices */
  const void* norms_gf;     /* fp16 [G, out_features], already divided by sqrt(128) */
  const void* lut;          /* table of the mode: fp16 / int8 / e4m3 [2^bit]; NULL = identity
                               (int8 path, 8-bit uniform codebook: w = idx - 128) */
  const void* rot;          /* fp16 [G, 128, 128] rotation matrices of the input groups */
  float extra_scale;        /* factor folded into the activation scales (int8 codebook step,
                               e4m3 table scale); 1 for DMQ_MODE_A16 */
} dmq_linear_desc;

/* The int8 GEMM behind dmq_linear_forward for 8-bit weights on a uniform grid and big batches
 * (wxa8_matmul_grouped_gf with IDENTITY_CB, triton_kernels_a8.py:769-799: w = idx - 128):
 * out[r, n] = sum_g x_scale[r, g] * norms_gf[g, n] * sum_k x_i8[r, g, k] * (idx[g, n, k] - 128),
 * 128 x 128 output tiles, both operands through LDS.  x_i8 [rows, x_row_bytes >= in_features]
 * (x_row_bytes % 16 == 0), x_scale fp16 [rows, scale_stride] with the codebook step folded in,
 * indices_gf u8 [G, out_features, 128], norms_gf fp16 [G, out_features] pre-scaled,
 * out fp16 [rows, out_stride]; out_features % 4 == 0, out_stride % 4 == 0. */
int dmq_linear_gemm_i8(const void* x_i8, long x_row_bytes, const void* x_scale_f16, int scale_stride,
                       const void* indices_gf, const void* norms_gf, int rows, int in_features,
                       int out_features, void* out_f16, long out_stride, void* stream);

/* 1 when dmq_linear_forward runs this Linear at this batch size through dmq_linear_gemm_i8. */
int dmq_linear_uses_i8_gemm(const dmq_linear_desc* linear, int rows);

/* Bytes of scratch dmq_linear_forward needs for batches of up to max_rows rows (0: bad descriptor). */
size_t dmq_linear_workspace_bytes(const dmq_linear_desc* linear, int max_rows);

/* x fp16 [rows, x_stride >= in_features] -> out fp16 [rows, out_stride >= out_features] (strides in
 * elements, x_stride % 8 == 0, out_stride % 4 == 0).  workspace: device memory, 256-byte aligned,
 * at least dmq_linear_workspace_bytes(linear, rows) bytes, any contents; calls that overlap on the
 * GPU need separate workspaces.  Allocates nothing, never synchronizes. */
int dmq_linear_forward(const dmq_linear_desc* linear, const void* x_f16, long x_stride, int rows,
                       void* out_f16, long out_stride, void* workspace, size_t workspace_bytes,
                       void* stream);

/* rms_norm of turboquant_utils/norm_kernels.py:79-117, :183-209 (Qwen3_5MoeRMSNorm.forward: the
 * norm in front of the MoE block): out = x * rsqrt(mean(x^2) + eps) * (1 + weight) in fp32, one
 * rounding to the activation type.  x / out fp16 (x_bf16 == 0) or bf16 [rows, n] with the given
 * row strides in elements; weight [n] in the activation type or fp32.  n and strides % 8 == 0. */
int dmq_rms_norm(const void* x, int x_bf16, const void* weight, int weight_fp32, long rows, int n,
                 long x_row_stride, long out_row_stride, float eps, void* out, void* stream);

/* fp16(out32 (+ add16)) over n elements (n % 4 == 0). */
int dmq_finalize_f16(const void* acc_f32, const void* add_f16, long n, void* out_f16, void* stream);
/* Zero-fill n bytes (n % 4 == 0) with a kernel (usable under graph capture). */
int dmq_fill_zero(void* ptr, long n_bytes, void* stream);

/* ------------------------------------------------------------------ whole layer */

typedef struct {
  int bit;
  int mode;                 /* mode of this pool (WxFP4 keeps bit-2 pools on DMQ_MODE_A8) */
  int major;                /* 1: rotate all tokens once (hoisted); 0: rotate routed rows only */
  int n_gate_up;            /* rows of the gate_up pool matrix (2*I*members) */
  int down_groups;          /* groups of the down pool matrix (I*members/128) */
  const void* gu_w;  const void* gu_norms;  const void* gu_lut;  const void* gu_rot;
  float gu_extra_scale;  int gu_w_scale_byte;
  const void* dn_w;  const void* dn_norms;  const void* dn_lut;  const void* dn_rot;
  float dn_extra_scale;  int dn_w_scale_byte;
} dmq_pool_desc;

typedef struct {
  int hidden, inter, experts, top_k, pools;    /* pools <= DMQ_MAX_POOLS */
  const dmq_pool_desc* pool;      /* host array [pools] */
  const void* slice_start;        /* device int32 [pools, experts] (2*start or -1) */
  const void* slice_count;        /* device int32 [pools, experts] (2*width of the pool's share) */
  /* Sub-expert layers (experts spread over several pools, shares of different widths): n_widths > 0
   * lists the distinct share widths (multiples of 128, at most 8), max_homes the largest number of
   * pools one expert lives in, col_start / home device int32 [pools, experts] as in dmq_gemm_pool.
   * n_widths == 0: every expert lives in exactly one pool with width `inter`. */
  int n_widths;
  int widths[8];
  int max_homes;
  const void* col_start;
  const void* home;
} dmq_layer_desc;

/* Bytes of workspace dmq_moe_ffn_forward needs for `tokens` tokens. */
size_t dmq_moe_workspace_bytes(const dmq_layer_desc* layer, int tokens);

/* WxA16BitPartitionedGroupMoE.forward (quantization/wxa16/bit_partitioned_moe.py:1059-1224)
 * and its WxA8 / WxFP8 / WxFP4 subclasses, routed experts only:
 *   x fp16 [tokens, hidden]; topk_idx int32 / topk_w fp32 [tokens, top_k];
 *   out fp16 [tokens, hidden] = sum_k w * down_e(silu(gate_e(x)) * up_e(x)) (+ add_f16).
 * tt <= 0 / ks == 0 / nbl <= 0 pick the tiling
 * (rows per tile, K split, feature blocks per workgroup) from tokens.  ks > 0 splits K over the
 * waves of a workgroup (1 or 4); ks = -2 / -4 shares the K range of the gate_up GEMM between
 * that many workgroups instead (k_split of dmq_gemm_args: tt == 1, at most 1024 routed rows). */
int dmq_moe_ffn_forward(const dmq_layer_desc* layer, const void* x, const void* topk_idx,
                        const void* topk_w, int tokens, const void* add_f16, void* out,
                        void* workspace, size_t workspace_bytes, int tt, int ks, int nbl,
                        void* stream);

/* Same forward with instrumentation, the role of the reference's CudaStageProfiler
 * (turboquant_utils/cuda_profiler.py:51-174): stage_events (optional) is a host array of 7
 * hipEvent_t recorded on `stream` before the first launch and after each stage (sort_prep,
 * rotation, merged_gate_up, act_quant_down, merged_down, combine); aux_out (optional) is a host
 * long[8] that receives tt, ks, the byte offset of counts[experts] inside the workspace,
 * max_items, the byte offset of n_items, nbl, the mask of pools whose SiLU*up rows the gate_up
 * launch rotates itself (bit i: pool i) and the tt of the first down launch. */
int dmq_moe_ffn_forward_staged(const dmq_layer_desc* layer, const void* x, const void* topk_idx,
                               const void* topk_w, int tokens, const void* add_f16, void* out,
                               void* workspace, size_t workspace_bytes, int tt, int ks, int nbl,
                               void* const* stage_events, void* aux_out, void* stream);

/* The router's output as the layer forward takes it: either its logits (softmax + top-k run
 * inside, quantization/wxa16/bit_partitioned_moe.py:1112-1120) or its own top-k (the HF tuple
 * form), plus the sigmoid gate of the always-on shared expert (:1101-1106, see
 * dmq_route_topk_shared). */
typedef struct {
  const void* logits;           /* [tokens, experts - n_shared] fp32 / fp16, or NULL */
  int logits_fp16;
  int renorm;                   /* divide the kept weights by their sum */
  const void* topk_idx;         /* logits == NULL: int32 [tokens, top_k - n_shared] */
  const void* topk_w;           /* logits == NULL: fp32  [tokens, top_k - n_shared] */
  const void* shared_gate_row;  /* fp16 [hidden] (n_shared > 0) */
  int n_shared;                 /* slices of the shared expert among layer->experts / top_k */
} dmq_router_args;

/* The whole layer from the router's output: dmq_moe_ffn_forward_staged plus the routing step.
 * layer->experts and layer->top_k count the n_shared always-on slices (experts E .. E+n_shared-1,
 * selected by every token with the gate value as routing weight).  For up to 1024 routed rows
 * and 512 experts shared columns, sort and work-item list are a single one-workgroup launch,
 * which also computes the top-k for up to 4 tokens; for more tokens the top-k shares the launch
 * of the whole-batch rotation.  stage_events / aux_out as in
 * dmq_moe_ffn_forward_staged (the first stage then includes the top-k); both may be NULL. */
int dmq_moe_ffn_forward_routed(const dmq_layer_desc* layer, const dmq_router_args* router,
                               const void* x, int tokens, const void* add_f16, void* out,
                               void* workspace, size_t workspace_bytes, int tt, int ks, int nbl,
                               void* const* stage_events, void* aux_out, void* stream);

/* What dmq_moe_ffn_forward_prenorm needs on top of the layer: the RMSNorm in front of the block
 * (turboquant_utils/norm_kernels.py:79-117: x = h * rsqrt(mean(h^2) + eps) * (1 + weight), fp32
 * arithmetic, one rounding to fp16) and the router projection (the `gate` Linear of
 * quantization/wxa16/bit_partitioned_moe.py:1112-1120). */
typedef struct {
  const void* norm_weight;      /* [hidden] fp16 or fp32 */
  int norm_weight_fp32;
  float eps;
  const void* gate_weight;      /* fp16 [experts - n_shared, hidden], row-major */
  void* state;                  /* device int32[1], zero before the first call; every call leaves it
                                   zero.  Calls that overlap on the GPU need separate words. */
  void* x_norm_out;             /* optional fp16 [tokens, hidden]: the normalized rows (same bits as
                                   dmq_rms_norm) */
  void* logits_out;             /* optional fp16 [tokens, experts - n_shared]: the router logits the
                                   top-k was taken from */
} dmq_prenorm_args;

/* dmq_moe_ffn_forward_routed for a decode step of at most 16 tokens that starts from the block's
 * pre-norm input h (fp16 [tokens, hidden]): the first launch computes the RMSNorm, the router
 * logits (fp32 accumulation, rounded to fp16 like an fp16 Linear), softmax + top-k and, for up to
 * 4 tokens, the routing step, next to the rotation of the gate_up input, which normalizes its
 * rows itself.  No norm launch, no router GEMM.  router carries renorm, n_shared and
 * shared_gate_row only (logits / topk_* must be NULL).  More than 16 tokens, more than 1024
 * routed experts, experts % 4 != 0 or a sub-expert layer return DMQ_ERR_LIMIT: such callers run
 * dmq_rms_norm, their router and dmq_moe_ffn_forward_routed. */
int dmq_moe_ffn_forward_prenorm(const dmq_layer_desc* layer, const dmq_router_args* router,
                                const dmq_prenorm_args* pre, const void* h, int tokens,
                                const void* add_f16, void* out, void* workspace,
                                size_t workspace_bytes, int tt, int ks, int nbl,
                                void* const* stage_events, void* aux_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif
