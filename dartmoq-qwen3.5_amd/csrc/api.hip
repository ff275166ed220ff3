// extern "C" surface of libdartmoq_hip.so: argument checks, workspace carving and launches.
#include "params.h"
#include "gemm_dispatch.h"

__global__ __launch_bounds__(256) void dmq_fill_zero_kernel(uint32_t* p, long n_words) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_words;
       i += (long)gridDim.x * blockDim.x)
    p[i] = 0u;
}

static inline int act_bytes_per_group(int mode) {
  return mode == DMQ_MODE_A16 ? 256 : (mode == DMQ_MODE_FP4 ? 64 : 128);
}

extern "C" {

int dmq_abi_version(void) { return 1; }

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
  if (!dmq_valid_bit(bit)) return DMQ_ERR_BIT;
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
  return dmq_route_topk_launch(logits, logits_fp16, tokens, experts, k, renorm, (float*)out_w,
                               (int*)out_idx, (hipStream_t)stream);
}

int dmq_route_permute(const void* topk_idx, const void* topk_w, int tokens, int k, int experts,
                      int pools, const void* slice_start, const void* slice_count, int tile_rows,
                      int max_tiles, void* counts, void* offsets, void* sorted_tokens,
                      void* sorted_weights, void* sorted_slots, void* gu_info, void* dn_info,
                      void* n_tiles, void* tiles, void* stream) {
  if (!topk_idx || !topk_w || !slice_start || !slice_count || !counts || !offsets ||
      !sorted_tokens || !sorted_weights || !gu_info || !dn_info || !n_tiles || !tiles)
    return DMQ_ERR_NULL;
  if (tokens <= 0 || k <= 0 || experts <= 0 || pools <= 0) return DMQ_ERR_SHAPE;
  if (tile_rows <= 0 || tile_rows % 16) return DMQ_ERR_ALIGN;
  PlanParams plan{(const int*)counts, experts, pools, tile_rows, max_tiles,
                  (const int*)slice_start, (const int*)slice_count, (int*)offsets, (int*)gu_info,
                  (int*)dn_info, (int*)n_tiles, (int*)tiles};
  return dmq_route_permute_launch((const int*)topk_idx, (const float*)topk_w, tokens, k, (int*)counts,
                                  plan, (int*)sorted_tokens, (float*)sorted_weights,
                                  (int*)sorted_slots, (hipStream_t)stream);
}

int dmq_build_tiles(const void* expert_info, int n_experts, int tile_rows, int max_tiles,
                    void* n_tiles, void* tiles, void* stream) {
  if (!expert_info || !n_tiles || !tiles) return DMQ_ERR_NULL;
  if (n_experts <= 0 || max_tiles <= 0) return DMQ_ERR_EMPTY;
  if (tile_rows <= 0 || tile_rows % 16) return DMQ_ERR_ALIGN;
  return dmq_tiles_from_info_launch((const int*)expert_info, n_experts, tile_rows, max_tiles,
                                    (int*)n_tiles, (int*)tiles, (hipStream_t)stream);
}

static int rotate_common(int mode, RotParams& p, long items, int tt, void* stream) {
  if (mode < DMQ_MODE_A16 || mode > DMQ_MODE_FP4) return DMQ_ERR_MODE;
  if (tt != 1 && tt != 4) return DMQ_ERR_MODE;
  if (!p.x || !p.rot || !p.out) return DMQ_ERR_NULL;
  if (mode != DMQ_MODE_A16 && !p.scale) return DMQ_ERR_NULL;
  if (p.groups <= 0) return DMQ_ERR_SHAPE;
  return dmq_rotate_dispatch(mode, p, items, tt, (hipStream_t)stream);
}

int dmq_rotate(int mode, const void* x, long x_stride, const void* row_index, const void* rot,
               int rows, int groups, void* out, long out_row_bytes, void* scale, int scale_stride,
               int scale_fp32, float extra_scale, int tt, void* stream) {
  if (rows <= 0) return DMQ_OK;
  RotParams p{(const __half*)x, x_stride, (const int*)row_index, (const __half*)rot, rows, groups, 1,
              nullptr, nullptr, nullptr, 0, (uint8_t*)out, out_row_bytes, scale, scale_stride,
              scale_fp32, extra_scale};
  if (tt != 1 && tt != 4) return DMQ_ERR_MODE;
  const long row_tiles = (rows + 16 * tt - 1) / (16 * tt);
  return rotate_common(mode, p, row_tiles * groups, tt, stream);
}

int dmq_rotate_tiled(int mode, const void* x, long x_stride, const void* row_index, const void* rot,
                     int rot_per_expert, int groups, const void* expert_info, const void* tiles, const void* n_tiles,
                     int tile_rows, int max_tiles, void* out, long out_row_bytes, void* scale,
                     int scale_stride, int scale_fp32, float extra_scale, int tt, void* stream) {
  if (!expert_info || !tiles || !n_tiles) return DMQ_ERR_NULL;
  if (max_tiles <= 0) return DMQ_OK;
  if (tt != 1 && tt != 4) return DMQ_ERR_MODE;
  if (tile_rows <= 0 || tile_rows % (16 * tt)) return DMQ_ERR_ALIGN;
  RotParams p{(const __half*)x, x_stride, (const int*)row_index, (const __half*)rot, 0, groups,
              rot_per_expert ? 1 : 0, (const int*)expert_info, (const int*)tiles, (const int*)n_tiles, tile_rows,
              (uint8_t*)out, out_row_bytes, scale, scale_stride, scale_fp32, extra_scale};
  const long items = (long)max_tiles * (tile_rows / (16 * tt)) * groups;
  return rotate_common(mode, p, items, tt, stream);
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
  if (a->mode < DMQ_MODE_A16 || a->mode > DMQ_MODE_FP4) return DMQ_ERR_MODE;
  if (!dmq_valid_bit(a->bit)) return DMQ_ERR_BIT;
  if (a->epi < DMQ_EPI_STORE || a->epi > DMQ_EPI_SCATTER) return DMQ_ERR_MODE;
  if (a->tt != 1 && a->tt != 2 && a->tt != 4) return DMQ_ERR_MODE;
  if (!a->act || !a->w || !a->norms || !a->expert_info || !a->tiles || !a->n_tiles || !a->out)
    return DMQ_ERR_NULL;
  if (a->mode != DMQ_MODE_FP4 && !a->lut) return DMQ_ERR_NULL;
  if (a->mode != DMQ_MODE_A16 && !a->act_scale) return DMQ_ERR_NULL;
  if (a->epi == DMQ_EPI_SCATTER && (!a->row_weight || !a->row_token)) return DMQ_ERR_NULL;
  if (a->n_experts <= 0 || a->max_tiles <= 0) return DMQ_ERR_EMPTY;
  if (a->groups <= 0 || a->n_out <= 0 || a->n_total <= 0) return DMQ_ERR_SHAPE;
  const int feat_per_wave = (a->epi == DMQ_EPI_SILU) ? 32 : 64;
  if (a->n_out % feat_per_wave) return DMQ_ERR_ALIGN;
  if (a->epi == DMQ_EPI_SILU && (a->half_width != a->n_out)) return DMQ_ERR_SHAPE;
  if (a->n_total % 16) return DMQ_ERR_ALIGN;
  if (a->act_row_bytes < (long)a->groups * act_bytes_per_group(a->mode)) return DMQ_ERR_SHAPE;

  GemmLaunch L;
  GemmParams& p = L.p;
  p.act = (const uint8_t*)a->act;
  p.act_row_bytes = a->act_row_bytes;
  p.act_scale = a->act_scale;
  p.act_scale_stride = a->act_scale_stride;
  p.row_index = (const int*)a->row_index;
  p.w = (const uint8_t*)a->w;
  p.norms = (const __half*)a->norms;
  p.lut = a->lut;
  p.n_total = a->n_total;
  p.groups = a->groups;
  p.n_out = a->n_out;
  p.half_width = a->half_width;
  p.slice_is_groups = a->slice_is_groups;
  p.w_scale_byte = a->w_scale_byte;
  p.expert_info = (const int*)a->expert_info;
  p.tiles = (const int*)a->tiles;
  p.n_tiles = (const int*)a->n_tiles;
  const int feat_per_block = 4 * feat_per_wave;
  p.n_blocks = (a->n_out + feat_per_block - 1) / feat_per_block;
  p.out = (__half*)a->out;
  p.out_stride = a->out_stride;
  p.out_accum = (float*)a->out;
  p.row_weight = (const float*)a->row_weight;
  p.row_token = (const int*)a->row_token;
  p.dbg_acc = (int*)a->dbg_acc;
  L.bit = a->bit;
  L.epi = a->epi;
  L.tt = a->tt;
  L.dbg = a->dbg_acc != nullptr;
  L.stream = (hipStream_t)stream;
  const long max_work = (long)a->max_tiles * p.n_blocks;
  const int resident = 256 * (a->tt == 1 ? 4 : (a->tt == 2 ? 2 : 1));
  L.grid = (int)(max_work < resident ? max_work : resident);
  switch (a->mode) {
    case DMQ_MODE_A16: return dmq_gemm_launch_a16(L);
    case DMQ_MODE_A8: return dmq_gemm_launch_a8(L);
    case DMQ_MODE_FP8: return dmq_gemm_launch_fp8(L);
    case DMQ_MODE_FP4: return dmq_gemm_launch_fp4(L);
  }
  return DMQ_ERR_MODE;
}

int dmq_finalize_f16(const void* acc_f32, const void* add_f16, long n, void* out_f16, void* stream) {
  if (!acc_f32 || !out_f16) return DMQ_ERR_NULL;
  if (n % 4) return DMQ_ERR_ALIGN;
  return dmq_finalize_launch((const float*)acc_f32, (const __half*)add_f16, n, (__half*)out_f16,
                             (hipStream_t)stream);
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
  int *counts, *offsets, *sorted_tokens, *gu_info, *dn_info, *n_tiles, *tiles;
  float *sorted_weights, *out32;
  uint8_t *xq, *xq_scale, *act, *actq, *actq_scale;
  int max_tiles, tile_rows;
  size_t bytes;
};

static inline size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

static int pick_tt(int tokens, int top_k, int experts) {
  const long avg = (long)tokens * top_k / (experts > 0 ? experts : 1);
  return avg <= 8 ? 1 : (avg <= 48 ? 2 : 4);
}

static MoeWorkspace carve(const dmq_layer_desc* L, int tokens, int tt, uint8_t* base) {
  MoeWorkspace w;
  const size_t R = (size_t)tokens * L->top_k;
  const size_t E = L->experts, P = L->pools, H = L->hidden, I = L->inter;
  w.tile_rows = 16 * tt;
  w.max_tiles = (int)(R / w.tile_rows + E);
  size_t off = 0;
  auto take = [&](size_t n) { uint8_t* p = base + off; off += align_up(n); return p; };
  w.counts = (int*)take(E * 4);
  w.offsets = (int*)take((E + 1) * 4);
  w.sorted_tokens = (int*)take(R * 4);
  w.sorted_weights = (float*)take(R * 4);
  w.gu_info = (int*)take(P * E * 16);
  w.dn_info = (int*)take(P * E * 16);
  w.n_tiles = (int*)take(P * 16);
  w.tiles = (int*)take(P * (size_t)w.max_tiles * 8);
  w.out32 = (float*)take((size_t)tokens * H * 4);
  w.xq = take(R * H * 2);
  w.xq_scale = take(R * (H / DMQ_GS) * 4);
  w.act = take(R * I * 2);
  w.actq = take(R * I * 2);
  w.actq_scale = take(R * (I / DMQ_GS) * 4);
  w.bytes = off;
  return w;
}

size_t dmq_moe_workspace_bytes(const dmq_layer_desc* layer, int tokens) {
  if (!layer || tokens <= 0) return 0;
  // tile size 16 gives the largest tile list; everything else is independent of tt
  return carve(layer, tokens, 1, nullptr).bytes;
}

int dmq_moe_ffn_forward(const dmq_layer_desc* layer, const void* x, const void* topk_idx,
                        const void* topk_w, int tokens, const void* add_f16, void* out,
                        void* workspace, size_t workspace_bytes, int tt, void* stream) {
  if (!layer || !x || !topk_idx || !topk_w || !out || !workspace || !layer->pool) return DMQ_ERR_NULL;
  if (tokens <= 0) return DMQ_ERR_EMPTY;
  const int H = layer->hidden, I = layer->inter, E = layer->experts, K = layer->top_k;
  if (H % DMQ_GS || I % DMQ_GS || H / DMQ_GS < 1 || I / DMQ_GS < 1) return DMQ_ERR_ALIGN;
  if (layer->pools <= 0 || E <= 0 || K <= 0) return DMQ_ERR_SHAPE;
  if (tt <= 0) tt = pick_tt(tokens, K, E);
  if (tt != 1 && tt != 2 && tt != 4) return DMQ_ERR_MODE;
  const int rot_tt = (tt == 4) ? 4 : 1;
  MoeWorkspace w = carve(layer, tokens, tt, (uint8_t*)workspace);
  if (w.bytes > workspace_bytes) return DMQ_ERR_LIMIT;
  const int R = tokens * K;
  int rc;

  rc = dmq_route_permute(topk_idx, topk_w, tokens, K, E, layer->pools, layer->slice_start,
                         layer->slice_count, w.tile_rows, w.max_tiles, w.counts, w.offsets,
                         w.sorted_tokens, w.sorted_weights, nullptr, w.gu_info, w.dn_info,
                         w.n_tiles, w.tiles, stream);
  if (rc) return rc;
  rc = dmq_fill_zero(w.out32, (long)tokens * H * 4, stream);
  if (rc) return rc;

  for (int pi = 0; pi < layer->pools; ++pi) {
    const dmq_pool_desc& pd = layer->pool[pi];
    const int mode = pd.mode;
    if (mode < DMQ_MODE_A16 || mode > DMQ_MODE_FP4) return DMQ_ERR_MODE;
    const int* gu_info = w.gu_info + (size_t)pi * E * 4;
    const int* dn_info = w.dn_info + (size_t)pi * E * 4;
    const int* n_tiles = w.n_tiles + pi * 4;
    const int* tiles = w.tiles + (size_t)pi * w.max_tiles * 2;
    const long code_row_bytes_h = (long)(H / DMQ_GS) * act_bytes_per_group(mode);
    const long code_row_bytes_i = (long)(I / DMQ_GS) * act_bytes_per_group(mode);
    const int sstride_h = (mode == DMQ_MODE_FP4) ? H / 32 : H / DMQ_GS;
    const int sstride_i = (mode == DMQ_MODE_FP4) ? I / 32 : I / DMQ_GS;

    // 1. gate_up input: rotate (+quantize) once per token (major pool) or per routed row
    if (pd.major) {
      rc = dmq_rotate(mode, x, H, nullptr, pd.gu_rot, tokens, H / DMQ_GS, w.xq, code_row_bytes_h,
                      w.xq_scale, sstride_h, 0, pd.gu_extra_scale, rot_tt, stream);
    } else {
      // gate_up rotation matrices do not depend on the expert
      rc = dmq_rotate_tiled(mode, x, H, w.sorted_tokens, pd.gu_rot, 0, H / DMQ_GS, gu_info, tiles,
                            n_tiles, w.tile_rows, w.max_tiles, w.xq, code_row_bytes_h, w.xq_scale,
                            sstride_h, 0, pd.gu_extra_scale, rot_tt, stream);
    }
    if (rc) return rc;

    // 2. gate_up GEMM with fused SiLU * up -> act[R, I]
    dmq_gemm_args g{};
    g.mode = mode; g.bit = pd.bit; g.epi = DMQ_EPI_SILU; g.tt = tt;
    g.act = w.xq; g.act_row_bytes = code_row_bytes_h;
    g.act_scale = (mode == DMQ_MODE_A16) ? nullptr : w.xq_scale; g.act_scale_stride = sstride_h;
    g.row_index = pd.major ? w.sorted_tokens : nullptr;
    g.w = pd.gu_w; g.norms = pd.gu_norms; g.lut = pd.gu_lut;
    g.n_total = pd.n_gate_up; g.groups = H / DMQ_GS; g.n_out = I; g.half_width = I;
    g.slice_is_groups = 0; g.w_scale_byte = pd.gu_w_scale_byte;
    g.expert_info = gu_info; g.n_experts = E; g.tiles = tiles; g.n_tiles = n_tiles;
    g.max_tiles = w.max_tiles;
    g.out = w.act; g.out_stride = I;
    rc = dmq_matmul_merged_gf(&g, stream);
    if (rc) return rc;

    // 3. down input: per-expert rotation (+quantize) of act
    rc = dmq_rotate_tiled(mode, w.act, I, nullptr, pd.dn_rot, 1, I / DMQ_GS, dn_info, tiles, n_tiles,
                          w.tile_rows, w.max_tiles, w.actq, code_row_bytes_i, w.actq_scale,
                          sstride_i, 0, pd.dn_extra_scale, rot_tt, stream);
    if (rc) return rc;

    // 4. down GEMM with fused routing weight + scatter-add into out32
    dmq_gemm_args d{};
    d.mode = mode; d.bit = pd.bit; d.epi = DMQ_EPI_SCATTER; d.tt = tt;
    d.act = w.actq; d.act_row_bytes = code_row_bytes_i;
    d.act_scale = (mode == DMQ_MODE_A16) ? nullptr : w.actq_scale; d.act_scale_stride = sstride_i;
    d.row_index = nullptr;
    d.w = pd.dn_w; d.norms = pd.dn_norms; d.lut = pd.dn_lut;
    d.n_total = H; d.groups = I / DMQ_GS; d.n_out = H; d.half_width = 0;
    d.slice_is_groups = 1; d.w_scale_byte = pd.dn_w_scale_byte;
    d.expert_info = dn_info; d.n_experts = E; d.tiles = tiles; d.n_tiles = n_tiles;
    d.max_tiles = w.max_tiles;
    d.out = w.out32; d.out_stride = H;
    d.row_weight = w.sorted_weights; d.row_token = w.sorted_tokens;
    rc = dmq_matmul_merged_gf(&d, stream);
    if (rc) return rc;
  }
  (void)R;
  return dmq_finalize_f16(w.out32, add_f16, (long)tokens * H, out, stream);
}

}  // extern "C"
