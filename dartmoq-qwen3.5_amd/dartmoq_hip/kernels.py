"""The backend callables of the reference, by their reference names.

The reference's MoE modules import their kernels from ``turboquant_utils.triton_kernels``,
``triton_kernels_a8``, ``triton_kernels_fp8``, ``triton_kernels_fp4`` and ``rotation``
(quantization/wxa16/bit_partitioned_moe.py:17-29, wxa8/...:32-41, wxfp8/...:28-37,
wxfp4/...:27-39).  This module offers the same names with the same positional arguments, return
values, dtype rule (non-fp16 inputs are computed in fp16 and cast back) and ValueErrors, on top
of libdartmoq_hip.so.  Every function allocates its outputs, launches on the current stream and
never synchronises, except where noted.  Tensors must live on the GPU.
"""

from __future__ import annotations

import math

import torch

from . import hostprep, ops
from ._lib import (EPI_STORE, MODE_A16, MODE_A8, MODE_FP4, MODE_FP8)
from .hostprep import (build_e2m1_codebook, build_fp8_codebook, build_int8_codebook,  # noqa: F401
                       generate_batch_rotation_matrices, generate_rotation_matrix,
                       is_uniform_codebook, uniform_codebook_step)
from .moe import HipStageProfiler as CudaStageProfiler  # noqa: F401  (cuda_profiler.py:51-174)
from .ops import fold_indices_to_e2m1  # noqa: F401  (triton_kernels_fp4.py:80-122)

GROUP_SIZE = ops.GROUP_SIZE


# ----------------------------------------------------------------------------- helpers

def _check_gs(group_size):
    if group_size != GROUP_SIZE:
        raise ValueError(f"group_size must be {GROUP_SIZE}, got {group_size}")


def _check_bit(bit_width, allowed, what):
    if bit_width not in allowed:
        raise ValueError(f"{what}: bit_width must be one of {sorted(allowed)}, got {bit_width}")


def _seed(seed) -> int:
    return int(seed.item()) if isinstance(seed, torch.Tensor) else int(seed)


def _norms(norms_gf, prescaled, group_size):
    """fp16 norms divided by sqrt(group_size) unless the caller already did."""
    if prescaled:
        return norms_gf.half().contiguous() if norms_gf.dtype != torch.float16 else norms_gf.contiguous()
    return (norms_gf.float() / math.sqrt(group_size)).half().contiguous()


def _info(expert_info, device, what):
    rows = [tuple(int(v) for v in row) for row in expert_info]
    if not rows:
        raise ValueError(f"{what}: empty expert list")
    n_slice = rows[0][3]
    if any(r[3] != n_slice for r in rows):
        raise ValueError(f"{what}: experts of a pool must share one slice_count, got "
                         f"{sorted({r[3] for r in rows})}")
    total = sum(r[1] for r in rows)
    return torch.tensor(rows, dtype=torch.int32, device=device), n_slice, total


def _w_scale_byte(w_s) -> int:
    """The pools of the reference carry one constant e8m0 byte (127 + E0) replicated over
    [N, K/32]; the kernels take the scalar.  Reading a tensor synchronises the stream."""
    if isinstance(w_s, torch.Tensor):
        return int(w_s.reshape(-1)[0].item())
    return int(w_s)


def _rows_major_f4(x_f4_t):
    """(K/2, B) pre-transposed e2m1 codes -> the row-major (B, K/2) buffer the kernels read
    (free for tensors made by rotate_quantize_fused_fp4, a copy otherwise)."""
    return x_f4_t.t().contiguous()


def _gemm(mode, bit, x_codes, x_scale, w_gf, norms, lut, info, *, groups, n_out, slice_is_groups,
          rows_total, w_scale_byte=127, cfg=None):
    tt = None
    if cfg is not None:                       # (BLOCK_B, ...) of the reference: rows per tile
        tt = max(1, min(4, int(cfg[0]) // 16))
        tt = 4 if tt >= 4 else (2 if tt >= 2 else 1)
    small = {}
    if tt is None and rows_total <= 16 and info.shape[0] == 1 and mode != MODE_FP4 and n_out % 16 == 0:
        # one matrix, a handful of rows: a workgroup per 16 features, its four waves splitting K
        tt, small = 1, {"ks": 4, "nt": 1}
    elif tt is None and rows_total > 64 and info.shape[0] == 1:
        # one matrix: the largest row tile that still gives every CU a workgroup (8-bit: 32 rows)
        blocks = (n_out + 255) // 256
        tt = next((t for t in ((2,) if bit == 8 else (4, 2))
                   if ((rows_total + 16 * t - 1) // (16 * t)) * blocks >= 256), 1)
    return ops.matmul_merged(mode, bit, EPI_STORE, x_codes, x_scale, w_gf, norms, lut, info,
                             groups=groups, n_out=n_out, slice_is_groups=slice_is_groups,
                             rows_total=rows_total, w_scale_byte=w_scale_byte, tt=tt, **small)


# ----------------------------------------------------------------------------- norm

def rms_norm(x, weight, eps):
    """turboquant_utils/norm_kernels.py:183-209 (Qwen3_5MoeRMSNorm.forward, the norm that feeds the
    MoE block): (x * rsqrt(mean(x^2) + eps) * (1 + weight)).type_as(x), fp32 inside."""
    return ops.rms_norm(x, weight, eps)


# ----------------------------------------------------------------------------- layout / rotation

def convert_to_group_first(indices_packed, norms, group_size, bit_width):
    """triton_kernels.py:1042-1069: ([N, G*ppg] u8, [N, G] f16) -> ([G, N, ppg], [G, N])."""
    return ops.convert_to_group_first(indices_packed, norms, group_size, bit_width, prescale=False)


def batch_rotate_input(x, group_size, seed_base):
    """rotation.py:176-212: x[B, K] -> x_rot[B, K], group g rotated by the matrix of seed
    seed_base + g * group_size.  The matrices are generated on the host (torch CPU QR)."""
    _check_gs(group_size)
    k = x.shape[1]
    rot = generate_batch_rotation_matrices(group_size, _seed(seed_base), k // group_size, group_size,
                                           device=x.device)
    out, _ = ops.rotate(MODE_A16, x.half() if x.dtype != torch.float16 else x, rot)
    return out if x.dtype == torch.float16 else out.to(x.dtype)


# ----------------------------------------------------------------------------- WxA16 GEMMs

def triton_fused_matmul_grouped_slice_rows_gf(x, indices_packed_gf, codebook, norms_gf, seed,
                                              group_size, in_features, row_start, row_end,
                                              bit_width: int = 4, x_is_rotated: bool = False,
                                              norms_prescaled: bool = False):
    """triton_kernels.py:1143-1251 (gate_up, one expert): rows [row_start, row_end) of the pool."""
    _check_bit(bit_width, {1, 2, 4, 8}, "slice_rows_gf")
    _check_gs(group_size)
    if in_features % group_size:
        raise ValueError(f"in_features ({in_features}) must be a multiple of group_size ({group_size})")
    orig = x.dtype
    xh = x if orig == torch.float16 else x.half()
    x_rot = xh if x_is_rotated else batch_rotate_input(xh, group_size, seed)
    b = x.shape[0]
    info = torch.tensor([[0, b, row_start, row_end - row_start]], dtype=torch.int32, device=x.device)
    out = _gemm(MODE_A16, bit_width, x_rot, None, indices_packed_gf, _norms(norms_gf, norms_prescaled,
                group_size), codebook.half(), info, groups=in_features // group_size,
                n_out=row_end - row_start, slice_is_groups=False, rows_total=b)
    return out if orig == torch.float16 else out.to(orig)


def triton_fused_matmul_grouped_slice_in_features_gf(x, indices_packed_gf, codebook, norms_gf, seed,
                                                     group_size, original_start, original_end,
                                                     full_in_features, bit_width: int = 4,
                                                     norms_prescaled: bool = False):
    """triton_kernels.py:1254-1354 (down, one expert): groups [start/gs, end/gs) of the pool;
    rotates x with seed + original_start."""
    _check_bit(bit_width, {1, 2, 4, 8}, "slice_in_features_gf")
    _check_gs(group_size)
    if original_start % group_size or (original_end - original_start) % group_size:
        raise ValueError(f"slice [{original_start}, {original_end}) must align to group_size {group_size}")
    orig = x.dtype
    xh = x if orig == torch.float16 else x.half()
    x_rot = batch_rotate_input(xh, group_size, _seed(seed) + original_start)
    b = x.shape[0]
    g0, gc = original_start // group_size, (original_end - original_start) // group_size
    info = torch.tensor([[0, b, g0, gc]], dtype=torch.int32, device=x.device)
    out = _gemm(MODE_A16, bit_width, x_rot, None, indices_packed_gf, _norms(norms_gf, norms_prescaled,
                group_size), codebook.half(), info, groups=gc, n_out=indices_packed_gf.shape[1],
                slice_is_groups=True, rows_total=b)
    return out if orig == torch.float16 else out.to(orig)


def triton_fused_matmul_merged_rows_gf(x_rot, indices_packed_gf, codebook, norms_gf, expert_info,
                                       group_size, in_features, bit_width: int = 4,
                                       norms_prescaled: bool = False, cfg=None):
    """triton_kernels.py:1482-1551: every expert of a bit pool in one launch (gate_up)."""
    _check_bit(bit_width, {1, 2, 4, 8}, "merged_rows_gf")
    _check_gs(group_size)
    if in_features % group_size:
        raise ValueError(f"in_features ({in_features}) must be a multiple of group_size ({group_size})")
    if in_features // group_size < 2:
        raise ValueError("merged rows kernel needs at least two groups")
    info, n_slice, total = _info(expert_info, x_rot.device, "merged_rows_gf")
    orig = x_rot.dtype
    xh = x_rot if orig == torch.float16 else x_rot.half()
    out = _gemm(MODE_A16, bit_width, xh, None, indices_packed_gf, _norms(norms_gf, norms_prescaled,
                group_size), codebook.half(), info, groups=in_features // group_size, n_out=n_slice,
                slice_is_groups=False, rows_total=x_rot.shape[0], cfg=cfg)
    return out if orig == torch.float16 else out.to(orig)


def triton_fused_matmul_merged_in_features_gf(x_rot, indices_packed_gf, codebook, norms_gf,
                                              expert_info, group_size, bit_width: int = 4,
                                              norms_prescaled: bool = False, cfg=None):
    """triton_kernels.py:1554-1615: every expert of a bit pool in one launch (down)."""
    _check_bit(bit_width, {1, 2, 4, 8}, "merged_in_features_gf")
    _check_gs(group_size)
    info, g_slice, total = _info(expert_info, x_rot.device, "merged_in_features_gf")
    if g_slice < 2:
        raise ValueError("merged in_features kernel needs at least two groups per expert")
    orig = x_rot.dtype
    xh = x_rot if orig == torch.float16 else x_rot.half()
    out = _gemm(MODE_A16, bit_width, xh, None, indices_packed_gf, _norms(norms_gf, norms_prescaled,
                group_size), codebook.half(), info, groups=g_slice, n_out=indices_packed_gf.shape[1],
                slice_is_groups=True, rows_total=x_rot.shape[0], cfg=cfg)
    return out if orig == torch.float16 else out.to(orig)


# Row-major (checkpoint layout) callables of the Linear path.  The kernels read the group-first
# layout only, so these convert on first sight of a weight tensor and keep the converted copy while
# the source tensor is alive and unmodified; modules that own their weights (dartmoq_hip.linear)
# convert once at load and do not come through here.
_GF_CACHE: dict[tuple, tuple] = {}


def _group_first_cached(indices_packed, norms, group_size, bit_width):
    if norms.dim() == 1:
        norms = norms.unsqueeze(1)
    key = (indices_packed.data_ptr(), norms.data_ptr(), tuple(indices_packed.shape), int(bit_width),
           indices_packed._version, norms._version, str(indices_packed.device))
    hit = _GF_CACHE.get(key)
    if hit is None:
        nh = norms if norms.dtype == torch.float16 else norms.half()
        hit = ops.convert_to_group_first(indices_packed.contiguous(), nh.contiguous(), group_size,
                                         bit_width, prescale=True)
        if len(_GF_CACHE) >= 64:
            _GF_CACHE.pop(next(iter(_GF_CACHE)))
        _GF_CACHE[key] = hit
    return hit


_RAGGED_CACHE: dict = {}


def _ragged_linear(indices_packed, codebook, norms, seed, group_size, in_features, bit_width):
    """A WxA16Linear over a row-major packed matrix whose last group is short; kept per
    (tensor, shape) like the group-first copies, since it pads and re-lays the weights out."""
    from .linear import WxA16Linear
    key = (indices_packed.data_ptr(), tuple(indices_packed.shape), norms.data_ptr(), _seed(seed),
           int(in_features), int(bit_width), indices_packed._version, norms._version)
    hit = _RAGGED_CACHE.get(key)
    if hit is None:
        hit = WxA16Linear(in_features, indices_packed.shape[0], bit_width, group_size, indices_packed,
                          codebook, norms, _seed(seed), device=indices_packed.device)
        if len(_RAGGED_CACHE) >= 64:
            _RAGGED_CACHE.pop(next(iter(_RAGGED_CACHE)))
        _RAGGED_CACHE[key] = hit
    return hit


def triton_fused_matmul_grouped(x, indices_packed, codebook, norms, seed, group_size, in_features,
                                bit_width: int = 4):
    """triton_kernels.py:600-684, the kernel of WxA16Linear.forward: x[B, K] times the whole packed
    matrix [N, K*bit/8] (row-major, bit 1/2/4/8), group g rotated with seed + g*group_size.
    A ragged last group (in_features % group_size != 0, the reference's per-group path :652-684)
    runs through a WxA16Linear, which pads that group once."""
    _check_bit(bit_width, {1, 2, 4, 8}, "matmul_grouped")
    _check_gs(group_size)
    if in_features % group_size:
        return _ragged_linear(indices_packed, codebook, norms, seed, group_size, in_features, bit_width)(x)
    idx_gf, norms_gf = _group_first_cached(indices_packed, norms, group_size, bit_width)
    return triton_fused_matmul_grouped_slice_rows_gf(
        x, idx_gf, codebook, norms_gf, seed, group_size, in_features, 0, indices_packed.shape[0],
        bit_width, norms_prescaled=True)


def triton_fused_matmul_grouped_slice_rows(x, indices_packed, codebook, norms, seed, group_size,
                                           in_features, row_start, row_end, bit_width: int = 4):
    """triton_kernels.py:686-771: output rows [row_start, row_end) of a row-major packed matrix."""
    _check_bit(bit_width, {1, 2, 4, 8}, "slice_rows")
    _check_gs(group_size)
    if in_features % group_size:
        n2 = norms if norms.dim() == 2 else norms.unsqueeze(1)
        return _ragged_linear(indices_packed[row_start:row_end], codebook, n2[row_start:row_end], seed,
                              group_size, in_features, bit_width)(x)
    idx_gf, norms_gf = _group_first_cached(indices_packed, norms, group_size, bit_width)
    return triton_fused_matmul_grouped_slice_rows_gf(
        x, idx_gf, codebook, norms_gf, seed, group_size, in_features, row_start, row_end, bit_width,
        norms_prescaled=True)


def triton_fused_matmul_grouped_slice_in_features(x, indices_packed, codebook, norms, seed,
                                                  group_size, original_start, original_end,
                                                  full_in_features, bit_width: int = 4):
    """triton_kernels.py:774-860: input features [original_start, original_end) of a row-major
    packed matrix; x[B, end-start] is rotated with seed + original_start."""
    _check_bit(bit_width, {1, 2, 4, 8}, "slice_in_features")
    _check_gs(group_size)
    if original_start % group_size:
        raise ValueError(f"original_start ({original_start}) must be aligned to group_size ({group_size})")
    idx_gf, norms_gf = _group_first_cached(indices_packed, norms, group_size, bit_width)
    return triton_fused_matmul_grouped_slice_in_features_gf(
        x, idx_gf, codebook, norms_gf, seed, group_size, original_start, original_end,
        full_in_features, bit_width, norms_prescaled=True)


# ----------------------------------------------------------------------------- activation quantizers

def rotate_quantize_fused(x, rot, group_size, num_groups, extra_scale: float = 1.0):
    """triton_kernels_a8.py:486-523: (int8 [B, K], fp16 scale [B, G]); scale = s * extra_scale."""
    _check_gs(group_size)
    return ops.rotate(MODE_A8, x, rot, extra_scale=extra_scale, scale_fp32=False)


def quantize_act_per_token_group(x_rot, group_size, extra_scale: float = 1.0):
    """triton_kernels_a8.py:384-421: (int8 [B, K], fp32 scale [B, G])."""
    _check_gs(group_size)
    return ops.quantize_act(MODE_A8, x_rot, extra_scale=extra_scale, scale_fp32=True)


def rotate_quantize_fused_fp8(x, rot, group_size, num_groups, extra_scale: float = 1.0):
    """triton_kernels_fp8.py:188-226: (e4m3 [B, K], fp16 scale [B, G])."""
    _check_gs(group_size)
    return ops.rotate(MODE_FP8, x, rot, extra_scale=extra_scale, scale_fp32=False)


def quantize_act_per_token_group_fp8(x_rot, group_size, extra_scale: float = 1.0):
    """triton_kernels_fp8.py:94-124: (e4m3 [B, K], fp32 scale [B, G])."""
    _check_gs(group_size)
    return ops.quantize_act(MODE_FP8, x_rot, extra_scale=extra_scale, scale_fp32=True)


def rotate_quantize_fused_fp4(x, rot, group_size, num_groups):
    """triton_kernels_fp4.py:1111-1135: (e2m1 codes pre-transposed [K/2, B], e8m0 bytes
    [B, K/32]).  The transposed tensor is a view of a row-major [B, K/2] buffer."""
    _check_gs(group_size)
    codes, scale = ops.rotate(MODE_FP4, x, rot)
    return codes.t(), scale


def quantize_act_e2m1_per32(x_rot):
    """triton_kernels_fp4.py:125-150: (packed e2m1 [B, K/2], e8m0 bytes [B, K/32])."""
    return ops.quantize_act(MODE_FP4, x_rot)


# ----------------------------------------------------------------------------- quantized-activation GEMMs

def _qa_slice_rows(mode, what, x_q, x_scale, idx_gf, lut, norms_gf, group_size, in_features, row_start,
                   row_end, bit_width, norms_prescaled, w_scale_byte=127):
    _check_bit(bit_width, {1, 2, 4} if mode == MODE_FP4 else {1, 2, 4, 8}, what)
    _check_gs(group_size)
    b = x_q.shape[0]
    info = torch.tensor([[0, b, row_start, row_end - row_start]], dtype=torch.int32, device=x_q.device)
    return _gemm(mode, bit_width, x_q, x_scale, idx_gf, _norms(norms_gf, norms_prescaled, group_size),
                 lut, info, groups=in_features // group_size, n_out=row_end - row_start,
                 slice_is_groups=False, rows_total=b, w_scale_byte=w_scale_byte)


def _qa_slice_in(mode, what, x_q, x_scale, idx_gf, lut, norms_gf, group_size, original_start,
                 original_end, bit_width, norms_prescaled, w_scale_byte=127):
    _check_bit(bit_width, {1, 2, 4} if mode == MODE_FP4 else {1, 2, 4, 8}, what)
    _check_gs(group_size)
    if original_start % group_size or (original_end - original_start) % group_size:
        raise ValueError(f"slice [{original_start}, {original_end}) must align to group_size {group_size}")
    b = x_q.shape[0]
    g0, gc = original_start // group_size, (original_end - original_start) // group_size
    info = torch.tensor([[0, b, g0, gc]], dtype=torch.int32, device=x_q.device)
    return _gemm(mode, bit_width, x_q, x_scale, idx_gf, _norms(norms_gf, norms_prescaled, group_size),
                 lut, info, groups=gc, n_out=idx_gf.shape[1], slice_is_groups=True, rows_total=b,
                 w_scale_byte=w_scale_byte)


def _qa_merged(mode, what, rows, x_q, x_scale, idx_gf, lut, norms_gf, expert_info, group_size,
               in_features, bit_width, norms_prescaled, cfg, w_scale_byte=127):
    _check_bit(bit_width, {1, 2, 4} if mode == MODE_FP4 else {1, 2, 4, 8}, what)
    _check_gs(group_size)
    info, n_slice, total = _info(expert_info, x_q.device, what)
    if rows:
        if in_features % group_size:
            raise ValueError(f"in_features ({in_features}) must be a multiple of group_size ({group_size})")
        groups, n_out = in_features // group_size, n_slice
    else:
        groups, n_out = n_slice, idx_gf.shape[1]
    return _gemm(mode, bit_width, x_q, x_scale, idx_gf, _norms(norms_gf, norms_prescaled, group_size),
                 lut, info, groups=groups, n_out=n_out, slice_is_groups=not rows,
                 rows_total=x_q.shape[0], w_scale_byte=w_scale_byte, cfg=cfg)


def wxa8_matmul_grouped_slice_rows_gf(x_i8, x_scale, indices_packed_gf, codebook_i8, norms_gf,
                                      group_size, in_features, row_start, row_end,
                                      bit_width: int = 2, norms_prescaled: bool = False):
    """triton_kernels_a8.py:584-624."""
    return _qa_slice_rows(MODE_A8, "wxa8 slice_rows", x_i8, x_scale.half(), indices_packed_gf,
                          codebook_i8, norms_gf, group_size, in_features, row_start, row_end,
                          bit_width, norms_prescaled)


def wxa8_matmul_grouped_slice_in_features_gf(x_i8, x_scale, indices_packed_gf, codebook_i8, norms_gf,
                                             group_size, original_start, original_end,
                                             bit_width: int = 2, norms_prescaled: bool = False):
    """triton_kernels_a8.py:723-766."""
    return _qa_slice_in(MODE_A8, "wxa8 slice_in_features", x_i8, x_scale.half(), indices_packed_gf,
                        codebook_i8, norms_gf, group_size, original_start, original_end, bit_width,
                        norms_prescaled)


def wxa8_matmul_merged_rows_gf(x_i8, x_scale, indices_packed_gf, codebook_i8, norms_gf, expert_info,
                               group_size, in_features, bit_width: int = 2,
                               norms_prescaled: bool = True, cfg=None):
    """triton_kernels_a8.py:959-1014."""
    return _qa_merged(MODE_A8, "wxa8 merged_rows", True, x_i8, x_scale.half(), indices_packed_gf,
                      codebook_i8, norms_gf, expert_info, group_size, in_features, bit_width,
                      norms_prescaled, cfg)


def wxa8_matmul_merged_in_features_gf(x_i8, x_scale, indices_packed_gf, codebook_i8, norms_gf,
                                      expert_info, group_size, bit_width: int = 2,
                                      norms_prescaled: bool = True, cfg=None):
    """triton_kernels_a8.py:1017-1068."""
    return _qa_merged(MODE_A8, "wxa8 merged_in_features", False, x_i8, x_scale.half(),
                      indices_packed_gf, codebook_i8, norms_gf, expert_info, group_size, 0, bit_width,
                      norms_prescaled, cfg)


def wxa8_matmul_grouped_gf(x_i8, x_scale, indices_packed_gf, codebook_i8, norms_gf, group_size,
                           num_groups, bit_width: int = 8, identity_cb: bool = False, cfg=None):
    """triton_kernels_a8.py:769-799, the kernel of WxA8Linear.forward: the whole matrix, norms_gf
    already divided by sqrt(group_size).  With identity_cb (8-bit uniform codebook) codebook_i8 is
    not read and the weights are idx - 128; the codebook step rides x_scale."""
    if identity_cb:
        if bit_width != 8:
            raise ValueError("identity_cb needs bit_width 8")
        codebook_i8 = None                      # the kernel computes idx - 128 itself
    return _qa_slice_rows(MODE_A8, "wxa8 grouped", x_i8, x_scale.half(), indices_packed_gf,
                          codebook_i8, norms_gf, group_size, num_groups * group_size, 0,
                          indices_packed_gf.shape[1], bit_width, True)


def wxfp8_matmul_grouped_gf(x_f8, x_scale, indices_packed_gf, cb_f8, norms_gf, group_size,
                            num_groups, bit_width: int, cfg=None):
    """triton_kernels_fp8.py:407-428: the whole matrix (WxFP8Linear.forward)."""
    return _qa_slice_rows(MODE_FP8, "wxfp8 grouped", x_f8, x_scale.half(), indices_packed_gf, cb_f8,
                          norms_gf, group_size, num_groups * group_size, 0,
                          indices_packed_gf.shape[1], bit_width, True)


def wxfp8_matmul_grouped_slice_rows_gf(x_f8, x_scale, indices_packed_gf, cb_f8, norms_gf, group_size,
                                       in_features, row_start, row_end, bit_width: int = 2,
                                       norms_prescaled: bool = False):
    """triton_kernels_fp8.py:431-467."""
    return _qa_slice_rows(MODE_FP8, "wxfp8 slice_rows", x_f8, x_scale.half(), indices_packed_gf, cb_f8,
                          norms_gf, group_size, in_features, row_start, row_end, bit_width,
                          norms_prescaled)


def wxfp8_matmul_grouped_slice_in_features_gf(x_f8, x_scale, indices_packed_gf, cb_f8, norms_gf,
                                              group_size, original_start, original_end,
                                              bit_width: int = 2, norms_prescaled: bool = False):
    """triton_kernels_fp8.py:470-513."""
    return _qa_slice_in(MODE_FP8, "wxfp8 slice_in_features", x_f8, x_scale.half(), indices_packed_gf,
                        cb_f8, norms_gf, group_size, original_start, original_end, bit_width,
                        norms_prescaled)


def wxfp8_matmul_merged_rows_gf(x_f8, x_scale, indices_packed_gf, cb_f8, norms_gf, expert_info,
                                group_size, in_features, bit_width: int = 2,
                                norms_prescaled: bool = True, cfg=None):
    """triton_kernels_fp8.py:641-696."""
    return _qa_merged(MODE_FP8, "wxfp8 merged_rows", True, x_f8, x_scale.half(), indices_packed_gf,
                      cb_f8, norms_gf, expert_info, group_size, in_features, bit_width, norms_prescaled,
                      cfg)


def wxfp8_matmul_merged_in_features_gf(x_f8, x_scale, indices_packed_gf, cb_f8, norms_gf, expert_info,
                                       group_size, bit_width: int = 2, norms_prescaled: bool = True,
                                       cfg=None):
    """triton_kernels_fp8.py:699-750."""
    return _qa_merged(MODE_FP8, "wxfp8 merged_in_features", False, x_f8, x_scale.half(),
                      indices_packed_gf, cb_f8, norms_gf, expert_info, group_size, 0, bit_width,
                      norms_prescaled, cfg)


def _folded(indices_packed_gf, nib, bit_width, w_e2m1_gf):
    if w_e2m1_gf is not None:
        return w_e2m1_gf
    return ops.fold_indices_to_e2m1(indices_packed_gf, nib, bit_width)


def wxfp4_matmul_grouped_slice_rows_gf_swapped(x_f4_t, x_s, indices_packed_gf, nib, w_s, norms_gf,
                                               group_size, in_features, row_start, row_end, bit_width,
                                               norms_prescaled=False, w_e2m1_gf=None):
    """triton_kernels_fp4.py:501-532.  norms_gf already carries the codebook residual."""
    _check_bit(bit_width, {1, 2, 4}, "wxfp4 slice_rows")
    return _qa_slice_rows(MODE_FP4, "wxfp4 slice_rows", _rows_major_f4(x_f4_t), x_s,
                          _folded(indices_packed_gf, nib, bit_width, w_e2m1_gf), None, norms_gf,
                          group_size, in_features, row_start, row_end, bit_width, norms_prescaled,
                          _w_scale_byte(w_s))


def wxfp4_matmul_grouped_slice_in_features_gf_swapped(x_f4_t, x_s, indices_packed_gf, nib, w_s,
                                                      norms_gf, group_size, original_start,
                                                      original_end, bit_width, norms_prescaled=False,
                                                      w_e2m1_gf=None):
    """triton_kernels_fp4.py:535-569."""
    _check_bit(bit_width, {1, 2, 4}, "wxfp4 slice_in_features")
    return _qa_slice_in(MODE_FP4, "wxfp4 slice_in_features", _rows_major_f4(x_f4_t), x_s,
                        _folded(indices_packed_gf, nib, bit_width, w_e2m1_gf), None, norms_gf,
                        group_size, original_start, original_end, bit_width, norms_prescaled,
                        _w_scale_byte(w_s))


def wxfp4_matmul_merged_rows_gf(x_f4_t, x_s, indices_packed_gf, nib, w_s, norms_gf, expert_info,
                                group_size, in_features, bit_width: int, norms_prescaled: bool = False,
                                w_e2m1_gf=None, cfg=None):
    """triton_kernels_fp4.py:740-808."""
    _check_bit(bit_width, {1, 2, 4}, "wxfp4 merged_rows")
    return _qa_merged(MODE_FP4, "wxfp4 merged_rows", True, _rows_major_f4(x_f4_t), x_s,
                      _folded(indices_packed_gf, nib, bit_width, w_e2m1_gf), None, norms_gf,
                      expert_info, group_size, in_features, bit_width, norms_prescaled, cfg,
                      _w_scale_byte(w_s))


def wxfp4_matmul_merged_in_features_gf(x_f4_t, x_s, indices_packed_gf, nib, w_s, norms_gf, expert_info,
                                       group_size, bit_width: int, norms_prescaled: bool = False,
                                       w_e2m1_gf=None, cfg=None):
    """triton_kernels_fp4.py:811-874."""
    _check_bit(bit_width, {1, 2, 4}, "wxfp4 merged_in_features")
    return _qa_merged(MODE_FP4, "wxfp4 merged_in_features", False, _rows_major_f4(x_f4_t), x_s,
                      _folded(indices_packed_gf, nib, bit_width, w_e2m1_gf), None, norms_gf,
                      expert_info, group_size, 0, bit_width, norms_prescaled, cfg, _w_scale_byte(w_s))
