"""Thin torch-tensor front end of the C ABI: pointer extraction, output allocation, checks.

torch is used for device memory and streams only; every computation below happens in
libdartmoq_hip.so.
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._lib import (EPI_SILU_ROT,  # noqa: F401
                   EPI_SCATTER, EPI_SILU, EPI_STORE, MODE_A16, MODE_A8, MODE_FP4, MODE_FP8, GemmArgs,
                   check, load)

GROUP_SIZE = 128
ROWS_TT = 8          # tt value of the persistent launch over 128-row work items (fp16 layers)
ITEM_WORDS = 8          # int32 words of a work-item record (DMQ_ITEM_WORDS)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("dartmoq_hip operates on GPU tensors only (no CPU fallback)")


def _check_bit(bit, allowed=(1, 2, 4)):
    if bit not in allowed:
        raise ValueError(f"bit_width must be one of {allowed}, got {bit}")


def act_bytes_per_group(mode: int) -> int:
    return {MODE_A16: 256, MODE_A8: 128, MODE_FP8: 128, MODE_FP4: 64}[mode]


# ----------------------------------------------------------------------------- packed format

def unpack_nbit(packed: torch.Tensor, bit_width: int, n: int | None = None) -> torch.Tensor:
    """uint8 (..., P) -> uint8 (..., P*8/bit) [:n]."""
    _check_bit(bit_width, (1, 2, 4, 8))
    _need_cuda(packed)
    packed = packed.contiguous()
    epb = 8 // bit_width
    out = torch.empty(packed.shape[:-1] + (packed.shape[-1] * epb,), dtype=torch.uint8,
                      device=packed.device)
    check(load().dmq_unpack_nbit(_ptr(packed), packed.numel(), bit_width, _ptr(out),
                                 _stream(packed.device)), "unpack_nbit")
    return out if n is None else out[..., :n]


def convert_to_group_first(indices_packed, norms, group_size, bit_width, prescale: bool = False):
    _check_bit(bit_width, (1, 2, 4, 8))
    if group_size != GROUP_SIZE:
        raise ValueError(f"group_size must be {GROUP_SIZE}, got {group_size}")
    _need_cuda(indices_packed, norms)
    indices_packed = indices_packed.contiguous()
    norms = norms.contiguous().to(torch.float16)
    ppg = group_size * bit_width // 8
    n_rows, packed_k = indices_packed.shape
    if packed_k % ppg:
        raise ValueError(f"packed row length {packed_k} is not a multiple of {ppg}")
    groups = packed_k // ppg
    idx_gf = torch.empty((groups, n_rows, ppg), dtype=torch.uint8, device=indices_packed.device)
    norms_gf = torch.empty((groups, n_rows), dtype=torch.float16, device=indices_packed.device)
    check(load().dmq_convert_to_group_first(_ptr(indices_packed), _ptr(norms), n_rows, groups,
                                            bit_width, int(prescale), _ptr(idx_gf), _ptr(norms_gf),
                                            _stream(idx_gf.device)), "convert_to_group_first")
    return idx_gf, norms_gf


def dequant_tile(idx_gf, codebook, norms_gf, g0, g_cnt, n0, n_cnt, bit_width):
    _check_bit(bit_width, (1, 2, 4, 8))
    _need_cuda(idx_gf, codebook)
    out = torch.empty((g_cnt, n_cnt, GROUP_SIZE), dtype=torch.float16, device=idx_gf.device)
    check(load().dmq_dequant_tile(_ptr(idx_gf), _ptr(codebook.contiguous()), _ptr(norms_gf),
                                  idx_gf.shape[1], g0, g_cnt, n0, n_cnt, bit_width, _ptr(out),
                                  _stream(out.device)), "dequant_tile")
    return out


def fold_indices_to_e2m1(indices_gf, nib, bit_width, group_size=GROUP_SIZE):
    if bit_width not in (1, 2, 4):
        raise ValueError(f"fold supports bit 1/2/4, got {bit_width}")
    _need_cuda(indices_gf)
    g, n, _ = indices_gf.shape
    out = torch.empty((g, n, group_size // 2), dtype=torch.uint8, device=indices_gf.device)
    nib = nib.to(indices_gf.device, torch.uint8).contiguous()
    check(load().dmq_fold_indices_to_e2m1(_ptr(indices_gf.contiguous()), _ptr(nib), g * n, bit_width,
                                          _ptr(out), _stream(out.device)), "fold_indices_to_e2m1")
    return out


# ----------------------------------------------------------------------------- routing

def route_topk(logits: torch.Tensor, top_k: int, renormalize: bool = False):
    _need_cuda(logits)
    if logits.dtype not in (torch.float32, torch.float16):
        logits = logits.float()
    logits = logits.contiguous()
    t, e = logits.shape
    w = torch.empty((t, top_k), dtype=torch.float32, device=logits.device)
    idx = torch.empty((t, top_k), dtype=torch.int32, device=logits.device)
    check(load().dmq_route_topk(_ptr(logits), int(logits.dtype == torch.float16), t, e, top_k,
                                int(renormalize), _ptr(w), _ptr(idx), _stream(logits.device)),
          "route_topk")
    return w, idx


def route_topk_shared(logits, topk_idx, topk_w, top_k: int, renormalize: bool, x: torch.Tensor,
                      gate_row: torch.Tensor, num_experts: int, n_shared: int):
    """Top-k (from ``logits``, or copied from ``topk_idx`` / ``topk_w`` when logits is None) widened
    by ``n_shared`` always-on columns: index num_experts + j, weight sigmoid(x . gate_row)."""
    _need_cuda(x, gate_row)
    if x.dtype != torch.float16 or gate_row.dtype != torch.float16:
        raise TypeError("x and gate_row must be fp16")
    x = x.contiguous()
    gate_row = gate_row.contiguous().reshape(-1)
    t, h = x.shape
    if gate_row.numel() != h:
        raise ValueError("gate_row must hold hidden values")
    w = torch.empty((t, top_k + n_shared), dtype=torch.float32, device=x.device)
    idx = torch.empty((t, top_k + n_shared), dtype=torch.int32, device=x.device)
    if logits is not None:
        _need_cuda(logits)
        if logits.dtype not in (torch.float32, torch.float16):
            logits = logits.float()
        logits = logits.contiguous()
        if logits.shape != (t, num_experts):
            raise ValueError("logits must be [tokens, num_experts]")
        args = (_ptr(logits), int(logits.dtype == torch.float16), None, None)
    else:
        _need_cuda(topk_idx, topk_w)
        topk_idx = topk_idx.to(torch.int32).contiguous()
        topk_w = topk_w.float().contiguous()
        if topk_idx.shape != (t, top_k) or topk_w.shape != (t, top_k):
            raise ValueError("topk_idx / topk_w must be [tokens, top_k]")
        args = (None, 0, _ptr(topk_idx), _ptr(topk_w))
    check(load().dmq_route_topk_shared(*args, t, num_experts, top_k, int(renormalize), _ptr(x),
                                       _ptr(gate_row), h, n_shared, _ptr(w), _ptr(idx),
                                       _stream(x.device)), "route_topk_shared")
    return w, idx


def route_permute(topk_idx, topk_w, num_experts, slice_start, slice_count, tile_rows=16,
                  static_scratch=False):
    """Device-side sort + pool partition.  Returns a dict of int32/fp32 device tensors.
    ``static_scratch``: go through dmq_route_permute_static, whose histograms live in the library's
    static device array instead of a scratch tensor (the entry point for callers that cannot
    allocate; calls that overlap on one GPU would race on that array)."""
    _need_cuda(topk_idx, topk_w, slice_start, slice_count)
    t, k = topk_idx.shape
    dev = topk_idx.device
    pools = slice_start.shape[0]
    rows = t * k
    max_items = rows // tile_rows + num_experts
    i32 = dict(dtype=torch.int32, device=dev)
    res = {
        "counts": torch.empty(num_experts, **i32),
        "offsets": torch.empty(num_experts + 1, **i32),
        "sorted_tokens": torch.empty(rows, **i32),
        "sorted_weights": torch.empty(rows, dtype=torch.float32, device=dev),
        "sorted_rows": torch.empty(rows, **i32),
        "gu_info": torch.empty((pools, num_experts, 4), **i32),
        "dn_info": torch.empty((pools, num_experts, 4), **i32),
        "n_items": torch.zeros(4, **i32),
        "items": torch.zeros((max_items, ITEM_WORDS), **i32),
        "max_items": max_items, "tile_rows": tile_rows,
    }
    if static_scratch:
        check(load().dmq_route_permute_static(
            _ptr(topk_idx.to(torch.int32).contiguous()), _ptr(topk_w.float().contiguous()), t, k,
            num_experts, pools, _ptr(slice_start.contiguous()), _ptr(slice_count.contiguous()),
            tile_rows, max_items, _ptr(res["counts"]), _ptr(res["offsets"]), _ptr(res["sorted_tokens"]),
            _ptr(res["sorted_weights"]), _ptr(res["sorted_rows"]), _ptr(res["gu_info"]),
            _ptr(res["dn_info"]), _ptr(res["n_items"]), _ptr(res["items"]), _stream(dev)),
            "route_permute_static")
        return res
    scratch = torch.empty(max(1, load().dmq_route_scratch_bytes(t, k, num_experts)),
                          dtype=torch.uint8, device=dev)
    check(load().dmq_route_permute(
        _ptr(topk_idx.to(torch.int32).contiguous()), _ptr(topk_w.float().contiguous()), t, k,
        num_experts, pools, _ptr(slice_start.contiguous()), _ptr(slice_count.contiguous()), tile_rows,
        max_items, _ptr(res["counts"]), _ptr(res["offsets"]), _ptr(res["sorted_tokens"]),
        _ptr(res["sorted_weights"]), _ptr(res["sorted_rows"]), _ptr(res["gu_info"]),
        _ptr(res["dn_info"]), _ptr(res["n_items"]), _ptr(res["items"]), _ptr(scratch),
        scratch.numel(), _stream(dev)), "route_permute")
    return res


def build_tiles(expert_info: torch.Tensor, rows_total: int, tile_rows: int, pool: int = 0):
    """(n_items int32[1], items int32[max_items, 4], max_items) for a device expert_info [E, 4]."""
    _need_cuda(expert_info)
    n_exp = expert_info.shape[0]
    max_items = rows_total // tile_rows + n_exp
    n_items = torch.zeros(4, dtype=torch.int32, device=expert_info.device)
    items = torch.zeros((max_items, ITEM_WORDS), dtype=torch.int32, device=expert_info.device)
    check(load().dmq_build_tiles(_ptr(expert_info), n_exp, tile_rows, max_items, pool, _ptr(n_items),
                                 _ptr(items), _stream(expert_info.device)), "build_tiles")
    return n_items, items, max_items


# ----------------------------------------------------------------------------- activations

def _alloc_codes(mode, rows, k, device, scale_fp32):
    groups = k // GROUP_SIZE
    if mode == MODE_A16:
        return torch.empty((rows, k), dtype=torch.float16, device=device), None, 0
    if mode == MODE_A8:
        codes = torch.empty((rows, k), dtype=torch.int8, device=device)
    elif mode == MODE_FP8:
        codes = torch.empty((rows, k), dtype=torch.float8_e4m3fn, device=device)
    else:
        codes = torch.empty((rows, k // 2), dtype=torch.uint8, device=device)
        return codes, torch.empty((rows, k // 32), dtype=torch.uint8, device=device), k // 32
    sdt = torch.float32 if scale_fp32 else torch.float16
    return codes, torch.empty((rows, groups), dtype=sdt, device=device), groups


def rotate(mode: int, x: torch.Tensor, rot: torch.Tensor, extra_scale: float = 1.0,
           scale_fp32: bool = False, tt: int | None = None):
    """Rotate (and quantize for mode != A16) x[B, K] with rot[G, 128, 128]."""
    _need_cuda(x, rot)
    if x.dtype != torch.float16:
        x = x.half()
    x = x.contiguous()
    rot = rot.contiguous()
    rows, k = x.shape
    groups = k // GROUP_SIZE
    if k != groups * GROUP_SIZE:
        raise ValueError(f"K ({k}) must be a multiple of {GROUP_SIZE}")
    if tuple(rot.shape) != (groups, GROUP_SIZE, GROUP_SIZE) or rot.dtype != torch.float16:
        raise ValueError(f"rot must be fp16 {(groups, GROUP_SIZE, GROUP_SIZE)}, got {tuple(rot.shape)}")
    codes, scale, sstride = _alloc_codes(mode, rows, k, x.device, scale_fp32)
    if tt is None:
        tt = 4 if rows >= 1024 else 1
    check(load().dmq_rotate(mode, _ptr(x), x.stride(0), None, _ptr(rot), rows, groups,
                            _ptr(codes), codes.stride(0) * codes.element_size(), _ptr(scale), sstride,
                            int(scale_fp32), float(extra_scale), tt, _stream(x.device)), "rotate")
    return codes, scale


def rotate_tiled(mode, x, rot, expert_info, n_items, items, tile_rows, max_items, rows_out,
                 rot_per_expert=True, extra_scale=1.0, row_index=None, tt=1):
    """Rotation of rows grouped by expert: rows of expert e use rot[slice_start_e + g] when
    ``rot_per_expert`` (else rot[g]); ``row_index`` gathers the input rows."""
    _need_cuda(x, rot, expert_info)
    x = x.contiguous()
    k = x.shape[1]
    groups = k // GROUP_SIZE
    codes, scale, sstride = _alloc_codes(mode, rows_out, k, x.device, False)
    check(load().dmq_rotate_tiled(mode, _ptr(x), x.stride(0), _ptr(row_index), _ptr(rot.contiguous()),
                                  int(rot_per_expert), groups, _ptr(expert_info), _ptr(items),
                                  _ptr(n_items), tile_rows, max_items, _ptr(codes),
                                  codes.stride(0) * codes.element_size(), _ptr(scale), sstride, 0,
                                  float(extra_scale), tt, _stream(x.device)), "rotate_tiled")
    return codes, scale


def quantize_act(mode: int, x_rot: torch.Tensor, extra_scale: float = 1.0, scale_fp32: bool = True):
    """Quantize already rotated activations (fp16 or fp32)."""
    _need_cuda(x_rot)
    if x_rot.dtype not in (torch.float16, torch.float32):
        x_rot = x_rot.float()
    x_rot = x_rot.contiguous()
    rows, k = x_rot.shape
    if k % GROUP_SIZE:
        raise ValueError(f"K ({k}) must be a multiple of group_size ({GROUP_SIZE})")
    codes, scale, sstride = _alloc_codes(mode, rows, k, x_rot.device, scale_fp32)
    check(load().dmq_quantize_act(mode, _ptr(x_rot), int(x_rot.dtype == torch.float32), x_rot.stride(0),
                                  rows, k // GROUP_SIZE, _ptr(codes),
                                  codes.stride(0) * codes.element_size(), _ptr(scale), sstride,
                                  int(scale_fp32), float(extra_scale), _stream(x_rot.device)),
          "quantize_act")
    return codes, scale


# ----------------------------------------------------------------------------- GEMM

def pick_tt(rows_total: int, n_experts: int) -> int:
    avg = rows_total / max(n_experts, 1)
    return 1 if avg <= 8 else (2 if avg <= 160 else 4)


def pick_ks(tt: int, rows_total: int) -> int:
    """Waves of a workgroup splitting K in a stand-alone GEMM launch."""
    return 4 if (tt == 1 and rows_total <= 16) else 1


def gemv_plane_count(groups: int) -> int:
    """Planes a rotating dot-product gate_up launch over ``groups`` groups of 128 writes."""
    nit = groups // 4
    return 128 // (16 * (1 if nit >= 4 else 4 // max(nit, 1)))


def gemm_pool(mode, bit, act, act_scale, w, norms, lut, expert_info, row_index=None, w_scale_byte=127):
    """One pool entry of a merged launch (a dict of device tensors and scalars)."""
    return dict(mode=mode, bit=bit, act=act, act_scale=act_scale, w=w, norms=norms, lut=lut,
                expert_info=expert_info, row_index=row_index, w_scale_byte=w_scale_byte)


def matmul_pools(mode, epi, pools, items, n_items, max_items, *, groups, n_out, slice_is_groups,
                 tt, ks=0, nbl=0, out, out_stride, half_width=0, act_row_bytes=None, act_scale_stride=None,
                 row_weight=None, row_slot=None, dbg_acc=None, post=None, k_split=0, k_split_items=0, rows_total=None,
                 item_tile_rows=0, split_ws=None, nt=0, roomy=0, spread=0, mode2=None, widths_apart=0, gemv=False,
                 gemv_planes=None):
    """Merged dequant-GEMM launch over up to four pools sharing one work-item list.  ``post``
    (EPI_SILU_ROT) = dict(rot=[per-pool fp16 rotation matrices], extra=[per-pool scale factors],
    out=codes tensor [rows, *], scale=scale tensor or None).  ``k_split`` = 2 or 4 (plain-store
    epilogue: up to 16) shares the groups of every (item, feature block) between that many
    workgroups (16-row tiles, SiLU and plain-store epilogues); ``rows_total`` then bounds the
    routed row indices and ``split_ws`` = (fp32 planes, zeroed int32 counters) may bring the
    scratch tensors in (allocated per call otherwise).  ``nt`` = 1: one n-tile per wave (plain
    store, tt = 1, ks = 4; any bit width): the launch of a Linear with a handful of rows.  ``item_tile_rows``: rows per work item
    when the list was built for a larger tile than 16 * tt.  ``gemv``: work items of at most four
    rows as dot products on the vector ALU (fp16 activations, 1/2/4-bit pools; SiLU, scatter, or,
    with ``gemv_planes``, SiLU + down rotation handed to the scatter launch as fp32 planes)."""
    a = GemmArgs()
    a.mode, a.epi, a.tt, a.ks, a.nbl, a.n_pools = mode, epi, tt, ks, nbl, len(pools)
    dev = None
    for i, p in enumerate(pools):
        _need_cuda(p["act"], p["w"], p["norms"], p["expert_info"])
        dev = p["act"].device
        _check_bit(p["bit"], (1, 2, 4, 8))
        q = a.pool[i]
        q.w, q.norms = p["w"].data_ptr(), p["norms"].data_ptr()
        q.lut = p["lut"].data_ptr() if p["lut"] is not None else None
        q.expert_info = p["expert_info"].data_ptr()
        q.act = p["act"].data_ptr()
        q.act_scale = p["act_scale"].data_ptr() if p["act_scale"] is not None else None
        q.row_index = p["row_index"].data_ptr() if p["row_index"] is not None else None
        q.n_total, q.bit, q.mode, q.w_scale_byte = p["w"].shape[1], p["bit"], p["mode"], int(p["w_scale_byte"])
    first = next(p for p in pools if p["mode"] == mode)
    if act_row_bytes is None:
        act_row_bytes = first["act"].stride(0) * first["act"].element_size()
    if act_scale_stride is None:
        act_scale_stride = first["act_scale"].stride(0) if first["act_scale"] is not None else 0
    a.act_row_bytes, a.act_scale_stride = act_row_bytes, act_scale_stride
    a.groups, a.n_out, a.half_width, a.slice_is_groups = groups, n_out, half_width, int(slice_is_groups)
    a.items, a.n_items, a.max_items = items.data_ptr(), n_items.data_ptr(), max_items
    a.out, a.out_stride = out.data_ptr(), out_stride
    a.row_weight = row_weight.data_ptr() if row_weight is not None else None
    a.row_slot = row_slot.data_ptr() if row_slot is not None else None
    a.dbg_acc = dbg_acc.data_ptr() if dbg_acc is not None else None
    if post is not None:
        for i, r in enumerate(post["rot"]):
            a.post_rot[i] = r.data_ptr() if r is not None else None
            a.post_extra_scale[i] = float(post["extra"][i])
        a.post_out = post["out"].data_ptr()
        a.post_row_bytes = post["out"].stride(0) * post["out"].element_size()
        if post.get("scale") is not None:
            a.post_scale = post["scale"].data_ptr()
            a.post_scale_stride = post["scale"].stride(0)
    a.item_tile_rows = int(item_tile_rows)
    a.nt = int(nt)
    a.roomy = int(roomy)
    a.spread = int(spread)
    a.mode2_on = 0 if mode2 is None else 1
    a.mode2 = 0 if mode2 is None else int(mode2)
    a.widths_apart = int(widths_apart)
    a.gemv = int(bool(gemv))
    if gemv and gemv_planes is not None:
        # fp32 planes [n_planes, rows, width] of partial sums of the rotated SiLU*up rows: written by
        # the gate_up launch (EPI_SILU_ROT, width = n_out), read by the down launch (EPI_SCATTER,
        # width = 128 * groups)
        if gemv_planes.dtype != torch.float32 or gemv_planes.dim() != 3 or not gemv_planes.is_contiguous():
            raise TypeError("gemv_planes must be a contiguous float32 tensor [planes, rows, width]")
        width = 128 * groups if epi == EPI_SCATTER else n_out
        if gemv_planes.shape[2] != width or gemv_planes.shape[0] < (1 if epi == EPI_SCATTER else gemv_plane_count(groups)):
            raise ValueError("gemv_planes does not fit this launch")
        if rows_total is not None and gemv_planes.shape[1] < rows_total:
            raise ValueError("gemv_planes holds fewer rows than the launch routes")
        a.split_partial, a.split_rows = gemv_planes.data_ptr(), gemv_planes.shape[1]
        a.gemv_planes = gemv_planes.shape[0] if epi == EPI_SCATTER else 0
    if tt == ROWS_TT:       # the persistent launch over 128-row work items: its queue words start at zero
        rows_queue = torch.zeros(16, dtype=torch.int32, device=dev)
        a.rows_queue = rows_queue.data_ptr()
    if k_split > 1:
        if rows_total is None:
            raise ValueError("k_split needs rows_total")
        width = n_out if epi == EPI_STORE else 2 * n_out
        n_counters = max_items * ((n_out + 127) // 128)
        if split_ws is not None:
            partial, counter = split_ws
            if partial.numel() < k_split * rows_total * width or counter.numel() < n_counters:
                raise ValueError("split_ws is too small for this launch")
        else:
            partial = torch.empty((k_split, rows_total, width), dtype=torch.float32, device=dev)
            counter = torch.zeros(n_counters, dtype=torch.int32, device=dev)
        a.k_split, a.split_rows = k_split, rows_total
        a.k_split_items = int(k_split_items)
        a.split_partial, a.split_counter = partial.data_ptr(), counter.data_ptr()
    check(load().dmq_matmul_merged_gf(ctypes.byref(a), _stream(dev)), "matmul_merged_gf")
    return out


def matmul_merged(mode, bit, epi, act, act_scale, w, norms, lut, expert_info, *, groups, n_out,
                  slice_is_groups, rows_total, out=None, out_stride=None, half_width=0,
                  row_index=None, w_scale_byte=127, row_weight=None, row_slot=None, tt=None, ks=0, nbl=0,
                  tiling=None, dbg_acc=None, post=None, k_split=0, item_tile_rows=0, split_ws=None, nt=0,
                  roomy=0, spread=0, widths_apart=0, gemv=False, gemv_planes=None):
    """One-pool merged dequant GEMM.  ``expert_info`` is an int32 device tensor [E, 4]."""
    _need_cuda(act, w, norms, expert_info)
    _check_bit(bit, (1, 2, 4, 8))
    n_exp = expert_info.shape[0]
    if tt is None:
        tt = pick_tt(rows_total, n_exp)
    if tiling is None:
        tiling = build_tiles(expert_info, rows_total, item_tile_rows or 16 * tt)
    n_items, items, max_items = tiling
    if out is None:
        if epi == EPI_SCATTER:
            raise ValueError("scatter epilogue needs a caller-provided fp16 slot buffer")
        out = torch.empty((rows_total, n_out), dtype=torch.float16, device=act.device)
        out_stride = n_out
    pool = gemm_pool(mode, bit, act, act_scale, w, norms, lut, expert_info, row_index, w_scale_byte)
    return matmul_pools(mode, epi, [pool], items, n_items, max_items, groups=groups, n_out=n_out,
                        slice_is_groups=slice_is_groups, tt=tt, ks=ks, nbl=nbl, out=out,
                        out_stride=out_stride if out_stride is not None else out.stride(0),
                        half_width=half_width, row_weight=row_weight, row_slot=row_slot,
                        dbg_acc=dbg_acc, post=post, k_split=k_split, rows_total=rows_total,
                        item_tile_rows=item_tile_rows, split_ws=split_ws, nt=nt, roomy=roomy, spread=spread, widths_apart=widths_apart,
                        gemv=gemv, gemv_planes=gemv_planes)


def linear_gemm_i8(x_i8: torch.Tensor, x_scale: torch.Tensor, indices_gf: torch.Tensor,
                   norms_gf: torch.Tensor) -> torch.Tensor:
    """int8 GEMM of a Linear whose 8-bit weights are idx - 128 (uniform codebook): x_i8 [rows, K]
    int8 with fp16 scales [rows, K/128] (codebook step folded in), indices_gf u8 [G, N, 128],
    norms_gf fp16 [G, N] pre-scaled -> fp16 [rows, N]."""
    _need_cuda(x_i8, x_scale, indices_gf, norms_gf)
    rows, k = x_i8.shape
    g, n, _ = indices_gf.shape
    if x_scale.dtype != torch.float16 or norms_gf.dtype != torch.float16:
        raise TypeError("x_scale and norms_gf must be fp16")
    out = torch.empty((rows, n), dtype=torch.float16, device=x_i8.device)
    check(load().dmq_linear_gemm_i8(_ptr(x_i8), x_i8.stride(0), _ptr(x_scale), x_scale.stride(0),
                                    _ptr(indices_gf), _ptr(norms_gf), rows, k, n, _ptr(out), n,
                                    _stream(x_i8.device)), "linear_gemm_i8")
    return out


def combine_slots(slots: torch.Tensor, top_k: int, add: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = fp16(sum_j slots[t*k + j] (+ add[t])), slots fp16 [T*k, H], summed in fp32."""
    _need_cuda(slots)
    if slots.dtype != torch.float16:
        raise TypeError("slots must be float16")
    rows, hidden = slots.shape
    tokens = rows // top_k
    out = torch.empty((tokens, hidden), dtype=torch.float16, device=slots.device)
    check(load().dmq_combine_slots(_ptr(slots), top_k, _ptr(add), tokens, hidden, _ptr(out),
                                   _stream(slots.device)), "combine_slots")
    return out


def finalize_f16(acc32: torch.Tensor, add: torch.Tensor | None = None) -> torch.Tensor:
    _need_cuda(acc32)
    out = torch.empty(acc32.shape, dtype=torch.float16, device=acc32.device)
    check(load().dmq_finalize_f16(_ptr(acc32), _ptr(add), acc32.numel(), _ptr(out),
                                  _stream(acc32.device)), "finalize_f16")
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """out = x * rsqrt(mean(x^2, -1) + eps) * (1 + weight) in fp32, rounded once to x.dtype
    (fp16 or bf16).  Rows may be strided (a chunk view) as long as their elements are contiguous."""
    _need_cuda(x, weight)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("rms_norm takes fp16 or bf16 activations")
    n = x.shape[-1]
    if x.stride(-1) != 1:
        x = x.contiguous()
    x2 = x.reshape(-1, n) if x.is_contiguous() else x
    if x2.dim() != 2:
        x2 = x.contiguous().reshape(-1, n)
    if weight.dtype not in (x.dtype, torch.float32):
        weight = weight.float()
    weight = weight.contiguous()
    if weight.numel() != n:
        raise ValueError("weight must hold one value per feature")
    out = torch.empty((x2.shape[0], n), dtype=x.dtype, device=x.device)
    check(load().dmq_rms_norm(_ptr(x2), int(x.dtype == torch.bfloat16), _ptr(weight),
                              int(weight.dtype == torch.float32), x2.shape[0], n, x2.stride(0), n,
                              float(eps), _ptr(out), _stream(x.device)), "rms_norm")
    return out.reshape(x.shape)


def quantize_weights(w: torch.Tensor, rot_f32: torch.Tensor, boundaries: torch.Tensor, bit_width: int):
    """TurboQuant quantizer on the GPU: w fp16 [N, K], rot fp32 [K/128, 128, 128], boundaries fp32
    [2^bit - 1] -> (indices_packed u8 [N, K*bit/8], norms fp16 [N, K/128])."""
    _check_bit(bit_width, (1, 2, 4, 8))
    _need_cuda(w, rot_f32, boundaries)
    if w.dtype != torch.float16:
        w = w.half()
    w = w.contiguous()
    n, k = w.shape
    groups = k // GROUP_SIZE
    if k != groups * GROUP_SIZE:
        raise ValueError(f"K ({k}) must be a multiple of {GROUP_SIZE}")
    rot_f32 = rot_f32.float().contiguous()
    boundaries = boundaries.float().contiguous()
    if tuple(rot_f32.shape) != (groups, GROUP_SIZE, GROUP_SIZE):
        raise ValueError(f"rot must be {(groups, GROUP_SIZE, GROUP_SIZE)}, got {tuple(rot_f32.shape)}")
    if boundaries.numel() != (1 << bit_width) - 1:
        raise ValueError(f"{(1 << bit_width) - 1} boundaries expected, got {boundaries.numel()}")
    idx = torch.empty((n, k * bit_width // 8), dtype=torch.uint8, device=w.device)
    norms = torch.empty((n, groups), dtype=torch.float16, device=w.device)
    check(load().dmq_quantize_weights(_ptr(w), w.stride(0), _ptr(rot_f32), _ptr(boundaries), n, groups,
                                      bit_width, _ptr(idx), _ptr(norms), _stream(w.device)),
          "quantize_weights")
    return idx, norms
