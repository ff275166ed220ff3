"""ctypes binding of libdartmoq_hip.so (the C ABI declared in include/dartmoq_hip.h).

The library is built in-tree by ``make -C dartmoq-qwen3.5_amd`` (hipcc, gfx950).  There is
no CPU fallback: a missing library raises on first use.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_long, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdartmoq_hip.so")

OK = 0
ABI_VERSION = 21
MAX_POOLS = 4
MODE_A16, MODE_A8, MODE_FP8, MODE_FP4 = 0, 1, 2, 3
EPI_STORE, EPI_SILU, EPI_SCATTER, EPI_SILU_ROT = 0, 1, 2, 3
MODE_BY_NAME = {"wxa16": MODE_A16, "wxa8": MODE_A8, "wxfp8": MODE_FP8, "wxfp4": MODE_FP4}

# status -> exception type, mirroring the reference wrappers (ValueError for bad bit widths,
# misaligned slices and inconsistent shapes; see turboquant_utils/triton_kernels.py:1500-1519)
_EXC = {1: ValueError, 2: ValueError, 3: ValueError, 4: ValueError, 5: ValueError,
        6: TypeError, 7: RuntimeError, 8: ValueError}


class GemmPool(Structure):
    _fields_ = [
        ("w", c_void_p), ("norms", c_void_p), ("lut", c_void_p), ("expert_info", c_void_p),
        ("act", c_void_p), ("act_scale", c_void_p), ("row_index", c_void_p),
        ("n_total", c_int), ("bit", c_int), ("mode", c_int), ("w_scale_byte", c_int),
        ("col_start", c_void_p), ("home", c_void_p),
    ]


class GemmArgs(Structure):
    _fields_ = [
        ("mode", c_int), ("epi", c_int), ("tt", c_int), ("ks", c_int), ("nbl", c_int),
        ("n_pools", c_int),
        ("pool", GemmPool * MAX_POOLS),
        ("act_row_bytes", c_long), ("act_scale_stride", c_int),
        ("groups", c_int), ("n_out", c_int), ("half_width", c_int), ("slice_is_groups", c_int),
        ("items", c_void_p), ("n_items", c_void_p), ("max_items", c_int),
        ("out", c_void_p), ("out_stride", c_long),
        ("row_weight", c_void_p), ("row_slot", c_void_p), ("dbg_acc", c_void_p),
        ("post_rot", c_void_p * MAX_POOLS), ("post_extra_scale", c_float * MAX_POOLS),
        ("post_out", c_void_p), ("post_row_bytes", c_long),
        ("post_scale", c_void_p), ("post_scale_stride", c_int),
        ("k_split", c_int), ("split_rows", c_int), ("split_partial", c_void_p), ("split_counter", c_void_p),
        ("item_tile_rows", c_int),
        ("nt", c_int),
        ("width_filter", c_int), ("home_filter", c_int), ("accumulate", c_int), ("roomy", c_int), ("spread", c_int), ("mode2_on", c_int), ("mode2", c_int), ("widths_apart", c_int),
        ("rows_queue", c_void_p), ("k_split_items", c_int), ("gemv", c_int), ("gemv_planes", c_int),
    ]


class PoolDesc(Structure):
    _fields_ = [
        ("bit", c_int), ("mode", c_int), ("major", c_int), ("n_gate_up", c_int),
        ("down_groups", c_int),
        ("gu_w", c_void_p), ("gu_norms", c_void_p), ("gu_lut", c_void_p), ("gu_rot", c_void_p),
        ("gu_extra_scale", c_float), ("gu_w_scale_byte", c_int),
        ("dn_w", c_void_p), ("dn_norms", c_void_p), ("dn_lut", c_void_p), ("dn_rot", c_void_p),
        ("dn_extra_scale", c_float), ("dn_w_scale_byte", c_int),
    ]


class LinearDesc(Structure):
    _fields_ = [
        ("mode", c_int), ("bit", c_int), ("in_features", c_int), ("out_features", c_int),
        ("indices_gf", c_void_p), ("norms_gf", c_void_p), ("lut", c_void_p), ("rot", c_void_p),
        ("extra_scale", c_float),
    ]


class LayerDesc(Structure):
    _fields_ = [
        ("hidden", c_int), ("inter", c_int), ("experts", c_int), ("top_k", c_int), ("pools", c_int),
        ("pool", POINTER(PoolDesc)), ("slice_start", c_void_p), ("slice_count", c_void_p),
        ("n_widths", c_int), ("widths", c_int * 8), ("max_homes", c_int),
        ("col_start", c_void_p), ("home", c_void_p),
    ]


class RouterArgs(Structure):
    _fields_ = [
        ("logits", c_void_p), ("logits_fp16", c_int), ("renorm", c_int),
        ("topk_idx", c_void_p), ("topk_w", c_void_p),
        ("shared_gate_row", c_void_p), ("n_shared", c_int),
    ]


class PrenormArgs(Structure):
    _fields_ = [
        ("norm_weight", c_void_p), ("norm_weight_fp32", c_int), ("eps", ctypes.c_float),
        ("gate_weight", c_void_p), ("state", c_void_p), ("x_norm_out", c_void_p),
        ("logits_out", c_void_p),
    ]


# name -> (restype, argtypes); the single source for the symbol-export test as well
PROTOTYPES = {
    "dmq_abi_version": (c_int, []),
    "dmq_status_string": (c_char_p, [c_int]),
    "dmq_unpack_nbit": (c_int, [c_void_p, c_long, c_int, c_void_p, c_void_p]),
    "dmq_convert_to_group_first": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                           c_void_p, c_void_p]),
    "dmq_dequant_tile": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                 c_int, c_void_p, c_void_p]),
    "dmq_fold_indices_to_e2m1": (c_int, [c_void_p, c_void_p, c_long, c_int, c_void_p, c_void_p]),
    "dmq_route_topk": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                               c_void_p]),
    "dmq_route_topk_shared": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                      c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "dmq_route_permute": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                  c_int, c_int] + [c_void_p] * 10 + [c_size_t, c_void_p]),
    "dmq_route_scratch_bytes": (c_size_t, [c_int, c_int, c_int]),
    "dmq_route_permute_static": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                         c_int, c_int] + [c_void_p] * 10),
    "dmq_build_tiles": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "dmq_rotate": (c_int, [c_int, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p,
                           c_long, c_void_p, c_int, c_int, c_float, c_int, c_void_p]),
    "dmq_rotate_tiled": (c_int, [c_int, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                 c_void_p, c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_int,
                                 c_int, c_float, c_int, c_void_p]),
    "dmq_quantize_act": (c_int, [c_int, c_void_p, c_int, c_long, c_int, c_int, c_void_p, c_long,
                                 c_void_p, c_int, c_int, c_float, c_void_p]),
    "dmq_matmul_merged_gf": (c_int, [POINTER(GemmArgs), c_void_p]),
    "dmq_combine_slots": (c_int, [c_void_p, c_int, c_void_p, c_long, c_int, c_void_p, c_void_p]),
    "dmq_finalize_f16": (c_int, [c_void_p, c_void_p, c_long, c_void_p, c_void_p]),
    "dmq_fill_zero": (c_int, [c_void_p, c_long, c_void_p]),
    "dmq_quantize_weights": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p,
                                     c_void_p, c_void_p]),
    "dmq_rms_norm": (c_int, [c_void_p, c_int, c_void_p, c_int, c_long, c_int, c_long, c_long, c_float,
                             c_void_p, c_void_p]),
    "dmq_linear_workspace_bytes": (c_size_t, [POINTER(LinearDesc), c_int]),
    "dmq_linear_uses_i8_gemm": (c_int, [POINTER(LinearDesc), c_int]),
    "dmq_linear_gemm_i8": (c_int, [c_void_p, c_long, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                                   c_int, c_void_p, c_long, c_void_p]),
    "dmq_linear_forward": (c_int, [POINTER(LinearDesc), c_void_p, c_long, c_int, c_void_p, c_long,
                                   c_void_p, c_size_t, c_void_p]),
    "dmq_moe_workspace_bytes": (c_size_t, [POINTER(LayerDesc), c_int]),
    "dmq_moe_ffn_forward": (c_int, [POINTER(LayerDesc), c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                    c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_void_p]),
    "dmq_moe_ffn_forward_staged": (c_int, [POINTER(LayerDesc), c_void_p, c_void_p, c_void_p, c_int,
                                           c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int,
                                           c_int, POINTER(c_void_p), POINTER(c_long), c_void_p]),
    "dmq_moe_ffn_forward_routed": (c_int, [POINTER(LayerDesc), POINTER(RouterArgs), c_void_p, c_int,
                                           c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int,
                                           c_int, POINTER(c_void_p), POINTER(c_long), c_void_p]),
    "dmq_moe_ffn_forward_prenorm": (c_int, [POINTER(LayerDesc), POINTER(RouterArgs), POINTER(PrenormArgs),
                                            c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t,
                                            c_int, c_int, c_int, POINTER(c_void_p), POINTER(c_long),
                                            c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(_HERE)}` "
                "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.dmq_abi_version() != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI {lib.dmq_abi_version()}, expected {ABI_VERSION}: rebuild")
        _lib = lib
    return _lib


def check(status: int, what: str = ""):
    if status != OK:
        msg = load().dmq_status_string(status).decode()
        raise _EXC.get(status, RuntimeError)(f"dartmoq_hip {what}: {msg} (status {status})")
