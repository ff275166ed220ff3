"""n-bit index packing and the group-first weight layout (oracle; test only).

Packing rule (turboquant_utils/quantize.py:35-100): element i of the last axis
lives in byte i // epb at bit offset (i % epb) * bit, epb = 8 // bit, i.e. the
first element of a byte occupies its least significant bits.
"""

from __future__ import annotations

import numpy as np
import torch

SUPPORTED_BITS = (1, 2, 4, 8)


def _check_bit(bit_width: int):
    if bit_width not in SUPPORTED_BITS:
        raise ValueError(f"bit_width must be one of {SUPPORTED_BITS}, got {bit_width}")


def pack_nbit(indices: torch.Tensor, bit_width: int) -> torch.Tensor:
    """Pack integer indices (..., N) into uint8 (..., ceil(N/epb)).

    Reference: turboquant_utils/quantize.py:35-71 (tail padded with zeros).
    """
    _check_bit(bit_width)
    epb = 8 // bit_width
    n = indices.shape[-1]
    pad = (-n) % epb
    idx = indices.to(torch.int64)
    if pad:
        idx = torch.nn.functional.pad(idx, (0, pad))
    lanes = idx.reshape(*idx.shape[:-1], -1, epb) & ((1 << bit_width) - 1)
    shifts = torch.arange(epb, dtype=torch.int64) * bit_width
    return (lanes << shifts).sum(dim=-1).to(torch.uint8)


def unpack_nbit(packed: torch.Tensor, bit_width: int, n: int) -> torch.Tensor:
    """Inverse of pack_nbit; returns int32 (..., n).

    Reference: turboquant_utils/quantize.py:74-100.
    """
    _check_bit(bit_width)
    epb = 8 // bit_width
    shifts = torch.arange(epb, dtype=torch.int32) * bit_width
    vals = (packed.to(torch.int32).unsqueeze(-1) >> shifts) & ((1 << bit_width) - 1)
    return vals.reshape(*packed.shape[:-1], -1)[..., :n].contiguous()


def unpack_nbit_np(packed: np.ndarray, bit_width: int) -> np.ndarray:
    """numpy twin of unpack_nbit over a flat byte array (all elements kept)."""
    _check_bit(bit_width)
    epb = 8 // bit_width
    shifts = (np.arange(epb) * bit_width).astype(np.uint8)
    vals = (packed[..., None] >> shifts) & np.uint8((1 << bit_width) - 1)
    return vals.reshape(*packed.shape[:-1], -1)


def convert_to_group_first(indices_packed: torch.Tensor, norms: torch.Tensor,
                           group_size: int, bit_width: int):
    """Row-major packed weights -> group-first layout.

    indices_packed [N, G*ppg] -> indices_gf [G, N, ppg]; norms [N, G] -> [G, N].
    Reference: turboquant_utils/triton_kernels.py:1042-1069.
    """
    _check_bit(bit_width)
    ppg = group_size // (8 // bit_width)
    n_rows, packed_k = indices_packed.shape
    groups = packed_k // ppg
    idx_gf = indices_packed.reshape(n_rows, groups, ppg).permute(1, 0, 2).contiguous()
    norms_gf = norms.t().contiguous()
    return idx_gf, norms_gf
