"""TurboQuant weight quantizer / dequantizer (oracle; test infrastructure only).

Weight model for W[N, K] with groups of ``gs`` columns (Appendix of the
reference's quantize.py):

    norm[n, g] = max(||W[n, g]||_2, 1e-8)
    Y          = (W[n, g] / norm) @ P_g^T * sqrt(gs)          P_g: seed + g*gs
    idx        = clamp(searchsorted(boundaries, Y), 0, L-1)
    W~[n, g]   = norm * (cb[idx] / sqrt(gs)) @ P_g

Reference: turboquant_utils/quantize.py:350-474 (quantize) and :478-826
(dequantize, row slice, column slice).
"""

from __future__ import annotations

import math

import torch

from .codebook import get_codebook, uniform_codebook_8bit
from .packing import pack_nbit, unpack_nbit, _check_bit
from .rotation import rotation_matrix


def quantize_packed(w: torch.Tensor, bit_width: int, group_size: int | None = None,
                    seed: int = 42, uniform_codebook: bool = False) -> dict:
    """Quantize W[N, K] and return the packed dictionary the reference stores.

    Keys mirror turboquant_quantize_packed_full (quantize.py:461-472):
    indices_packed u8 [N, K*bit/8], codebook fp16 [2^bit], norms fp16 [N, G],
    seed, group_size, shape, bit_width, rotation, orig_dtype, codebook_type.
    """
    _check_bit(bit_width)
    if uniform_codebook and bit_width != 8:
        raise ValueError("uniform_codebook is only defined for bit_width == 8")
    n_rows, k = w.shape
    gs = k if group_size is None else int(group_size)
    if uniform_codebook:
        cents, bounds = uniform_codebook_8bit()
        cb_type = "uniform"
    else:
        cents, bounds = get_codebook(bit_width)
        cb_type = "lloydmax"

    norms_cols, idx_cols = [], []
    for g0 in range(0, k, gs):
        g1 = min(g0 + gs, k)
        d = g1 - g0
        wg = w[:, g0:g1].float()
        nrm = wg.norm(dim=1, keepdim=True).clamp(min=1e-8)          # quantize.py:416
        p = rotation_matrix(d, seed + g0)                           # quantize.py:427
        y = (wg / nrm) @ p.T * math.sqrt(d)                         # quantize.py:428-432
        idx = torch.searchsorted(bounds, y.reshape(-1)).clamp(0, cents.numel() - 1)
        idx_cols.append(idx.reshape(n_rows, d).to(torch.uint8))
        norms_cols.append(nrm.squeeze(1))

    full_idx = torch.cat(idx_cols, dim=1)
    norms = torch.stack(norms_cols, dim=1) if len(norms_cols) > 1 else norms_cols[0]
    return {
        "indices_packed": pack_nbit(full_idx, bit_width),
        "codebook": cents.half(),
        "norms": norms.half(),
        "seed": int(seed),
        "group_size": gs,
        "shape": (n_rows, k),
        "bit_width": bit_width,
        "rotation": "qr",
        "orig_dtype": str(w.dtype),
        "codebook_type": cb_type,
    }


def dequantize_packed(packed: dict, row_start: int = 0, row_end: int | None = None,
                      col_start: int = 0, col_end: int | None = None,
                      out_dtype: torch.dtype | None = torch.float32) -> torch.Tensor:
    """Dequantize rows [row_start,row_end) x columns [col_start,col_end).

    Covers turboquant_dequantize_packed (quantize.py:478-556), the row slice
    (:560-678) and the column slice (:682-826): whole groups overlapping the
    column window are rebuilt, then cropped.  Arithmetic is fp32; the reference
    finally casts to the original dtype, pass ``out_dtype=torch.float16`` for
    that behaviour.
    """
    n_rows, k = packed["shape"]
    gs = packed["group_size"]
    bit = packed["bit_width"]
    seed = packed["seed"]
    row_end = n_rows if row_end is None else min(row_end, n_rows)
    col_end = k if col_end is None else min(col_end, k)
    row_start, col_start = max(row_start, 0), max(col_start, 0)
    if row_start >= row_end or col_start >= col_end:
        return torch.zeros((max(row_end - row_start, 0), max(col_end - col_start, 0)),
                           dtype=out_dtype or torch.float32)
    cb = packed["codebook"].float()
    norms = packed["norms"].float()
    if norms.dim() == 1:
        norms = norms.unsqueeze(1)
    # only the bytes of the groups that overlap the column window are unpacked (the reference
    # unpacks the whole matrix first, :733: same values, a pool-sized temporary per call)
    g_first = (col_start // gs) * gs
    g_last = min(-(-col_end // gs) * gs, k)
    epb = 8 // bit
    idx = unpack_nbit(packed["indices_packed"][row_start:row_end, g_first // epb:-(-g_last // epb)],
                      bit, g_last - g_first).long()
    norms = norms[row_start:row_end]
    out = torch.zeros((row_end - row_start, col_end - col_start), dtype=torch.float32)
    for g0 in range(g_first, col_end, gs):
        g1 = min(g0 + gs, k)
        d = g1 - g0
        p = rotation_matrix(d, seed + g0)
        wg = (cb[idx[:, g0 - g_first:g1 - g_first]] / math.sqrt(d)) @ p * norms[:, g0 // gs].unsqueeze(1)
        lo, hi = max(col_start, g0), min(col_end, g1)
        out[:, lo - col_start:hi - col_start] = wg[:, lo - g0:hi - g0]
    return out if out_dtype is None else out.to(out_dtype)


def rotated_space_weights(packed: dict, row_start: int = 0, row_end: int | None = None,
                          group_start: int = 0, group_end: int | None = None) -> torch.Tensor:
    """cb[idx] * norm / sqrt(gs) without the inverse rotation, fp32 [rows, groups*gs].

    This is the matrix the fused kernels contract the *rotated* activation with:
    y[b, n] = sum_g (norm[n,g]/sqrt(gs)) * sum_k xrot[b,g,k] * cb[idx[n,g,k]]
    (turboquant_utils/triton_kernels.py:893-991).
    """
    n_rows, k = packed["shape"]
    gs = packed["group_size"]
    row_end = n_rows if row_end is None else row_end
    groups = k // gs
    group_end = groups if group_end is None else group_end
    idx = unpack_nbit(packed["indices_packed"][row_start:row_end], packed["bit_width"], k).long()
    idx = idx[:, group_start * gs:group_end * gs]
    cb = packed["codebook"].float()
    norms = packed["norms"].float()[row_start:row_end, group_start:group_end]
    w = cb[idx].reshape(idx.shape[0], group_end - group_start, gs)
    w = w * (norms / math.sqrt(gs)).unsqueeze(-1)
    return w.reshape(idx.shape[0], -1)
