"""Seeded Haar rotations for the block-QR scheme (oracle; test only).

Recipe (turboquant_utils/rotation.py:53-116): a CPU ``torch.Generator`` seeded
with ``seed`` draws a d x d standard normal matrix, ``torch.linalg.qr`` factors
it and every column of Q is multiplied by the sign of the matching diagonal
entry of R.  Matrices are always produced on the CPU so the quantizer and the
inference side see identical values.
"""

from __future__ import annotations

import torch

_CACHE: dict[tuple[int, int], torch.Tensor] = {}


def rotation_matrix(d: int, seed: int) -> torch.Tensor:
    """fp32 [d, d] orthogonal matrix for (d, seed).  rotation.py:53-116."""
    key = (int(d), int(seed))
    hit = _CACHE.get(key)
    if hit is not None:
        return hit
    gen = torch.Generator().manual_seed(int(seed))
    gauss = torch.randn(d, d, generator=gen)
    q, r = torch.linalg.qr(gauss)
    q = q * torch.sign(torch.diag(r)).unsqueeze(0)
    if len(_CACHE) >= 8192:
        _CACHE.pop(next(iter(_CACHE)))
    _CACHE[key] = q
    return q


def batch_rotation_matrices(d: int, seed_base: int, num_groups: int, stride: int,
                            dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """[num_groups, d, d]; group i uses seed_base + i*stride.  rotation.py:127-173."""
    mats = [rotation_matrix(d, seed_base + i * stride).to(dtype) for i in range(num_groups)]
    return torch.stack(mats, 0).contiguous()


def batch_rotate_input(x: torch.Tensor, group_size: int, seed_base: int,
                       out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x[B, K] -> x_rot[B, K], x_rot[:, g] = x[:, g] @ P_g^T  (rotation.py:176-212).

    The reference multiplies in the activation dtype (fp16 bmm) and returns that
    dtype.  Here the product is formed in fp32 from the fp16-rounded matrices
    and rounded once to ``out_dtype`` (default: dtype of x), which is what an
    fp32-accumulating matrix unit produces.
    """
    b, k = x.shape
    g = k // group_size
    mats = batch_rotation_matrices(group_size, seed_base, g, group_size, dtype=x.dtype)
    return rotate_with(x, mats, out_dtype)


def rotate_with(x: torch.Tensor, mats: torch.Tensor,
                out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Apply explicit per-group matrices: out[b, g, j] = sum_k x[b, g, k] * mats[g, j, k]."""
    b, k = x.shape
    g, d, _ = mats.shape
    xg = x.float().reshape(b, g, d).transpose(0, 1)           # [g, b, d]
    yr = torch.bmm(xg, mats.float().transpose(1, 2))          # [g, b, d]
    y = yr.transpose(0, 1).reshape(b, k)
    return y.to(out_dtype if out_dtype is not None else x.dtype).contiguous()
