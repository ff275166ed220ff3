"""TurboQuant weight quantizer on the GPU.

Mirror of turboquant_quantize_packed_full (turboquant_utils/quantize.py:350-474) for the "qr"
rotation and group size 128: the reference loops over groups with torch ops (normalise, rotate
with the fp32 matrix of seed + g*128, scale by sqrt(128), searchsorted against the Lloyd-Max or
uniform boundaries, pack); here one kernel does all of it for the whole matrix.  The returned
dictionary has the reference's keys, so it feeds from_packed / WxA16Linear.from_packed / the
checkpoint writer unchanged.
"""

from __future__ import annotations

import torch

from . import hostprep, ops

GROUP_SIZE = ops.GROUP_SIZE


def uniform_codebook_8bit():
    """cb[i] = (i - 128) * 3.5 / 128 and its mid-point boundaries (quantize.py:394-402)."""
    step = 3.5 / 128.0
    cents = (torch.arange(256, dtype=torch.float32) - 128) * step
    bounds = (torch.arange(255, dtype=torch.float32) - 127.5) * step
    return cents, bounds


def rotation_matrices_f32(seed: int, groups: int, device) -> torch.Tensor:
    """fp32 [groups, 128, 128]: the quantizer multiplies by the unrounded matrices
    (rotation.py:53-116), the inference path by their fp16 cast."""
    return torch.stack([hostprep.generate_rotation_matrix(GROUP_SIZE, seed + g * GROUP_SIZE)
                        for g in range(groups)], 0).to(device)


@torch.no_grad()
def turboquant_quantize_packed_full(w: torch.Tensor, bit_width: int, group_size: int = GROUP_SIZE,
                                    seed: int = 42, rotation: str = "qr",
                                    uniform_codebook: bool = False) -> dict:
    if bit_width not in (1, 2, 4, 8):
        raise ValueError(f"bit_width must be 1/2/4/8, got {bit_width}")
    if uniform_codebook and bit_width != 8:
        raise ValueError(f"uniform_codebook needs bit_width 8, got {bit_width}")
    if group_size != GROUP_SIZE:
        raise ValueError(f"group_size must be {GROUP_SIZE}, got {group_size}")
    if rotation != "qr":
        raise ValueError(f"rotation must be 'qr', got {rotation!r}")
    if not w.is_cuda:
        raise RuntimeError("the quantizer runs on the GPU only (no CPU fallback)")
    n, k = w.shape
    if k % group_size:
        raise ValueError(f"in_features ({k}) must be a multiple of group_size ({group_size})")
    cents, bounds = uniform_codebook_8bit() if uniform_codebook else hostprep.get_codebook(bit_width)
    rot = rotation_matrices_f32(int(seed), k // group_size, w.device)
    idx, norms = ops.quantize_weights(w, rot, bounds.to(w.device), bit_width)
    if norms.shape[1] == 1:
        norms = norms[:, 0].contiguous()              # one group: [N], as quantize.py:449 returns it
    return {"indices_packed": idx, "codebook": cents.half(), "norms": norms, "seed": int(seed),
            "group_size": group_size, "shape": (n, k), "bit_width": bit_width, "rotation": rotation,
            "orig_dtype": str(w.dtype), "codebook_type": "uniform" if uniform_codebook else "lloydmax"}
