"""Per-token activation quantizers (oracle; test infrastructure only).

Inputs are *already rotated* activations.  Three codes:

* int8 per 128 : turboquant_utils/triton_kernels_a8.py:384-421
* e4m3 per 128 : turboquant_utils/triton_kernels_fp8.py:94-124
* e2m1 per 32 + e8m0 scale : turboquant_utils/triton_kernels_fp4.py:125-150

All arithmetic is IEEE fp32 (division, round half to even) exactly as the
torch expressions of the reference evaluate on a CPU.
"""

from __future__ import annotations

import torch

from .luts import E2M1_GRID, E2M1_MAX, E4M3_MAX


def quantize_act_int8(x_rot: torch.Tensor, group_size: int, extra_scale: float = 1.0):
    """(q int8 [B, K], scale fp32 [B, K/gs]).

    scale = max(amax/127, 1e-8); q = clamp(rne(x/scale), -127, 127); the
    returned scale is multiplied by ``extra_scale`` (the codebook step) after
    the division (triton_kernels_a8.py:415-421).
    """
    b, k = x_rot.shape
    if k % group_size:
        raise ValueError(f"K ({k}) must be a multiple of group_size ({group_size})")
    xg = x_rot.reshape(b, k // group_size, group_size).float()
    scale = (xg.abs().amax(dim=-1) / 127.0).clamp(min=1e-8)
    q = (xg / scale.unsqueeze(-1)).round().clamp_(-127, 127).to(torch.int8)
    if extra_scale != 1.0:
        scale = scale * extra_scale
    return q.reshape(b, k).contiguous(), scale.contiguous()


def quantize_act_fp8(x_rot: torch.Tensor, group_size: int, extra_scale: float = 1.0):
    """(q float8_e4m3fn [B, K], scale fp32 [B, K/gs]); saturating at +-448.

    Reference: triton_kernels_fp8.py:115-124.
    """
    b, k = x_rot.shape
    if k % group_size:
        raise ValueError(f"K ({k}) must be a multiple of group_size ({group_size})")
    xg = x_rot.reshape(b, k // group_size, group_size).float()
    scale = (xg.abs().amax(dim=-1) / E4M3_MAX).clamp(min=1e-8)
    q = (xg / scale.unsqueeze(-1)).clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    if extra_scale != 1.0:
        scale = scale * extra_scale
    return q.reshape(b, k).contiguous(), scale.contiguous()


def quantize_act_e2m1(x_rot: torch.Tensor):
    """(packed u8 [B, K/2], scale_byte u8 [B, K/32]); MX blocks of 32.

    e = ceil(log2(max(amax, 1e-30) / 6)); byte = clamp(e + 127, 0, 254);
    y = clamp(x / 2^e, -6, 6); magnitude = argmin |grid - |y|| (ties -> the
    smaller magnitude); nibble = magnitude | (y < 0) << 3; even k in the low
    nibble (triton_kernels_fp4.py:138-150).
    """
    b, k = x_rot.shape
    if k % 32:
        raise ValueError(f"K ({k}) must be a multiple of 32")
    xb = x_rot.float().reshape(b, k // 32, 32)
    amax = xb.abs().amax(dim=-1, keepdim=True).clamp(min=1e-30)
    e = torch.ceil(torch.log2(amax / E2M1_MAX))
    s = torch.pow(2.0, e).clamp(min=1e-30)
    scale_b = (e + 127.0).clamp(0, 254).to(torch.uint8).reshape(b, k // 32)
    y = (xb / s).clamp(-E2M1_MAX, E2M1_MAX)
    grid = torch.tensor(E2M1_GRID)
    mag = torch.argmin((y.abs().unsqueeze(-1) - grid).abs(), dim=-1)
    nib = ((mag & 0x7).to(torch.uint8) | ((y < 0).to(torch.uint8) << 3)).reshape(b, k)
    packed = nib[:, 0::2] | (nib[:, 1::2] << 4)
    return packed.contiguous(), scale_b.contiguous()


def dequant_act_e2m1(packed: torch.Tensor, scale_b: torch.Tensor) -> torch.Tensor:
    """Inverse map of quantize_act_e2m1 to fp32 [B, K] (for error measurements)."""
    b, kh = packed.shape
    nib = torch.stack([packed & 0xF, packed >> 4], dim=-1).reshape(b, kh * 2)
    grid = torch.tensor(E2M1_GRID)
    val = grid[(nib & 7).long()]
    val = torch.where((nib & 8) != 0, -val, val)
    scale = torch.pow(2.0, scale_b.float() - 127.0).repeat_interleave(32, dim=1)
    return val * scale
