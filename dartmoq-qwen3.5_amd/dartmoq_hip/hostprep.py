"""Load-time host preparation: rotation matrices and codebook look-up tables.

These run once per checkpoint on the CPU with torch, exactly where the reference runs them
(rotation matrices are always generated on the CPU so that quantizer and inference agree,
turboquant_utils/rotation.py:78-80).  Nothing here is on the per-token path.
"""

from __future__ import annotations

import math

import torch

E4M3_MAX = 448.0
E2M1_GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
FP4_BITS = (1, 4)            # pools that run on the MX fp4 path in wxfp4 mode (bit 2 stays int8)

_ROT_CACHE: dict[tuple[int, int], torch.Tensor] = {}
_BATCH_CACHE: dict[tuple, torch.Tensor] = {}


def generate_rotation_matrix(d: int, seed: int = 42) -> torch.Tensor:
    """Haar orthogonal matrix: QR of a seeded CPU Gaussian, columns signed by diag(R).

    Same recipe as turboquant_utils/rotation.py:53-116.
    """
    key = (int(d), int(seed))
    q = _ROT_CACHE.get(key)
    if q is None:
        g = torch.randn(d, d, generator=torch.Generator().manual_seed(int(seed)))
        q, r = torch.linalg.qr(g)
        q = q * torch.sign(torch.diag(r)).unsqueeze(0)
        if len(_ROT_CACHE) >= 4096:
            _ROT_CACHE.pop(next(iter(_ROT_CACHE)))
        _ROT_CACHE[key] = q
    return q


def generate_batch_rotation_matrices(d: int, seed_base: int, num_groups: int, stride: int,
                                     device=None, dtype=torch.float16) -> torch.Tensor:
    """[num_groups, d, d], group i seeded seed_base + i*stride (rotation.py:127-173).  Batches of
    up to 64 matrices (the per-call rotations of the Linear path) are kept per device like the
    reference's batch cache; the large per-pool batches are owned by their modules instead."""
    key = (int(d), int(seed_base), int(num_groups), int(stride), str(device), str(dtype))
    hit = _BATCH_CACHE.get(key)
    if hit is not None:
        return hit
    mats = torch.stack([generate_rotation_matrix(d, seed_base + i * stride).to(dtype)
                        for i in range(num_groups)], 0).contiguous()
    if device is not None:
        mats = mats.to(device)
    if num_groups <= 64:
        if len(_BATCH_CACHE) >= 512:
            _BATCH_CACHE.pop(next(iter(_BATCH_CACHE)))
        _BATCH_CACHE[key] = mats
    return mats


def build_int8_codebook(codebook: torch.Tensor):
    """(cb_i8, cb_step), cb ~= cb_i8 * cb_step (triton_kernels_a8.py:526-550)."""
    cb = codebook.detach().float().cpu()
    top = cb.abs().max()
    if top <= 0:
        raise ValueError("all-zero codebook cannot be converted to int8")
    step = (top / 127.0).item()
    return (cb / step).round().clamp_(-127, 127).to(torch.int8).contiguous(), step


def uniform_codebook_step(codebook: torch.Tensor) -> float:
    """Step of a uniform 256-level codebook cb[i] = (i - 128) * step, from its end points
    (quantization/wxa8/linear.py:35-47)."""
    cb = codebook.float()
    if cb.numel() != 256:
        raise ValueError(f"an 8-bit codebook has 256 levels, got {cb.numel()}")
    step = float((cb[-1] - cb[0]) / 255.0)
    if step <= 0:
        raise ValueError(f"illegal codebook step {step}")
    return step


def is_uniform_codebook(codebook: torch.Tensor, rel_tol: float = 1e-2) -> bool:
    """Constant spacing between neighbouring levels (quantization/wxa8/linear.py:50-62)."""
    if codebook.numel() != 256:
        return False
    d = codebook.float()[1:] - codebook.float()[:-1]
    mean = d.mean().abs()
    if mean <= 0:
        return False
    return bool((d - d.mean()).abs().max() < rel_tol * mean)


def build_int8_lut(codebook: torch.Tensor, round_lloyd_max_8bit: bool = False):
    """int8 look-up table and step of a codebook for the int8 path: the rounded table of
    build_int8_codebook for 1/2/4-bit codebooks; for uniform 8-bit codebooks the identity
    w = idx - 128 with the uniform step, which is what the reference's IDENTITY_CB kernels compute
    (quantization/wxa8/linear.py:130-159).  A Lloyd-Max 8-bit codebook is refused for a Linear, as
    in the reference (:79-98); the bit pools of a MoE layer pass ``round_lloyd_max_8bit``: the
    reference rounds the codebook of every pool to int8 whatever its width
    (quantization/wxa8/bit_partitioned_moe.py:78-82), levels near zero merging
    (triton_kernels_a8.py:539-542)."""
    if codebook.numel() == 256:
        if is_uniform_codebook(codebook):
            q = (torch.arange(256, dtype=torch.int16) - 128).to(torch.int8)
            return q, uniform_codebook_step(codebook)
        if not round_lloyd_max_8bit:
            raise ValueError("the int8 path takes 8-bit weights only with a uniform codebook")
    return build_int8_codebook(codebook)


def int8_lut_for_launch(codebook: torch.Tensor, device, round_lloyd_max_8bit: bool = False):
    """(table or None, step) as the int8 GEMM launches take it: 8-bit uniform codebooks pass no
    table (the kernels compute w = idx - 128 from the index bytes), everything else its rounded
    int8 table on the device."""
    q, step = build_int8_lut(codebook, round_lloyd_max_8bit)
    identity = codebook.numel() == 256 and is_uniform_codebook(codebook)
    return (None if identity else q.to(device)), step


def build_fp8_codebook(codebook: torch.Tensor, n_coarse: int = 512):
    """(cb_e4m3, cb_scale) by the log-grid scale search of triton_kernels_fp8.py:35-87."""
    cb = codebook.detach().float().cpu()
    top = cb.abs().max()
    if top <= 0:
        raise ValueError("all-zero codebook cannot be converted to fp8")

    def lut_at(s):
        return (cb / s).clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)

    def err_at(s):
        return ((lut_at(s).float() * s - cb).norm() / cb.norm()).item()

    s0 = (top / E4M3_MAX).item()
    mid = torch.log10(torch.tensor(s0))
    coarse = torch.logspace(mid - 1.0, mid + 1.0, n_coarse).tolist()
    best_s, best_e = s0, float("inf")
    for s in coarse:
        e = err_at(s)
        if e < best_e:
            best_s, best_e = s, e
    span = coarse[1] / coarse[0] if len(coarse) > 1 else 1.0
    for ratio in (span ** 0.5, span ** 0.25):
        for s in [best_s * ratio ** (i / 64.0 - 0.5) for i in range(64)]:
            e = err_at(s)
            if e < best_e:
                best_s, best_e = s, e
    return lut_at(best_s).contiguous(), best_s


def build_e2m1_codebook(codebook: torch.Tensor):
    """(nib, E0, residual, relerr), cb ~= e2m1(nib) * 2^E0 * residual (triton_kernels_fp4.py:32-77)."""
    cb = codebook.detach().float().cpu()
    top = cb.abs().max()
    if top <= 0:
        raise ValueError("all-zero codebook cannot be converted to e2m1")
    grid = torch.tensor(E2M1_GRID)

    def fit(s):
        y = (cb / s).clamp(-6.0, 6.0)
        mag = torch.argmin((y.abs().unsqueeze(-1) - grid).abs(), dim=-1)
        nib = ((mag & 7) | ((y < 0).to(torch.uint8) << 3).long()).to(torch.uint8)
        rec = grid[mag] * y.sign() * s
        return nib, ((rec - cb).norm() / cb.norm()).item()

    s0 = top / 6.0
    best_s, best_e, best_nib = s0, float("inf"), None
    for s in [s0 * (2.0 ** (i / 16.0)) for i in range(-16, 17)]:
        nib, e = fit(s)
        if e < best_e:
            best_s, best_e, best_nib = s, e, nib
    for _ in range(2):
        span = 2.0 ** (1 / 16)
        lo, hi = best_s / span, best_s * span
        for s in [lo * (hi / lo) ** (i / 64.0) for i in range(65)]:
            nib, e = fit(s)
            if e < best_e:
                best_s, best_e, best_nib = s, e, nib
    e0 = math.floor(math.log2(best_s))
    return best_nib.contiguous(), int(e0), float(best_s / (2.0 ** e0)), best_e


_CODEBOOKS: dict[int, tuple[torch.Tensor, torch.Tensor]] = {}


def get_codebook(bit_width: int):
    """Lloyd-Max centroids / interior boundaries for N(0,1) (turboquant_utils/codebook.py:18-100):
    200 Lloyd iterations from a uniform split of [-3.5, 3.5]."""
    hit = _CODEBOOKS.get(bit_width)
    if hit is not None:
        return hit
    import numpy as np
    from scipy.stats import norm
    levels = 2 ** bit_width
    edges = np.linspace(-3.5, 3.5, levels + 1)
    edges[0], edges[-1] = -1e10, 1e10
    cents = np.zeros(levels)
    for _ in range(200):
        for i in range(levels):
            lo, hi = edges[i], edges[i + 1]
            mass = norm.cdf(hi) - norm.cdf(lo)
            cents[i] = ((norm.pdf(lo) - norm.pdf(hi)) / mass if mass > 1e-15
                        else (max(lo, -3.5) + min(hi, 3.5)) / 2)
        for i in range(1, levels):
            edges[i] = (cents[i - 1] + cents[i]) / 2
    out = (torch.tensor(cents, dtype=torch.float32), torch.tensor(edges[1:-1], dtype=torch.float32))
    _CODEBOOKS[bit_width] = out
    return out
