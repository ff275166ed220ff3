"""Codebook -> low-precision LUT builders (oracle; test infrastructure only).

Each builder factors the fp16 codebook as ``cb[i] ~= lut[i] * scale`` so the
GEMM can run on integer / fp8 / fp4 matrix cores:

* int8   turboquant_utils/triton_kernels_a8.py:526-550
* e4m3   turboquant_utils/triton_kernels_fp8.py:35-87
* e2m1   turboquant_utils/triton_kernels_fp4.py:32-77, fold :80-122
"""

from __future__ import annotations

import math

import torch

from .packing import unpack_nbit

E4M3_MAX = 448.0
E2M1_GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
E2M1_MAX = 6.0


def build_int8_codebook(codebook: torch.Tensor):
    """(cb_i8 int8 [L], cb_step float): cb ~= cb_i8 * cb_step, cb_step = max|cb|/127.

    Reference: triton_kernels_a8.py:543-550 (round half to even, clamp +-127).
    """
    cb = codebook.float()
    top = cb.abs().max()
    if top <= 0:
        raise ValueError("all-zero codebook cannot be converted to int8")
    step = (top / 127.0).item()
    q = (cb / step).round().clamp_(-127, 127).to(torch.int8)
    return q.contiguous(), step


def _relerr(cb: torch.Tensor, rec: torch.Tensor) -> float:
    return ((rec - cb).norm() / cb.norm()).item()


def build_fp8_codebook(codebook: torch.Tensor, n_coarse: int = 512):
    """(cb_e4m3 float8_e4m3fn [L], cb_scale float): cb ~= cb_e4m3 * cb_scale.

    Scale search of triton_kernels_fp8.py:35-87: a log grid of ``n_coarse``
    points over one decade either side of max|cb|/448 (torch.logspace in fp32),
    then two refinement rounds of 64 points spanning sqrt / fourth root of the
    coarse ratio around the incumbent; strict ``<`` keeps the first minimum.
    """
    cb = codebook.float()
    top = cb.abs().max()
    if top <= 0:
        raise ValueError("all-zero codebook cannot be converted to fp8")

    def lut_at(s: float) -> torch.Tensor:
        return (cb / s).clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)

    def err_at(s: float) -> float:
        return _relerr(cb, lut_at(s).float() * s)

    s0 = (top / E4M3_MAX).item()
    centre = torch.log10(torch.tensor(s0))
    coarse = torch.logspace(centre - 1.0, centre + 1.0, n_coarse).tolist()
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


def _fit_e2m1(cb: torch.Tensor, s, grid: torch.Tensor):
    y = (cb / s).clamp(-E2M1_MAX, E2M1_MAX)
    mag = torch.argmin((y.abs().unsqueeze(-1) - grid).abs(), dim=-1)
    nib = ((mag & 0x7) | ((y < 0).to(torch.uint8) << 3).long()).to(torch.uint8)
    rec = grid[mag] * y.sign() * s
    return nib, _relerr(cb, rec)


def build_e2m1_codebook(codebook: torch.Tensor):
    """(nib u8 [L], E0 int, residual float, relerr): cb ~= e2m1(nib) * 2^E0 * residual.

    Reference: triton_kernels_fp4.py:32-77.  Coarse sweep s0 * 2^(i/16) for
    i in [-16, 16], then two rounds of 65 log-spaced points across
    [best / 2^(1/16), best * 2^(1/16)].  argmin ties resolve to the smaller
    magnitude; nib = sign << 3 | magnitude index.
    """
    cb = codebook.float()
    top = cb.abs().max()
    if top <= 0:
        raise ValueError("all-zero codebook cannot be converted to e2m1")
    grid = torch.tensor(E2M1_GRID)
    s0 = top / E2M1_MAX
    best_s, best_e, best_nib = s0, float("inf"), None
    for s in [s0 * (2.0 ** (i / 16.0)) for i in range(-16, 17)]:
        nib, e = _fit_e2m1(cb, s, grid)
        if e < best_e:
            best_s, best_e, best_nib = s, e, nib
    for _ in range(2):
        span = 2.0 ** (1 / 16)
        lo, hi = best_s / span, best_s * span
        for s in [lo * (hi / lo) ** (i / 64.0) for i in range(65)]:
            nib, e = _fit_e2m1(cb, s, grid)
            if e < best_e:
                best_s, best_e, best_nib = s, e, nib
    e0 = math.floor(math.log2(best_s))
    residual = float(best_s / (2.0 ** e0))
    return best_nib.contiguous(), int(e0), residual, best_e


def e2m1_value(nib: torch.Tensor) -> torch.Tensor:
    """Decode e2m1 nibbles (sign<<3 | mag) to fp32."""
    grid = torch.tensor(E2M1_GRID)
    mag = grid[(nib & 0x7).long()]
    return torch.where((nib & 0x8) != 0, -mag, mag)


def fold_indices_to_e2m1(indices_gf: torch.Tensor, nib: torch.Tensor,
                         bit_width: int, group_size: int) -> torch.Tensor:
    """[G, N, gs*bit/8] codebook indices -> [G, N, gs/2] packed e2m1 bytes.

    byte j of a row holds nib[idx[2j]] | nib[idx[2j+1]] << 4
    (triton_kernels_fp4.py:80-122).
    """
    if bit_width not in (1, 2, 4):
        raise ValueError(f"fold supports bit 1/2/4, got {bit_width}")
    g, n, _ = indices_gf.shape
    idx = unpack_nbit(indices_gf, bit_width, group_size).long()      # [G, N, gs]
    nb = nib[idx]
    return (nb[..., 0::2] | (nb[..., 1::2] << 4)).to(torch.uint8).contiguous()
