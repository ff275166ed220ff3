"""GPU parity of the reference-named callables (dartmoq_hip.kernels) against the CPU oracle.

The weights are real TurboQuant quantizations of random matrices, so the comparison
x @ dequantize(W)^T exercises rotation seeds, slice semantics and norm scaling of every wrapper.
fp16 outputs: max |a-b| / max |b| <= 1e-2 and cosine >= 0.9999 against the fp32 oracle.
"""

import math

import pytest
import torch

from oracle import actquant, luts, packing, rotation, turboquant
from tests.helpers import cosine, max_rel

pytestmark = pytest.mark.gpu

GS = 128


def _quantized(n_rows, k, bit, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n_rows, k, generator=g) * 0.02).half()
    return turboquant.quantize_packed(w, bit, GS, seed=seed)


def _gf(packed):
    from dartmoq_hip import kernels
    return kernels.convert_to_group_first(packed["indices_packed"].cuda(), packed["norms"].cuda(), GS,
                                          packed["bit_width"])


def _close(out, ref):
    assert max_rel(out, ref) <= 1e-2, max_rel(out, ref)
    assert cosine(out, ref) >= 0.9999, cosine(out, ref)


@pytest.mark.parametrize("bit", [1, 2, 4])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_slice_rows_and_in_features_gf(bit, dtype):
    from dartmoq_hip import kernels
    k, n = 512, 384
    packed = _quantized(n, k, bit, seed=42 + bit)
    idx_gf, norms_gf = _gf(packed)
    x = (torch.randn(9, k, generator=torch.Generator().manual_seed(bit)) * 0.5).to(dtype)
    # gate_up style: rows [128, 384) of the pool, x not rotated yet
    out = kernels.triton_fused_matmul_grouped_slice_rows_gf(
        x.cuda(), idx_gf, packed["codebook"].cuda(), norms_gf, packed["seed"], GS, k, 128, 384, bit)
    assert out.dtype == dtype and tuple(out.shape) == (9, 256)
    ref = x.float() @ turboquant.dequantize_packed(packed, 128, 384).T
    _close(out.float(), ref)
    # the same rows with the rotation hoisted by the caller
    x_rot = kernels.batch_rotate_input(x.cuda(), GS, packed["seed"])
    out2 = kernels.triton_fused_matmul_grouped_slice_rows_gf(
        x_rot, idx_gf, packed["codebook"].cuda(), norms_gf, packed["seed"], GS, k, 128, 384, bit,
        x_is_rotated=True)
    _close(out2.float(), ref)
    # down style: input features [128, 384) of the pool, rotation seed + original_start inside
    xs = (torch.randn(5, 256, generator=torch.Generator().manual_seed(7)) * 0.5).to(dtype)
    out3 = kernels.triton_fused_matmul_grouped_slice_in_features_gf(
        xs.cuda(), idx_gf, packed["codebook"].cuda(), norms_gf, packed["seed"], GS, 128, 384, k, bit)
    assert out3.dtype == dtype and tuple(out3.shape) == (5, n)
    ref3 = xs.float() @ turboquant.dequantize_packed(packed, col_start=128, col_end=384).T
    _close(out3.float(), ref3)


@pytest.mark.parametrize("bit", [2, 4])
def test_merged_wrappers_equal_per_expert_wrappers(bit):
    from dartmoq_hip import kernels
    k, inter, n_exp = 256, 128, 3
    packed = _quantized(2 * inter * n_exp, k, bit, seed=50 + bit)
    idx_gf, norms_gf = _gf(packed)
    cb = packed["codebook"].cuda()
    counts = [5, 0, 37]
    x = (torch.randn(sum(counts), k, generator=torch.Generator().manual_seed(3)) * 0.5).half().cuda()
    x_rot = kernels.batch_rotate_input(x, GS, packed["seed"])
    info, cur = [], 0
    for e, c in enumerate(counts):
        info.append((cur, c, e * 2 * inter, 2 * inter))
        cur += c
    merged = kernels.triton_fused_matmul_merged_rows_gf(x_rot, idx_gf, cb, norms_gf, info, GS, k, bit)
    assert tuple(merged.shape) == (sum(counts), 2 * inter)
    for ts, c, ss, sc in info:
        if c == 0:
            continue
        one = kernels.triton_fused_matmul_grouped_slice_rows_gf(
            x_rot[ts:ts + c], idx_gf, cb, norms_gf, packed["seed"], GS, k, ss, ss + sc, bit,
            x_is_rotated=True)
        torch.testing.assert_close(merged[ts:ts + c].float().cpu(), one.float().cpu(),
                                   rtol=2e-3, atol=2e-3 * one.abs().max().item())
        ref = x[ts:ts + c].float().cpu() @ turboquant.dequantize_packed(packed, ss, ss + sc).T
        _close(merged[ts:ts + c].float(), ref)


def test_wrapper_errors_match_reference_behaviour():
    from dartmoq_hip import kernels
    packed = _quantized(256, 256, 2, seed=1)
    idx_gf, norms_gf = _gf(packed)
    cb = packed["codebook"].cuda()
    x = torch.zeros(4, 256, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):                     # unsupported bit width
        kernels.triton_fused_matmul_grouped_slice_rows_gf(x, idx_gf, cb, norms_gf, 1, GS, 256, 0, 128, 3)
    with pytest.raises(ValueError):                     # inconsistent slice_count inside a pool
        kernels.triton_fused_matmul_merged_rows_gf(x, idx_gf, cb, norms_gf,
                                                   [(0, 2, 0, 128), (2, 2, 128, 64)], GS, 256, 2)
    with pytest.raises(ValueError):                     # empty expert list
        kernels.triton_fused_matmul_merged_rows_gf(x, idx_gf, cb, norms_gf, [], GS, 256, 2)
    with pytest.raises(ValueError):                     # merged path needs >= 2 groups
        kernels.triton_fused_matmul_merged_rows_gf(x[:, :128], idx_gf[:1], cb, norms_gf[:1],
                                                   [(0, 4, 0, 128)], GS, 128, 2)
    with pytest.raises(ValueError):                     # misaligned original_start
        kernels.triton_fused_matmul_grouped_slice_in_features_gf(x[:, :128], idx_gf, cb, norms_gf, 1,
                                                                 GS, 64, 192, 256, 2)
    with pytest.raises(ValueError):                     # wxfp4 has no 8-bit pools
        kernels.wxfp4_matmul_merged_rows_gf(x, x, idx_gf, cb, 127, norms_gf, [(0, 4, 0, 128)], GS,
                                            256, 8)


@pytest.mark.parametrize("mode", ["a8", "fp8", "fp4"])
def test_quantized_activation_wrappers(mode):
    """rotate+quantize wrappers return the reference's layouts and feed the merged GEMM wrappers."""
    from dartmoq_hip import kernels
    bit, k, inter = 2, 256, 128
    packed = _quantized(2 * inter * 2, k, bit, seed=60)
    idx_gf, norms_gf = _gf(packed)
    norms_pre = (norms_gf.float() / math.sqrt(GS)).half()
    cb = packed["codebook"]
    counts = [6, 11]
    b = sum(counts)
    x = (torch.randn(b, k, generator=torch.Generator().manual_seed(9)) * 0.5).half()
    rot = kernels.generate_batch_rotation_matrices(GS, packed["seed"], k // GS, GS, device="cuda")
    x_rot = rotation.batch_rotate_input(x.float(), GS, packed["seed"])
    info = [(0, counts[0], 0, 2 * inter), (counts[0], counts[1], 2 * inter, 2 * inter)]
    w_rot = turboquant.rotated_space_weights(packed)              # fp32 [N, K] in rotated space
    ref = torch.cat([x_rot[ts:ts + c] @ w_rot[ss:ss + sc].T for ts, c, ss, sc in info])
    if mode == "a8":
        lut, step = kernels.build_int8_codebook(cb)
        codes, scale = kernels.rotate_quantize_fused(x.cuda(), rot, GS, k // GS, step)
        assert codes.dtype == torch.int8 and scale.dtype == torch.float16
        assert tuple(codes.shape) == (b, k) and tuple(scale.shape) == (b, k // GS)
        c2, s2 = kernels.quantize_act_per_token_group(kernels.batch_rotate_input(x.cuda(), GS,
                                                      packed["seed"]), GS, step)
        assert c2.dtype == torch.int8 and s2.dtype == torch.float32
        out = kernels.wxa8_matmul_merged_rows_gf(codes, scale, idx_gf, lut.cuda(), norms_pre, info, GS,
                                                 k, bit, norms_prescaled=True)
        tol = 3e-2                                                # int8 activations + int8 LUT
    elif mode == "fp8":
        lut, s = kernels.build_fp8_codebook(cb)
        codes, scale = kernels.rotate_quantize_fused_fp8(x.cuda(), rot, GS, k // GS, s)
        assert codes.dtype == torch.float8_e4m3fn and scale.dtype == torch.float16
        out = kernels.wxfp8_matmul_merged_rows_gf(codes, scale, idx_gf, lut.cuda(), norms_pre, info, GS,
                                                  k, bit, norms_prescaled=True)
        tol = 8e-2                                                # e4m3 activations and weights
    else:
        nib, e0, resid, _ = kernels.build_e2m1_codebook(cb)
        x_t, x_s = kernels.rotate_quantize_fused_fp4(x.cuda(), rot, GS, k // GS)
        assert tuple(x_t.shape) == (k // 2, b) and tuple(x_s.shape) == (b, k // 32)
        p_ref, s_ref = actquant.quantize_act_e2m1(x_rot)
        # the fused kernel rotates on the matrix cores; codes may differ from the fp32 oracle
        # only where a value sits within rounding of a grid midpoint
        same = (x_t.t().cpu() == p_ref).float().mean().item()
        assert same > 0.97
        folded = kernels.fold_indices_to_e2m1(idx_gf, nib, bit)
        w_s = torch.full((2 * inter * 2, k // 32), 127 + e0, dtype=torch.uint8, device="cuda")
        out = kernels.wxfp4_matmul_merged_rows_gf(x_t, x_s, idx_gf, nib.cuda(), w_s,
                                                  (norms_pre.float() * resid).half(), info, GS, k, bit,
                                                  norms_prescaled=True, w_e2m1_gf=folded)
        tol = 0.3                                                 # e2m1 activations and weights
    assert out.dtype == torch.float16 and tuple(out.shape) == (b, 2 * inter)
    err = (out.float().cpu() - ref).norm() / ref.norm()
    assert err < tol, err.item()


def test_stage_profiler_alias():
    from dartmoq_hip import kernels
    prof = kernels.CudaStageProfiler(enabled=True)
    prof.begin_round()
    with prof.stage("noop"):
        torch.zeros(8, device="cuda").add_(1)
    stats = prof.end_round()
    assert stats["noop"]["calls"] == 1 and stats["noop"]["ms"] >= 0.0
