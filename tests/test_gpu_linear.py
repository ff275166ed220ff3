"""GPU parity: quantized Linear layers (the Linears of the shared expert) and the un-sliced
callables of the reference's Linear path, against the CPU oracle.

fp32 reference: x @ dequantize(W)^T (WxA16Linear.dequantize, quantization/wxa16/linear.py:160-221).
WxA16 is held to the north-star bound (max relative error <= 1e-2, cosine >= 0.9999); the
activation-quantized modes are compared with the oracle's restatement of their dataflow.
"""

import pytest
import torch

from oracle import moe, turboquant
from oracle.rotation import batch_rotation_matrices, rotate_with
from tests.helpers import cosine, max_rel, relerr

pytestmark = pytest.mark.gpu


def _packed(n, k, bit, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).half()
    return turboquant.quantize_packed(w, bit, 128, seed=seed + 5)


def _dataflow(packed, x, mode):
    gs = packed["group_size"]
    n, k = packed["shape"]
    w_lut, norms, extra, wbs = moe._lut_weights(packed, mode)
    rot = batch_rotation_matrices(gs, packed["seed"], k // gs, gs, torch.float16)
    codes, scale = moe.quantize_activation(rotate_with(x.half(), rot, torch.float32), mode, gs, extra)
    return moe.lut_gemm(codes, scale, w_lut, norms, gs, wbs)


@pytest.mark.parametrize("bit", [1, 2, 4])
@pytest.mark.parametrize("rows", [1, 33, 300])
def test_wxa16_linear_matches_dequantized_matmul(bit, rows):
    import dartmoq_hip
    packed = _packed(384, 512, bit, seed=bit)
    lin = dartmoq_hip.WxA16Linear.from_packed(packed)
    x = torch.randn(rows, 512, generator=torch.Generator().manual_seed(rows)).half()
    out = lin(x.cuda()).float().cpu()
    ref = x.float() @ turboquant.dequantize_packed(packed).T
    assert out.shape == (rows, 384)
    assert relerr(out, ref) < 2e-3
    assert max_rel(out, ref) <= 1e-2 and cosine(out, ref) >= 0.9999
    assert relerr(out, _dataflow(packed, x, "wxa16")) < 1.5e-3


@pytest.mark.parametrize("mode,cls,tight", [("wxa8", "WxA8Linear", 6e-3), ("wxfp8", "WxFP8Linear", 2e-2)])
def test_quantized_activation_linears(mode, cls, tight):
    import dartmoq_hip
    packed = _packed(256, 640, 4, seed=9)
    lin = getattr(dartmoq_hip, cls).from_wxa16(dartmoq_hip.WxA16Linear.from_packed(packed))
    x = torch.randn(70, 640, generator=torch.Generator().manual_seed(4)).half()
    out = lin(x.cuda()).float().cpu()
    assert relerr(out, _dataflow(packed, x, mode)) < tight
    ref = x.float() @ turboquant.dequantize_packed(packed).T
    assert relerr(out, ref) < {"wxa8": 0.02, "wxfp8": 0.075}[mode]


@pytest.mark.parametrize("k", [200, 448])
@pytest.mark.parametrize("bit,mode", [(4, "wxa16"), (2, "wxa16"), (1, "wxa16"), (4, "wxa8"), (4, "wxfp8")])
def test_ragged_in_features(k, bit, mode):
    """in_features not a multiple of the group size: the last group has d = k % 128 columns, its own
    d x d rotation (seed + g_start) and scale 1 / sqrt(d), the reference's per-group path
    (turboquant_utils/triton_kernels.py:618-650); here the group is padded to 128 once at load."""
    import dartmoq_hip
    packed = _packed(192, k, bit, seed=k + bit)
    assert packed["indices_packed"].shape == (192, k * bit // 8) and packed["norms"].shape == (192, -(-k // 128))
    lin = dartmoq_hip.WxA16Linear.from_packed(packed)
    if mode != "wxa16":
        lin = {"wxa8": dartmoq_hip.WxA8Linear, "wxfp8": dartmoq_hip.WxFP8Linear}[mode].from_wxa16(lin)
    x = torch.randn(45, k, generator=torch.Generator().manual_seed(k)).half()
    out = lin(x.cuda()).float().cpu()
    ref = x.float() @ turboquant.dequantize_packed(packed).T
    assert relerr(out, ref) < {"wxa16": 2e-3, "wxa8": 0.02, "wxfp8": 0.075}[mode], relerr(out, ref)
    if mode == "wxa16":
        assert max_rel(out, ref) <= 1e-2 and cosine(out, ref) >= 0.9999
    assert torch.equal(lin.forward_by_pieces(x.cuda()).float().cpu(), out)
    if mode == "wxa16":
        # the reference's un-sliced callables take the same route
        from dartmoq_hip import kernels as K
        ip, cb, nm = packed["indices_packed"].cuda(), packed["codebook"].cuda(), packed["norms"].cuda()
        full = K.triton_fused_matmul_grouped(x.cuda(), ip, cb, nm, packed["seed"], 128, k, bit)
        assert torch.equal(full.float().cpu(), out)
        part = K.triton_fused_matmul_grouped_slice_rows(x.cuda(), ip, cb, nm, packed["seed"], 128, k, 64, 192, bit)
        assert relerr(part.float().cpu(), ref[:, 64:192]) < 2e-3


def test_linear_bias_shapes_and_dtypes():
    import dartmoq_hip
    packed = _packed(128, 256, 2, seed=3)
    bias = torch.linspace(-1, 1, 128).half()
    lin = dartmoq_hip.WxA16Linear.from_packed(packed, bias=bias)
    x = torch.randn(2, 5, 256, generator=torch.Generator().manual_seed(8))
    ref = x.reshape(-1, 256).half().float() @ turboquant.dequantize_packed(packed).T + bias.float()
    out = lin(x.cuda().bfloat16())
    assert out.dtype == torch.bfloat16 and out.shape == (2, 5, 128)
    assert relerr(out.float().cpu().reshape(-1, 128), ref) < 1e-2       # bf16 in and out
    out16 = lin(x.cuda().half())
    assert relerr(out16.float().cpu().reshape(-1, 128), ref) < 2e-3
    with pytest.raises(ValueError):
        lin(torch.zeros(3, 128, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError):
        lin(torch.zeros(3, 256, dtype=torch.float16))


def test_linear_constructor_errors():
    import dartmoq_hip
    packed = _packed(128, 256, 2, seed=3)
    with pytest.raises(ValueError):
        dartmoq_hip.WxA16Linear(256, 128, 3, 128, packed["indices_packed"], packed["codebook"],
                                packed["norms"], 1)
    with pytest.raises(ValueError):
        dartmoq_hip.WxA16Linear(256, 128, 2, 64, packed["indices_packed"], packed["codebook"],
                                packed["norms"], 1)
    with pytest.raises(ValueError):
        dartmoq_hip.WxA16Linear(256, 64, 2, 128, packed["indices_packed"], packed["codebook"],
                                packed["norms"], 1)
    with pytest.raises(TypeError):
        dartmoq_hip.WxA8Linear.from_wxa16(object())


def test_reference_module_duck_typing():
    import types
    import dartmoq_hip
    packed = _packed(128, 256, 4, seed=6)
    ref_lin = types.SimpleNamespace(
        in_features=256, out_features=128, bit_width=4, group_size=128,
        packed_indices=packed["indices_packed"], codebook=packed["codebook"], norms=packed["norms"],
        seed=torch.tensor(packed["seed"]), rotation="qr", bias=None, orig_dtype=torch.float16,
        codebook_type="lloydmax")
    a = dartmoq_hip.WxA16Linear.from_reference_module(ref_lin)
    b = dartmoq_hip.WxA16Linear.from_packed(packed)
    x = torch.randn(9, 256, generator=torch.Generator().manual_seed(1)).half().cuda()
    assert torch.equal(a(x), b(x))


def test_unsliced_callables_by_reference_names():
    """triton_fused_matmul_grouped and its row-major slice variants; wxa8 / wxfp8 grouped_gf."""
    from dartmoq_hip import kernels as K
    packed = _packed(256, 512, 2, seed=11)
    w = turboquant.dequantize_packed(packed)
    x = torch.randn(40, 512, generator=torch.Generator().manual_seed(3)).half()
    dev = lambda t: t.cuda()
    ip, cb, nm = dev(packed["indices_packed"]), dev(packed["codebook"]), dev(packed["norms"])
    out = K.triton_fused_matmul_grouped(x.cuda(), ip, cb, nm, packed["seed"], 128, 512, 2)
    assert relerr(out.float().cpu(), x.float() @ w.T) < 2e-3
    # second call hits the converted-layout cache and gives the same bits
    assert torch.equal(out, K.triton_fused_matmul_grouped(x.cuda(), ip, cb, nm, torch.tensor(packed["seed"]),
                                                          128, 512, 2))
    rows = K.triton_fused_matmul_grouped_slice_rows(x.cuda(), ip, cb, nm, packed["seed"], 128, 512, 64, 192, 2)
    assert torch.equal(rows, out[:, 64:192])
    xs = x[:, 128:384].contiguous()
    part = K.triton_fused_matmul_grouped_slice_in_features(xs.cuda(), ip, cb, nm, packed["seed"], 128,
                                                           128, 384, 512, 2)
    assert relerr(part.float().cpu(), xs.float() @ w[:, 128:384].T) < 2e-3
    with pytest.raises(ValueError):
        K.triton_fused_matmul_grouped(x.cuda(), ip, cb, nm, packed["seed"], 128, 512, 3)
    with pytest.raises(ValueError):
        K.triton_fused_matmul_grouped(x.cuda(), ip, cb, nm, packed["seed"], 128, 500, 2)
    with pytest.raises(ValueError):
        K.triton_fused_matmul_grouped_slice_in_features(xs.cuda(), ip, cb, nm, packed["seed"], 128, 64, 320,
                                                        512, 2)

    idx_gf, norms_gf = K.convert_to_group_first(ip, nm, 128, 2)
    norms_pre = (norms_gf.float() / 128 ** 0.5).half()
    rot = K.generate_batch_rotation_matrices(128, packed["seed"], 4, 128, device="cuda")
    cb_i8, step = K.build_int8_codebook(packed["codebook"])
    x_i8, x_s = K.rotate_quantize_fused(x.cuda(), rot, 128, 4, extra_scale=step)
    o8 = K.wxa8_matmul_grouped_gf(x_i8, x_s, idx_gf, cb_i8.cuda(), norms_pre, 128, 4, 2)
    assert relerr(o8.float().cpu(), _dataflow(packed, x, "wxa8")) < 6e-3
    with pytest.raises(ValueError):
        K.wxa8_matmul_grouped_gf(x_i8, x_s, idx_gf, cb_i8.cuda(), norms_pre, 128, 4, 2, identity_cb=True)
    cb_f8, sc = K.build_fp8_codebook(packed["codebook"])
    x_f8, x_s8 = K.rotate_quantize_fused_fp8(x.cuda(), rot, 128, 4, extra_scale=sc)
    of8 = K.wxfp8_matmul_grouped_gf(x_f8, x_s8, idx_gf, cb_f8.cuda(), norms_pre, 128, 4, 2)
    assert relerr(of8.float().cpu(), _dataflow(packed, x, "wxfp8")) < 2e-2


@pytest.mark.parametrize("cls,mode,tol", [("WxA16Linear", "wxa16", 1.5e-3), ("WxA8Linear", "wxa8", 6e-3),
                                          ("WxFP8Linear", "wxfp8", 2e-2)])
@pytest.mark.parametrize("bit", [1, 2, 4, 8])
@pytest.mark.parametrize("rows", [1, 16, 17, 64])
def test_linears_with_a_handful_of_rows(cls, mode, tol, bit, rows):
    """The small-batch launches of a Linear: one n-tile per wave with K split over the waves (up
    to 16 rows), K split over the waves of four n-tiles or shared between workgroups (up to 64);
    16 groups, so every wave and every workgroup gets several."""
    import dartmoq_hip
    n, k = 320, 2048
    packed = (turboquant.quantize_packed((torch.randn(n, k, generator=torch.Generator().manual_seed(bit)) * 0.02).half(),
                                         bit, 128, seed=11, uniform_codebook=True)
              if bit == 8 else _packed(n, k, bit, seed=bit))
    lin = dartmoq_hip.WxA16Linear.from_packed(packed)
    if cls != "WxA16Linear":
        lin = getattr(dartmoq_hip, cls).from_wxa16(lin)
    x = torch.randn(rows, k, generator=torch.Generator().manual_seed(rows)).half()
    out = lin(x.cuda())
    assert torch.equal(out, lin(x.cuda()))                        # same bits on every call
    assert torch.equal(out, lin.forward_by_pieces(x.cuda()))      # the C entry = its two launches
    out = out.float().cpu()
    assert out.shape == (rows, n)
    assert relerr(out, _dataflow(packed, x, mode)) < tol
    if mode == "wxa16":
        ref = x.float() @ turboquant.dequantize_packed(packed).T
        assert max_rel(out, ref) <= 1e-2 and cosine(out, ref) >= 0.9999
    # a row's result does not depend on the rows batched with it (same launch shape)
    if rows == 16:
        alone = lin(x[:5].cuda()).float().cpu()
        assert torch.equal(alone, out[:5])


_BIG = {}


def _big_packed(bit):
    if bit not in _BIG:
        _BIG[bit] = _packed8(1024, 512, seed=3, uniform=True) if bit == 8 else _packed(1024, 512, bit, seed=3)
    return _BIG[bit]


@pytest.mark.parametrize("cls,mode,tol", [("WxA16Linear", "wxa16", 1.5e-3), ("WxA8Linear", "wxa8", 6e-3),
                                          ("WxFP8Linear", "wxfp8", 2e-2)])
@pytest.mark.parametrize("bit", [4, 8])
@pytest.mark.parametrize("rows", [65, 1100, 2100, 4200, 6200])
def test_linear_entry_point_equals_its_pieces(cls, mode, tol, bit, rows):
    """dmq_linear_forward against dmq_rotate + dmq_matmul_merged_gf issued one by one, over the
    launch shapes of bigger batches (1024 features = 4 blocks: 16-row tiles with K shared by two
    workgroups at 65 and 1100 rows, 32-row tiles at 2100, 64-row tiles at 4200 unless the weights
    are 8-bit; 6200 rows of 8-bit weights on the int8 path: the 128 x 128-tile int8 GEMM), with an
    input whose rows are strided; and against the oracle's dataflow."""
    import dartmoq_hip
    packed = _big_packed(bit)
    lin = dartmoq_hip.WxA16Linear.from_packed(packed)
    if cls != "WxA16Linear":
        lin = getattr(dartmoq_hip, cls).from_wxa16(lin)
    wide = torch.randn(rows, 640, generator=torch.Generator().manual_seed(rows)).half()
    x = wide.cuda()[:, :512]                                      # row stride 640
    out = lin(x)
    assert torch.equal(out, lin.forward_by_pieces(x))
    assert torch.equal(out, lin(x.contiguous()))
    assert relerr(out.float().cpu(), _dataflow(packed, wide[:, :512], mode)) < tol


def test_int8_gemm_of_uniform_8bit_weights():
    """dmq_linear_gemm_i8 (128 x 128 tiles, weights idx - 128 as a plain MFMA operand) on ragged
    shapes (300 rows, 320 features: partial tiles both ways) against the look-up kernel's
    table-free path and the oracle's int8 dataflow; the group sums are exact integers in both
    kernels and are scaled and added in the same order."""
    from dartmoq_hip import kernels as K, ops
    packed = _packed8(320, 512, seed=6, uniform=True)
    x = torch.randn(300, 512, generator=torch.Generator().manual_seed(2)).half()
    idx_gf, norms_gf = K.convert_to_group_first(packed["indices_packed"].cuda(), packed["norms"].cuda(), 128, 8)
    norms_pre = (norms_gf.float() / 128 ** 0.5).half()
    rot = K.generate_batch_rotation_matrices(128, packed["seed"], 4, 128, device="cuda")
    x_i8, x_s = K.rotate_quantize_fused(x.cuda(), rot, 128, 4, extra_scale=K.uniform_codebook_step(packed["codebook"]))
    out = ops.linear_gemm_i8(x_i8, x_s, idx_gf, norms_pre)
    dummy = torch.zeros(256, dtype=torch.int8, device="cuda")
    lut_path = K.wxa8_matmul_grouped_gf(x_i8, x_s, idx_gf, dummy, norms_pre, 128, 4, 8, identity_cb=True)
    assert out.shape == (300, 320)
    assert relerr(out.float().cpu(), lut_path.float().cpu()) < 5e-4
    assert relerr(out.float().cpu(), _dataflow(packed, x, "wxa8")) < 6e-3
    assert torch.equal(out, ops.linear_gemm_i8(x_i8, x_s, idx_gf, norms_pre))


def test_int8_gemm_exact_integers():
    """dmq_linear_gemm_i8 on operands whose result is an exact small integer: activation codes in
    [-3, 3], weights idx - 128 in [-2, 2], unit scales and norms.  Every group sum is an int32 the
    matrix cores must deliver exactly, their fp32 scaling and sum are exact, and the fp16 store of
    an integer below 2048 is exact, so the output must equal an int64 matmul bit for bit (ragged
    shape: partial tiles in rows and features)."""
    from dartmoq_hip import ops
    rows, k, n = 203, 384, 200
    g = torch.Generator().manual_seed(11)
    x = torch.randint(-3, 4, (rows, k), generator=g, dtype=torch.int8)
    w = torch.randint(-2, 3, (n, k), generator=g, dtype=torch.int64)
    idx_gf = (w + 128).to(torch.uint8).reshape(n, k // 128, 128).permute(1, 0, 2).contiguous()
    ones_s = torch.ones(rows, k // 128, dtype=torch.float16)
    ones_n = torch.ones(k // 128, n, dtype=torch.float16)
    out = ops.linear_gemm_i8(x.cuda(), ones_s.cuda(), idx_gf.cuda(), ones_n.cuda())
    ref = x.long() @ w.t()
    assert ref.abs().max() < 2048 and ref.abs().max() > 100
    assert torch.equal(out.cpu().long(), ref)
    # power-of-two scales and norms keep everything exact: the scale and norm factors reach the
    # right row and feature
    s2 = (2.0 ** torch.randint(-2, 3, (rows, k // 128), generator=g)).half()
    n2 = (2.0 ** torch.randint(-3, 2, (k // 128, n), generator=g)).half()
    out2 = ops.linear_gemm_i8(x.cuda(), s2.cuda(), idx_gf.cuda(), n2.cuda()).cpu()
    xg = x.double().reshape(rows, k // 128, 128)
    wg = w.double().reshape(n, k // 128, 128)
    ref2 = torch.einsum("rgk,ngk,rg,gn->rn", xg, wg, s2.double(), n2.double())
    # the scaled sums (multiples of 2^-5 below 2^14) are exact in fp32; the fp16 store rounds once
    assert torch.equal(out2, ref2.float().half())


# ----------------------------------------------------------------------------- 8-bit codebooks

def _packed8(n, k, seed, uniform):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).half()
    return turboquant.quantize_packed(w, 8, 128, seed=seed + 5, uniform_codebook=uniform)


@pytest.mark.parametrize("uniform", [True, False])
@pytest.mark.parametrize("rows", [3, 40, 200])
def test_wxa16_linear_8bit(uniform, rows):
    """8-bit indices (the attention / shared-expert Linears of a real checkpoint), uniform grid
    and 256-level Lloyd-Max, through the 256-entry fp16 table."""
    import dartmoq_hip
    packed = _packed8(256, 384, seed=2, uniform=uniform)
    lin = dartmoq_hip.WxA16Linear.from_packed(packed)
    x = torch.randn(rows, 384, generator=torch.Generator().manual_seed(rows)).half()
    out = lin(x.cuda()).float().cpu()
    ref = x.float() @ turboquant.dequantize_packed(packed).T
    assert relerr(out, ref) < 2e-3
    assert max_rel(out, ref) <= 1e-2 and cosine(out, ref) >= 0.9999


def test_dequant_tile_8bit_is_exact():
    from dartmoq_hip import ops
    from oracle import packing
    packed = _packed8(64, 256, seed=9, uniform=True)
    idx_gf, norms_gf = packing.convert_to_group_first(packed["indices_packed"], packed["norms"], 128, 8)
    tile = ops.dequant_tile(idx_gf.cuda(), packed["codebook"].cuda(), None, 0, 2, 0, 64, 8).cpu()
    want = packed["codebook"][idx_gf.long()]                      # [G, N, 128] one index per byte
    assert torch.equal(tile, want)


def test_wxa8_linear_8bit_identity_codebook():
    """int8 path on 8-bit uniform weights: w = idx - 128, step folded into the activation scale
    (the reference's IDENTITY_CB); a Lloyd-Max 8-bit codebook is refused like the reference does."""
    import dartmoq_hip
    from dartmoq_hip import kernels as K
    packed = _packed8(256, 512, seed=4, uniform=True)
    lin = dartmoq_hip.WxA8Linear.from_wxa16(dartmoq_hip.WxA16Linear.from_packed(packed))
    x = torch.randn(70, 512, generator=torch.Generator().manual_seed(1)).half()
    out = lin(x.cuda()).float().cpu()
    ideal = _dataflow(packed, x, "wxa8")
    assert relerr(out, ideal) < 6e-3
    ref = x.float() @ turboquant.dequantize_packed(packed).T
    assert relerr(out, ref) < 0.02
    # the reference-named kernel with identity_cb=True: same numbers from explicit pieces
    idx_gf, norms_gf = K.convert_to_group_first(packed["indices_packed"].cuda(), packed["norms"].cuda(), 128, 8)
    norms_pre = (norms_gf.float() / 128 ** 0.5).half()
    rot = K.generate_batch_rotation_matrices(128, packed["seed"], 4, 128, device="cuda")
    step = K.uniform_codebook_step(packed["codebook"])
    assert step == pytest.approx(3.5 / 128, rel=1e-3) and K.is_uniform_codebook(packed["codebook"])
    x_i8, x_s = K.rotate_quantize_fused(x.cuda(), rot, 128, 4, extra_scale=step)
    dummy = torch.zeros(256, dtype=torch.int8, device="cuda")
    o = K.wxa8_matmul_grouped_gf(x_i8, x_s, idx_gf, dummy, norms_pre, 128, 4, 8, identity_cb=True)
    # (the class shares K between two workgroups at this size, the callable does not: the fp32
    # group sums meet in another order, so the fp16 results agree to rounding, not bit for bit)
    assert relerr(o.float().cpu(), out) < 5e-4
    # ... and the table-free kernel gives the bits of the look-up kernel fed the identity table
    table = (torch.arange(256, dtype=torch.int16) - 128).to(torch.int8).cuda()
    o_tab = K.wxa8_matmul_grouped_gf(x_i8, x_s, idx_gf, table, norms_pre, 128, 4, 8, identity_cb=False)
    assert torch.equal(o, o_tab)
    lloyd = _packed8(128, 256, seed=4, uniform=False)
    with pytest.raises(ValueError):
        dartmoq_hip.WxA8Linear.from_wxa16(dartmoq_hip.WxA16Linear.from_packed(lloyd))


@pytest.mark.parametrize("uniform", [True, False])
def test_wxfp8_linear_8bit(uniform):
    import dartmoq_hip
    packed = _packed8(128, 256, seed=6, uniform=uniform)
    lin = dartmoq_hip.WxFP8Linear.from_wxa16(dartmoq_hip.WxA16Linear.from_packed(packed))
    x = torch.randn(33, 256, generator=torch.Generator().manual_seed(2)).half()
    out = lin(x.cuda()).float().cpu()
    assert relerr(out, _dataflow(packed, x, "wxfp8")) < 2e-2
    assert relerr(out, x.float() @ turboquant.dequantize_packed(packed).T) < 0.075
