"""GPU parity: the long-stretch dequant GEMM (work items of 128 rows, fp16 pools).

The kernel multiplies the norm into the fp16 weight operand and runs the MFMAs of a (row, feature)
in the order of the 32-row kernel, so its outputs must equal that kernel's bit for bit, whatever the
number of rows of an expert; the 32-row kernel itself is checked against the fp32 oracle in
test_gpu_gemm.py, and one case here repeats that check directly.
"""

import math

import pytest
import torch

from oracle import codebook, moe, packing

pytestmark = pytest.mark.gpu

A16 = 0
STORE, SILU, SCATTER = 0, 1, 2
ROWS_TT = 8

# ragged experts: empty, a single row, around every tile-class edge (32 / 64 / 128) and several items
COUNTS = [1, 0, 31, 32, 33, 64, 65, 127, 128, 129, 300, 16, 5]


def _pool(bit, n_rows, k, seed):
    g = torch.Generator().manual_seed(seed)
    groups = k // 128
    idx_gf = torch.randint(0, 256, (groups, n_rows, 128 * bit // 8), dtype=torch.uint8, generator=g)
    norms_gf = ((torch.rand(groups, n_rows, generator=g) * 0.2 + 0.02) / math.sqrt(128)).half()
    cb = codebook.get_codebook(bit)[0].half()
    return idx_gf, norms_gf, cb


def _starts(counts):
    out, cur = [], 0
    for c in counts:
        out.append(cur)
        cur += c
    return out, cur


@pytest.mark.parametrize("bit", [1, 2, 4])
@pytest.mark.parametrize("k", [512, 1024])
def test_rows_store_equals_32_row_kernel_and_oracle(bit, k):
    from dartmoq_hip import ops
    n_slice = 256
    starts, rows_total = _starts(COUNTS)
    idx_gf, norms_gf, cb = _pool(bit, n_slice * len(COUNTS), k, 500 + bit)
    g = torch.Generator().manual_seed(k + bit)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half()
    info = [(starts[e], COUNTS[e], e * n_slice, n_slice) for e in range(len(COUNTS))]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    kw = dict(groups=k // 128, n_out=n_slice, slice_is_groups=False, rows_total=rows_total)
    tens = (x.cuda(), None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev)
    want = ops.matmul_merged(A16, bit, STORE, *tens, tt=2, **kw)
    got = ops.matmul_merged(A16, bit, STORE, *tens, tt=ROWS_TT, **kw)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # and against the fp32 dequantize-then-matmul contraction
    w = cb.float()[packing.unpack_nbit(idx_gf, bit, 128).long()]
    ref = torch.zeros(rows_total, n_slice)
    for e, (ts, cnt, ss, sc) in enumerate(info):
        if cnt == 0:
            continue
        wl = w[:, ss:ss + sc].permute(1, 0, 2).reshape(n_slice, -1)
        ref[ts:ts + cnt] = moe.lut_gemm(x[ts:ts + cnt].float(), torch.ones(cnt, k // 128), wl,
                                        norms_gf[:, ss:ss + sc].float().t(), 128)
    torch.testing.assert_close(got.cpu().float(), ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("bit", [2, 4])
def test_rows_silu_scatter_and_gather_equal_32_row_kernel(bit):
    """SiLU*up epilogue with a row gather on the input, and the down shape (slices in groups) with
    the routing-weighted scatter."""
    from dartmoq_hip import ops
    k, inter, hidden = 512, 256, 512
    starts, rows_total = _starts(COUNTS)
    n_exp = len(COUNTS)
    g = torch.Generator().manual_seed(77 + bit)
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter * n_exp, k, 600 + bit)
    tokens = 97
    x = (torch.randn(tokens, k, generator=g) * 0.5).half().cuda()
    row_index = torch.randint(0, tokens, (rows_total,), generator=g).int().cuda()
    info = [(starts[e], COUNTS[e], e * 2 * inter, 2 * inter) for e in range(n_exp)]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    kw = dict(groups=k // 128, n_out=inter, half_width=inter, slice_is_groups=False,
              rows_total=rows_total, row_index=row_index)
    tens = (x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev)
    want = ops.matmul_merged(A16, bit, SILU, *tens, tt=2, **kw)
    got = ops.matmul_merged(A16, bit, SILU, *tens, tt=ROWS_TT, **kw)
    torch.cuda.synchronize()
    assert want.abs().max() > 0
    assert torch.equal(got, want)

    # the down shape contracts inter / 128 groups per expert: the kernel wants a multiple of four
    inter4 = 512
    didx, dnorms, dcb = _pool(bit, hidden, inter4 * n_exp, 700 + bit)
    dinfo = [(starts[e], COUNTS[e], e * (inter4 // 128), inter4 // 128) for e in range(n_exp)]
    dinfo_dev = torch.tensor(dinfo, dtype=torch.int32).cuda()
    a = (torch.randn(rows_total, inter4, generator=g) * 0.5).half().cuda()
    slot = torch.randperm(rows_total, generator=g).int().cuda()
    wts = torch.rand(rows_total, generator=g).cuda()
    outs = []
    for tt in (2, ROWS_TT):
        slots = torch.full((rows_total, hidden), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_merged(A16, bit, SCATTER, a, None, didx.cuda(), dnorms.cuda(), dcb.cuda(), dinfo_dev,
                          groups=inter4 // 128, n_out=hidden, slice_is_groups=True, rows_total=rows_total,
                          out=slots, out_stride=hidden, row_weight=wts, row_slot=slot, tt=tt)
        torch.cuda.synchronize()
        outs.append(slots.cpu())
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


@pytest.mark.parametrize("bit", [1, 2, 4])
def test_rows_fused_down_rotation_equals_32_row_kernel(bit):
    """DMQ_EPI_SILU_ROT through the 128-row kernel: same rotated fp16 rows as the 32-row kernel."""
    from dartmoq_hip import ops
    from dartmoq_hip._lib import EPI_SILU_ROT
    k, inter = 512, 256
    n_exp = len(COUNTS)
    starts, rows_total = _starts(COUNTS)
    g = torch.Generator().manual_seed(31 + bit)
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter * n_exp, k, 800 + bit)
    x = (torch.randn(rows_total, k, generator=g) * 0.7).half().cuda()
    info = [(starts[e], COUNTS[e], e * 2 * inter, 2 * inter) for e in range(n_exp)]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    rot = (torch.randn(n_exp * inter // 128, 128, 128, generator=g) / 128 ** 0.5).half().cuda()
    tens = (x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev)
    outs = []
    for tt in (2, ROWS_TT):
        codes = torch.full((rows_total, inter), float("nan"), dtype=torch.float16, device="cuda")
        dummy = torch.empty((rows_total, inter), dtype=torch.float16, device="cuda")
        ops.matmul_merged(A16, bit, EPI_SILU_ROT, *tens, groups=k // 128, n_out=inter, half_width=inter,
                          slice_is_groups=False, rows_total=rows_total, tt=tt, out=dummy, out_stride=inter,
                          post=dict(rot=[rot], extra=[1.0], out=codes, scale=None))
        torch.cuda.synchronize()
        outs.append(codes.cpu())
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


def test_rows_argument_errors():
    from dartmoq_hip import ops
    idx_gf, norms_gf, cb = _pool(2, 256, 384, 1)
    x = torch.zeros(16, 384, dtype=torch.float16, device="cuda")
    info = torch.tensor([[0, 16, 0, 256]], dtype=torch.int32).cuda()
    with pytest.raises(ValueError):            # three groups: the 128-row kernel needs a multiple of four
        ops.matmul_merged(A16, 2, STORE, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info,
                          groups=3, n_out=256, slice_is_groups=False, rows_total=16, tt=ROWS_TT)
    idx_gf, norms_gf, cb = _pool(2, 128, 512, 1)
    x = torch.zeros(16, 512, dtype=torch.float16, device="cuda")
    info = torch.tensor([[0, 16, 0, 128]], dtype=torch.int32).cuda()
    with pytest.raises(ValueError):            # a block of the plain-store epilogue is 256 features
        ops.matmul_merged(A16, 2, STORE, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info,
                          groups=4, n_out=128, slice_is_groups=False, rows_total=16, tt=ROWS_TT)


@pytest.mark.parametrize("epi", ["store", "silu_rot", "scatter"])
def test_rows_many_units_keep_the_pipeline_full(epi):
    """Several hundred work items of every tile class, so that workgroups run many units one after
    the other (loads of a unit's last steps go to the next unit, units drawn from the queues while
    the previous one runs, other workgroups' queues emptied at the end): bits of the 32-row kernel."""
    from dartmoq_hip import ops
    from dartmoq_hip._lib import EPI_SILU_ROT
    bit = 2
    g = torch.Generator().manual_seed(91)
    n_exp = 300
    counts = torch.randint(0, 260, (n_exp,), generator=g).tolist()
    counts[7] = 1500                                     # one expert with many full stretches
    starts, rows_total = _starts(counts)
    if epi == "scatter":                                 # down shape: slices in groups, K = 512, 1024 features out
        k, hidden = 512, 1024
        didx, dnorms, dcb = _pool(bit, hidden, k * n_exp, 41)
        dinfo = torch.tensor([(starts[e], counts[e], e * (k // 128), k // 128) for e in range(n_exp)],
                             dtype=torch.int32).cuda()
        a = (torch.randn(rows_total, k, generator=g) * 0.5).half().cuda()
        slot = torch.randperm(rows_total, generator=g).int().cuda()
        wts = torch.rand(rows_total, generator=g).cuda()
        outs = []
        for tt in (2, ROWS_TT):
            slots = torch.full((rows_total, hidden), float("nan"), dtype=torch.float16, device="cuda")
            ops.matmul_merged(A16, bit, SCATTER, a, None, didx.cuda(), dnorms.cuda(), dcb.cuda(), dinfo,
                              groups=k // 128, n_out=hidden, slice_is_groups=True, rows_total=rows_total,
                              out=slots, out_stride=hidden, row_weight=wts, row_slot=slot, tt=tt)
            torch.cuda.synchronize()
            outs.append(slots.cpu())
        assert not torch.isnan(outs[0].float()).any()
        assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
        return
    k, inter = 1024, 256
    n_rows = (inter if epi == "store" else 2 * inter) * n_exp
    idx_gf, norms_gf, cb = _pool(bit, n_rows, k, 43)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half().cuda()
    width = n_rows // n_exp
    info = torch.tensor([(starts[e], counts[e], e * width, width) for e in range(n_exp)],
                        dtype=torch.int32).cuda()
    tens = (x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info)
    outs = []
    for tt in (2, ROWS_TT):
        if epi == "store":
            out = ops.matmul_merged(A16, bit, STORE, *tens, groups=k // 128, n_out=inter,
                                    slice_is_groups=False, rows_total=rows_total, tt=tt)
        else:
            rot = (torch.randn(n_exp * inter // 128, 128, 128, generator=torch.Generator().manual_seed(5))
                   / 128 ** 0.5).half().cuda()
            out = torch.full((rows_total, inter), float("nan"), dtype=torch.float16, device="cuda")
            dummy = torch.empty((rows_total, inter), dtype=torch.float16, device="cuda")
            ops.matmul_merged(A16, bit, EPI_SILU_ROT, *tens, groups=k // 128, n_out=inter, half_width=inter,
                              slice_is_groups=False, rows_total=rows_total, tt=tt, out=dummy,
                              out_stride=inter, post=dict(rot=[rot], extra=[1.0], out=out, scale=None))
        torch.cuda.synchronize()
        outs.append(out.cpu())
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
