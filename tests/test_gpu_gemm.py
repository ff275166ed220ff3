"""GPU parity: merged codebook-dequant GEMMs in all four precision modes.

Each case feeds the kernel and the oracle the *same* activation codes / scales and the same
packed pool, so the comparison isolates the GEMM: int32 accumulators are exact, fp16 outputs
match fp32 maths to fp16 rounding.
"""

import math

import pytest
import torch

from oracle import actquant, codebook, luts, moe, packing, routing

pytestmark = pytest.mark.gpu

A16, A8, FP8, FP4 = 0, 1, 2, 3
STORE, SILU, SCATTER = 0, 1, 2


def _gemv_groups_ok(groups):
    return groups % 4 == 0 and groups // 4 in (1, 2, 4, 6, 8)


def _pool(bit, n_rows, k, seed):
    """Random packed pool in group-first layout (indices, prescaled fp16 norms, codebook)."""
    g = torch.Generator().manual_seed(seed)
    groups = k // 128
    idx_gf = torch.randint(0, 256, (groups, n_rows, 128 * bit // 8), dtype=torch.uint8, generator=g)
    norms_gf = ((torch.rand(groups, n_rows, generator=g) * 0.2 + 0.02) / math.sqrt(128)).half()
    cb = codebook.get_codebook(bit)[0].half()
    return idx_gf, norms_gf, cb


def _expert_rows(counts):
    info, cur = [], 0
    for c in counts:
        info.append(cur)
        cur += c
    return info, cur


def _mode_inputs(mode, x_rot, cb):
    """(act codes tensor for the GPU, scale tensor or None, oracle codes fp32, oracle scale fp32,
    lut for the GPU, oracle lut values fp32, w block scale, norm factor, w_scale_byte)."""
    b, k = x_rot.shape
    if mode == A16:
        xh = x_rot.half()
        return xh, None, xh.float(), torch.ones(b, k // 128), cb, cb.float(), 1.0, 1.0, 127
    if mode == A8:
        q, step = luts.build_int8_codebook(cb)
        codes, s = actquant.quantize_act_int8(x_rot, 128, step)
        return codes, s.half(), codes.float(), s.half().float(), q, q.float(), 1.0, 1.0, 127
    if mode == FP8:
        q, scale = luts.build_fp8_codebook(cb)
        codes, s = actquant.quantize_act_fp8(x_rot, 128, scale)
        return codes, s.half(), codes.float(), s.half().float(), q, q.float(), 1.0, 1.0, 127
    nib, e0, resid, _ = luts.build_e2m1_codebook(cb)
    p, sb = actquant.quantize_act_e2m1(x_rot)
    return (p, sb, actquant.dequant_act_e2m1(p, sb), torch.ones(b, k // 128), nib,
            luts.e2m1_value(nib), 2.0 ** e0, resid, 127 + e0)


def _run_case(mode, bit, tt, counts, k, n_slice, slice_is_groups, seed, roomy=0, spread=0):
    from dartmoq_hip import ops
    n_exp = len(counts)
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(seed)
    if slice_is_groups:                       # down: weight [G_total = n_exp * k/128, N = n_slice]
        idx_gf, norms_gf, cb = _pool(bit, n_slice, k * n_exp, seed)
        info = [(starts[e], counts[e], e * (k // 128), k // 128) for e in range(n_exp)]
    else:                                     # gate_up: weight [G = k/128, N = n_exp * n_slice]
        idx_gf, norms_gf, cb = _pool(bit, n_slice * n_exp, k, seed)
        info = [(starts[e], counts[e], e * n_slice, n_slice) for e in range(n_exp)]
    x_rot = torch.randn(rows_total, k, generator=g) * 0.7
    act, scale, o_codes, o_scale, lut, o_lut, wbs, nfac, wsb = _mode_inputs(mode, x_rot, cb)
    norms_used = (norms_gf.float() * nfac).half() if mode == FP4 else norms_gf
    w_dev = idx_gf.cuda()
    if mode == FP4:
        w_dev = ops.fold_indices_to_e2m1(w_dev, lut, bit)
    idx = packing.unpack_nbit(idx_gf, bit, 128).long()           # [G, N, 128]
    w_vals = o_lut[idx]                                           # lut[idx] fp32

    ref = torch.zeros(rows_total, n_slice)
    for e, (ts, cnt, ss, sc) in enumerate(info):
        if cnt == 0:
            continue
        if slice_is_groups:
            wl = w_vals[ss:ss + sc].permute(1, 0, 2).reshape(n_slice, -1)
            nl = norms_used[ss:ss + sc].float().t()
        else:
            wl = w_vals[:, ss:ss + sc].permute(1, 0, 2).reshape(n_slice, -1)
            nl = norms_used[:, ss:ss + sc].float().t()
        ref[ts:ts + cnt] = moe.lut_gemm(o_codes[ts:ts + cnt], o_scale[ts:ts + cnt], wl, nl, 128, wbs)

    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    out = ops.matmul_merged(
        mode, bit, STORE, act.cuda(), None if scale is None else scale.cuda(), w_dev,
        norms_used.cuda(), None if mode == FP4 else lut.cuda(), info_dev, groups=k // 128,
        n_out=n_slice, slice_is_groups=slice_is_groups, rows_total=rows_total, w_scale_byte=wsb, tt=tt,
        roomy=roomy, spread=spread)
    torch.cuda.synchronize()
    return out.cpu().float(), ref


@pytest.mark.parametrize("mode", [A16, A8, FP8, FP4])
@pytest.mark.parametrize("bit", [1, 2, 4])
@pytest.mark.parametrize("tt", [1, 2, 4])
def test_merged_rows_gate_up(mode, bit, tt):
    counts = [3, 0, 17, 64, 1, 130]            # ragged, an empty expert, several tiles
    out, ref = _run_case(mode, bit, tt, counts, k=512, n_slice=128, slice_is_groups=False,
                         seed=100 + 10 * mode + bit)
    # only the fp16 rounding of the output (and fp32 summation order) separates the two
    torch.testing.assert_close(out, ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("mode", [A16, A8, FP8])
@pytest.mark.parametrize("bit", [1, 2, 4])
def test_two_per_cu_instance_gives_the_same_bits(mode, bit):
    """16-row tiles have a second kernel instance (two waves per SIMD, registers instead of scratch
    for the 4-bit weight ring): same arithmetic, so the same bits."""
    counts = [3, 0, 17, 64, 1, 130]
    lean, ref = _run_case(mode, bit, 1, counts, k=512, n_slice=128, slice_is_groups=False,
                          seed=100 + 10 * mode + bit)
    roomy, _ = _run_case(mode, bit, 1, counts, k=512, n_slice=128, slice_is_groups=False,
                         seed=100 + 10 * mode + bit, roomy=1)
    assert torch.equal(lean, roomy)
    torch.testing.assert_close(roomy, ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("mode", [A16, A8, FP4])
@pytest.mark.parametrize("tt", [1, 2, 4])
def test_items_dealt_out_one_per_xcd_give_the_same_bits(mode, tt):
    """spread: work item i goes to XCD i % 8 instead of every XCD taking a contiguous eighth of the
    list; a different schedule of the same work."""
    counts = [3, 0, 17, 64, 1, 130, 300, 5, 33]
    a, ref = _run_case(mode, 2, tt, counts, k=256, n_slice=192, slice_is_groups=False, seed=200 + mode + tt)
    b, _ = _run_case(mode, 2, tt, counts, k=256, n_slice=192, slice_is_groups=False, seed=200 + mode + tt,
                     spread=1)
    assert torch.equal(a, b)
    torch.testing.assert_close(b, ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("main", [A8, FP8, FP4])
@pytest.mark.parametrize("roomy", [0, 1])
def test_two_modes_in_one_launch_give_the_bits_of_two_launches(main, roomy):
    """mode2: the fp16 pool (4-bit weights) rides the launch of a quantized pool (2-bit weights);
    every work item runs the body of its pool's mode, so the result is that of one launch per mode."""
    from dartmoq_hip import ops
    k, inter = 384, 128
    counts0, counts1 = [5, 40, 0, 17], [21, 2]
    r0, r1 = sum(counts0), sum(counts1)
    rows = r0 + r1
    g = torch.Generator().manual_seed(77 + main)
    x_rot = torch.randn(rows, k, generator=g) * 0.7
    pools = []
    infos = []
    for pi, (mode, bit, counts, first_row) in enumerate([(main, 2, counts0, 0), (A16, 4, counts1, r0)]):
        idx_gf, norms_gf, cb = _pool(bit, 2 * inter * len(counts), k, 300 + pi)
        act, scale, _, _, lut, _, _, nfac, wsb = _mode_inputs(mode, x_rot, cb)
        norms_used = (norms_gf.float() * nfac).half() if mode == FP4 else norms_gf
        w_dev = idx_gf.cuda()
        if mode == FP4:
            w_dev = ops.fold_indices_to_e2m1(w_dev, lut, bit)
        # one row pitch for both pools (that of the fp16 rows), as in the layer's activation buffers
        buf = torch.zeros(rows, 2 * k, dtype=torch.uint8)
        raw = act.contiguous().view(torch.uint8).reshape(rows, -1)
        buf[:, :raw.shape[1]] = raw
        starts = [first_row + sum(counts[:e]) for e in range(len(counts))]
        info = torch.tensor([(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(len(counts))],
                            dtype=torch.int32).cuda()
        infos.append(info)
        pools.append(dict(w=w_dev, norms=norms_used.cuda(), lut=None if mode == FP4 else lut.cuda(),
                          expert_info=info, act=buf.cuda(), act_scale=None if scale is None else scale.cuda(),
                          row_index=None, bit=bit, mode=mode, w_scale_byte=wsb))
    lists = [ops.build_tiles(infos[pi], rows, 16, pool=pi) for pi in range(2)]
    n = [int(l[0][0]) for l in lists]
    items = torch.cat([lists[0][1][:n[0]], lists[1][1][:n[1]]]).contiguous()
    n_items = torch.tensor([n[0] + n[1], 0, 0, 0], dtype=torch.int32).cuda()
    scale_stride = pools[0]["act_scale"].stride(0)
    common = dict(groups=k // 128, n_out=inter, half_width=inter, slice_is_groups=False, tt=1,
                  out_stride=inter, act_row_bytes=2 * k, act_scale_stride=scale_stride, roomy=roomy)
    both = torch.full((rows, inter), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_pools(main, SILU, pools, items, n_items, items.shape[0], out=both, mode2=A16, **common)
    apart = torch.full((rows, inter), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_pools(main, SILU, pools, items, n_items, items.shape[0], out=apart, **common)
    assert torch.isnan(apart[r0:].float()).all() and not torch.isnan(apart[:r0].float()).any()
    ops.matmul_pools(A16, SILU, pools, items, n_items, items.shape[0], out=apart, spread=1, **common)
    torch.cuda.synchronize()
    assert not torch.isnan(both.float()).any()
    assert torch.equal(both, apart)


@pytest.mark.parametrize("mode", [A16, A8])
@pytest.mark.parametrize("roomy", [0, 1])
def test_both_index_widths_in_one_launch_give_the_bits_of_two_launches(mode, roomy):
    """16-row tiles: a 2-bit pool and an 8-bit pool of one mode ride one launch (the default) or one
    launch per index width (widths_apart); the same work either way.  The 8-bit table is a 256-entry
    fp16 grid in WxA16 and the identity idx - 128 in WxA8."""
    from dartmoq_hip import ops
    k, inter = 512, 128
    counts0, counts1 = [5, 40, 0, 17], [21, 2]
    r0, r1 = sum(counts0), sum(counts1)
    rows = r0 + r1
    g = torch.Generator().manual_seed(91 + mode)
    x_rot = torch.randn(rows, k, generator=g) * 0.7
    cb2 = codebook.get_codebook(2)[0].half()
    act, scale, _, _, lut2, _, _, _, wsb = _mode_inputs(mode, x_rot, cb2)
    lut8 = None if mode == A8 else (torch.arange(256).float() - 128).mul(3.0 / 128).half()
    pools, infos = [], []
    for pi, (bit, counts, first_row, lut) in enumerate([(2, counts0, 0, lut2), (8, counts1, r0, lut8)]):
        idx_gf, norms_gf, _ = _pool(2, 2 * inter * len(counts), k, 400 + pi)
        if bit == 8:                                   # one index byte per weight
            idx_gf = torch.randint(0, 256, (k // 128, 2 * inter * len(counts), 128), dtype=torch.uint8,
                                   generator=g)
        starts = [first_row + sum(counts[:e]) for e in range(len(counts))]
        info = torch.tensor([(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(len(counts))],
                            dtype=torch.int32).cuda()
        infos.append(info)
        pools.append(dict(w=idx_gf.cuda(), norms=norms_gf.cuda(), lut=None if lut is None else lut.cuda(),
                          expert_info=info, act=act.cuda(), act_scale=None if scale is None else scale.cuda(),
                          row_index=None, bit=bit, mode=mode, w_scale_byte=wsb))
    lists = [ops.build_tiles(infos[pi], rows, 16, pool=pi) for pi in range(2)]
    n = [int(l[0][0]) for l in lists]
    items = torch.cat([lists[0][1][:n[0]], lists[1][1][:n[1]]]).contiguous()
    n_items = torch.tensor([n[0] + n[1], 0, 0, 0], dtype=torch.int32).cuda()
    common = dict(groups=k // 128, n_out=inter, half_width=inter, slice_is_groups=False, tt=1,
                  out_stride=inter, act_row_bytes=act.element_size() * k,
                  act_scale_stride=0 if scale is None else scale.stride(0), roomy=roomy)
    one = torch.full((rows, inter), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_pools(mode, SILU, pools, items, n_items, items.shape[0], out=one, **common)
    two = torch.full((rows, inter), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_pools(mode, SILU, pools, items, n_items, items.shape[0], out=two, widths_apart=1, **common)
    torch.cuda.synchronize()
    assert not torch.isnan(one.float()).any()
    assert torch.equal(one, two)
    # K shared by 2 or 4 workgroups per block (partial sums added in fp32 by the last to arrive):
    # the same sums in another order
    for apart in (0, 1):
        for share in (2, 4):
            got = torch.full((rows, inter), float("nan"), dtype=torch.float16, device="cuda")
            ops.matmul_pools(mode, SILU, pools, items, n_items, items.shape[0], out=got, widths_apart=apart,
                             k_split=share, rows_total=rows, **common)
            torch.cuda.synchronize()
            torch.testing.assert_close(got.float(), one.float(), rtol=2e-3,
                                       atol=2e-3 * one.float().abs().max().item())


@pytest.mark.parametrize("mode", [A16, A8])
def test_k_shared_for_the_leading_items_only(mode):
    """16-row tiles, a list that begins with the items of a 4-bit pool (n_items[1] of them) followed
    by those of a 2-bit pool: with k_split_items the leading items share K between four workgroups
    and give the bits of a launch that shares every item, the others run one workgroup per block
    and give the bits of a launch that shares nothing."""
    from dartmoq_hip import ops
    k, inter = 1024, 256
    counts0, counts1 = [3, 0, 20], [5, 40, 0, 17, 1]
    r0, r1 = sum(counts0), sum(counts1)
    rows = r0 + r1
    g = torch.Generator().manual_seed(17 + mode)
    x_rot = torch.randn(rows, k, generator=g) * 0.7
    pools, infos = [], []
    act = scale = None
    for pi, (bit, counts, first_row) in enumerate([(4, counts0, 0), (2, counts1, r0)]):
        cb = codebook.get_codebook(bit)[0].half()
        act, scale, _, _, lut, _, _, _, wsb = _mode_inputs(mode, x_rot, cb)
        idx_gf, norms_gf, _ = _pool(bit, 2 * inter * len(counts), k, 500 + pi)
        starts = [first_row + sum(counts[:e]) for e in range(len(counts))]
        info = torch.tensor([(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(len(counts))],
                            dtype=torch.int32).cuda()
        infos.append(info)
        pools.append(dict(w=idx_gf.cuda(), norms=norms_gf.cuda(), lut=lut.cuda(), expert_info=info,
                          act=act.cuda(), act_scale=None if scale is None else scale.cuda(),
                          row_index=None, bit=bit, mode=mode, w_scale_byte=wsb))
    lists = [ops.build_tiles(infos[pi], rows, 16, pool=pi) for pi in range(2)]
    n = [int(l[0][0]) for l in lists]
    items = torch.cat([lists[0][1][:n[0]], lists[1][1][:n[1]]]).contiguous()
    n_items = torch.tensor([n[0] + n[1], n[0], 0, 0], dtype=torch.int32).cuda()
    common = dict(groups=k // 128, n_out=inter, half_width=inter, slice_is_groups=False, tt=1,
                  out_stride=inter, act_row_bytes=act.element_size() * k,
                  act_scale_stride=0 if scale is None else scale.stride(0))

    def run(**kw):
        out = torch.full((rows, inter), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_pools(mode, SILU, pools, items, n_items, items.shape[0] + 3, out=out, **common, **kw)
        torch.cuda.synchronize()
        assert not torch.isnan(out.float()).any()
        return out

    none = run()
    every = run(k_split=4, rows_total=rows)
    for bound in (n[0], n[0] + 2, 1):
        lead = run(k_split=4, rows_total=rows, k_split_items=bound)
        if bound >= n[0]:
            assert torch.equal(lead[:r0], every[:r0])
            assert torch.equal(lead[r0:], none[r0:])
        else:        # a bound below the prefix count: only that many items are shared
            first = int(items[0, 4])                       # rows of the first item
            assert torch.equal(lead[:first], every[:first])
            assert torch.equal(lead[first:], none[first:])
    torch.testing.assert_close(every.float(), none.float(), rtol=2e-3, atol=2e-3 * none.float().abs().max().item())


@pytest.mark.parametrize("mode", [A16, A8, FP8, FP4])
@pytest.mark.parametrize("bit", [1, 2, 4])
def test_merged_in_features_down(mode, bit):
    counts = [5, 33, 0, 16]
    out, ref = _run_case(mode, bit, 1, counts, k=256, n_slice=256, slice_is_groups=True,
                         seed=200 + 10 * mode + bit)
    torch.testing.assert_close(out, ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("tt", [1, 2, 4])
@pytest.mark.parametrize("bit", [1, 2, 4])
def test_wxa8_int32_accumulators_exact(bit, tt):
    """Per-group int32 accumulators of the i8 matrix cores equal an int64 numpy matmul, in the
    16-, 32- and 64-row kernels (the last two serve the prefill batches); full-range int8 codes."""
    from dartmoq_hip import ops
    counts = [7, 20, 1, 70, 0, 130]
    k, n_slice = 384, 128
    starts, rows_total = _expert_rows(counts)
    idx_gf, norms_gf, cb = _pool(bit, n_slice * len(counts), k, 300 + bit)
    q_lut, step = luts.build_int8_codebook(cb)
    g = torch.Generator().manual_seed(bit)
    codes, s = actquant.quantize_act_int8(torch.randn(rows_total, k, generator=g), 128, step)
    info = [(starts[e], counts[e], e * n_slice, n_slice) for e in range(len(counts))]
    dbg = torch.zeros(rows_total, k // 128, n_slice, dtype=torch.int32, device="cuda")
    ops.matmul_merged(A8, bit, STORE, codes.cuda(), s.half().cuda(), idx_gf.cuda(), norms_gf.cuda(),
                      q_lut.cuda(), torch.tensor(info, dtype=torch.int32).cuda(), groups=k // 128,
                      n_out=n_slice, slice_is_groups=False, rows_total=rows_total, tt=tt, ks=1, dbg_acc=dbg)
    torch.cuda.synchronize()
    w = q_lut.long()[packing.unpack_nbit(idx_gf, bit, 128).long()]          # [G, N, 128]
    for e, (ts, cnt, ss, sc) in enumerate(info):
        if cnt == 0:
            continue
        a = codes[ts:ts + cnt].long().reshape(cnt, k // 128, 128)
        ref = torch.einsum("bgk,gnk->bgn", a, w[:, ss:ss + sc])
        assert torch.equal(dbg[ts:ts + cnt].cpu().long(), ref)


def test_silu_and_scatter_epilogues():
    """gate_up with fused SiLU*up and down with fused weight + scatter-add (WxA16, 2-bit)."""
    from dartmoq_hip import ops
    bit, k, inter, hidden = 2, 256, 128, 256
    counts = [9, 40, 2]                        # 51 rows = 17 tokens x 3 slots
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(5)
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter * len(counts), k, 41)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half()
    info = [(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(len(counts))]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    common = dict(groups=k // 128, slice_is_groups=False, rows_total=rows_total, tt=1)
    gu = ops.matmul_merged(A16, bit, STORE, x.cuda(), None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(),
                           info_dev, n_out=2 * inter, **common).float().cpu()
    act = ops.matmul_merged(A16, bit, SILU, x.cuda(), None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(),
                            info_dev, n_out=inter, half_width=inter, **common).float().cpu()
    ref_act = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    torch.testing.assert_close(act, ref_act, rtol=4e-3, atol=4e-3 * ref_act.abs().max().item())

    # scatter: routing-weighted rows land in their (token, slot) rows, combine adds the slots
    didx, dnorms, dcb = _pool(bit, hidden, inter * len(counts), 43)
    a = (torch.randn(rows_total, inter, generator=g) * 0.5).half()
    dinfo = [(starts[e], counts[e], e * (inter // 128), inter // 128) for e in range(len(counts))]
    dinfo_dev = torch.tensor(dinfo, dtype=torch.int32).cuda()
    top_k = 3
    slot = torch.randperm(rows_total, generator=g).int()          # rows_total == 17 tokens * 3
    wts = torch.rand(rows_total, generator=g)
    dcommon = dict(groups=inter // 128, n_out=hidden, slice_is_groups=True, rows_total=rows_total, tt=1)
    dn = ops.matmul_merged(A16, bit, STORE, a.cuda(), None, didx.cuda(), dnorms.cuda(), dcb.cuda(),
                           dinfo_dev, **dcommon).float().cpu()
    slots = torch.full((rows_total, hidden), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_merged(A16, bit, SCATTER, a.cuda(), None, didx.cuda(), dnorms.cuda(), dcb.cuda(),
                      dinfo_dev, out=slots, out_stride=hidden, row_weight=wts.cuda(),
                      row_slot=slot.cuda(), **dcommon)
    out = ops.combine_slots(slots, top_k).float().cpu()
    ref_slots = torch.zeros(rows_total, hidden)
    ref_slots[slot.long()] = dn * wts.unsqueeze(1)
    ref = ref_slots.reshape(rows_total // top_k, top_k, hidden).sum(1)
    torch.testing.assert_close(out, ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("tt,ks", [(1, 4), (1, 1), (2, 1), (4, 1)])
def test_k_split_variants_agree(tt, ks):
    """Every (row tile, K split) instantiation computes the same GEMM."""
    from dartmoq_hip import ops
    bit, k, n_slice = 2, 1024, 256
    counts = [3, 70, 0, 21]
    starts, rows_total = _expert_rows(counts)
    idx_gf, norms_gf, cb = _pool(bit, n_slice * len(counts), k, 77)
    g = torch.Generator().manual_seed(tt * 10 + ks)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half()
    info = [(starts[e], counts[e], e * n_slice, n_slice) for e in range(len(counts))]
    out = ops.matmul_merged(A16, bit, STORE, x.cuda(), None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(),
                            torch.tensor(info, dtype=torch.int32).cuda(), groups=k // 128,
                            n_out=n_slice, slice_is_groups=False, rows_total=rows_total, tt=tt, ks=ks)
    w = cb.float()[packing.unpack_nbit(idx_gf, bit, 128).long()]
    ref = torch.zeros(rows_total, n_slice)
    for e, (ts, cnt, ss, sc) in enumerate(info):
        wl = w[:, ss:ss + sc].permute(1, 0, 2).reshape(n_slice, -1)
        ref[ts:ts + cnt] = moe.lut_gemm(x[ts:ts + cnt].float(), torch.ones(cnt, k // 128), wl,
                                        norms_gf[:, ss:ss + sc].float().t(), 128)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=2e-3, atol=2e-3 * ref.abs().max().item())


@pytest.mark.parametrize("tt", [1, 2, 4])
@pytest.mark.parametrize("epi", ["silu", "store", "scatter"])
def test_blocks_per_workgroup_identical(tt, epi):
    """A workgroup walking 2, 3 or all feature blocks stores exactly what one block per
    workgroup stores (same arithmetic, only the schedule differs)."""
    from dartmoq_hip import ops
    bit, k = 2, 512
    counts = [5, 70, 0, 33]
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(900 + tt)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half().cuda()
    if epi == "silu":
        inter = 512                                            # 4 blocks of 128 features
        idx_gf, norms_gf, cb = _pool(bit, 2 * inter * len(counts), k, 91)
        info = [(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(len(counts))]
        kw = dict(n_out=inter, half_width=inter, slice_is_groups=False)
        mode_epi = SILU
    else:
        n_slice = 1024                                         # 4 blocks of 256 features
        idx_gf, norms_gf, cb = _pool(bit, n_slice * len(counts), k, 92)
        info = [(starts[e], counts[e], e * n_slice, n_slice) for e in range(len(counts))]
        kw = dict(n_out=n_slice, slice_is_groups=False)
        mode_epi = STORE if epi == "store" else SCATTER
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    slot = torch.randperm(rows_total, generator=g).int().cuda()
    wts = torch.rand(rows_total, generator=g).cuda()
    outs = []
    for nbl in (1, 2, 3, 4):
        extra = {}
        if mode_epi == SCATTER:
            extra = dict(out=torch.zeros(rows_total, kw["n_out"], dtype=torch.float16, device="cuda"),
                         out_stride=kw["n_out"], row_weight=wts, row_slot=slot)
        out = ops.matmul_merged(A16, bit, mode_epi, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(),
                                info_dev, groups=k // 128, rows_total=rows_total, tt=tt, ks=1, nbl=nbl,
                                **kw, **extra)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    assert outs[0].abs().max() > 0
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


def test_gemm_argument_errors():
    from dartmoq_hip import ops
    x = torch.zeros(16, 256, dtype=torch.float16, device="cuda")
    idx_gf, norms_gf, cb = _pool(2, 128, 256, 1)
    info = torch.tensor([[0, 16, 0, 128]], dtype=torch.int32).cuda()
    with pytest.raises(ValueError):            # unsupported bit width
        ops.matmul_merged(A16, 3, STORE, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info,
                          groups=2, n_out=128, slice_is_groups=False, rows_total=16, tt=1)
    with pytest.raises(ValueError):            # n_out not a multiple of the wave tile
        ops.matmul_merged(A16, 2, STORE, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info,
                          groups=2, n_out=100, slice_is_groups=False, rows_total=16, tt=1)
    with pytest.raises(ValueError):            # activation rows shorter than groups * 128
        ops.matmul_merged(A16, 2, STORE, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info,
                          groups=4, n_out=128, slice_is_groups=False, rows_total=16, tt=1)


@pytest.mark.parametrize("mode,bit", [(A16, 2), (A8, 2), (FP8, 2), (FP4, 2), (A16, 8), (A8, 8)])
@pytest.mark.parametrize("tt,nbl", [(1, 1), (2, 2), (4, 1)])
def test_fused_down_rotation_equals_separate_kernels(mode, bit, tt, nbl):
    """DMQ_EPI_SILU_ROT: the gate_up GEMM hands over the rotated (+ quantized) input of the down
    projection.  It must be bit for bit what the SiLU epilogue followed by the per-expert rotation
    kernel produces (same fp16 SiLU*up rows, same MFMA order, same quantizer).  8-bit pools: a
    256-entry fp16 grid in WxA16, the identity idx - 128 (no table) in WxA8."""
    from dartmoq_hip import ops
    from dartmoq_hip._lib import EPI_SILU_ROT
    k, inter = 256, 256
    counts = [9, 70, 0, 33]
    n_exp = len(counts)
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(17 + mode)
    idx_gf, norms_gf, cb = _pool(2, 2 * inter * n_exp, k, 91)
    x_rot = torch.randn(rows_total, k, generator=g) * 0.7
    act, scale, _oc, _os, lut, _ol, _wbs, nfac, wsb = _mode_inputs(mode, x_rot, cb)
    if bit == 8:                                       # one index byte per weight
        idx_gf = torch.randint(0, 256, (k // 128, 2 * inter * n_exp, 128), dtype=torch.uint8, generator=g)
        lut = None if mode == A8 else (torch.arange(256).float() - 128).mul(3.0 / 128).half()
    norms_used = (norms_gf.float() * nfac).half() if mode == FP4 else norms_gf
    w_dev = idx_gf.cuda()
    if mode == FP4:
        w_dev = ops.fold_indices_to_e2m1(w_dev, lut, bit)
    info = [(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(n_exp)]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    dinfo = [(starts[e], counts[e], e * (inter // 128), inter // 128) for e in range(n_exp)]
    dinfo_dev = torch.tensor(dinfo, dtype=torch.int32).cuda()
    rot = (torch.randn(n_exp * inter // 128, 128, 128, generator=g) / 128 ** 0.5).half().cuda()
    extra = 0.37
    tiling = ops.build_tiles(info_dev, rows_total, 16 * tt)
    n_items, items, max_items = tiling
    common = dict(groups=k // 128, n_out=inter, half_width=inter, slice_is_groups=False,
                  rows_total=rows_total, w_scale_byte=wsb, tt=tt, nbl=nbl, tiling=tiling)
    args = (mode, bit)
    tens = (act.cuda(), None if scale is None else scale.cuda(), w_dev, norms_used.cuda(),
            None if (mode == FP4 or lut is None) else lut.cuda(), info_dev)
    silu = ops.matmul_merged(*args, SILU, *tens, **common)
    # the rotation kernel takes the down slice of an expert from its own work items
    dn_items, ditems, dmax = ops.build_tiles(dinfo_dev, rows_total, 16 * tt)
    want_codes, want_scale = ops.rotate_tiled(mode, silu, rot, dinfo_dev, dn_items, ditems, 16 * tt,
                                              dmax, rows_total, rot_per_expert=True,
                                              extra_scale=extra, tt=tt)
    codes, sc, _ = ops._alloc_codes(mode, rows_total, inter, "cuda", False)
    codes.view(torch.uint8).fill_(0x5a)
    want = want_codes.clone()
    ops.matmul_merged(*args, EPI_SILU_ROT, *tens, out=silu, out_stride=inter,
                      post=dict(rot=[rot], extra=[extra], out=codes, scale=sc), **common)
    torch.cuda.synchronize()
    assert torch.equal(codes.view(torch.uint8), want.view(torch.uint8))
    if sc is not None:
        assert torch.equal(sc.view(torch.uint8), want_scale.view(torch.uint8))
    if tt == 1 and bit != 8 and mode != FP4:
        # the two-per-CU instance (256-byte table rows, look-ups of the next group issued ahead)
        codes2, sc2, _ = ops._alloc_codes(mode, rows_total, inter, "cuda", False)
        codes2.view(torch.uint8).fill_(0x5a)
        ops.matmul_merged(*args, EPI_SILU_ROT, *tens, out=silu, out_stride=inter, roomy=1,
                          post=dict(rot=[rot], extra=[extra], out=codes2, scale=sc2), **common)
        torch.cuda.synchronize()
        assert torch.equal(codes2.view(torch.uint8), want.view(torch.uint8))
        if sc2 is not None:
            assert torch.equal(sc2.view(torch.uint8), want_scale.view(torch.uint8))


@pytest.mark.parametrize("mode", [A16, A8, FP4])
@pytest.mark.parametrize("tt,item_rows", [(1, 64), (2, 64), (1, 32)])
def test_work_items_larger_than_the_launch_tile(mode, tt, item_rows):
    """item_tile_rows: one work-item list (64- or 32-row items) serves a launch with smaller row
    tiles; every item is walked as item_tile_rows / (16 tt) tiles and the output equals, bit for
    bit, the launch over items of its own tile size (ragged counts, an empty expert, counts that
    end inside the first sub-tile)."""
    from dartmoq_hip import ops
    bit, k, n_slice = 2, 256, 128
    counts = [70, 3, 0, 33, 64, 17]
    n_exp = len(counts)
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(23 + mode)
    idx_gf, norms_gf, cb = _pool(bit, n_slice * n_exp, k, 5)
    x_rot = torch.randn(rows_total, k, generator=g) * 0.7
    act, scale, _oc, _os, lut, _ol, _wbs, nfac, wsb = _mode_inputs(mode, x_rot, cb)
    norms_used = (norms_gf.float() * nfac).half() if mode == FP4 else norms_gf
    w_dev = idx_gf.cuda()
    if mode == FP4:
        w_dev = ops.fold_indices_to_e2m1(w_dev, lut, bit)
    info = torch.tensor([(starts[e], counts[e], e * n_slice, n_slice) for e in range(n_exp)],
                        dtype=torch.int32).cuda()
    args = (mode, bit, STORE, act.cuda(), None if scale is None else scale.cuda(), w_dev,
            norms_used.cuda(), None if mode == FP4 else lut.cuda(), info)
    kw = dict(groups=k // 128, n_out=n_slice, slice_is_groups=False, rows_total=rows_total,
              w_scale_byte=wsb, tt=tt)
    own = ops.matmul_merged(*args, **kw)
    big = ops.matmul_merged(*args, item_tile_rows=item_rows, **kw)
    torch.cuda.synchronize()
    assert torch.equal(own, big)
    with pytest.raises(ValueError):                 # not a multiple of the launch tile
        ops.matmul_merged(*args, item_tile_rows=48, **dict(kw, tt=2))


@pytest.mark.parametrize("bit", [1, 2, 4])
@pytest.mark.parametrize("k,inter", [(512, 128), (1024, 256), (2048, 512), (3072, 256), (4096, 128)])
def test_dot_product_launch_for_a_few_rows_per_expert(bit, k, inter):
    """Decode steps of at most four tokens: the vector-ALU launch (gemv) against the MFMA launch and
    against fp32 maths, gate_up with SiLU * up and down with weight + scatter.  Experts with one to
    four rows and an expert with none."""
    from dartmoq_hip import ops
    counts = [1, 4, 0, 2, 3, 1]
    n_exp = len(counts)
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(100 + bit + k)
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter * n_exp, k, 7 + bit)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half()
    info = [(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(n_exp)]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    args = (A16, bit, SILU, x.cuda(), None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev)
    common = dict(groups=k // 128, slice_is_groups=False, rows_total=rows_total, tt=1, n_out=inter,
                  half_width=inter)
    mfma = ops.matmul_merged(*args, **common).float().cpu()
    got = ops.matmul_merged(*args, gemv=True, **common).float().cpu()
    w = (cb.float()[packing.unpack_nbit(idx_gf, bit, 128).long()] * norms_gf.float().unsqueeze(-1))
    ref = torch.zeros(rows_total, inter)
    for e, (ts, cnt, ss, sc) in enumerate(info):
        we = w[:, ss:ss + sc].permute(1, 0, 2).reshape(sc, k)
        gu = x[ts:ts + cnt].float() @ we.t()
        ref[ts:ts + cnt] = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    scale = ref.abs().max().item()
    torch.testing.assert_close(got, ref, rtol=2e-3, atol=2e-3 * scale)
    torch.testing.assert_close(got, mfma, rtol=4e-3, atol=4e-3 * scale)

    # down: K = k again (groups of the expert's slice), n_out = 256 features, scattered
    hidden, top_k = 256, 1
    didx, dnorms, dcb = _pool(bit, hidden, k * n_exp, 9 + bit)
    a = (torch.randn(rows_total, k, generator=g) * 0.5).half()
    dinfo = [(starts[e], counts[e], e * (k // 128), k // 128) for e in range(n_exp)]
    dinfo_dev = torch.tensor(dinfo, dtype=torch.int32).cuda()
    slot = torch.randperm(rows_total, generator=g).int()
    wts = torch.rand(rows_total, generator=g)
    dargs = (A16, bit, SCATTER, a.cuda(), None, didx.cuda(), dnorms.cuda(), dcb.cuda(), dinfo_dev)
    dcommon = dict(groups=k // 128, n_out=hidden, slice_is_groups=True, rows_total=rows_total, tt=1,
                   out_stride=hidden, row_weight=wts.cuda(), row_slot=slot.cuda())
    outs = []
    for gemv in (False, True):
        slots = torch.full((rows_total, hidden), float("nan"), dtype=torch.float16, device="cuda")
        ops.matmul_merged(*dargs, out=slots, gemv=gemv, **dcommon)
        outs.append(slots.float().cpu())
    dw = (dcb.float()[packing.unpack_nbit(didx, bit, 128).long()] * dnorms.float().unsqueeze(-1))
    dref = torch.zeros(rows_total, hidden)
    for e, (ts, cnt, ss, sc) in enumerate(dinfo):
        we = dw[ss:ss + sc].permute(1, 0, 2).reshape(hidden, k)
        dref[slot[ts:ts + cnt].long()] = (a[ts:ts + cnt].float() @ we.t()) * wts[ts:ts + cnt].unsqueeze(1)
    dscale = dref.abs().max().item()
    torch.testing.assert_close(outs[1], dref, rtol=2e-3, atol=2e-3 * dscale)
    torch.testing.assert_close(outs[1], outs[0], rtol=4e-3, atol=4e-3 * dscale)


def test_dot_product_launch_rejects_what_it_does_not_cover():
    from dartmoq_hip import ops
    bit, k, inter = 2, 640, 128                               # 5 groups: not a multiple of 4
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter, k, 3)
    x = torch.zeros(1, k).half().cuda()
    info_dev = torch.tensor([(0, 1, 0, 2 * inter)], dtype=torch.int32).cuda()
    with pytest.raises(ValueError):
        ops.matmul_merged(A16, bit, SILU, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev,
                          groups=k // 128, slice_is_groups=False, rows_total=1, tt=1, n_out=inter,
                          half_width=inter, gemv=True)
    # 8-bit pools, activation-quantized modes and 32-row tiles keep the MFMA launch
    k = 512
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter, k, 3)
    x = torch.zeros(1, k).half().cuda()
    common = dict(groups=k // 128, slice_is_groups=False, rows_total=1, n_out=inter, half_width=inter, gemv=True)
    idx8 = torch.zeros((k // 128, 2 * inter, 128), dtype=torch.uint8)
    lut8 = (torch.arange(256).float() - 128).mul(3.0 / 128).half()
    with pytest.raises(ValueError):
        ops.matmul_merged(A16, 8, SILU, x, None, idx8.cuda(), norms_gf.cuda(), lut8.cuda(), info_dev, tt=1, **common)
    with pytest.raises(ValueError):
        ops.matmul_merged(A16, bit, SILU, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev, tt=2, **common)
    codes = torch.zeros(1, k, dtype=torch.int8).cuda()
    with pytest.raises(ValueError):
        ops.matmul_merged(A8, bit, SILU, codes, torch.ones(1, k // 128).half().cuda(), idx_gf.cuda(),
                          norms_gf.cuda(), torch.zeros(4, dtype=torch.int8).cuda(), info_dev, tt=1, **common)
    # planes of the wrong width or too few planes
    from dartmoq_hip._lib import EPI_SILU_ROT
    rot = torch.zeros(1, 128, 128).half().cuda()
    dummy = torch.empty((1, inter), dtype=torch.float16, device="cuda")
    post = dict(rot=[rot], extra=[1.0], out=dummy, scale=None)
    with pytest.raises(ValueError):
        ops.matmul_merged(A16, bit, EPI_SILU_ROT, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev,
                          tt=1, out=dummy, out_stride=inter, post=post,
                          gemv_planes=torch.zeros(2, 1, 2 * inter, device="cuda"), **common)
    with pytest.raises(ValueError):
        ops.matmul_merged(A16, bit, EPI_SILU_ROT, x, None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev,
                          tt=1, out=dummy, out_stride=inter, post=post,
                          gemv_planes=torch.zeros(1, 1, inter, device="cuda"), **common)


@pytest.mark.parametrize("bit", [1, 2, 4])
@pytest.mark.parametrize("k,inter", [(512, 512), (1024, 1024), (2048, 512), (3072, 128)])
def test_dot_product_launch_with_the_down_rotation_fused(bit, k, inter):
    """The dot-product gate_up launch hands the rotated input of the down projection over as fp32
    planes of partial sums; the dot-product down launch adds them up.  The sum of the planes is the
    stand-alone rotation of the launch's own SiLU*up rows up to the order of the fp32 sums, the
    down launch fed with planes equals the down launch fed with that sum rounded to fp16 bit for
    bit, and a second run gives the same bits."""
    from dartmoq_hip import ops
    from dartmoq_hip._lib import EPI_SILU_ROT
    counts = [2, 0, 4, 1, 3]
    n_exp = len(counts)
    starts, rows_total = _expert_rows(counts)
    g = torch.Generator().manual_seed(300 + bit + k)
    idx_gf, norms_gf, cb = _pool(bit, 2 * inter * n_exp, k, 17 + bit)
    x = (torch.randn(rows_total, k, generator=g) * 0.5).half()
    info = [(starts[e], counts[e], e * 2 * inter, 2 * inter) for e in range(n_exp)]
    info_dev = torch.tensor(info, dtype=torch.int32).cuda()
    dinfo = [(starts[e], counts[e], e * (inter // 128), inter // 128) for e in range(n_exp)]
    dinfo_dev = torch.tensor(dinfo, dtype=torch.int32).cuda()
    rot = (torch.randn(n_exp * inter // 128, 128, 128, generator=g) / 128 ** 0.5).half().cuda()
    tiling = ops.build_tiles(info_dev, rows_total, 16)
    common = dict(groups=k // 128, n_out=inter, half_width=inter, slice_is_groups=False,
                  rows_total=rows_total, tt=1, tiling=tiling, gemv=True)
    tens = (x.cuda(), None, idx_gf.cuda(), norms_gf.cuda(), cb.cuda(), info_dev)
    silu = ops.matmul_merged(A16, bit, SILU, *tens, **common)
    dn_tiling = ops.build_tiles(dinfo_dev, rows_total, 16)
    dn_items, ditems, dmax = dn_tiling
    want, _ = ops.rotate_tiled(A16, silu, rot, dinfo_dev, dn_items, ditems, 16, dmax, rows_total,
                               rot_per_expert=True, extra_scale=1.0, tt=1)
    n_planes = ops.gemv_plane_count(k // 128)
    runs = []
    for _ in range(2):
        planes = torch.full((n_planes, rows_total, inter), float("nan"), device="cuda")
        dummy = torch.empty((rows_total, inter), dtype=torch.float16, device="cuda")
        ops.matmul_merged(A16, bit, EPI_SILU_ROT, *tens, out=dummy, out_stride=inter,
                          post=dict(rot=[rot], extra=[1.0], out=dummy, scale=None),
                          gemv_planes=planes, **common)
        torch.cuda.synchronize()
        runs.append(planes.clone())
    assert torch.equal(runs[0].view(torch.int32), runs[1].view(torch.int32))
    got = runs[0].sum(0)
    scale = want.float().abs().max().item()
    torch.testing.assert_close(got, want.float(), rtol=2e-3, atol=2e-3 * scale)

    # the down launch: planes in, against the same launch fed with the fp16 sum of the planes
    hidden = 256
    didx, dnorms, dcb = _pool(bit, hidden, inter * n_exp, 19 + bit)
    if not _gemv_groups_ok(inter // 128):                    # the down launch covers 4, 8, 16, 24, 32 groups
        return
    summed = runs[0][0].clone()
    for pl in range(1, n_planes):
        summed += runs[0][pl]
    slot = torch.randperm(rows_total, generator=g).int().cuda()
    wts = torch.rand(rows_total, generator=g).cuda()
    dargs = (A16, bit, SCATTER)
    dtens = (None, didx.cuda(), dnorms.cuda(), dcb.cuda(), dinfo_dev)
    dcommon = dict(groups=inter // 128, n_out=hidden, slice_is_groups=True, rows_total=rows_total, tt=1,
                   out_stride=hidden, row_weight=wts, row_slot=slot, tiling=dn_tiling, gemv=True)
    a = torch.full((rows_total, hidden), float("nan"), dtype=torch.float16, device="cuda")
    b = torch.full((rows_total, hidden), float("nan"), dtype=torch.float16, device="cuda")
    ops.matmul_merged(*dargs, summed.half(), *dtens, out=a, **dcommon)
    ops.matmul_merged(*dargs, dummy, *dtens, out=b, gemv_planes=runs[0], **dcommon)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
