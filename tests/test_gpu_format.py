"""GPU parity: packed format kernels (bit-exact against the oracle)."""

import math

import pytest
import torch

from oracle import codebook, luts, packing

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_unpack_bit_exact(bit):
    from dartmoq_hip import ops
    g = torch.Generator().manual_seed(bit)
    packed = torch.randint(0, 256, (37, 96), dtype=torch.uint8, generator=g)
    ref = packing.unpack_nbit(packed, bit, 96 * 8 // bit).to(torch.uint8)
    got = ops.unpack_nbit(packed.cuda(), bit).cpu()
    assert torch.equal(got, ref)


@pytest.mark.parametrize("bit", [1, 2, 4])
def test_group_first_and_prescale_bit_exact(bit):
    from dartmoq_hip import ops
    g = torch.Generator().manual_seed(10 + bit)
    n_rows, groups = 48, 5
    ppg = 128 * bit // 8
    idx = torch.randint(0, 256, (n_rows, groups * ppg), dtype=torch.uint8, generator=g)
    norms = (torch.rand(n_rows, groups, generator=g) * 3 + 0.01).half()
    ref_idx, ref_norms = packing.convert_to_group_first(idx, norms, 128, bit)
    got_idx, got_norms = ops.convert_to_group_first(idx.cuda(), norms.cuda(), 128, bit)
    assert torch.equal(got_idx.cpu(), ref_idx)
    assert torch.equal(got_norms.cpu().view(torch.int16), ref_norms.view(torch.int16))
    # pre-division by sqrt(128) is evaluated on the fp16 tensor like the reference does
    _, got_scaled = ops.convert_to_group_first(idx.cuda(), norms.cuda(), 128, bit, prescale=True)
    ref_scaled = ref_norms / math.sqrt(128)
    assert torch.equal(got_scaled.cpu().view(torch.int16), ref_scaled.view(torch.int16))


@pytest.mark.parametrize("bit", [1, 2, 4])
def test_dequant_tile_bit_exact(bit):
    """Dequantized weight tiles: codebook[idx] must come out bit for bit."""
    from dartmoq_hip import ops
    g = torch.Generator().manual_seed(20 + bit)
    groups, n_rows = 3, 80
    ppg = 128 * bit // 8
    idx_gf = torch.randint(0, 256, (groups, n_rows, ppg), dtype=torch.uint8, generator=g)
    cb = codebook.get_codebook(bit)[0].half()
    idx = packing.unpack_nbit(idx_gf, bit, 128).long()
    ref = cb[idx]                                            # [G, N, 128]
    got = ops.dequant_tile(idx_gf.cuda(), cb.cuda(), None, 1, 2, 16, 48, bit).cpu()
    assert torch.equal(got.view(torch.int16), ref[1:3, 16:64].contiguous().view(torch.int16))
    norms = (torch.rand(groups, n_rows, generator=g) + 0.05).half()
    got_n = ops.dequant_tile(idx_gf.cuda(), cb.cuda(), norms.cuda(), 0, 3, 0, 80, bit).cpu()
    ref_n = (ref.float() * norms.float().unsqueeze(-1)).half()
    assert torch.equal(got_n.view(torch.int16), ref_n.view(torch.int16))


@pytest.mark.parametrize("bit", [1, 2, 4])
def test_fold_to_e2m1_bit_exact(bit):
    from dartmoq_hip import ops
    g = torch.Generator().manual_seed(30 + bit)
    idx_gf = torch.randint(0, 256, (2, 33, 128 * bit // 8), dtype=torch.uint8, generator=g)
    nib, _e0, _res, _err = luts.build_e2m1_codebook(codebook.get_codebook(bit)[0].half())
    ref = luts.fold_indices_to_e2m1(idx_gf, nib, bit, 128)
    got = ops.fold_indices_to_e2m1(idx_gf.cuda(), nib, bit).cpu()
    assert torch.equal(got, ref)


def test_bad_bit_width_raises():
    from dartmoq_hip import ops
    with pytest.raises(ValueError):
        ops.unpack_nbit(torch.zeros(4, 4, dtype=torch.uint8, device="cuda"), 3)
    with pytest.raises(ValueError):
        ops.fold_indices_to_e2m1(torch.zeros(1, 1, 16, dtype=torch.uint8, device="cuda"),
                                 torch.zeros(256, dtype=torch.uint8), 8)
