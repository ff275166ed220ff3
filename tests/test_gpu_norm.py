"""GPU parity: RMSNorm in front of the MoE block against the oracle's torch formula."""

import pytest
import torch

from oracle import norm

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,n", [(1, 2048), (77, 3072), (300, 128), (16, 256), (5, 8)])
@pytest.mark.parametrize("w32", [False, True])
def test_rms_norm_matches_oracle(dtype, rows, n, w32):
    from dartmoq_hip import kernels as K
    g = torch.Generator().manual_seed(rows + n)
    x = (torch.randn(rows, n, generator=g) * 3).to(dtype)
    w = (torch.randn(n, generator=g) * 0.1).to(torch.float32 if w32 else dtype)
    ref = norm.rms_norm(x, w, 1e-6)
    out = K.rms_norm(x.cuda(), w.cuda(), 1e-6)
    assert out.dtype == dtype and out.shape == x.shape
    # fp32 inside, one rounding: at most one unit in the last place of the output type where the
    # sum of squares was accumulated in another order
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=ulp, atol=1e-6)
    assert (out.cpu() == ref).float().mean() > 0.99


def test_rms_norm_strided_rows_and_errors():
    from dartmoq_hip import kernels as K
    g = torch.Generator().manual_seed(3)
    big = torch.randn(40, 512, generator=g).half()
    view = big[:, :256]                                  # row stride 512, 256 contiguous elements
    w = torch.zeros(256).half()
    out = K.rms_norm(view.cuda(), w.cuda(), 1e-6)
    torch.testing.assert_close(out.cpu().float(), norm.rms_norm(view, w, 1e-6).float(), rtol=2.0 ** -10, atol=1e-6)
    x3 = torch.randn(2, 3, 128, generator=g).half()
    assert K.rms_norm(x3.cuda(), torch.zeros(128).half().cuda(), 1e-6).shape == (2, 3, 128)
    with pytest.raises(TypeError):
        K.rms_norm(torch.zeros(2, 128, device="cuda"), torch.zeros(128, device="cuda"), 1e-6)
    with pytest.raises(ValueError):
        K.rms_norm(torch.zeros(2, 128, dtype=torch.float16, device="cuda"),
                   torch.zeros(64, dtype=torch.float16, device="cuda"), 1e-6)
    with pytest.raises(RuntimeError):
        K.rms_norm(torch.zeros(2, 128, dtype=torch.float16), torch.zeros(128, dtype=torch.float16), 1e-6)
