"""GPU parity: the layer forward that starts from the block's pre-norm hidden states (RMSNorm,
router projection and top-k inside the first launch; at most 16 tokens).

* the normalized rows it can hand back are the bits of the stand-alone RMSNorm kernel and match
  oracle.norm.rms_norm to one fp16 rounding;
* its router logits match the fp32 product of the oracle's normalized rows and the gate weight to
  fp16 rounding, and the top-k taken from them is oracle.routing.route_topk's on every token
  whose k-th and (k+1)-th logits are further apart than that rounding;
* its output is, bit for bit, the output of the routed forward fed the same normalized rows and
  the same logits (one launch instead of three in front of the GEMMs changes no value).
"""

import dataclasses

import pytest
import torch

from oracle import moe, norm, routing
from tests.helpers import make_module, relerr

pytestmark = pytest.mark.gpu

EPS = 1e-6


def _case(layer, tokens, seed, weight_dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    h = (torch.randn(tokens, layer.hidden, generator=g) * 3.0).half()
    h[0, 7] = 40.0                                                     # an outlier in the mean square
    wn = (torch.randn(layer.hidden, generator=g) * 0.1).to(weight_dtype)
    wg = (torch.randn(layer.num_experts, layer.hidden, generator=g) * 0.06).half()
    return h, wn, wg


def _run(layer, mode, tokens, seed, weight_dtype=torch.float16):
    from dartmoq_hip import ops
    h, wn, wg = _case(layer, tokens, seed, weight_dtype)
    mod = make_module(layer, mode)
    mod.gate_weight = wg.cuda()
    logits = torch.empty(tokens, layer.num_experts, dtype=torch.float16, device="cuda")
    out, xn = mod.forward_prenorm(h.cuda(), wn.cuda(), EPS, return_normed=True, logits_out=logits, fused=True)
    torch.cuda.synchronize()
    # the stand-alone kernel's bits
    xk = ops.rms_norm(h.cuda(), wn.cuda(), EPS)
    assert torch.equal(xn.view(torch.int16), xk.view(torch.int16))
    # the oracle's rows to one rounding
    xo = norm.rms_norm(h, wn, EPS)
    ulp = (xn.cpu().view(torch.int16).int() - xo.view(torch.int16).int()).abs()
    assert ulp.max() <= 1 and (ulp != 0).float().mean() < 2e-3
    # logits: fp32 product rounded to fp16
    lo = xn.cpu().float() @ wg.float().t()
    torch.testing.assert_close(logits.cpu().float(), lo, rtol=2e-3, atol=2e-3)
    # top-k from those logits = the oracle's wherever the cut is not within rounding
    w_ref, idx_ref = routing.route_topk(lo, layer.top_k)
    srt = lo.sort(dim=-1, descending=True).values
    safe = (srt[:, layer.top_k - 1] - srt[:, layer.top_k]) > 8e-3
    w_dev, idx_dev = mod.route(xn, router_logits=logits)
    k = layer.top_k
    assert torch.equal(idx_dev[:, :k].cpu().long()[safe].sort(-1).values, idx_ref[safe].sort(-1).values)
    # the same values as the routed forward on the same rows and logits
    want = mod.forward(xn, router_logits=logits)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    return h, xo, lo, safe, out.cpu().float()


@pytest.mark.parametrize("mode", ["wxa16", "wxa8", "wxfp8", "wxfp4"])
@pytest.mark.parametrize("tokens", [1, 3, 4, 5, 11, 16])
def test_prenorm_forward_is_the_routed_forward(small_layer, mode, tokens):
    h, xo, lo, safe, out = _run(small_layer, mode, tokens, seed=100 + tokens)
    if mode == "wxa16" and bool(safe.all()):
        w, idx = routing.route_topk(lo.half().float(), small_layer.top_k)
        ideal = moe.quantized_forward(small_layer, xo, idx, w, mode)
        assert relerr(out, ideal) < 5e-3


@pytest.mark.parametrize("tokens", [1, 4, 9, 16])
def test_prenorm_forward_with_shared_expert_and_fp32_norm_weight(small_layer, tokens):
    layer = moe.add_shared_expert(dataclasses.replace(small_layer, shared=None), 2 * small_layer.inter,
                                  seed=77)
    _run(layer, "wxa8", tokens, seed=200 + tokens, weight_dtype=torch.float32)
    _run(layer, "wxa16", tokens, seed=300 + tokens)


def test_prenorm_forward_twice_and_beyond_the_limit(small_layer):
    """The state word is left ready for the next call; more than 16 tokens take the separate steps."""
    mod = make_module(small_layer, "wxa16")
    h, wn, wg = _case(small_layer, 6, 5)
    mod.gate_weight = wg.cuda()
    a = mod.forward_prenorm(h.cuda(), wn.cuda(), EPS)
    b = mod.forward_prenorm(h.cuda(), wn.cuda(), EPS)
    c = mod.forward_prenorm(h[:2].cuda(), wn.cuda(), EPS)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(a[:2], c)
    assert int(mod._prenorm_state.abs().sum()) == 0
    # a replaced gate weight is picked up (the module keeps an fp16 copy of it)
    wg2 = wg.flip(0).contiguous()
    mod.gate_weight = wg2.cuda()
    lg = torch.empty(6, small_layer.num_experts, dtype=torch.float16, device="cuda")
    _o, xn6 = mod.forward_prenorm(h.cuda(), wn.cuda(), EPS, return_normed=True, logits_out=lg)
    torch.testing.assert_close(lg.float().cpu(), xn6.float().cpu() @ wg2.float().t(), rtol=2e-3, atol=2e-3)
    mod.gate_weight = wg.cuda()
    h40, _wn, _wg = _case(small_layer, 40, 6)
    out, xn = mod.forward_prenorm(h40.cuda(), wn.cuda(), EPS, return_normed=True)
    want = mod.forward(xn, router_logits=torch.matmul(xn, wg.cuda().t()))
    assert torch.equal(out, want)


def test_prenorm_entry_rejects_what_it_does_not_take(small_layer):
    import ctypes
    from dartmoq_hip import _lib
    mod = make_module(small_layer, "wxa16")
    h, wn, wg = _case(small_layer, 17, 1)
    mod.gate_weight = wg.cuda()
    mod.forward_prenorm(h[:1].cuda(), wn.cuda(), EPS)          # sets the state word up
    desc = mod._descriptor()[0]
    ws = mod._get_workspace(17)
    router = _lib.RouterArgs()
    pre = _lib.PrenormArgs()
    wn_d, hd = wn.cuda(), h.cuda()
    out = torch.empty_like(hd)
    pre.norm_weight = wn_d.data_ptr()
    pre.eps = EPS
    pre.gate_weight = mod._gate_f16.data_ptr()
    pre.state = mod._prenorm_state.data_ptr()
    rc = _lib.load().dmq_moe_ffn_forward_prenorm(
        ctypes.byref(desc), ctypes.byref(router), ctypes.byref(pre), hd.data_ptr(), 17, None,
        out.data_ptr(), ws.data_ptr(), ws.numel(), 0, 0, 0, None, None, None)
    assert rc != 0                                             # more than 16 tokens
    pre.state = None
    rc = _lib.load().dmq_moe_ffn_forward_prenorm(
        ctypes.byref(desc), ctypes.byref(router), ctypes.byref(pre), hd.data_ptr(), 4, None,
        out.data_ptr(), ws.data_ptr(), ws.numel(), 0, 0, 0, None, None, None)
    assert rc != 0                                             # no state word


@pytest.mark.parametrize("tokens", [2, 7])
def test_prenorm_forward_is_graph_capturable(small_layer, tokens):
    """The pre-norm forward allocates nothing, never synchronises and leaves its state word zero,
    so it can be captured in a HIP graph: every replay, with eager work of the same module in
    between, reproduces the eager result bit for bit."""
    h, wn, wg = _case(small_layer, tokens, 40 + tokens)
    mod = make_module(small_layer, "wxa8")
    mod.gate_weight = wg.cuda()
    hd, wnd = h.cuda(), wn.cuda()
    ref = mod.forward_prenorm(hd, wnd, EPS, fused=True).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            mod.forward_prenorm(hd, wnd, EPS, fused=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = mod.forward_prenorm(hd, wnd, EPS, fused=True)
    for _ in range(4):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, ref)
        other = mod.forward_prenorm(hd.flip(0).contiguous(), wnd, EPS, fused=True)
        torch.cuda.synchronize()
        assert torch.equal(other.flip(0), ref)
    assert int(mod._prenorm_state.abs().sum()) == 0
