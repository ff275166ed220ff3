"""GPU parity: top-k router and device-side permutation / pool partition."""

import pytest
import torch

from oracle import routing

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,experts,k,skew", [(1, 256, 8, True), (64, 256, 8, True),
                                                   (300, 256, 8, False), (17, 16, 4, True),
                                                   (5, 100, 3, False)])
def test_topk_matches_oracle(tokens, experts, k, skew):
    from dartmoq_hip import ops
    logits = routing.zipf_logits(tokens, experts, seed=tokens + experts, skew=skew)
    ref_w, ref_idx = routing.route_topk(logits, k)
    w, idx = ops.route_topk(logits.cuda(), k)
    assert torch.equal(idx.cpu().long(), ref_idx)            # indices are exact
    torch.testing.assert_close(w.cpu(), ref_w, rtol=2e-6, atol=1e-9)
    ref_wn, _ = routing.route_topk(logits, k, renormalize=True)
    wn, _ = ops.route_topk(logits.cuda(), k, renormalize=True)
    torch.testing.assert_close(wn.cpu(), ref_wn, rtol=4e-6, atol=1e-9)


def test_topk_ties_pick_lowest_index():
    from dartmoq_hip import ops
    logits = torch.zeros(3, 128)
    logits[1, 70] = 1.0
    logits[2, [5, 90, 127]] = 2.0
    _w, idx = ops.route_topk(logits.cuda(), 4)
    assert idx[0].tolist() == [0, 1, 2, 3]
    assert idx[1].tolist() == [70, 0, 1, 2]
    assert idx[2].tolist() == [5, 90, 127, 0]


def _slices(expert_bit, inter, bits):
    e = len(expert_bit)
    start = torch.full((len(bits), e), -1, dtype=torch.int32)
    count = torch.zeros((len(bits), e), dtype=torch.int32)
    for pi, b in enumerate(bits):
        cur = 0
        for ex in range(e):
            if expert_bit[ex] == b:
                start[pi, ex] = 2 * cur
                count[pi, ex] = 2 * inter
                cur += inter
    return start, count


@pytest.mark.parametrize("tokens,tile_rows", [(1, 16), (64, 16), (500, 32), (2048, 64)])
def test_permute_matches_oracle(tokens, tile_rows):
    from dartmoq_hip import ops
    experts, k, inter = 64, 8, 256
    expert_bit = [4 if e % 9 == 0 else (1 if e % 13 == 5 else 2) for e in range(experts)]
    bits = [4, 2, 1]
    logits = routing.zipf_logits(tokens, experts, seed=tokens)
    w, idx = routing.route_topk(logits, k)
    toks, wts, slots, offs = routing.sort_by_expert(idx, w, experts)
    start, count = _slices(expert_bit, inter, bits)
    res = ops.route_permute(idx.cuda().int(), w.cuda(), experts, start.cuda(), count.cuda(), tile_rows)
    torch.cuda.synchronize()
    assert torch.equal(res["offsets"].cpu().long(), offs)
    assert torch.equal(res["counts"].cpu().long(), offs[1:] - offs[:-1])
    assert torch.equal(res["sorted_tokens"].cpu().long(), toks)
    assert torch.equal(res["sorted_rows"].cpu().long(), toks * k + slots)
    assert torch.equal(res["sorted_weights"].cpu(), wts)
    # pool partition: expert_info rows and the layer's work-item list (pool-major)
    exp_items = []
    for pi, b in enumerate(bits):
        gu = res["gu_info"][pi].cpu()
        dn = res["dn_info"][pi].cpu()
        for e in range(experts):
            member = expert_bit[e] == b
            cnt = int(offs[e + 1] - offs[e]) if member else 0
            assert gu[e, 0] == offs[e] and gu[e, 1] == cnt
            assert dn[e, 0] == offs[e] and dn[e, 1] == cnt
            if member:
                assert gu[e, 2] == start[pi, e] and gu[e, 3] == 2 * inter
                assert dn[e, 2] == start[pi, e] // 256 and dn[e, 3] == inter // 128
            exp_items += [(pi, e, i, int(offs[e]), cnt, int(start[pi, e]), int(start[pi, e]) // 256, 0)
                          for i in range(-(-cnt // tile_rows))]
    n = int(res["n_items"][0])
    assert n == len(exp_items)
    assert [tuple(r) for r in res["items"][:n].cpu().tolist()] == exp_items


@pytest.mark.parametrize("tokens,experts,k", [(700, 100, 3), (1000, 37, 1), (333, 300, 5), (5000, 256, 8),
                                                   (113, 257, 9), (128, 512, 8), (60, 513, 8), (129, 512, 8),
                                                   (2100, 600, 8), (900, 1100, 6), (2048, 200, 8), (2049, 200, 8),
                                                   (16384, 16, 1), (5461, 30, 3)])
def test_permute_odd_shapes(tokens, experts, k):
    """Tokens whose k rows straddle the 64-row steps of the sort, expert counts off the wave size;
    the cases with more than 512 experts take the separate planning and scatter launches, the
    others the launch that does both: counting the rows itself up to 16384 routed rows (2048 x 8,
    16384 x 1 and 5461 x 3 sit at that limit, 2049 x 8 just past it), reading the chunk histogram
    beyond."""
    from dartmoq_hip import ops
    logits = routing.zipf_logits(tokens, experts, seed=7 * tokens + k)
    w, idx = routing.route_topk(logits, k)
    toks, wts, slots, offs = routing.sort_by_expert(idx, w, experts)
    start = torch.arange(experts, dtype=torch.int32).reshape(1, experts) * 512
    count = torch.full((1, experts), 512, dtype=torch.int32)
    res = ops.route_permute(idx.cuda().int(), w.cuda(), experts, start.cuda(), count.cuda(), 16)
    torch.cuda.synchronize()
    assert torch.equal(res["offsets"].cpu().long(), offs)
    assert torch.equal(res["sorted_tokens"].cpu().long(), toks)
    assert torch.equal(res["sorted_rows"].cpu().long(), toks * k + slots)
    assert torch.equal(res["sorted_weights"].cpu(), wts)
    n = int(res["n_items"][0])
    assert n == int(sum(-(-int(c) // 16) for c in (offs[1:] - offs[:-1])))
