"""GPU test of the launch-shape tuner: a short search on a small layer, and a forward under the
resulting table."""

import pytest
import torch

from oracle import moe, routing
from tests.helpers import make_module, relerr

pytestmark = pytest.mark.gpu


def test_search_times_the_shapes_and_the_table_drives_the_forward(small_layer, tmp_path):
    from dartmoq_hip import autotune
    mods = [make_module(small_layer, "wxa16") for _ in range(2)]
    space = [{"tt": 1, "ks": 1, "nbl": 0}, {"tt": 1, "ks": 4, "nbl": 0}, {"tt": 2, "ks": 1, "nbl": 1},
             {"tt": 2, "ks": 4, "nbl": 0},             # filtered out: K split needs 16-row tiles
             {"tt": 1, "ks": -2, "nbl": 0}, {"tt": 4, "ks": 1, "nbl": 2}]
    results = autotune.run_full_autotune(mods, [3, 40], str(tmp_path), skew=True, n_warmup=1, n_repeat=3,
                                         variants=2, configs=space, prelude_s=0.05)
    for res in results:
        assert res["params"]["total_configs"] == 5 and res["params"]["failed_count"] == 0
        assert len(res["results"]) == 6 and sum(r["is_baseline"] for r in res["results"]) == 1
        times = [r["median_ms"] for r in res["results"]]
        assert times == sorted(times) and all(0 < t < 50 for t in times)
        assert res["best"]["median_ms"] <= res["baseline"]["median_ms"]
    assert all(m.tt_override == 0 and m.ks_override == 0 for m in mods)
    table = autotune.generate_config_table(str(tmp_path), min_gain=0.0)
    assert [e["tokens"] for e in table["entries"]] == [3, 40]

    # a forward under a table: same bits as the explicit override of the same shape, right values
    forced = {"entries": [{"tokens": 3, "tt": 1, "ks": 4, "nbl": 0}, {"tokens": 40, "tt": 2, "ks": 1, "nbl": 1}]}
    mod = mods[0]
    for tokens, (tt, ks, nbl) in ((3, (1, 4, 0)), (40, (2, 1, 1))):
        g = torch.Generator().manual_seed(tokens)
        x = torch.randn(tokens, small_layer.hidden, generator=g).half()
        logits = routing.zipf_logits(tokens, small_layer.num_experts, tokens)
        w, idx = routing.route_topk(logits, small_layer.top_k)
        autotune.apply_config_table(mod, forced)
        out = mod.forward(x.cuda(), router_logits=logits.cuda())
        autotune.apply_config_table(mod, None)
        mod.tt_override, mod.ks_override, mod.nbl_override = tt, ks, nbl
        want = mod.forward(x.cuda(), router_logits=logits.cuda())
        mod.tt_override = mod.ks_override = mod.nbl_override = 0
        assert torch.equal(out, want)
        ideal = moe.quantized_forward(small_layer, x, idx, w, "wxa16")
        assert relerr(out.float().cpu(), ideal) < 3e-3


@pytest.mark.parametrize("tokens", [3, 300])
def test_validity_filter_agrees_with_the_library(small_layer, tokens):
    """Every shape of the search space: the library takes it exactly when the tuner's filter says so
    (H = 256: K cannot be shared four ways; 1200 routed rows: not between workgroups at all)."""
    from dartmoq_hip import autotune
    mod = make_module(small_layer, "wxa16")
    g = torch.Generator().manual_seed(tokens)
    x = torch.randn(tokens, small_layer.hidden, generator=g).half().cuda()
    logits = routing.zipf_logits(tokens, small_layer.num_experts, tokens).cuda()
    want = mod.forward(x, router_logits=logits).float()
    scale = want.abs().max().item()
    seen = {True: 0, False: 0}
    for cfg in autotune.generate_configs():
        valid = autotune.is_config_valid(cfg, tokens, mod.top_k + mod.n_shared, mod.hidden_size)
        mod.tt_override, mod.ks_override, mod.nbl_override = cfg["tt"], cfg["ks"], cfg["nbl"]
        try:
            out = mod.forward(x, router_logits=logits).float()
            accepted = True
        except ValueError:
            accepted = False
        finally:
            mod.tt_override = mod.ks_override = mod.nbl_override = 0
        assert accepted == valid, cfg
        seen[valid] += 1
        if accepted:                                   # any shape computes the same layer
            torch.testing.assert_close(out, want, rtol=4e-3, atol=4e-3 * scale)
    assert seen[True] > 10 and seen[False] > 10
