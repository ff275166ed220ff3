"""Host logic of the launch-shape tuner (dartmoq_hip.autotune): search space, validity filter,
table generation and the lookup a module's forward does.  No GPU."""

import json
import types

from dartmoq_hip import autotune
from dartmoq_hip.moe import WxA16BitPartitionedGroupMoE


def test_search_space_and_validity_filter():
    cfgs = autotune.generate_configs()
    assert len(cfgs) == 3 * 5 * 4 and {"tt": 2, "ks": 1, "nbl": 4} in cfgs
    ok = lambda tt, ks, tokens=8, hidden=2048: autotune.is_config_valid({"tt": tt, "ks": ks, "nbl": 0}, tokens, 8, hidden)
    assert ok(1, 4) and ok(1, -4) and ok(2, 1) and ok(4, 0)
    assert not ok(2, 4) and not ok(4, -2)            # K is split or shared with 16-row tiles only
    assert not ok(1, -4, hidden=768)                 # 6 groups do not divide by 4
    assert ok(1, -2, hidden=768)
    assert not ok(1, -2, tokens=129)                 # 1032 routed rows: beyond the shared form's scratch
    assert not autotune.is_config_valid({"tt": 3, "ks": 1, "nbl": 0}, 8, 8, 2048)
    assert not autotune.is_config_valid({"tt": 1, "ks": 1, "nbl": 3}, 8, 8, 2048)


def _result(tokens, best_cfg, speedup):
    return {"params": {"tokens": tokens}, "baseline": {"config": dict(autotune.AUTO), "median_ms": 1.0},
            "best": {"config": best_cfg, "median_ms": 1.0 / speedup, "tflops": 1.0, "speedup": speedup},
            "results": []}


def test_table_keeps_the_library_choice_within_noise_and_lookup_is_nearest_on_a_log_scale(tmp_path):
    autotune.save_result(_result(8, {"tt": 1, "ks": 4, "nbl": 1}, 1.10), str(tmp_path / "tokens_8.json"))
    autotune.save_result(_result(64, {"tt": 2, "ks": 1, "nbl": 2}, 1.01), str(tmp_path / "tokens_64.json"))
    autotune.save_result(_result(2048, {"tt": 4, "ks": 1, "nbl": 0}, 1.05), str(tmp_path / "tokens_2048.json"))
    (tmp_path / "notes.txt").write_text("ignored")
    table = autotune.generate_config_table(str(tmp_path))
    assert [e["tokens"] for e in table["entries"]] == [8, 64, 2048]
    assert table["entries"][1]["tt"] == 0 and table["entries"][1]["speedup"] == 1.0     # 1 % is noise
    assert autotune.lookup_config(table, 1) == {"tt": 1, "ks": 4, "nbl": 1}
    assert autotune.lookup_config(table, 20) == {"tt": 1, "ks": 4, "nbl": 1}           # 20 / 8 < 64 / 20
    assert autotune.lookup_config(table, 30) == dict(autotune.AUTO)
    assert autotune.lookup_config(table, 100000) == {"tt": 4, "ks": 1, "nbl": 0}
    assert autotune.lookup_config(None, 5) == dict(autotune.AUTO)
    assert json.loads(json.dumps(table)) == table


def test_module_forward_takes_overrides_first_then_the_table_then_the_library_choice():
    table = {"entries": [{"tokens": 4, "tt": 1, "ks": -4, "nbl": 0}, {"tokens": 512, "tt": 2, "ks": 1, "nbl": 2}]}
    m = types.SimpleNamespace(tt_override=0, ks_override=0, nbl_override=0, tile_table=None, top_k=8, n_shared=0,
                              hidden_size=2048)
    tiling = lambda tokens: WxA16BitPartitionedGroupMoE._tiling(m, tokens)
    assert tiling(4) == (0, 0, 0)
    m.tile_table = table
    assert tiling(2) == (1, -4, 0) and tiling(400) == (2, 1, 2)
    m.hidden_size = 768                    # K cannot be shared four ways: the library's own choice
    assert tiling(2) == (0, 0, 0)
    m.hidden_size = 2048
    m.tt_override = 4
    assert tiling(2) == (4, 0, 0)
