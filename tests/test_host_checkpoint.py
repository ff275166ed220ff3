"""Checkpoint format (meta.json + safetensors): writer/reader round trip on the CPU, and a layer
loaded from a checkpoint against the same layer built in memory on the GPU.

The key names, meta.json fields and the qmeta seed cross-check follow the reference
(qwen35_quant_io.py:36-125, :128-190, :241-292, :348-413).
"""

import dataclasses
import json
import os
import warnings

import pytest
import torch

from oracle import moe, routing
from tests.helpers import make_module, pools_dict

LAYER = "model.layers.3.mlp"


def _layer_dict(layer, gate_weight=None):
    return {"pools": pools_dict(layer), "num_experts": layer.num_experts, "hidden_size": layer.hidden,
            "intermediate_size": layer.inter, "top_k": layer.top_k, "gate_weight": gate_weight,
            "shared_expert": layer.shared}


@pytest.fixture(scope="module")
def shared_layer(small_layer):
    return moe.add_shared_expert(dataclasses.replace(small_layer, shared=None), 2 * small_layer.inter,
                                 seed=77)


@pytest.mark.parametrize("shards", [1, 3])
def test_round_trip_and_format(tmp_path, shared_layer, shards):
    from dartmoq_hip import checkpoint
    layer = shared_layer
    gate = torch.randn(layer.num_experts, layer.hidden).half()
    meta = checkpoint.save_layers(str(tmp_path), {LAYER: _layer_dict(layer, gate)},
                                  quant_args={"seed": 42}, shards=shards)
    # the fields restore_quant_metadata / from_metadata read
    on_disk = json.load(open(os.path.join(tmp_path, "meta.json")))
    assert on_disk == json.loads(json.dumps(meta))
    lm = on_disk["layers"][LAYER]
    assert lm["type"] == "wxa16_moe" and lm["num_experts"] == layer.num_experts
    assert set(lm["bits"]) == set(layer.pools) and lm["bit_list"] == [int(b) for b in layer.pools]
    for b, p in layer.pools.items():
        assert lm["expert_offsets"][b] == list(p.expert_offsets)
        assert lm["bits"][b]["gate_up"]["seed"] == 42 + int(b)
        assert lm["bits"][b]["down"]["shape"] == [layer.hidden, p.expert_offsets[-1]]
    assert on_disk["modules"][LAYER + ".shared_expert.down_proj"]["type"] == "wxa16_linear"
    assert checkpoint.list_layers(str(tmp_path)) == [LAYER]
    if shards > 1:
        assert os.path.isfile(os.path.join(tmp_path, "model.safetensors.index.json"))

    back = checkpoint.read_layer(str(tmp_path), LAYER)
    assert back["num_experts"] == layer.num_experts and back["top_k"] == layer.top_k
    assert torch.equal(back["gate_weight"], gate)
    assert list(back["pools"]) == list(layer.pools)          # processing order is kept
    for b, p in layer.pools.items():
        for which, src in (("gate_up", p.gate_up), ("down", p.down)):
            got = back["pools"][b][which]
            for k in ("indices_packed", "codebook", "norms"):
                assert torch.equal(got[k], src[k])
            assert got["seed"] == src["seed"] and tuple(got["shape"]) == tuple(src["shape"])
            assert got["bit_width"] == int(b) and got["group_size"] == 128
        assert back["pools"][b]["expert_offsets"] == list(p.expert_offsets)
    for name in ("gate", "up", "down"):
        for k in ("indices_packed", "codebook", "norms"):
            assert torch.equal(back["shared_expert"][name][k], layer.shared[name][k])
        assert back["shared_expert"][name]["seed"] == layer.shared[name]["seed"]
    assert torch.equal(back["shared_expert"]["gate_row"].reshape(-1), layer.shared["gate_row"].reshape(-1))


def test_errors_and_seed_cross_check(tmp_path, small_layer):
    from dartmoq_hip import checkpoint
    checkpoint.save_layers(str(tmp_path), {LAYER: _layer_dict(small_layer)})
    with pytest.raises(KeyError):
        checkpoint.read_layer(str(tmp_path), "model.layers.9.mlp")
    assert checkpoint.read_layer(str(tmp_path), LAYER)["shared_expert"] is None
    # meta.json from another quantization run: seeds disagree with the qmeta scalars
    path = os.path.join(tmp_path, "meta.json")
    meta = json.load(open(path))
    first = next(iter(meta["layers"][LAYER]["bits"]))
    meta["layers"][LAYER]["bits"][first]["down"]["seed"] += 1
    json.dump(meta, open(path, "w"))
    with warnings.catch_warnings(record=True) as rec:
        warnings.simplefilter("always")
        checkpoint.read_layer(str(tmp_path), LAYER)
    assert any("qmeta seed mismatch" in str(w.message) for w in rec)
    # a tensor whose shape disagrees with meta.json is refused
    meta["layers"][LAYER]["bits"][first]["down"]["seed"] -= 1
    meta["layers"][LAYER]["bits"][first]["down"]["norms_shape"][0] += 1
    json.dump(meta, open(path, "w"))
    with pytest.raises(ValueError):
        checkpoint.read_layer(str(tmp_path), LAYER)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["wxa16", "wxa8"])
def test_loaded_layer_equals_in_memory_layer(tmp_path, shared_layer, mode):
    from dartmoq_hip import checkpoint
    layer = shared_layer
    g = torch.Generator().manual_seed(4)
    gate = (torch.randn(layer.num_experts, layer.hidden, generator=g) * 0.1).half()
    checkpoint.save_layers(str(tmp_path), {LAYER: _layer_dict(layer, gate)}, shards=2)
    loaded = checkpoint.load_moe_layer(str(tmp_path), LAYER, mode=mode)
    direct = make_module(layer, mode)
    x = torch.randn(21, layer.hidden, generator=g).half().cuda()
    logits = routing.zipf_logits(21, layer.num_experts, 4).cuda()
    assert torch.equal(loaded.forward(x, router_logits=logits), direct.forward(x, router_logits=logits))
    # the router weight of the checkpoint drives the forward when no logits are given
    y = loaded.forward(x)
    ref_logits = (x @ gate.cuda().t())
    assert torch.equal(y, direct.forward(x, router_logits=ref_logits))
