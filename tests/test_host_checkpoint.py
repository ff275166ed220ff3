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


# ----------------------------------------------------------------------------- reference-written fixture
# tests/golden/ckpt_tiny was written by the reference's save_quantized_model over a tiny model
# assembled from the reference's classes (tests/golden/make_ckpt_fixture.py); expected.json holds
# outputs computed with the reference's own CPU dequantizers.

CKPT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ckpt_tiny")
FIX_LAYERS = ("model.layers.0.mlp", "model.layers.1.mlp")


def _fixture_case(path):
    exp = json.load(open(os.path.join(CKPT, "expected.json")))[path]
    x = torch.tensor(exp["x_fp16_bits"], dtype=torch.int16).view(torch.float16).reshape(4, -1)
    return (x, torch.tensor(exp["topk_idx"]), torch.tensor(exp["topk_w"], dtype=torch.float32),
            torch.tensor(exp["y_routed"]), torch.tensor(exp["y_shared"]))


def _oracle_layer(d):
    layer = moe.MoELayer(d["hidden_size"], d["intermediate_size"], d["num_experts"], d["top_k"], 128)
    for b, p in d["pools"].items():
        layer.pools[b] = moe.BitPool(int(b), p["gate_up"], p["down"], p["expert_offsets"])
    layer.shared = d["shared_expert"]
    return layer


def test_reads_checkpoint_written_by_the_reference():
    from safetensors import safe_open
    from dartmoq_hip import checkpoint
    assert checkpoint.list_layers(CKPT) == list(FIX_LAYERS)
    meta = json.load(open(os.path.join(CKPT, "meta.json")))
    raw = safe_open(os.path.join(CKPT, "model.safetensors"), framework="pt", device="cpu")
    for path in FIX_LAYERS:
        d = checkpoint.read_layer(CKPT, path)
        lm = meta["layers"][path]
        assert (d["num_experts"], d["hidden_size"], d["top_k"]) == (4, 256, 2)
        assert d["intermediate_size"] == lm["intermediate_size"]
        assert list(d["pools"]) == [str(b) for b in lm["bit_list"]] == ["4", "2"]
        for b, p in d["pools"].items():
            assert p["expert_offsets"] == lm["expert_offsets"][b]
            for which in ("gate_up", "down"):
                assert p[which]["seed"] == 42 + int(b) + (1000 if which == "down" else 0)
                assert p[which]["bit_width"] == int(b) and p[which]["group_size"] == 128
                for k in ("indices_packed", "codebook", "norms"):
                    assert torch.equal(p[which][k], raw.get_tensor(f"{path}.bit_weights.{b}.{which}_{k}"))
            total = p["expert_offsets"][-1]
            assert tuple(p["gate_up"]["shape"]) == (2 * total, 256)
            assert tuple(p["down"]["shape"]) == (256, total)
        assert torch.equal(d["gate_weight"], raw.get_tensor(f"{path}.gate.weight"))
        sh = d["shared_expert"]
        assert sh["gate"]["bit_width"] == (4 if path.endswith("0.mlp") else 8)
        assert sh["down"]["codebook_type"] == ("lloydmax" if path.endswith("0.mlp") else "uniform")
        assert torch.equal(sh["gate_row"], raw.get_tensor(f"{path}.shared_expert_gate.weight"))
    # layer 1 is the --slices 2 layout: experts 0 and 2 live in both pools
    offs = checkpoint.read_layer(CKPT, FIX_LAYERS[1])["pools"]
    homes = [sum(1 for p in offs.values() if p["expert_offsets"][e + 1] > p["expert_offsets"][e])
             for e in range(4)]
    assert homes == [2, 1, 2, 1]


@pytest.mark.parametrize("path", FIX_LAYERS)
def test_oracle_on_reference_checkpoint_matches_reference_dequant_outputs(path):
    """The oracle's dequantize-then-matmul forward over the tensors the reader returns equals what
    the reference's own dequantizers give (routed part incl. the sum over the pools of a split
    expert, and the gated shared expert)."""
    from dartmoq_hip import checkpoint
    layer = _oracle_layer(checkpoint.read_layer(CKPT, path))
    x, idx, w, y_routed, y_shared = _fixture_case(path)
    shared = layer.shared
    layer.shared = None
    routed = moe.reference_forward(layer, x, idx, w)
    # the reference's dequantizers return the weight dtype (fp16: one rounding per weight, relative
    # 2^-11), the oracle keeps fp32
    from tests.helpers import relerr
    assert relerr(routed, y_routed) < 5e-4
    layer.shared = shared
    assert relerr(moe.shared_expert_forward(layer, x.float()), y_shared) < 5e-4


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["wxa16", "wxa8", "wxfp8", "wxfp4"])
@pytest.mark.parametrize("path", FIX_LAYERS)
def test_gpu_forward_of_reference_checkpoint(path, mode):
    """load_moe_layer on the reference-written checkpoint, router's own top-k handed over: output
    against the reference-dequantizer expectation (fp32) within the mode's error."""
    from dartmoq_hip import checkpoint
    from tests.helpers import relerr
    bound = {"wxa16": 2e-3, "wxa8": 0.03, "wxfp8": 0.09, "wxfp4": 0.35}[mode]
    mod = checkpoint.load_moe_layer(CKPT, path, mode=mode)
    x, idx, w, y_routed, y_shared = _fixture_case(path)
    out = mod.forward(x.cuda(), topk_idx=idx.int().cuda(), topk_w=w.cuda()).float().cpu()
    want = y_routed + y_shared
    assert relerr(out, want) < bound, (mode, relerr(out, want))
    # and the router weight of the checkpoint reproduces that top-k
    out2 = mod.forward(x.cuda()).float().cpu()
    assert relerr(out2, want) < bound


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["wxa16", "wxa8", "wxfp8", "wxfp4"])
@pytest.mark.parametrize("tokens,tt", [(1, 0), (37, 0), (300, 2), (300, 4)])
def test_gpu_sub_expert_layer_matches_dataflow_oracle(mode, tokens, tt):
    """model.layers.1.mlp of the fixture (experts cut into sub-experts over two pools, an 8-bit
    uniform shared expert narrower than the routed experts) at several batch sizes and tilings,
    against the oracle's kernel-dataflow forward on the tensors the reader returns."""
    from dartmoq_hip import checkpoint
    from tests.helpers import relerr
    d = checkpoint.read_layer(CKPT, FIX_LAYERS[1])
    layer = _oracle_layer(d)
    mod = checkpoint.load_moe_layer(CKPT, FIX_LAYERS[1], mode=mode)
    mod.tt_override = tt
    g = torch.Generator().manual_seed(tokens)
    x = torch.randn(tokens, layer.hidden, generator=g).half()
    w, idx = routing.route_topk(routing.zipf_logits(tokens, layer.num_experts, tokens), layer.top_k)
    out = mod.forward(x.cuda(), topk_idx=idx.int().cuda(), topk_w=w.cuda()).float().cpu()
    ideal = moe.quantized_forward(layer, x, idx, w, mode)
    tight = {"wxa16": 3e-3, "wxa8": 6e-3, "wxfp8": 2e-2, "wxfp4": 6e-2}[mode]
    assert relerr(out, ideal) < tight, (mode, relerr(out, ideal))
    # splitting the batch leaves every row unchanged
    if tokens > 100:
        a = mod.forward(x[:111].cuda(), topk_idx=idx[:111].int().cuda(), topk_w=w[:111].cuda())
        b = mod.forward(x[111:].cuda(), topk_idx=idx[111:].int().cuda(), topk_w=w[111:].cuda())
        assert torch.equal(torch.cat([a, b]).float().cpu(), out)
