"""Reader (and writer) of the reference's quantized checkpoint format for the MoE FFN layer.

A checkpoint directory holds ``meta.json`` (everything that is not a tensor: seeds, group size,
shapes, expert_offsets per bit pool, the quantized Linears by module path) and
``model.safetensors`` or shards listed in ``model.safetensors.index.json`` (every tensor under
its state_dict key, plus the seeds once more as ``qmeta/...`` int64 scalars).  This module follows
save_quantized_model / collect_quant_metadata / restore_quant_metadata of the reference
(qwen35_quant_io.py:36-125, :128-190, :241-292, :348-413, :612-628) for the part of a checkpoint
one MoE FFN layer needs:

    <layer>.bit_weights.<bit>.gate_up_indices_packed | gate_up_codebook | gate_up_norms
    <layer>.bit_weights.<bit>.down_indices_packed   | down_codebook   | down_norms
    <layer>.gate.weight                      router [E, H]
    <layer>.shared_expert.{gate_proj,up_proj,down_proj}.{packed_indices,norms,codebook}
    <layer>.shared_expert_gate.weight        [1, H]

Tensors are read with safetensors (nothing from the files is executed) and only the keys of the
requested layer are touched, so a 35B checkpoint is never loaded whole.
"""

from __future__ import annotations

import json
import os
import warnings

import torch

SHARED_LINEARS = ("gate_proj", "up_proj", "down_proj")
_TENSOR_KEYS = ("indices_packed", "codebook", "norms")


def _read_meta(quant_dir: str) -> dict:
    with open(os.path.join(quant_dir, "meta.json"), "r", encoding="utf-8") as f:
        return json.load(f)


class _TensorSource:
    """Key -> tensor over a single safetensors file or an index of shards."""

    def __init__(self, quant_dir: str):
        from safetensors import safe_open
        self._open = safe_open
        self.dir = quant_dir
        idx = os.path.join(quant_dir, "model.safetensors.index.json")
        if os.path.isfile(idx):
            with open(idx, "r", encoding="utf-8") as f:
                self.weight_map = json.load(f)["weight_map"]
        else:
            self.weight_map = None
        self._handles: dict[str, object] = {}

    def _file_of(self, key: str) -> str:
        if self.weight_map is None:
            return "model.safetensors"
        if key not in self.weight_map:
            raise KeyError(key)
        return self.weight_map[key]

    def _handle(self, fname: str):
        h = self._handles.get(fname)
        if h is None:
            h = self._open(os.path.join(self.dir, fname), framework="pt", device="cpu")
            self._handles[fname] = h
        return h

    def has(self, key: str) -> bool:
        try:
            return key in self._handle(self._file_of(key)).keys()
        except KeyError:
            return False

    def get(self, key: str) -> torch.Tensor:
        h = self._handle(self._file_of(key))
        if key not in h.keys():
            raise KeyError(f"{key} not in checkpoint {self.dir}")
        return h.get_tensor(key)


def list_layers(quant_dir: str) -> list:
    """Module paths of the quantized MoE layers in a checkpoint (keys of meta['layers'])."""
    return list(_read_meta(quant_dir).get("layers", {}).keys())


def _packed_from(src: _TensorSource, prefix: str, which: str, m: dict, where: str) -> dict:
    packed = {k: src.get(f"{prefix}.{which}_{k}") for k in _TENSOR_KEYS}
    packed.update(seed=int(m["seed"]), group_size=int(m["group_size"]), shape=tuple(m["shape"]),
                  bit_width=int(m["bit_width"]), rotation=m.get("rotation", "qr"),
                  orig_dtype=m.get("orig_dtype"))
    for k in _TENSOR_KEYS:
        want = m.get(f"{k}_shape")
        if want is not None and list(packed[k].shape) != list(want):
            raise ValueError(f"{where}.{which}_{k}: shape {list(packed[k].shape)} != meta {want}")
    return packed


def _check_seed(src: _TensorSource, key: str, want: int):
    """qmeta cross-check (qwen35_quant_io.py:153-187): a mismatch means meta.json and the tensor
    file do not belong together; a missing key is an older checkpoint."""
    if not src.has(key):
        return
    got = int(src.get(key).item())
    if got != int(want):
        warnings.warn(f"qmeta seed mismatch at {key}: meta.json has {want}, tensors have {got} "
                      "(files may not belong together)")


def read_layer(quant_dir: str, layer_path: str) -> dict:
    """Everything ``from_packed`` needs for one layer, on the CPU:
    {"pools", "num_experts", "hidden_size", "intermediate_size", "top_k", "gate_weight",
     "shared_expert" (or None)}."""
    meta = _read_meta(quant_dir)
    layers = meta.get("layers", {})
    if layer_path not in layers:
        raise KeyError(f"{layer_path} is not a quantized MoE layer of {quant_dir}; "
                       f"layers: {list(layers)[:4]}...")
    lm = layers[layer_path]
    if lm.get("type") != "wxa16_moe":
        raise ValueError(f"{layer_path}: unsupported layer type {lm.get('type')!r}")
    src = _TensorSource(quant_dir)
    pools = {}
    order = [str(b) for b in lm.get("bit_list", [])] or list(lm["bits"].keys())
    for bit_str in order:
        bm = lm["bits"][bit_str]
        prefix = f"{layer_path}.bit_weights.{bit_str}"
        pools[bit_str] = {
            "gate_up": _packed_from(src, prefix, "gate_up", bm["gate_up"], prefix),
            "down": _packed_from(src, prefix, "down", bm["down"], prefix),
            "expert_offsets": [int(v) for v in lm["expert_offsets"][bit_str]],
        }
        for which in ("gate_up", "down"):
            _check_seed(src, f"qmeta/{layer_path}/bits/{bit_str}/{which}/seed", bm[which]["seed"])
    gate_key = f"{layer_path}.gate.weight"
    gate_weight = src.get(gate_key) if src.has(gate_key) else None
    shared = None
    mods = meta.get("modules", {})
    lin_paths = {n: f"{layer_path}.shared_expert.{n}" for n in SHARED_LINEARS}
    if all(p in mods for p in lin_paths.values()):
        shared = {}
        for name, path in lin_paths.items():
            m = mods[path]
            if m.get("type") != "wxa16_linear":
                raise ValueError(f"{path}: unsupported module type {m.get('type')!r}")
            if m.get("has_bias"):
                raise ValueError(f"{path}: a biased shared-expert Linear is not supported")
            shared[name.split("_")[0]] = {
                "indices_packed": src.get(f"{path}.packed_indices"), "norms": src.get(f"{path}.norms"),
                "codebook": src.get(f"{path}.codebook"), "seed": int(m["seed"]),
                "group_size": int(m["group_size"]), "bit_width": int(m["bit_width"]),
                "shape": (int(m["out_features"]), int(m["in_features"])),
                "rotation": m.get("rotation", "qr"), "codebook_type": m.get("codebook_type", "lloydmax")}
            _check_seed(src, f"qmeta/{path}/seed", m["seed"])
        shared["gate_row"] = src.get(f"{layer_path}.shared_expert_gate.weight")
    return {"pools": pools, "num_experts": int(lm["num_experts"]), "hidden_size": int(lm["hidden_size"]),
            "intermediate_size": int(lm["intermediate_size"]), "top_k": int(lm["top_k"]),
            "gate_weight": gate_weight, "shared_expert": shared}


def load_moe_layer(quant_dir: str, layer_path: str, mode: str = "wxa16", renormalize: bool = False,
                   device="cuda"):
    """Checkpoint -> ready module (the role of restore_quant_metadata + convert_model_to_wxa8 /
    wxfp8 / wxfp4 for one layer, qwen35_quant_io.py:348-413, :416-532)."""
    from .moe import WxA16BitPartitionedGroupMoE, convert_moe
    d = read_layer(quant_dir, layer_path)
    moe = WxA16BitPartitionedGroupMoE.from_packed(
        d["pools"], d["num_experts"], d["hidden_size"], d["intermediate_size"], d["top_k"],
        gate_weight=d["gate_weight"], renormalize=renormalize, device=device,
        shared_expert=d["shared_expert"])
    return convert_moe(moe, mode) if mode != "wxa16" else moe


# ----------------------------------------------------------------------------- writer

def _packed_meta(packed: dict) -> dict:
    return {"seed": packed.get("seed"), "group_size": packed.get("group_size"),
            "shape": list(packed["shape"]), "bit_width": packed.get("bit_width"),
            "rotation": packed.get("rotation"), "orig_dtype": packed.get("orig_dtype"),
            "indices_packed_shape": list(packed["indices_packed"].shape),
            "codebook_shape": list(packed["codebook"].shape),
            "norms_shape": list(packed["norms"].shape)}


def save_layers(quant_dir: str, layers: dict, quant_args: dict | None = None, shards: int = 1) -> dict:
    """Write layers in the reference's checkpoint format.  ``layers`` maps a module path to the
    dictionary ``read_layer`` returns (pools, sizes, gate_weight, shared_expert).  ``shards`` > 1
    spreads the tensors over that many files with an index, like a sharded checkpoint."""
    from safetensors.torch import save_file
    os.makedirs(quant_dir, exist_ok=True)
    meta = {"base_model": None, "model_class": "Qwen3_5MoeForCausalLM", "quant_args": quant_args or {},
            "modules": {}, "layers": {}}
    sd = {}
    cpu = lambda t: t.detach().cpu().contiguous()
    for path, d in layers.items():
        inter = int(d["intermediate_size"])
        lm = {"type": "wxa16_moe", "num_experts": int(d["num_experts"]),
              "hidden_size": int(d["hidden_size"]), "intermediate_size": inter,
              "top_k": int(d["top_k"]), "bit_list": [int(b) for b in d["pools"]],
              "inter_size_by_bit": {str(b): inter for b in d["pools"]},
              "expert_offsets": {}, "bits": {}, "enable_timing": False}
        for bit_str, p in d["pools"].items():
            lm["expert_offsets"][bit_str] = [int(v) for v in p["expert_offsets"]]
            lm["bits"][bit_str] = {"gate_up": _packed_meta(p["gate_up"]), "down": _packed_meta(p["down"])}
            for which in ("gate_up", "down"):
                for k in _TENSOR_KEYS:
                    sd[f"{path}.bit_weights.{bit_str}.{which}_{k}"] = cpu(p[which][k])
                sd[f"qmeta/{path}/bits/{bit_str}/{which}/seed"] = torch.tensor(
                    int(p[which]["seed"]), dtype=torch.int64)
        meta["layers"][path] = lm
        if d.get("gate_weight") is not None:
            sd[f"{path}.gate.weight"] = cpu(d["gate_weight"])
        sh = d.get("shared_expert")
        if sh is not None:
            for name in SHARED_LINEARS:
                packed = sh[name.split("_")[0]]
                lp = f"{path}.shared_expert.{name}"
                n, k = (int(v) for v in packed["shape"])
                meta["modules"][lp] = {
                    "type": "wxa16_linear", "in_features": k, "out_features": n,
                    "bit_width": int(packed["bit_width"]), "group_size": int(packed["group_size"]),
                    "seed": int(packed["seed"]), "rotation": packed.get("rotation", "qr"),
                    "orig_dtype": str(packed.get("orig_dtype", "torch.float16")), "has_bias": False,
                    "indices_packed_shape": list(packed["indices_packed"].shape),
                    "codebook_shape": list(packed["codebook"].shape),
                    "norms_shape": list(packed["norms"].shape), "bias_shape": None,
                    "codebook_type": packed.get("codebook_type", "lloydmax")}
                sd[f"{lp}.packed_indices"] = cpu(packed["indices_packed"])
                sd[f"{lp}.norms"] = cpu(packed["norms"])
                sd[f"{lp}.codebook"] = cpu(packed["codebook"])
                sd[f"qmeta/{lp}/seed"] = torch.tensor(int(packed["seed"]), dtype=torch.int64)
            sd[f"{path}.shared_expert_gate.weight"] = cpu(sh["gate_row"]).reshape(1, -1)
    if quant_args and quant_args.get("seed") is not None:
        sd["qmeta/quant_args/seed"] = torch.tensor(int(quant_args["seed"]), dtype=torch.int64)
    with open(os.path.join(quant_dir, "meta.json"), "w", encoding="utf-8") as f:
        json.dump(meta, f, indent=1, ensure_ascii=False)
    if shards <= 1:
        save_file(sd, os.path.join(quant_dir, "model.safetensors"))
    else:
        keys = sorted(sd)
        weight_map = {}
        for i in range(shards):
            part = {k: sd[k] for k in keys[i::shards]}
            fname = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
            save_file(part, os.path.join(quant_dir, fname))
            weight_map.update({k: fname for k in part})
        with open(os.path.join(quant_dir, "model.safetensors.index.json"), "w", encoding="utf-8") as f:
            json.dump({"metadata": {}, "weight_map": weight_map}, f)
    return meta
