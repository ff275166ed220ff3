"""Write tests/golden/ckpt_tiny/ (meta.json + model.safetensors) with the reference's own writer.

Run once in the build container (needs /root/reference; never on the GPU box):

    python tests/golden/make_ckpt_fixture.py

A tiny CPU model is assembled from the reference's classes (WxA16BitPartitionedGroupMoE,
WxA16Weights, WxA16Linear; weights quantized by turboquant_quantize_packed_full) and saved by
save_quantized_model (qwen35_quant_io.py:241-292), which calls collect_quant_metadata /
_moe_meta / _linear_meta (:36-125) and _build_qmeta_tensors.  Two MoE layers, H = 256, 4 experts,
top-2, one shared expert each:

  model.layers.0.mlp   every expert in exactly one bit pool (pools 4 and 2), I = 128
  model.layers.1.mlp   --slices 2 layout: I = 256, every expert cut into two sub-experts of 128
                       neurons; expert 0 and 2 have one sub-expert in pool 4 and one in pool 2,
                       expert 1 both in pool 2, expert 3 both in pool 4

The files are data (tensors and JSON), a few hundred KB.
"""

import os
import sys

import torch
import torch.nn as nn

REF = os.environ.get("DARTMOQ_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ckpt_tiny")
H, E, TOP_K, GS = 256, 4, 2, 128


def main():
    sys.path.insert(0, REF)
    from quantization.wxa16.bit_partitioned_moe import WxA16BitPartitionedGroupMoE, WxA16Weights
    from quantization.wxa16.linear import WxA16Linear
    from turboquant_utils.quantize import turboquant_quantize_packed_full
    from qwen35_quant_io import save_quantized_model

    g = torch.Generator().manual_seed(2024)

    def lin(n_in, n_out):
        m = nn.Linear(n_in, n_out, bias=False)
        with torch.no_grad():
            m.weight.copy_(torch.randn(n_out, n_in, generator=g) * 0.02)
        return m.half()

    class SharedMLP(nn.Module):
        def __init__(self, inter, bit, seed, uniform):
            super().__init__()
            kw = dict(bit_width=bit, group_size=GS, seed=seed, keep_on_gpu=True, uniform_codebook=uniform)
            self.gate_proj = WxA16Linear.from_linear(lin(H, inter), **kw)
            self.up_proj = WxA16Linear.from_linear(lin(H, inter), **kw)
            self.down_proj = WxA16Linear.from_linear(lin(inter, H), **kw)

    def build_moe(inter, widths_by_bit, shared):
        """widths_by_bit: {bit: [neurons of expert e in this pool, ...]}"""
        moe = WxA16BitPartitionedGroupMoE(gate=lin(H, E), num_experts=E, hidden_size=H,
                                          intermediate_size=inter, top_k=TOP_K, shared_expert=shared,
                                          shared_expert_gate=lin(H, 1))
        moe.enable_timing = False
        for bit, widths in widths_by_bit.items():
            total = sum(widths)
            gu = (torch.randn(2 * total, H, generator=g) * 0.02).half()
            dn = (torch.randn(H, total, generator=g) * 0.02).half()
            gu_p = turboquant_quantize_packed_full(gu, bit_width=bit, group_size=GS, seed=42 + bit)
            dn_p = turboquant_quantize_packed_full(dn, bit_width=bit, group_size=GS, seed=42 + bit + 1000)
            w = WxA16Weights(bit, H)
            w.set_packed_data(gu_p, dn_p)
            moe.bit_weights[str(bit)] = w
            offs = torch.zeros(E + 1, dtype=torch.long)
            offs[1:] = torch.tensor(widths, dtype=torch.long).cumsum(0)
            moe.expert_offsets[str(bit)] = offs
            moe.inter_size_by_bit[bit] = total
            moe.bit_list.append(bit)
        return moe

    class Layer(nn.Module):
        def __init__(self, mlp):
            super().__init__()
            self.mlp = mlp

    class Tiny(nn.Module):
        def __init__(self, layers):
            super().__init__()
            self.model = nn.Module()
            self.model.layers = nn.ModuleList(layers)

    layer0 = build_moe(128, {4: [128, 0, 0, 128], 2: [0, 128, 128, 0]},
                       SharedMLP(128, 4, seed=42, uniform=False))
    layer1 = build_moe(256, {4: [128, 0, 128, 256], 2: [128, 256, 128, 0]},
                       SharedMLP(128, 8, seed=43, uniform=True))
    model = Tiny([Layer(layer0), Layer(layer1)])
    os.makedirs(OUT, exist_ok=True)
    save_quantized_model(model, OUT, base_model_path=None, quant_args={"seed": 42, "slices": 2},
                         verbose=False)
    # Expected outputs for fixed inputs, computed with the reference's own CPU dequantizers
    # (dequantize-then-matmul in fp32, the algorithm of reference_forward_fp16 in
    # turboquant_utils/test_triton_mp_moe_e2e_bench.py:167-292): softmax -> top-k without
    # renormalisation, the expert output summed over every pool the expert lives in
    # (quantization/wxa16/bit_partitioned_moe.py:818-822), plus the gated shared expert (:1101-1106).
    import json
    from turboquant_utils.quantize import (turboquant_dequantize_packed, turboquant_dequantize_packed_cols,
                                           turboquant_dequantize_packed_rows)
    expected = {}
    for li, moe in enumerate((layer0, layer1)):
        x = (torch.randn(4, H, generator=g) * 0.5).half()
        logits = x.float() @ moe.gate.weight.float().t()
        w, idx = torch.topk(torch.softmax(logits, dim=-1), TOP_K, dim=-1)
        y = torch.zeros(4, H)
        for t in range(4):
            for j in range(TOP_K):
                e = int(idx[t, j])
                for bit_str, bw in moe.bit_weights.items():
                    offs = moe.expert_offsets[bit_str]
                    s0, s1 = int(offs[e]), int(offs[e + 1])
                    if s1 <= s0:
                        continue
                    wgu = turboquant_dequantize_packed_rows(bw.gate_up_packed, 2 * s0, 2 * s1).float()
                    wdn = turboquant_dequantize_packed_cols(bw.down_packed, s0, s1).float()
                    gu = wgu @ x[t].float()
                    act = torch.nn.functional.silu(gu[:s1 - s0]) * gu[s1 - s0:]
                    y[t] += w[t, j] * (wdn @ act)
        sh = moe.shared_expert

        def dq(linm):
            return turboquant_dequantize_packed({
                "indices_packed": linm.packed_indices, "codebook": linm.codebook, "norms": linm.norms,
                "seed": linm.seed, "group_size": linm.group_size,
                "shape": (linm.out_features, linm.in_features), "bit_width": linm.bit_width,
                "rotation": linm.rotation, "orig_dtype": "torch.float16"}).float()
        xs = x.float()
        hidden = torch.nn.functional.silu(xs @ dq(sh.gate_proj).t()) * (xs @ dq(sh.up_proj).t())
        gate = torch.sigmoid(xs @ moe.shared_expert_gate.weight.float().t())
        y_shared = (hidden @ dq(sh.down_proj).t()) * gate
        expected[f"model.layers.{li}.mlp"] = {
            "x_fp16_bits": x.view(torch.int16).flatten().tolist(),
            "topk_idx": idx.tolist(), "topk_w": w.tolist(),
            "y_routed": [[float("%.9g" % v) for v in r] for r in y.tolist()],
            "y_shared": [[float("%.9g" % v) for v in r] for r in y_shared.tolist()]}
    with open(os.path.join(OUT, "expected.json"), "w") as fh:
        json.dump(expected, fh)
    for f in sorted(os.listdir(OUT)):
        print(f, os.path.getsize(os.path.join(OUT, f)))


if __name__ == "__main__":
    main()
