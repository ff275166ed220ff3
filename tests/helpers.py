"""Shared helpers for the parity tests (oracle object -> HIP module, error metrics)."""

import torch


def pools_dict(layer):
    """oracle MoELayer -> the ``pools`` argument of WxA16BitPartitionedGroupMoE.from_packed."""
    return {b: {"gate_up": p.gate_up, "down": p.down, "expert_offsets": p.expert_offsets}
            for b, p in layer.pools.items()}


def make_module(layer, mode="wxa16", device="cuda"):
    import dartmoq_hip
    moe = dartmoq_hip.WxA16BitPartitionedGroupMoE.from_packed(
        pools_dict(layer), layer.num_experts, layer.hidden, layer.inter, layer.top_k, device=device,
        shared_expert=layer.shared)
    return dartmoq_hip.convert_moe(moe, mode) if mode != "wxa16" else moe


def relerr(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def max_rel(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| / max |b| (the reference script's criterion, test_triton_mp_moe_e2e_bench.py:275-292)."""
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu().flatten(), b.double().cpu().flatten()
    return (torch.dot(a, b) / (a.norm() * b.norm()).clamp_min(1e-30)).item()
