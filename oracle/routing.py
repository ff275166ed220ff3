"""Router, expert sort and bit-pool partition (oracle; test infrastructure only).

Follows quantization/wxa16/bit_partitioned_moe.py of the reference:
router :1112-1120, sort :1125-1138, pool partition :1014-1057 and the host
tile list of turboquant_utils/triton_kernels_a8.py:938-956.

Tie rule (the reference leaves it to torch.topk / an unstable argsort): the
top-k picks the *lowest expert index* among equal logits and the sort is
stable, so rows of one expert stay in ascending (token, slot) order.
"""

from __future__ import annotations

import numpy as np
import torch


def route_topk(logits: torch.Tensor, top_k: int, renormalize: bool = False):
    """softmax over experts, then top-k.  Returns (weights fp32 [T,k], idx int64 [T,k]).

    Selection is made on the logits (softmax is monotone) with a stable
    descending sort; weights are exp(l - max) / sum in fp32.  ``renormalize``
    divides by the sum of the kept weights (HF TopKRouter form); the plain
    Linear gate of the reference does not (:1117-1118).
    """
    lg = logits.float()
    order = torch.sort(lg, dim=-1, descending=True, stable=True).indices[:, :top_k]
    probs = torch.softmax(lg, dim=-1)
    w = torch.gather(probs, 1, order)
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    return w, order


def sort_by_expert(topk_idx: torch.Tensor, topk_w: torch.Tensor, num_experts: int):
    """Stable counting sort of the T*k routed rows by expert.

    Returns (sorted_tokens int64 [R], sorted_weights [R], sorted_slots int64 [R],
    offsets int64 [E+1]) where rows offsets[e]:offsets[e+1] belong to expert e.
    Reference: bit_partitioned_moe.py:1125-1138 (tokens_per_expert there is
    offsets[1:]).
    """
    t, k = topk_idx.shape
    flat_e = topk_idx.reshape(-1).long()
    order = torch.sort(flat_e, stable=True).indices
    counts = torch.bincount(flat_e, minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    return order // k, topk_w.reshape(-1)[order], order % k, offsets


def pool_members(expert_offsets: dict, offsets: torch.Tensor):
    """{bit_str: [(expert, bit, start, end, token_start, count)]}, _merged_pools :1014-1037.

    ``expert_offsets[bit_str]`` is the cumulative neuron offset list (E+1) of
    that pool; experts with a zero-width slice or no routed rows are skipped.
    """
    pools: dict[str, list] = {}
    num_experts = offsets.numel() - 1
    for e in range(num_experts):
        ts, te = int(offsets[e]), int(offsets[e + 1])
        if te <= ts:
            continue
        for bit_str, offs in expert_offsets.items():
            s, t = int(offs[e]), int(offs[e + 1])
            if t > s:
                pools.setdefault(bit_str, []).append((e, int(bit_str), s, t, ts, te - ts))
    return pools


def expert_info_rows(members):
    """gate_up expert_info rows [cursor, n, 2*start, 2*inter] (:1039-1047)."""
    inter = members[0][3] - members[0][2]
    info, cur = [], 0
    for _e, _b, start, _end, _ts, n in members:
        info.append((cur, n, 2 * start, 2 * inter))
        cur += n
    return info


def expert_info_groups(members, group_size: int):
    """down expert_info rows [cursor, n, start/gs, inter/gs] (:1049-1057)."""
    inter = members[0][3] - members[0][2]
    info, cur = [], 0
    for _e, _b, start, _end, _ts, n in members:
        info.append((cur, n, start // group_size, inter // group_size))
        cur += n
    return info


def merged_block_info(expert_info, block_b: int, block_n: int, n_extent: int) -> np.ndarray:
    """int32 [num_blocks, 3] = (expert_idx, block_b, block_n), triton_kernels_a8.py:938-956."""
    blocks = []
    for e, (_ts, cnt, _ss, sc) in enumerate(expert_info):
        if cnt <= 0 or sc <= 0:
            continue
        for b in range(-(-cnt // block_b)):
            for n in range(-(-n_extent // block_n)):
                blocks.append((e, b, n))
    if not blocks:
        raise ValueError("merged kernel: empty block list (no active experts)")
    return np.asarray(blocks, dtype=np.int32)


def zipf_logits(num_tokens: int, num_experts: int, seed: int, alpha: float = 1.1,
                skew: bool = True) -> torch.Tensor:
    """randn router logits plus a per-expert Zipf(alpha) log-bias under a seeded permutation."""
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(num_tokens, num_experts, generator=gen)
    if skew:
        perm = torch.randperm(num_experts, generator=torch.Generator().manual_seed(seed + 7919))
        bias = torch.empty(num_experts)
        bias[perm] = -alpha * torch.log(torch.arange(1, num_experts + 1, dtype=torch.float32))
        logits = logits + bias
    return logits
