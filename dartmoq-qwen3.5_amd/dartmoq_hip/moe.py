"""Bit-partitioned quantized MoE FFN layer on MI355X.

Host-side mirror of WxA16BitPartitionedGroupMoE and its WxA8 / WxFP8 / WxFP4 subclasses
(quantization/{wxa16,wxa8,wxfp8,wxfp4}/bit_partitioned_moe.py of the reference).  The module
keeps the checkpoint tensors of the reference format (per bit pool: packed indices, fp16
norms, fp16 codebook for gate_up [2*I*E_pool, H] and down [H, I*E_pool] plus cumulative
``expert_offsets``), derives the runtime layout once (group-first indices, norms divided by
sqrt(128), resident rotation matrices, per-mode look-up tables) and runs the whole routed
forward through one C call that allocates nothing and never synchronizes with the host.
"""

from __future__ import annotations

import ctypes
import math

import torch

from . import hostprep, ops
from ._lib import (MODE_A16, MODE_A8, MODE_BY_NAME, MODE_FP4, MODE_FP8, LayerDesc, PoolDesc,
                   PrenormArgs, RouterArgs, check, load)

GROUP_SIZE = 128


def _lib_max_pools() -> int:
    from ._lib import MAX_POOLS
    return MAX_POOLS


class BitPoolWeights:
    """Runtime form of one bit pool (the reference's WxA16Weights, :32-265, after
    _build_group_first :177-233 and the subclasses' _get_bit_context)."""

    def __init__(self, bit: int, gate_up: dict, down: dict, expert_offsets, device):
        self.bit = int(bit)
        self.expert_offsets = [int(v) for v in expert_offsets]
        self.gate_up_meta = {k: v for k, v in gate_up.items() if not torch.is_tensor(v)}
        self.down_meta = {k: v for k, v in down.items() if not torch.is_tensor(v)}
        gs = int(gate_up["group_size"])
        if gs != GROUP_SIZE or int(down["group_size"]) != GROUP_SIZE:
            raise ValueError(f"group_size must be {GROUP_SIZE}")
        self.gu_codebook = gate_up["codebook"].to(device, torch.float16).contiguous()
        self.dn_codebook = down["codebook"].to(device, torch.float16).contiguous()
        # group-first relayout + norms / sqrt(gs) on the GPU; row-major originals are not kept
        self.gu_idx, self.gu_norms = ops.convert_to_group_first(
            gate_up["indices_packed"].to(device), gate_up["norms"].to(device), gs, bit, prescale=True)
        self.dn_idx, self.dn_norms = ops.convert_to_group_first(
            down["indices_packed"].to(device), down["norms"].to(device), gs, bit, prescale=True)
        self.n_gate_up, self.hidden = gate_up["shape"]
        self.down_in = down["shape"][1]
        # resident rotations: gate_up [H/gs, gs, gs]; down one matrix per global group,
        # seed = down_seed + j*gs  (== seed + original_start + g*gs, triton_kernels.py:1310)
        self.gu_rot = hostprep.generate_batch_rotation_matrices(
            gs, int(gate_up["seed"]), self.hidden // gs, gs, device)
        self.dn_rot = hostprep.generate_batch_rotation_matrices(
            gs, int(down["seed"]), self.down_in // gs, gs, device)
        self._mode_ctx: dict[int, dict] = {}

    def context(self, mode: int) -> dict:
        """Per-mode look-up tables and scale constants, built on first use."""
        ctx = self._mode_ctx.get(mode)
        if ctx is not None:
            return ctx
        dev = self.gu_idx.device
        ctx = {"gu_w": self.gu_idx, "dn_w": self.dn_idx, "gu_norms": self.gu_norms,
               "dn_norms": self.dn_norms, "gu_extra": 1.0, "dn_extra": 1.0, "gu_wsb": 127,
               "dn_wsb": 127}
        if mode == MODE_A16:
            ctx["gu_lut"], ctx["dn_lut"] = self.gu_codebook, self.dn_codebook
        elif mode == MODE_A8:
            gq, gstep = hostprep.int8_lut_for_launch(self.gu_codebook, dev, round_lloyd_max_8bit=True)
            dq, dstep = hostprep.int8_lut_for_launch(self.dn_codebook, dev, round_lloyd_max_8bit=True)
            ctx.update(gu_lut=gq, dn_lut=dq, gu_extra=gstep, dn_extra=dstep)
        elif mode == MODE_FP8:
            gq, gs_ = hostprep.build_fp8_codebook(self.gu_codebook)
            dq, ds_ = hostprep.build_fp8_codebook(self.dn_codebook)
            ctx.update(gu_lut=gq.to(dev), dn_lut=dq.to(dev), gu_extra=gs_, dn_extra=ds_)
        elif mode == MODE_FP4:
            # cb ~= e2m1(nib) * 2^E0 * residual: 2^E0 rides the weight e8m0 byte, the residual is
            # folded into a copy of the norms (wxfp4/bit_partitioned_moe.py:94-100), indices are
            # folded to packed e2m1 once (fold_indices_to_e2m1, triton_kernels_fp4.py:80-122)
            gn, ge0, gres, _ = hostprep.build_e2m1_codebook(self.gu_codebook)
            dn, de0, dres, _ = hostprep.build_e2m1_codebook(self.dn_codebook)
            ctx.update(
                gu_lut=None, dn_lut=None, gu_nib=gn.to(dev), dn_nib=dn.to(dev),
                gu_wsb=127 + ge0, dn_wsb=127 + de0,
                gu_norms=(self.gu_norms.float() * gres).half().contiguous(),
                dn_norms=(self.dn_norms.float() * dres).half().contiguous(),
                gu_w=ops.fold_indices_to_e2m1(self.gu_idx, gn, self.bit),
                dn_w=ops.fold_indices_to_e2m1(self.dn_idx, dn, self.bit))
        else:
            raise ValueError(f"unknown mode {mode}")
        self._mode_ctx[mode] = ctx
        return ctx


class WxA16BitPartitionedGroupMoE:
    """Quantized MoE layer; ``forward(hidden_states)`` returns the routed-expert sum.

    Mirrors the constructor fields and ``forward`` contract of the reference class
    (quantization/wxa16/bit_partitioned_moe.py:268-318, :1059-1224).
    """

    MODE = "wxa16"
    rotation_hoist_threshold = 1.5
    SHARED_KEY = "shared"

    def __init__(self, num_experts: int, hidden_size: int, intermediate_size: int, top_k: int,
                 gate_weight: torch.Tensor | None = None, renormalize: bool = False, device="cuda"):
        self.num_experts = num_experts
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.top_k = top_k
        self.device = torch.device(device)
        self.gate_weight = None if gate_weight is None else gate_weight.to(self.device)
        self.renormalize = renormalize
        self.bit_weights: dict[str, BitPoolWeights] = {}
        self.expert_offsets: dict[str, list] = {}
        self.bit_list: list[int] = []
        # always-on shared expert, run as n_shared extra experts of the routed path (see
        # attach_shared_expert); its pool sits in bit_weights under SHARED_KEY
        self.n_shared = 0
        self.shared_intermediate_size = 0
        self.shared_gate_row = None
        self._desc = None
        self._workspace = None
        self._gate_f16 = None       # fp16 copy of gate_weight and the state word of forward_prenorm
        self._gate_src = None
        self._prenorm_state = None
        self.tt_override = 0        # activation tiles of 16 rows per wave (0 = pick from tokens)
        self.ks_override = 0        # waves splitting K inside a workgroup (0 = pick from tt)
        self.nbl_override = 0       # feature blocks per workgroup of the GEMMs (0 = pick from tokens)
        self.tile_table = None      # launch shapes by token count (dartmoq_hip.autotune.apply_config_table)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_packed(cls, pools: dict, num_experts: int, hidden_size: int, intermediate_size: int,
                    top_k: int, gate_weight=None, renormalize=False, device="cuda",
                    shared_expert: dict | None = None):
        """pools: {bit_str: {"gate_up": packed, "down": packed, "expert_offsets": [E+1]}} in
        processing order (the ModuleDict order of the reference).  shared_expert (optional):
        see attach_shared_expert."""
        moe = cls(num_experts, hidden_size, intermediate_size, top_k, gate_weight, renormalize, device)
        for bit_str, p in pools.items():
            bit = int(bit_str)
            if bit not in (1, 2, 4, 8):
                raise ValueError(f"bit_width must be 1/2/4/8, got {bit}")
            offs = [int(v) for v in p["expert_offsets"]]
            if len(offs) != num_experts + 1:
                raise ValueError("expert_offsets must have num_experts + 1 entries")
            widths = {b - a for a, b in zip(offs[:-1], offs[1:]) if b > a}
            if any(w_ % GROUP_SIZE or w_ > intermediate_size for w_ in widths):
                raise ValueError(f"the share of an expert in a pool must be a multiple of {GROUP_SIZE} "
                                 f"neurons and at most {intermediate_size}, got widths {sorted(widths)}")
            moe.bit_weights[bit_str] = BitPoolWeights(bit, p["gate_up"], p["down"], offs, moe.device)
            moe.expert_offsets[bit_str] = offs
            moe.bit_list.append(bit)
        if len(moe.bit_weights) > _lib_max_pools():
            raise ValueError(f"at most {_lib_max_pools()} bit pools per layer")
        # An expert may be cut into sub-experts that live in several pools (the --slices layout,
        # quantization/wxa16/bit_partitioned_moe.py:499-521): its shares must add up to the
        # expert's intermediate size, its output is the sum over its pools (:818-822).
        for ex in range(num_experts):
            total = sum(o[ex + 1] - o[ex] for o in moe.expert_offsets.values())
            if total != intermediate_size:
                raise ValueError(f"the shares of expert {ex} add up to {total} neurons, "
                                 f"expected {intermediate_size}")
        if shared_expert is not None:
            moe.attach_shared_expert(shared_expert)
        return moe

    def attach_shared_expert(self, shared: dict):
        """Add the always-on shared expert of the reference layer
        (``final += shared_expert(x) * sigmoid(shared_expert_gate(x))``,
        quantization/wxa16/bit_partitioned_moe.py:1101-1106).

        shared = {"gate": packed, "up": packed, "down": packed, "gate_row": fp16 [1, H] or [H]}:
        the three quantized Linears of the shared MLP in the row-major packed format of
        WxA16Linear (quantization/wxa16/linear.py:27-80; all three share bit width, codebook and
        seed, dartmoq_utils.py:884) and the weight of the sigmoid gate.  The shared width must be a
        multiple of the routed experts' width I: the neurons are cut into I_s / I slices which
        join the routed path as extra experts E, E+1, ... that every token selects with the gate
        value as its routing weight, so the shared expert costs no extra launches."""
        if self.n_shared:
            raise ValueError("shared expert already attached")
        if len(self.bit_weights) + 1 > _lib_max_pools():
            raise ValueError(f"at most {_lib_max_pools()} pools per layer including the shared expert")
        gate, up, down = shared["gate"], shared["up"], shared["down"]
        inter = self.intermediate_size
        i_s, h = (int(v) for v in gate["shape"])
        if h != self.hidden_size or tuple(up["shape"]) != (i_s, h) or tuple(down["shape"]) != (h, i_s):
            raise ValueError("shared expert shapes must be gate/up [I_s, H], down [H, I_s]")
        if i_s % GROUP_SIZE:
            raise ValueError(f"shared intermediate size {i_s} must be a multiple of {GROUP_SIZE}")
        # slices of the routed experts' width when that divides the shared width, else the widest
        # multiple of 128 that does (the layer then runs as a sub-expert layer: shares of several widths)
        inter = max(w_ for w_ in range(GROUP_SIZE, inter + 1, GROUP_SIZE) if i_s % w_ == 0)
        bit = int(gate["bit_width"])
        if bit not in (1, 2, 4, 8) or int(up["bit_width"]) != bit or int(down["bit_width"]) != bit:
            raise ValueError(f"shared expert bit_width must be 1/2/4/8 and equal for gate/up/down, got {bit}")
        if int(up["seed"]) != int(gate["seed"]):
            raise ValueError("gate and up of the shared expert must share the rotation seed")
        if not torch.equal(gate["codebook"].cpu().half(), up["codebook"].cpu().half()):
            raise ValueError("gate and up of the shared expert must share the codebook")
        m = i_s // inter
        # rows of slice v: gate[v*I:(v+1)*I] then up[v*I:(v+1)*I], the layout of a routed expert
        def interleave(a, b):
            a = a.reshape(m, inter, -1)
            b = b.reshape(m, inter, -1)
            return torch.cat([a, b], dim=1).reshape(2 * i_s, -1).contiguous()
        gu = dict(gate)
        gu["indices_packed"] = interleave(gate["indices_packed"], up["indices_packed"])
        gn, un = gate["norms"], up["norms"]
        if gn.dim() == 1:
            gn, un = gn.unsqueeze(1), un.unsqueeze(1)
        gu["norms"] = interleave(gn, un)
        gu["shape"] = (2 * i_s, h)
        e = self.num_experts
        offs = [0] * (e + 1) + [inter * (v + 1) for v in range(m)]
        for key, o in self.expert_offsets.items():
            o.extend([o[-1]] * m)
            self.bit_weights[key].expert_offsets = list(o)
        self.bit_weights[self.SHARED_KEY] = BitPoolWeights(bit, gu, dict(down), offs, self.device)
        self.expert_offsets[self.SHARED_KEY] = offs
        self.bit_list.append(bit)
        self.n_shared = m
        self.shared_intermediate_size = i_s
        self.shared_gate_row = shared["gate_row"].reshape(-1).to(self.device, torch.float16).contiguous()
        if self.shared_gate_row.numel() != h:
            raise ValueError("gate_row must hold hidden_size values")
        self._desc = None
        self._workspace = None
        return self

    @classmethod
    def from_reference_module(cls, ref, gate_weight=None, renormalize=False, device="cuda"):
        """Build from a loaded module of the reference (duck-typed, nothing is imported):
        ``ref.bit_weights[bit_str]`` must offer ``gate_up_packed`` / ``down_packed`` dictionaries
        (indices_packed, norms, codebook, seed, group_size, shape — the WxA16Weights properties,
        quantization/wxa16/bit_partitioned_moe.py:78-150), ``ref.expert_offsets[bit_str]`` the
        E+1 neuron offsets (:324), plus num_experts / hidden_size / intermediate_size / top_k
        (:290-293).  ``ref.shared_expert`` (gate_proj / up_proj / down_proj as WxA16Linear) and
        ``ref.shared_expert_gate`` (:294-295) are attached when present.  Tensors are copied to
        ``device`` once; the reference module is not modified."""
        pools = {}
        for bit_str in ref.bit_weights.keys():
            w = ref.bit_weights[bit_str]
            offs = ref.expert_offsets[bit_str]
            offs = offs.cpu().tolist() if torch.is_tensor(offs) else list(offs)
            pools[str(bit_str)] = {"gate_up": dict(w.gate_up_packed), "down": dict(w.down_packed),
                                   "expert_offsets": offs}
        shared = None
        sh, sh_gate = getattr(ref, "shared_expert", None), getattr(ref, "shared_expert_gate", None)
        if sh is not None and sh_gate is not None:
            # WxA16Linear buffers (quantization/wxa16/linear.py:66-69) of the shared MLP
            def packed(lin):
                return {"indices_packed": lin.packed_indices, "norms": lin.norms,
                        "codebook": lin.codebook, "seed": int(lin.seed),
                        "group_size": int(lin.group_size), "bit_width": int(lin.bit_width),
                        "shape": (int(lin.out_features), int(lin.in_features))}
            shared = {"gate": packed(sh.gate_proj), "up": packed(sh.up_proj),
                      "down": packed(sh.down_proj), "gate_row": sh_gate.weight}
        return cls.from_packed(pools, int(ref.num_experts), int(ref.hidden_size),
                               int(ref.intermediate_size), int(ref.top_k), gate_weight, renormalize,
                               device, shared_expert=shared)

    @classmethod
    def from_wxa16(cls, moe: "WxA16BitPartitionedGroupMoE"):
        """Switch an already loaded layer to this precision mode in place (no tensor copies),
        like WxA8BitPartitionedGroupMoE.from_wxa16 (wxa8/bit_partitioned_moe.py:47-61)."""
        if not isinstance(moe, WxA16BitPartitionedGroupMoE):
            raise TypeError(f"expected WxA16BitPartitionedGroupMoE, got {type(moe)}")
        moe.__class__ = cls
        moe._desc = None
        return moe

    # ------------------------------------------------------------------ descriptors
    def pool_mode(self, bit: int) -> int:
        mode = MODE_BY_NAME[self.MODE]
        if mode == MODE_FP4 and bit not in hostprep.FP4_BITS:
            # bit-2 pools (wxfp4/bit_partitioned_moe.py:50,296-299) and the 8-bit Linears of the
            # shared expert (:8) stay on the int8 path
            return MODE_A8
        return mode

    # How the Linears of the shared expert run when the layer is switched to an activation-quantized
    # mode: "wxa8" (the reference's default, also for wxfp8 / wxfp4 layers), "wxfp8" (its opt-in
    # attn="wxfp8" of convert_model_to_wxfp8) or "wxa16".
    shared_attn = "wxa8"

    def shared_pool_mode(self, bw: "BitPoolWeights") -> int:
        """Precision mode of the shared expert's pool.  The reference converts these Linears on
        their own rule (qwen35_quant_io.py:416-532): a WxA16 layer keeps them fp16; the other
        modes move an 8-bit Linear to int8 only when its codebook is the uniform grid (a Lloyd-Max
        codebook would lose levels on the int8 grid) and never to fp8 unless asked to
        (attn="wxfp8"); anything else stays on the fp16 path.  The reference decides per Linear;
        a pool has one mode for its gate_up and its down projection, so a shared expert with one
        uniform and one Lloyd-Max codebook runs both projections in fp16 here (the reference would
        run the uniform one in int8)."""
        mode = MODE_BY_NAME[self.MODE]
        if mode == MODE_A16 or self.shared_attn == "wxa16" or bw.bit != 8:
            return MODE_A16
        if mode == MODE_FP8 and self.shared_attn == "wxfp8":
            return MODE_FP8
        uniform = hostprep.is_uniform_codebook(bw.gu_codebook.cpu()) and \
            hostprep.is_uniform_codebook(bw.dn_codebook.cpu())
        return MODE_A8 if uniform else MODE_A16

    def _descriptor(self):
        if self._desc is not None:
            return self._desc
        e = self.num_experts + self.n_shared
        top_k = self.top_k + self.n_shared
        n_pools = len(self.bit_weights)
        start = torch.full((n_pools, e), -1, dtype=torch.int32)
        count = torch.zeros((n_pools, e), dtype=torch.int32)
        pool_arr = (PoolDesc * n_pools)()
        keep = []
        for pi, (bit_str, bw) in enumerate(self.bit_weights.items()):
            members = 0
            for ex in range(e):
                s, t = bw.expert_offsets[ex], bw.expert_offsets[ex + 1]
                if t > s:
                    start[pi, ex] = 2 * s
                    count[pi, ex] = 2 * (t - s)
                    members += 1
            mode = self.shared_pool_mode(bw) if bit_str == self.SHARED_KEY else self.pool_mode(bw.bit)
            ctx = bw.context(mode)
            keep.append(ctx)
            d = pool_arr[pi]
            d.bit, d.mode = bw.bit, mode
            # expected routed rows of the pool exceed threshold * T  <=>  share * top_k > threshold
            # (the shared pool sees every token: rotating by token never does more work)
            d.major = int(bit_str == self.SHARED_KEY or
                          members * self.top_k > self.rotation_hoist_threshold * self.num_experts)
            d.n_gate_up, d.down_groups = bw.n_gate_up, bw.down_in // GROUP_SIZE
            d.gu_w, d.gu_norms = ctx["gu_w"].data_ptr(), ctx["gu_norms"].data_ptr()
            d.gu_lut = ctx["gu_lut"].data_ptr() if ctx["gu_lut"] is not None else None
            d.gu_rot = bw.gu_rot.data_ptr()
            d.gu_extra_scale, d.gu_w_scale_byte = ctx["gu_extra"], ctx["gu_wsb"]
            d.dn_w, d.dn_norms = ctx["dn_w"].data_ptr(), ctx["dn_norms"].data_ptr()
            d.dn_lut = ctx["dn_lut"].data_ptr() if ctx["dn_lut"] is not None else None
            d.dn_rot = bw.dn_rot.data_ptr()
            d.dn_extra_scale, d.dn_w_scale_byte = ctx["dn_extra"], ctx["dn_wsb"]
        slice_start = start.to(self.device)
        slice_count = count.to(self.device)
        desc = LayerDesc()
        desc.hidden, desc.inter = self.hidden_size, self.intermediate_size
        desc.experts, desc.top_k, desc.pools = e, top_k, n_pools
        desc.pool = ctypes.cast(pool_arr, ctypes.POINTER(PoolDesc))
        desc.slice_start, desc.slice_count = slice_start.data_ptr(), slice_count.data_ptr()
        # Sub-expert layers: per (pool, expert) the first column of the pool's share inside the
        # expert's SiLU*up row (shares packed in pool order) and the rank of the pool among the
        # expert's pools; the distinct share widths; the largest number of pools per expert.
        widths_all = (count // 2)
        homes_per_expert = (count > 0).sum(0)
        sub = bool((homes_per_expert > 1).any()) or bool(((count > 0) & (widths_all != self.intermediate_size)).any())
        col_start = home = None
        if sub:
            col = torch.zeros((n_pools, e), dtype=torch.int32)
            rank = torch.zeros((n_pools, e), dtype=torch.int32)
            run_col = torch.zeros(e, dtype=torch.int32)
            run_rank = torch.zeros(e, dtype=torch.int32)
            for pi in range(n_pools):
                member = count[pi] > 0
                col[pi] = torch.where(member, run_col, torch.zeros_like(run_col))
                rank[pi] = torch.where(member, run_rank, torch.zeros_like(run_rank))
                run_col = run_col + widths_all[pi]
                run_rank = run_rank + member.int()
            widths = sorted({int(v) for v in widths_all[count > 0].tolist()})
            if len(widths) > 8:
                raise ValueError(f"at most 8 distinct share widths per layer, got {widths}")
            desc.n_widths = len(widths)
            for i, w_ in enumerate(widths):
                desc.widths[i] = w_
            desc.max_homes = int(homes_per_expert.max())
            col_start, home = col.to(self.device), rank.to(self.device)
            desc.col_start, desc.home = col_start.data_ptr(), home.data_ptr()
        self._desc = (desc, pool_arr, slice_start, slice_count, keep, col_start, home)
        return self._desc

    def _get_workspace(self, tokens: int) -> torch.Tensor:
        desc = self._descriptor()[0]
        need = load().dmq_moe_workspace_bytes(ctypes.byref(desc), tokens)
        if self._workspace is None or self._workspace.numel() < need:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self._workspace

    # ------------------------------------------------------------------ forward
    def route(self, x: torch.Tensor, router_logits: torch.Tensor | None = None):
        """softmax -> top-k (bit_partitioned_moe.py:1112-1120); logits default to x @ W_g^T."""
        if router_logits is None:
            if self.gate_weight is None:
                raise ValueError("no gate weight: pass router_logits or topk_idx/topk_w")
            router_logits = torch.matmul(x, self.gate_weight.t().to(x.dtype))
        if self.n_shared:
            return ops.route_topk_shared(router_logits, None, None, self.top_k, self.renormalize,
                                         x, self.shared_gate_row, self.num_experts, self.n_shared)
        return ops.route_topk(router_logits, self.top_k, self.renormalize)

    def widen_topk(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_w: torch.Tensor):
        """Append the shared-expert columns to a router's own top-k: (weights, indices) of shape
        [T, top_k + n_shared] (unchanged when the layer has no shared expert)."""
        if not self.n_shared or topk_idx.shape[-1] == self.top_k + self.n_shared:
            return topk_w, topk_idx
        return ops.route_topk_shared(None, topk_idx, topk_w, self.top_k, False, x,
                                     self.shared_gate_row, self.num_experts, self.n_shared)

    def _router_args(self, x, router_logits, topk_idx, topk_w):
        """dmq_router_args for this call plus the tensors it points into (kept alive by the caller)."""
        r = RouterArgs()
        keep = []
        if topk_idx is None:
            if router_logits is None:
                if self.gate_weight is None:
                    raise ValueError("no gate weight: pass router_logits or topk_idx/topk_w")
                router_logits = torch.matmul(x, self.gate_weight.t().to(x.dtype))
            if router_logits.dtype not in (torch.float32, torch.float16):
                router_logits = router_logits.float()
            router_logits = router_logits.contiguous()
            if tuple(router_logits.shape) != (x.shape[0], self.num_experts):
                raise ValueError("router_logits must be [tokens, num_experts]")
            keep.append(router_logits)
            r.logits = router_logits.data_ptr()
            r.logits_fp16 = int(router_logits.dtype == torch.float16)
            r.renorm = int(self.renormalize)
        else:
            if topk_idx.shape[-1] == self.top_k + self.n_shared and self.n_shared:
                # already widened by widen_topk: hand the router's own columns over
                topk_idx, topk_w = topk_idx[:, :self.top_k], topk_w[:, :self.top_k]
            topk_idx = topk_idx.to(torch.int32).contiguous()
            topk_w = topk_w.float().contiguous()
            if tuple(topk_idx.shape) != (x.shape[0], self.top_k) or topk_w.shape != topk_idx.shape:
                raise ValueError("topk_idx / topk_w must be [tokens, top_k]")
            keep += [topk_idx, topk_w]
            r.topk_idx, r.topk_w = topk_idx.data_ptr(), topk_w.data_ptr()
        if self.n_shared:
            r.shared_gate_row = self.shared_gate_row.data_ptr()
            r.n_shared = self.n_shared
        return r, keep

    def _tiling(self, tokens: int):
        """(tt, ks, nbl) handed to the library: explicit overrides, else the tuned table's entry for
        this batch size where the library accepts it, else zeros (the library's own choice)."""
        if self.tt_override or self.ks_override or self.nbl_override or not self.tile_table:
            return int(self.tt_override), int(self.ks_override), int(self.nbl_override)
        from . import autotune
        cfg = autotune.lookup_config(self.tile_table, tokens)
        if not autotune.is_config_valid(cfg, tokens, self.top_k + self.n_shared, self.hidden_size):
            return 0, 0, 0
        return cfg["tt"], cfg["ks"], cfg["nbl"]

    @torch.no_grad()
    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor | None = None,
                topk_idx: torch.Tensor | None = None, topk_w: torch.Tensor | None = None,
                residual: torch.Tensor | None = None) -> torch.Tensor:
        shape = hidden_states.shape
        x = hidden_states.reshape(-1, shape[-1])
        if not x.is_cuda:
            raise RuntimeError("dartmoq_hip layers run on the GPU only (no CPU fallback)")
        orig_dtype = x.dtype
        if x.dtype != torch.float16:
            x = x.half()
        x = x.contiguous()
        tokens = x.shape[0]
        if tokens == 0:                         # an empty batch has an empty output
            return torch.empty(shape, dtype=orig_dtype, device=x.device)
        router, keep = self._router_args(x, router_logits, topk_idx, topk_w)
        desc = self._descriptor()[0]
        ws = self._get_workspace(tokens)
        out = torch.empty_like(x)
        add = None if residual is None else residual.reshape(-1, shape[-1]).half().contiguous()
        stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
        check(load().dmq_moe_ffn_forward_routed(
            ctypes.byref(desc), ctypes.byref(router), x.data_ptr(), tokens,
            None if add is None else add.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(),
            *self._tiling(tokens), None, None, stream),
            "moe_ffn_forward_routed")
        del keep
        if orig_dtype != torch.float16:
            out = out.to(orig_dtype)
        return out.reshape(shape)

    __call__ = forward

    PRENORM_MAX_TOKENS = 16      # what dmq_moe_ffn_forward_prenorm takes
    PRENORM_AUTO_TOKENS = 8      # up to here forward_prenorm picks it by itself (measured: H=2048,
                                 # 256 experts, top-8: 1 token 57.7 -> 39.7 us, 4 tokens 54.6 -> 46.8,
                                 # 8 tokens 61.7 -> 60.1, 16 tokens 81.8 -> 86.3: the last router
                                 # workgroup takes the top-k of four tokens at a time)

    @torch.no_grad()
    def forward_prenorm(self, hidden_states_prenorm: torch.Tensor, norm_weight: torch.Tensor,
                        eps: float = 1e-6, residual: torch.Tensor | None = None,
                        return_normed: bool = False, logits_out: torch.Tensor | None = None,
                        fused: bool | None = None):
        """The layer from the block's pre-norm hidden states for a decode step of at most 16
        tokens: RMSNorm (out = h * rsqrt(mean(h^2) + eps) * (1 + weight),
        turboquant_utils/norm_kernels.py:79-117), the router projection with this module's
        ``gate_weight``, softmax + top-k (quantization/wxa16/bit_partitioned_moe.py:1112-1120) and
        the rotation of the gate_up input are one launch (dmq_moe_ffn_forward_prenorm); no norm
        kernel and no router GEMM run in front of the layer.  ``fused`` None picks that launch up
        to 8 tokens, True up to 16; more tokens (or False) take the separate steps (ops.rms_norm,
        the router GEMM, forward).  Returns the output, or (output, normalized input) with
        ``return_normed``.  ``logits_out`` (fp16 [tokens, num_experts], optional) receives the
        router logits."""
        shape = hidden_states_prenorm.shape
        h = hidden_states_prenorm.reshape(-1, shape[-1])
        if not h.is_cuda:
            raise RuntimeError("dartmoq_hip layers run on the GPU only (no CPU fallback)")
        if self.gate_weight is None:
            raise ValueError("forward_prenorm needs the module's gate_weight")
        orig_dtype = h.dtype
        tokens = h.shape[0]
        if tokens == 0:
            empty = torch.empty(shape, dtype=orig_dtype, device=h.device)
            return (empty, empty.clone()) if return_normed else empty
        limit = self.PRENORM_AUTO_TOKENS if fused is None else (self.PRENORM_MAX_TOKENS if fused else 0)
        if tokens > limit:
            x = ops.rms_norm(h, norm_weight, eps)
            logits = torch.matmul(x, self.gate_weight.t().to(x.dtype))
            if logits_out is not None:
                logits_out.copy_(logits)
            out = self.forward(x.reshape(shape), router_logits=logits, residual=residual)
            return (out, x.reshape(shape)) if return_normed else out
        if h.dtype != torch.float16:
            h = h.half()
        h = h.contiguous()
        if norm_weight.dtype not in (torch.float16, torch.float32):
            norm_weight = norm_weight.float()
        norm_weight = norm_weight.to(h.device).contiguous()
        if self._gate_f16 is None or self._gate_src is not self.gate_weight:
            self._gate_src = self.gate_weight          # a new gate_weight tensor refreshes the copy
            self._gate_f16 = self.gate_weight.to(device=h.device, dtype=torch.float16).contiguous()
        if self._prenorm_state is None:
            self._prenorm_state = torch.zeros(64, dtype=torch.int32, device=h.device)
        router = RouterArgs()
        router.renorm = int(self.renormalize)
        if self.n_shared:
            router.shared_gate_row = self.shared_gate_row.data_ptr()
            router.n_shared = self.n_shared
        x_norm = torch.empty_like(h) if return_normed else None
        pre = PrenormArgs()
        pre.norm_weight = norm_weight.data_ptr()
        pre.norm_weight_fp32 = int(norm_weight.dtype == torch.float32)
        pre.eps = float(eps)
        pre.gate_weight = self._gate_f16.data_ptr()
        pre.state = self._prenorm_state.data_ptr()
        pre.x_norm_out = None if x_norm is None else x_norm.data_ptr()
        if logits_out is not None:
            if (logits_out.dtype != torch.float16 or not logits_out.is_contiguous()
                    or tuple(logits_out.shape) != (tokens, self.num_experts)):
                raise ValueError("logits_out must be a contiguous fp16 [tokens, num_experts] tensor")
            pre.logits_out = logits_out.data_ptr()
        desc = self._descriptor()[0]
        ws = self._get_workspace(tokens)
        out = torch.empty_like(h)
        add = None if residual is None else residual.reshape(-1, shape[-1]).half().contiguous()
        stream = ctypes.c_void_p(torch.cuda.current_stream(h.device).cuda_stream)
        check(load().dmq_moe_ffn_forward_prenorm(
            ctypes.byref(desc), ctypes.byref(router), ctypes.byref(pre), h.data_ptr(), tokens,
            None if add is None else add.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(),
            *self._tiling(tokens), None, None, stream),
            "moe_ffn_forward_prenorm")
        if orig_dtype != torch.float16:
            out = out.to(orig_dtype)
            x_norm = None if x_norm is None else x_norm.to(orig_dtype)
        out = out.reshape(shape)
        return (out, x_norm.reshape(shape)) if return_normed else out

    # ------------------------------------------------------------------ accounting
    def weight_bytes_per_expert(self, bit: int) -> int:
        """Algorithmic packed-weight bytes of one expert: indices + fp16 norms."""
        h, i = self.hidden_size, self.intermediate_size
        return 3 * h * i * bit // 8 + 6 * h * i // GROUP_SIZE

    def flops_per_token(self) -> int:
        return 6 * self.hidden_size * (self.top_k * self.intermediate_size + self.shared_intermediate_size)


class WxA8BitPartitionedGroupMoE(WxA16BitPartitionedGroupMoE):
    MODE = "wxa8"


class WxFP8BitPartitionedGroupMoE(WxA16BitPartitionedGroupMoE):
    MODE = "wxfp8"


class WxFP4BitPartitionedGroupMoE(WxA8BitPartitionedGroupMoE):
    MODE = "wxfp4"


MOE_CLASS_BY_MODE = {
    "wxa16": WxA16BitPartitionedGroupMoE, "wxa8": WxA8BitPartitionedGroupMoE,
    "wxfp8": WxFP8BitPartitionedGroupMoE, "wxfp4": WxFP4BitPartitionedGroupMoE,
}


def convert_moe(moe: WxA16BitPartitionedGroupMoE, mode: str) -> WxA16BitPartitionedGroupMoE:
    """convert_model_to_wxa8 / wxfp8 / wxfp4 for one layer (qwen35_quant_io.py:416-532)."""
    return MOE_CLASS_BY_MODE[mode].from_wxa16(moe)


class HipStageProfiler:
    """Event-pair stage timer on the current stream (the role of the reference's
    CudaStageProfiler, turboquant_utils/cuda_profiler.py:51-174): ``begin_round()``,
    ``with stage(name)``, ``end_round() -> {stage: {"ms": total, "calls": n}}``."""

    def __init__(self, enabled: bool = True):
        self.enabled = enabled
        self._pairs = []

    def begin_round(self):
        self._pairs = []
        if self.enabled:
            torch.cuda.synchronize()

    class _Stage:
        def __init__(self, prof, name):
            self.prof, self.name = prof, name

        def __enter__(self):
            if self.prof.enabled:
                self.start = torch.cuda.Event(enable_timing=True)
                self.stop = torch.cuda.Event(enable_timing=True)
                self.start.record()
            return self

        def __exit__(self, *exc):
            if self.prof.enabled:
                self.stop.record()
                self.prof._pairs.append((self.name, self.start, self.stop))
            return False

    def stage(self, name: str):
        return HipStageProfiler._Stage(self, name)

    def end_round(self) -> dict:
        if not self.enabled:
            return {}
        torch.cuda.synchronize()
        stats: dict[str, dict] = {}
        for name, a, b in self._pairs:
            s = stats.setdefault(name, {"ms": 0.0, "calls": 0})
            s["ms"] += a.elapsed_time(b)
            s["calls"] += 1
        return stats


STAGE_NAMES = ("sort_prep", "rotation", "merged_gate_up", "act_quant_down", "merged_down", "combine")


@torch.no_grad()
def forward_staged(moe: WxA16BitPartitionedGroupMoE, x: torch.Tensor,
                   topk_idx: torch.Tensor | None = None, topk_w: torch.Tensor | None = None,
                   tt: int = 0, ks: int = 0, nbl: int = 0, profile: bool = True,
                   router_logits: torch.Tensor | None = None):
    """dmq_moe_ffn_forward_routed with instrumentation: the production forward with an event
    recorded on the launch stream after every stage (sort_prep includes the top-k when
    ``router_logits`` are given instead of ``topk_idx`` / ``topk_w``).  Returns (out fp16 [T, H], {stage: ms}, aux) where aux carries the
    per-expert routed-row counts (for byte accounting) and the tiling that was used.  Stage names
    follow the reference's profiler: sort_prep, rotation (rotation_hoisted / act_quant),
    merged_gate_up (with silu_mul fused), act_quant_down, merged_down (routing weight and scatter
    fused), combine (the add of the scattered rows)."""
    x = x.half().contiguous()
    tokens = x.shape[0]
    router, keep = moe._router_args(x, router_logits, topk_idx, topk_w)
    desc = moe._descriptor()[0]
    ws = moe._get_workspace(tokens)
    out = torch.empty_like(x)
    stream = torch.cuda.current_stream(x.device)
    events = [torch.cuda.Event(enable_timing=True) for _ in range(len(STAGE_NAMES) + 1)]
    handles = (ctypes.c_void_p * len(events))()
    if profile:
        for i, ev in enumerate(events):
            ev.record(stream)                       # materialise the HIP event behind the object
            handles[i] = ev.cuda_event
    aux = (ctypes.c_long * 8)()
    check(load().dmq_moe_ffn_forward_routed(
        ctypes.byref(desc), ctypes.byref(router), x.data_ptr(), tokens, None,
        out.data_ptr(), ws.data_ptr(), ws.numel(), int(tt or moe.tt_override),
        int(ks or moe.ks_override), int(nbl or moe.nbl_override), handles if profile else None, aux,
        ctypes.c_void_p(stream.cuda_stream)), "moe_ffn_forward_routed")
    torch.cuda.synchronize(x.device)
    stats = {}
    if profile:
        for i, name in enumerate(STAGE_NAMES):
            stats[name] = events[i].elapsed_time(events[i + 1])
    counts = ws[aux[2]:aux[2] + 4 * (moe.num_experts + moe.n_shared)].view(torch.int32).clone()
    n_items = int(ws[aux[4]:aux[4] + 4].view(torch.int32).item())
    return out, stats, {"counts": counts, "tt": int(aux[0]), "ks": int(aux[1]), "nbl": int(aux[5]),
                        "n_items": n_items, "fused_rot_pools": int(aux[6]), "down_tt": int(aux[7])}
