"""Quantized Linear layers on MI355X: WxA16Linear and its WxA8 / WxFP8 variants.

Host-side mirror of quantization/wxa16/linear.py:27-260 (WxA16Linear: row-major packed indices,
fp16 norms [N, G], fp16 codebook, one rotation seed; forward = triton_fused_matmul_grouped),
quantization/wxa8/linear.py:79-159 (fused rotate + int8 quantize, integer GEMM) and
quantization/wxfp8/linear.py:37-100 (e4m3 activations and look-up table).  These are the Linears
of the shared expert of the MoE layer.  Like the reference's WxA8Linear._ensure_gf the module
converts the checkpoint layout to group-first once (norms divided by sqrt(128)) and keeps the
rotation matrices and the per-mode look-up table resident; a forward is one call of
dmq_linear_forward: two launches (rotate (+quantize), dequant GEMM) on the current stream, the
GEMM shaped by batch size.

Bit widths 1, 2, 4 and 8 are built, all through a codebook look-up.  8-bit weights run on the int8
path only with a uniform codebook (then the table is the identity w = idx - 128 and the step rides
the activation scale, the reference's IDENTITY_CB); the fp16 and e4m3 paths take any codebook.
"""

from __future__ import annotations

import torch

import ctypes

from . import hostprep, ops
from ._lib import EPI_STORE, MODE_A16, MODE_A8, MODE_FP8, LinearDesc, check, load

GROUP_SIZE = ops.GROUP_SIZE
SPLIT_MAX_ROWS = 64          # batches up to this size split K between waves or workgroups


_SPLIT_WS: dict = {}
_WORKSPACE: dict = {}


def _workspace(device, desc, rows: int) -> torch.Tensor:
    """Scratch of dmq_linear_forward, shared by the Linears of a (device, stream): launches on one
    stream run one after the other.  Grows to the largest request."""
    dev = torch.device(device)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(dev).cuda_stream)
    need = load().dmq_linear_workspace_bytes(ctypes.byref(desc), rows)
    if need == 0:
        raise ValueError("dmq_linear_workspace_bytes refused the Linear descriptor")
    ws = _WORKSPACE.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        _WORKSPACE[key] = ws
    return ws


def _split_workspace(device, k: int, rows: int, n_out: int, items: int):
    """fp32 planes and arrival counters of the K-sharing launches, one set per (device, stream):
    launches on one stream run one after the other and every launch leaves the counters zero."""
    dev = torch.device(device)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(dev).cuda_stream)
    need_p = k * rows * n_out
    need_c = items * ((n_out + 127) // 128)
    ws = _SPLIT_WS.get(key)
    if ws is None or ws[0].numel() < need_p or ws[1].numel() < need_c:
        ws = (torch.empty(max(need_p, ws[0].numel() if ws else 0), dtype=torch.float32, device=dev),
              torch.zeros(max(need_c, ws[1].numel() if ws else 0), dtype=torch.int32, device=dev))
        _SPLIT_WS[key] = ws
    return ws


class WxA16Linear:
    MODE = MODE_A16

    def __init__(self, in_features: int, out_features: int, bit_width: int, group_size: int,
                 packed_indices: torch.Tensor, codebook: torch.Tensor, norms: torch.Tensor, seed: int,
                 rotation: str = "qr", bias=None, orig_dtype: torch.dtype = torch.float16,
                 codebook_type: str = "lloydmax", device="cuda"):
        if bit_width not in (1, 2, 4, 8):
            raise ValueError(f"bit_width must be 1/2/4/8, got {bit_width}")
        if group_size != GROUP_SIZE:
            raise ValueError(f"group_size must be {GROUP_SIZE}, got {group_size}")
        if in_features % (8 // bit_width):
            raise ValueError(f"in_features ({in_features}) must fill whole bytes of {bit_width}-bit indices")
        if rotation != "qr":
            raise ValueError(f"rotation must be 'qr', got {rotation!r}")
        self.in_features, self.out_features = int(in_features), int(out_features)
        self.bit_width, self.group_size = int(bit_width), int(group_size)
        self.seed = int(seed.item()) if isinstance(seed, torch.Tensor) else int(seed)
        self.rotation, self.orig_dtype, self.codebook_type = rotation, orig_dtype, codebook_type
        self.device = torch.device(device)
        self.n_groups = -(-self.in_features // self.group_size)
        # A ragged last group (in_features % 128 = d > 0: the reference's per-group path,
        # turboquant_utils/triton_kernels.py:618-650, rotates it with a d x d matrix seeded
        # seed + g_start and scales by 1 / sqrt(d)) is widened to a full group once, here: index
        # bytes and activation columns padded with zeros, the d x d rotation in the corner of a
        # 128 x 128 matrix of zeros, the group's norm times sqrt(128 / d).
        self.k_padded = self.n_groups * self.group_size
        self.last_dim = self.in_features - (self.n_groups - 1) * self.group_size
        ppg = self.group_size * self.bit_width // 8
        row_bytes = self.in_features * self.bit_width // 8
        if tuple(packed_indices.shape) != (self.out_features, row_bytes):
            raise ValueError(f"packed_indices must be {(self.out_features, row_bytes)}, "
                             f"got {tuple(packed_indices.shape)}")
        if norms.dim() == 1:
            norms = norms.unsqueeze(1)
        if tuple(norms.shape) != (self.out_features, self.n_groups):
            raise ValueError(f"norms must be {(self.out_features, self.n_groups)}, got {tuple(norms.shape)}")
        self.codebook = codebook.to(self.device, torch.float16).contiguous()
        self.bias = None if bias is None else bias.to(self.device)
        # group-first relayout, norms / sqrt(gs): the row-major originals are not kept on the device
        packed_indices = packed_indices.to(self.device)
        norms = norms.to(self.device).half()
        full_groups = self.n_groups
        if self.k_padded != self.in_features:
            full_groups -= 1
            packed_indices = torch.nn.functional.pad(packed_indices, (0, self.n_groups * ppg - row_bytes))
            norms = norms.float()
            norms[:, -1] *= (self.group_size / self.last_dim) ** 0.5
            norms = norms.half()
        self.indices_gf, self.norms_gf = ops.convert_to_group_first(
            packed_indices.contiguous(), norms.contiguous(), self.group_size, self.bit_width, prescale=True)
        self.rot = hostprep.generate_batch_rotation_matrices(self.group_size, self.seed, full_groups,
                                                             self.group_size, self.device)
        if full_groups != self.n_groups:
            last = torch.zeros((1, self.group_size, self.group_size), dtype=torch.float16, device=self.device)
            small = hostprep.generate_rotation_matrix(self.last_dim, self.seed + full_groups * self.group_size)
            last[0, :self.last_dim, :self.last_dim] = small.to(self.device, torch.float16)
            self.rot = torch.cat([self.rot, last], 0).contiguous()
        self._ctx: dict[int, tuple] = {}
        self._info: dict[int, torch.Tensor] = {}
        self._tile_cache: dict = {}
        self._desc: dict = {}

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_packed(cls, packed: dict, bias=None, device="cuda"):
        """packed: the dictionary turboquant_quantize_packed_full returns (quantize.py:350-474):
        indices_packed, norms, codebook, seed, group_size, shape, bit_width."""
        n, k = (int(v) for v in packed["shape"])
        return cls(k, n, int(packed["bit_width"]), int(packed["group_size"]), packed["indices_packed"],
                   packed["codebook"], packed["norms"], packed["seed"],
                   rotation=packed.get("rotation", "qr"), bias=bias,
                   codebook_type=packed.get("codebook_type", "lloydmax"), device=device)

    @classmethod
    def from_reference_module(cls, lin, device="cuda"):
        """Build from a loaded WxA16Linear of the reference (duck-typed buffers and attributes,
        quantization/wxa16/linear.py:54-80); the module is not modified."""
        return cls(lin.in_features, lin.out_features, lin.bit_width, lin.group_size, lin.packed_indices,
                   lin.codebook, lin.norms, lin.seed, rotation=getattr(lin, "rotation", "qr"),
                   bias=getattr(lin, "bias", None),
                   orig_dtype=getattr(lin, "orig_dtype", torch.float16),
                   codebook_type=getattr(lin, "codebook_type", "lloydmax"), device=device)

    @classmethod
    def from_wxa16(cls, linear: "WxA16Linear"):
        """Switch a loaded layer to this precision mode in place (no tensor copies), like
        WxA8Linear.from_wxa16 (quantization/wxa8/linear.py:79-98)."""
        if not isinstance(linear, WxA16Linear):
            raise TypeError(f"expected WxA16Linear, got {type(linear)}")
        if cls.MODE == MODE_A8 and linear.bit_width == 8 and not hostprep.is_uniform_codebook(linear.codebook):
            raise ValueError("WxA8Linear takes 8-bit weights only with a uniform codebook")
        linear.__class__ = cls
        return linear

    # ------------------------------------------------------------------ forward
    def _mode_ctx(self):
        """(look-up table, activation extra scale) of this precision mode, built on first use."""
        ctx = self._ctx.get(self.MODE)
        if ctx is None:
            if self.MODE == MODE_A16:
                ctx = (self.codebook, 1.0)
            elif self.MODE == MODE_A8:
                ctx = hostprep.int8_lut_for_launch(self.codebook, self.device)
            else:
                q, scale = hostprep.build_fp8_codebook(self.codebook)
                ctx = (q.to(self.device), scale)
            self._ctx[self.MODE] = ctx
        return ctx

    def _expert_info(self, rows: int) -> torch.Tensor:
        info = self._info.get(rows)
        if info is None:
            if len(self._info) >= 64:
                self._info.pop(next(iter(self._info)))
            info = torch.tensor([[0, rows, 0, self.out_features]], dtype=torch.int32, device=self.device)
            self._info[rows] = info
        return info

    def _tiling(self, rows: int) -> dict:
        """A Linear is a single "expert": with 16-row tiles its launch has rows / 16 x
        out_features / 256 workgroups, far too few for 256 CUs when the rows are few.  Up to 16
        rows every wave takes one n-tile and the four waves of a workgroup split K (a workgroup per
        16 features: 35 -> 10 us for an 8-bit 4096 x 4096 matrix, 15 -> 10 us for a 4-bit one).  Up
        to 64 rows the waves still split K over four n-tiles each, except for 8-bit weights, whose
        K range is shared between four workgroups instead (fp32 partial sums, added in a fixed
        order by the last workgroup to arrive: 35 -> 21 us).  Bigger batches: see below.  The same
        policy as linear_shape() of the library, which forward() runs."""
        if rows <= 16:
            return {"tt": 1, "ks": 4, "nt": 1}
        k = 0
        if rows <= SPLIT_MAX_ROWS:
            if self.bit_width != 8:
                return {"tt": 1, "ks": 4}
            tt = 1
            k = 4 if self.n_groups % 4 == 0 else (2 if self.n_groups % 2 == 0 else 0)
        else:
            # the largest row tile that still gives every CU a workgroup (8-bit: at most 32 rows);
            # 16-row tiles on less than half the CUs: two workgroups share K
            blocks = (self.out_features + 255) // 256
            wgs = lambda t: ((rows + 16 * t - 1) // (16 * t)) * blocks
            tt = next((t for t in ((2,) if self.bit_width == 8 else (4, 2)) if wgs(t) >= 256), 1)
            if tt == 1 and wgs(1) <= 128 and self.n_groups % 2 == 0:
                k = 2
        if k <= 1:
            return {"tt": tt}
        # counters: one per (work item, feature block); the item list has rows // 16 + 1 slots
        partial, counter = _split_workspace(self.device, k, rows, self.out_features, rows // 16 + 1)
        return {"tt": 1, "ks": 1, "k_split": k, "split_ws": (partial, counter)}

    def _tiles(self, rows: int, tile_rows: int):
        """Work-item list of a batch of `rows` rows (device tensors, kept per batch size)."""
        key = (rows, tile_rows)
        t = self._tile_cache.get(key)
        if t is None:
            if len(self._tile_cache) >= 64:
                self._tile_cache.pop(next(iter(self._tile_cache)))
            t = ops.build_tiles(self._expert_info(rows), rows, tile_rows)
            self._tile_cache[key] = t
        return t

    def _descriptor(self) -> LinearDesc:
        d = self._desc.get(self.MODE)
        if d is None:
            lut, extra = self._mode_ctx()
            d = LinearDesc()
            d.mode, d.bit = self.MODE, self.bit_width
            d.in_features, d.out_features = self.k_padded, self.out_features
            d.indices_gf, d.norms_gf = self.indices_gf.data_ptr(), self.norms_gf.data_ptr()
            d.lut = lut.data_ptr() if lut is not None else None
            d.rot, d.extra_scale = self.rot.data_ptr(), float(extra)
            self._desc[self.MODE] = d
        return d

    @torch.no_grad()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """One call of dmq_linear_forward: the rotation (+ quantization) launch and the GEMM launch."""
        if not x.is_cuda:
            raise RuntimeError("dartmoq_hip layers run on the GPU only (no CPU fallback)")
        shape = x.shape
        if shape[-1] != self.in_features:
            raise ValueError(f"expected {self.in_features} input features, got {shape[-1]}")
        x2 = x.reshape(-1, self.in_features)
        src = x2 if x2.dtype == torch.float16 else x2.half()
        if self.k_padded != self.in_features:
            src = torch.nn.functional.pad(src, (0, self.k_padded - self.in_features))
        if src.stride(1) != 1 or src.stride(0) % 8:
            src = src.contiguous()
        rows = src.shape[0]
        out = torch.empty((rows, self.out_features), dtype=torch.float16, device=x.device)
        if rows:
            desc = self._descriptor()
            ws = _workspace(self.device, desc, rows)
            check(load().dmq_linear_forward(ctypes.byref(desc), src.data_ptr(), src.stride(0), rows,
                                            out.data_ptr(), self.out_features, ws.data_ptr(), ws.numel(),
                                            ops._stream(x.device)), "linear_forward")
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out.reshape(*shape[:-1], self.out_features).to(x.dtype)

    @torch.no_grad()
    def forward_by_pieces(self, x: torch.Tensor) -> torch.Tensor:
        """The same two launches issued through the generic entry points (dmq_rotate, then
        dmq_matmul_merged_gf over a one-matrix work list): what forward does inside one C call,
        kept as its cross-check."""
        if not x.is_cuda:
            raise RuntimeError("dartmoq_hip layers run on the GPU only (no CPU fallback)")
        shape = x.shape
        if shape[-1] != self.in_features:
            raise ValueError(f"expected {self.in_features} input features, got {shape[-1]}")
        x2 = x.reshape(-1, self.in_features)
        src = x2 if x2.dtype == torch.float16 else x2.half()
        if self.k_padded != self.in_features:
            src = torch.nn.functional.pad(src, (0, self.k_padded - self.in_features))
        rows = src.shape[0]
        if rows == 0:
            return torch.empty(*shape[:-1], self.out_features, dtype=x.dtype, device=x.device)
        lut, extra = self._mode_ctx()
        codes, scale = ops.rotate(self.MODE, src, self.rot, extra_scale=extra, scale_fp32=False)
        if load().dmq_linear_uses_i8_gemm(ctypes.byref(self._descriptor()), rows):
            # 8-bit uniform weights, int8 path, a big batch: the plain int8 GEMM
            out = ops.linear_gemm_i8(codes, scale, self.indices_gf, self.norms_gf)
            if self.bias is not None:
                out = out + self.bias.to(out.dtype)
            return out.reshape(*shape[:-1], self.out_features).to(x.dtype)
        tiling = self._tiling(rows)
        tt = tiling.get("tt") or ops.pick_tt(rows, 1)
        tiling["tt"] = tt
        out = ops.matmul_merged(self.MODE, self.bit_width, EPI_STORE, codes,
                                None if self.MODE == MODE_A16 else scale, self.indices_gf,
                                self.norms_gf, lut, self._expert_info(rows), groups=self.n_groups,
                                n_out=self.out_features, slice_is_groups=False, rows_total=rows,
                                tiling=self._tiles(rows, 16 * tt), **tiling)
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out.reshape(*shape[:-1], self.out_features).to(x.dtype)

    __call__ = forward

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bit_width={self.bit_width}, group_size={self.group_size}, rotation={self.rotation}")


class WxA8Linear(WxA16Linear):
    """int8 activations per token and group, int8 codebook look-up, i32 accumulation."""
    MODE = MODE_A8


class WxFP8Linear(WxA16Linear):
    """e4m3 activations per token and group, e4m3 codebook look-up, fp32 accumulation."""
    MODE = MODE_FP8
