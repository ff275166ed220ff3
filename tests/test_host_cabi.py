"""CPU checks of the host side: the C-ABI library loads and exports every declared symbol,
argument validation returns the documented status codes without touching a GPU, and the
load-time host helpers agree with the oracle and the golden vectors."""

import ctypes
import json
import os
import re

import pytest
import torch

from oracle import codebook as ocodebook, luts as oluts, moe as omoe, rotation as orotation

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dartmoq_hip.h")
GOLDEN = os.path.join(ROOT, "tests", "golden", "lut_fixtures.json")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dmq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from dartmoq_hip import _lib
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 19
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/dartmoq_hip.h but not exported"
    assert set(declared) == set(_lib.PROTOTYPES), "ctypes prototypes and header disagree"
    assert lib.dmq_abi_version() == _lib.ABI_VERSION == 21
    assert lib.dmq_status_string(0) == b"ok"
    assert b"bit width" in lib.dmq_status_string(1)


def test_argument_validation_without_gpu():
    """Entry points reject bad arguments before any launch (status codes, no compute)."""
    from dartmoq_hip import _lib
    lib = _lib.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.dmq_convert_to_group_first(p, p, 4, 4, 3, 0, p, p, None) == 1           # bad bit
    assert lib.dmq_dequant_tile(p, p, None, 16, 0, 1, 8, 16, 2, p, None) == 3          # n0+n_cnt > N
    assert lib.dmq_fold_indices_to_e2m1(p, p, 4, 8, p, None) == 1
    assert lib.dmq_route_topk(None, 0, 1, 8, 2, 0, p, p, None) == 6                   # null logits
    assert lib.dmq_build_tiles(p, 4, 24, 8, 0, p, p, None) == 2                       # tile not /16
    assert lib.dmq_finalize_f16(p, None, 7, p, None) == 2
    assert lib.dmq_fill_zero(p, 6, None) == 2
    a = _lib.GemmArgs()
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 8                       # no pools
    a.n_pools = 1
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 1                       # bit 0
    a.pool[0].bit, a.mode, a.tt = 2, 9, 1
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5                       # bad mode
    a.mode, a.ks = 0, 3
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5                       # bad K split
    a.ks = 0
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 6                       # null pointers
    assert lib.dmq_combine_slots(p, 8, None, 4, 6, p, None) == 2                      # hidden % 8
    with pytest.raises(ValueError):
        _lib.check(2, "demo")
    with pytest.raises(TypeError):
        _lib.check(6, "demo")
    assert lib.dmq_moe_workspace_bytes(None, 4) == 0


def test_workspace_size_formula():
    from dartmoq_hip import _lib
    lib = _lib.load()
    d = _lib.LayerDesc()
    d.hidden, d.inter, d.experts, d.top_k, d.pools = 2048, 512, 256, 8, 3
    small = lib.dmq_moe_workspace_bytes(ctypes.byref(d), 64)
    big = lib.dmq_moe_workspace_bytes(ctypes.byref(d), 4096)
    r = 4096 * 8
    # dominated by the fp16 slot rows [R, H], x codes by routed row [R, H] and by token
    # [pools, T, H] (2 bytes per element) and act / act codes [R, I]
    main = r * 2048 * 2 + r * 2048 * 2 + 3 * 4096 * 2048 * 2 + 2 * r * 512 * 2
    assert big >= main
    assert big < 1.15 * main + (1 << 22)
    assert small < big


def test_cpu_tensors_are_rejected():
    from dartmoq_hip import ops
    with pytest.raises(RuntimeError):
        ops.unpack_nbit(torch.zeros(2, 2, dtype=torch.uint8), 2)
    with pytest.raises(RuntimeError):
        ops.quantize_act(1, torch.zeros(2, 128, dtype=torch.float16))
    with pytest.raises(ValueError):
        ops.unpack_nbit(torch.zeros(2, 2, dtype=torch.uint8), 3)


def test_host_helpers_match_oracle_and_golden():
    from dartmoq_hip import hostprep, synthetic
    golden = json.load(open(GOLDEN))
    for bit in (1, 2, 4):
        cents, bounds = hostprep.get_codebook(bit)
        o_cents, o_bounds = ocodebook.get_codebook(bit)
        assert torch.equal(cents, o_cents) and torch.equal(bounds, o_bounds)
        cb = cents.half()
        g = golden[str(bit)]
        q, step = hostprep.build_int8_codebook(cb)
        assert q.tolist() == g["int8"] and step == g["int8_step"]
        f8, s8 = hostprep.build_fp8_codebook(cb)
        assert f8.view(torch.uint8).tolist() == g["e4m3_bytes"] and s8 == g["e4m3_scale"]
        nib, e0, resid, _ = hostprep.build_e2m1_codebook(cb)
        assert nib.tolist() == g["e2m1_nib"] and e0 == g["e2m1_e0"] and resid == g["e2m1_residual"]
    assert torch.equal(hostprep.generate_rotation_matrix(128, 1046), orotation.rotation_matrix(128, 1046))
    mats = hostprep.generate_batch_rotation_matrices(128, 44, 3, 128)
    assert torch.equal(mats, orotation.batch_rotation_matrices(128, 44, 3, 128))
    assert synthetic.assign_bits(256, {2: 0.979, 1: 0.010, 4: 0.011}, 42) == \
        omoe.assign_bits(256, {2: 0.979, 1: 0.010, 4: 0.011}, 42)


def test_synthetic_quantizer_matches_oracle_on_cpu():
    """The benchmark's layer builder produces the same packed checkpoint tensors as the oracle."""
    from dartmoq_hip import synthetic
    from oracle import turboquant
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(96, 256, generator=g) * 0.02).half()
    for bit in (1, 2, 4):
        a = synthetic.quantize_packed(w, bit, 42 + bit)
        b = turboquant.quantize_packed(w, bit, 128, seed=42 + bit)
        assert torch.equal(a["indices_packed"], b["indices_packed"])
        assert torch.equal(a["norms"], b["norms"]) and torch.equal(a["codebook"], b["codebook"])
        assert a["shape"] == b["shape"] and a["seed"] == b["seed"]


def test_module_construction_errors():
    import dartmoq_hip
    with pytest.raises(TypeError):
        dartmoq_hip.WxA8BitPartitionedGroupMoE.from_wxa16(object())
    with pytest.raises(ValueError):
        dartmoq_hip.WxA16BitPartitionedGroupMoE.from_packed(
            {"3": {"gate_up": {}, "down": {}, "expert_offsets": [0, 1]}}, 1, 128, 128, 1, device="cpu")
    with pytest.raises(ValueError):
        dartmoq_hip.WxA16BitPartitionedGroupMoE.from_packed(
            {"2": {"gate_up": {}, "down": {}, "expert_offsets": [0, 128, 384]}}, 2, 128, 128, 1,
            device="cpu")


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_argument_validation_of_later_entry_points():
    """Status codes of the routing / norm / quantizer / routed-forward entry points for bad
    arguments (rejected before any launch)."""
    from dartmoq_hip import _lib
    lib = _lib.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.dmq_rms_norm(p, 0, p, 0, 4, 12, 16, 16, 1e-6, p, None) == 2            # n % 8
    assert lib.dmq_rms_norm(p, 0, None, 0, 4, 16, 16, 16, 1e-6, p, None) == 6         # no weight
    assert lib.dmq_rms_norm(p, 0, p, 0, 4, 16, 8, 16, 1e-6, p, None) == 3             # stride < n
    assert lib.dmq_rms_norm(p, 0, p, 0, 0, 16, 16, 16, 1e-6, p, None) == 0            # nothing to do
    assert lib.dmq_quantize_weights(p, 128, p, p, 4, 1, 3, p, p, None) == 1           # bit 3
    assert lib.dmq_quantize_weights(p, 64, p, p, 4, 1, 4, p, p, None) == 2            # row shorter than K
    assert lib.dmq_quantize_weights(p, 128, None, p, 4, 1, 4, p, p, None) == 6
    assert lib.dmq_route_topk_shared(None, 0, None, None, 4, 8, 2, 0, p, p, 128, 1, p, p, None) == 6
    assert lib.dmq_route_topk_shared(p, 0, None, None, 4, 8, 2, 0, None, p, 128, 1, p, p, None) == 6
    assert lib.dmq_route_topk_shared(p, 0, None, None, 4, 8, 2, 0, p, p, 128, -1, p, p, None) == 3
    d = _lib.LayerDesc()
    r = _lib.RouterArgs()
    assert lib.dmq_moe_ffn_forward_routed(ctypes.byref(d), ctypes.byref(r), p, 4, None, p, p, 64, 0, 0, 0,
                                          None, None, None) == 6                       # no pools / router
    a = _lib.GemmArgs()
    a.n_pools, a.mode, a.tt, a.epi = 1, 0, 1, 3
    a.pool[0].bit = 8
    a.pool[0].mode = 0
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) in (5, 6)                  # fused rotation: no 8-bit pools
    a.epi = 7
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5                       # unknown epilogue


def test_linear_entry_point_validation():
    """dmq_linear_forward / dmq_linear_workspace_bytes reject bad descriptors before any launch."""
    from dartmoq_hip import _lib
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096 + 256)
    base = ctypes.addressof(buf)
    p = ctypes.c_void_p((base + 255) // 256 * 256)
    d = _lib.LinearDesc()
    d.mode, d.bit, d.in_features, d.out_features, d.extra_scale = 0, 4, 256, 128, 1.0
    assert lib.dmq_linear_workspace_bytes(ctypes.byref(d), 0) == 0
    small = lib.dmq_linear_workspace_bytes(ctypes.byref(d), 16)
    big = lib.dmq_linear_workspace_bytes(ctypes.byref(d), 4096)
    assert 0 < small < big and big >= 4096 * 256 * 2              # the rotated fp16 rows at least
    d8 = _lib.LinearDesc()
    d8.mode, d8.bit, d8.in_features, d8.out_features = 1, 8, 512, 128
    # 17 .. 64 rows of 8-bit weights add the fp32 planes of the shared K range
    assert lib.dmq_linear_workspace_bytes(ctypes.byref(d8), 64) >= 64 * 512 + 4 * 64 * 128 * 4
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, p, 4096, None) == 6   # no weights
    d.indices_gf = d.norms_gf = d.lut = d.rot = p
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 0, p, 128, p, 4096, None) == 0   # no rows
    assert lib.dmq_linear_forward(ctypes.byref(d), None, 256, 4, p, 128, p, 4096, None) == 6
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 128, 4, p, 128, p, 4096, None) == 3   # x_stride < K
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 260, 4, p, 128, p, 4096, None) == 2   # x_stride % 8
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, p, 64, None) == 8     # workspace too small
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, ctypes.c_void_p(p.value + 4), 4096,
                                  None) == 2                                                # unaligned
    d.lut = None
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, p, 4096, None) == 6   # table missing
    d.lut, d.mode = p, 3
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, p, 4096, None) == 5   # no WxFP4 Linear
    d.mode, d.bit = 0, 3
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, p, 4096, None) == 1
    d.bit, d.out_features = 4, 100
    assert lib.dmq_linear_forward(ctypes.byref(d), p, 256, 4, p, 128, p, 4096, None) == 2


def test_k_sharing_argument_validation():
    """k_split of the merged GEMM: 2 or 4 workgroups per block (8 and 16 with the plain-store
    epilogue only), 16-row tiles, never the scatter epilogue, groups divisible, scratch present
    (all rejected before any launch)."""
    from dartmoq_hip import _lib
    lib = _lib.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    a = _lib.GemmArgs()
    a.mode, a.epi, a.tt, a.n_pools = 0, _lib.EPI_SILU, 1, 1
    q = a.pool[0]
    q.w = q.norms = q.lut = q.expert_info = q.act = p
    q.n_total, q.bit, q.mode = 256, 2, 0
    a.items = a.n_items = a.out = p
    a.max_items, a.groups, a.n_out, a.half_width, a.act_row_bytes = 4, 4, 128, 128, 1024
    a.k_split = 3
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5
    a.k_split = 2
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 6           # no scratch
    a.split_partial = a.split_counter = p
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 3           # split_rows missing
    a.split_rows, a.tt = 16, 2
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5           # 16-row tiles only
    a.tt, a.epi = 1, _lib.EPI_SCATTER
    a.row_weight = a.row_slot = p
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5           # not the scatter epilogue
    a.epi, a.k_split = _lib.EPI_SILU, 8
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5           # 8 only with the plain store
    a.epi = _lib.EPI_STORE
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 2           # 4 groups, 8 workgroups
    a.k_split, a.nt = 0, 1
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5           # one n-tile per wave: ks = 4 only
    a.ks, a.tt = 4, 2
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5           # ... and 16-row tiles
    a.tt, a.nt = 1, 3
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 5           # 0, 1 or 4
    a.nt, a.ks = 0, 0
    a.epi, a.k_split, a.groups, a.act_row_bytes = _lib.EPI_SILU, 4, 6, 2048
    assert lib.dmq_matmul_merged_gf(ctypes.byref(a), None) == 2           # 6 groups, 4 workgroups


def test_ctypes_structs_match_the_header_layout(tmp_path):
    """Size and the offset of the last field of every argument struct, as gcc lays the header out,
    against the ctypes mirror: a field missing on one side shifts everything behind it (and ctypes
    accepts an assignment to a field it does not know without a word)."""
    import ctypes
    import shutil
    import subprocess
    from dartmoq_hip import _lib
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    pairs = [("dmq_gemm_pool", _lib.GemmPool), ("dmq_gemm_args", _lib.GemmArgs),
             ("dmq_pool_desc", _lib.PoolDesc), ("dmq_linear_desc", _lib.LinearDesc),
             ("dmq_layer_desc", _lib.LayerDesc), ("dmq_router_args", _lib.RouterArgs),
             ("dmq_prenorm_args", _lib.PrenormArgs)]
    lines = ['#include "dartmoq_hip.h"', "#include <stdio.h>", "#include <stddef.h>", "int main(void) {"]
    for cname, cls in pairs:
        last = cls._fields_[-1][0]
        lines.append(f'  printf("%zu %zu\\n", sizeof({cname}), offsetof({cname}, {last}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.dirname(HEADER), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    for (cname, cls), line in zip(pairs, out):
        size, off = (int(v) for v in line.split())
        last = cls._fields_[-1][0]
        assert ctypes.sizeof(cls) == size, f"{cname}: ctypes {ctypes.sizeof(cls)} bytes, header {size}"
        assert getattr(cls, last).offset == off, f"{cname}.{last}: ctypes offset differs from the header"
