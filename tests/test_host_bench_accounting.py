"""The algorithmic bytes and flops bench.py prices its rooflines with, against the per-unit
figures of the benchmark definition: per routed expert 3*H*I*bit/8 bytes of packed indices plus
6*H*I/128 bytes of fp16 norms (1,622,016 / 835,584 / 442,368 B at H = 2048, I = 512 for 4 / 2 / 1
bit; 2,506,752 / 4,866,048 B at H = 3072, I = 1024 for 2 / 4 bit), 6*H*I flop per expert and
token, and 2*T*H*2 bytes of activations in and out (no GPU needed)."""

import importlib.util
import os
import types

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _module(hidden, inter, expert_bits, shared_bit=None, shared_slices=0):
    """A stand-in with the fields bench.py reads: pools keyed by bit, every expert in the pool of
    its bit, the shared expert as `shared_slices` always-on experts of a pool of their own."""
    n = len(expert_bits)
    pools = {}
    for bit in sorted(set(expert_bits), reverse=True):
        offs, cur = [0], 0
        for e in range(n + shared_slices):
            if e < n and expert_bits[e] == bit:
                cur += inter
            offs.append(cur)
        pools[str(bit)] = types.SimpleNamespace(bit=bit, expert_offsets=offs)
    if shared_slices:
        offs, cur = [0], 0
        for e in range(n + shared_slices):
            if e >= n:
                cur += inter
            offs.append(cur)
        pools["shared"] = types.SimpleNamespace(bit=shared_bit, expert_offsets=offs)
    m = types.SimpleNamespace(hidden_size=hidden, intermediate_size=inter, num_experts=n,
                              n_shared=shared_slices, bit_weights=pools, top_k=8,
                              shared_intermediate_size=shared_slices * inter)
    m.weight_bytes_per_expert = lambda bit: 3 * hidden * inter * bit // 8 + 6 * hidden * inter // 128
    m.flops_per_token = lambda: 6 * hidden * (8 * inter + shared_slices * inter)
    return m


def test_per_expert_bytes_and_flops(bench):
    m = _module(2048, 512, [4, 2, 1, 2])
    assert [m.weight_bytes_per_expert(b) for b in (4, 2, 1)] == [1622016, 835584, 442368]
    counts = [3, 0, 1, 5]                                   # expert 1 gets no row
    total, per_pool = bench.layer_bytes(m, counts)
    assert total == 1622016 + 442368 + 835584
    assert per_pool == {"4": (1, 3, 4), "2": (1, 5, 2), "1": (1, 1, 1)}
    assert m.flops_per_token() == 8 * 6 * 2048 * 512 == 50331648
    big = _module(3072, 1024, [2, 4], shared_bit=4, shared_slices=1)
    assert [big.weight_bytes_per_expert(b) for b in (2, 4)] == [2506752, 4866048]
    assert big.flops_per_token() == 9 * 6 * 3072 * 1024 == 169869312


def test_kernel_work_splits_the_layer_between_its_two_gemms(bench):
    hidden, inter, tokens = 2048, 512, 7
    m = _module(hidden, inter, [4, 2, 1, 2])
    counts = [3, 0, 1, 5]
    w = bench.kernel_work(m, counts, tokens, fused_pools=0b101)
    layer_weights = 1622016 + 442368 + 835584
    assert w["layer_bytes"] == layer_weights + 2 * tokens * hidden * 2
    assert w["rows"] == 9 and w["distinct"] == 3
    # gate_up holds two thirds of an expert's indices and norms, down one third
    gu_w = sum(2 * hidden * inter * b // 8 + 4 * hidden * inter // 128 for b in (4, 2, 1))
    dn_w = sum(hidden * inter * b // 8 + 2 * hidden * inter // 128 for b in (4, 2, 1))
    assert gu_w + dn_w == layer_weights
    assert w["gu_bytes"] == gu_w + 3 * tokens * hidden * 2 + 9 * inter * 2     # rotated input once per pool
    assert w["dn_bytes"] == dn_w + 9 * inter * 2 + tokens * hidden * 2
    assert w["gu_flops"] == 2.0 * 9 * hidden * 2 * inter and w["dn_flops"] == 2.0 * 9 * inter * hidden
    assert w["gu_flops"] + w["dn_flops"] == 9 * 6 * hidden * inter
    # the fused down rotation is listed apart: pools 0 (4-bit, 3 rows) and 2 (1-bit, 1 row)
    assert w["gu_extra_flops"] == 2.0 * (3 + 1) * inter * 128
    assert w["gu_extra_bytes"] == 2 * (inter // 128) * 128 * 128 * 2


def test_roofline_picks_the_binding_roof(bench):
    r = bench.roofline_of(nbytes=8.0e6, flops=1.0e9, ms=0.01, mode="wxa16")       # 1 us of HBM, 0.4 us of MFMA
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert r["achieved"] == pytest.approx(800.0) and r["frac"] == pytest.approx(0.1)
    r = bench.roofline_of(nbytes=1.2e8, flops=6.87e10, ms=0.1, mode="wxa16")      # 15 us of HBM, 27.5 us of MFMA
    assert r["bound"] == "mfma" and r["unit"] == "TFLOP/s" and r["peak"] == 2500.0
    assert r["frac"] == pytest.approx(6.87e10 / 1e-4 / 2.5e15)
    r8 = bench.roofline_of(1.2e8, 6.87e10, 0.1, "wxa8")           # 15 us of HBM, 13.7 us of int8 MFMA
    assert r8["bound"] == "hbm"
