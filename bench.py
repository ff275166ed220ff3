#!/usr/bin/env python3
"""MoE-layer throughput benchmark on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--tokens 2048] [--sweep 1,16,64,256,4096] [--mode wxa16]

A step is one pass of the hot path (device top-k routing, permutation, rotation, gate_up
dequant-GEMM + SiLU*up, per-expert rotation, down dequant-GEMM + scatter-add, fp16 store) over
one batch of synthetic tokens of BASELINE configs[1]: H=2048, 256 experts, top-8, I=512, WxA16
with mixed bit pools at ~2 bpw and Zipf(1.1)-skewed routing.  Inputs are resident in HBM when
the timed region starts.  The 2 bpw layer (~216 MB packed) fits in the 256 MB Infinity Cache, so
the steps rotate through three independent copies of the layer; a small batch touches few
experts, so its steps also cycle through router logits with the expert axis rolled until the
distinct weights of one cycle exceed twice that cache (`weight_copies_rotated`, `logit_variants`,
`cycle_weight_bytes` of every entry).

Defaults: 50 untimed warm-up steps and 500 timed ones (about 0.15 s of GPU work).  The GPU takes
tens of milliseconds of sustained load to reach its working clocks, so every measurement starts
with an untimed prelude of fixed length (`clock_prelude_s` in the JSON) of the same forwards:
short and long runs then read the same time per step.

`modes` holds the activation-quantized modes on the configurations named for them (configs[2]
WxA8, configs[4] WxFP8 and WxFP4; the all-4-bit layer, uniform routing) at 2048 and 64 tokens, each
with the roofline of its gate_up launch; `sweep` the decode sizes of the main configuration.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the merged gate_up dequant-GEMM),
timed live with events on the stream it runs on, on its algorithmic bytes and flops: packed
indices, norms and activation rows; the down-projection rotation the same launch performs is
listed beside them as `extra_bytes` / `extra_flops`.  `roofline_down` is the same for the down
dequant-GEMM.  `cpu_baseline` is the CPU
oracle (dequantize-then-matmul, fp32) timed on the host cores on a bounded sample.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG_DIR = os.path.join(ROOT, "dartmoq-qwen3.5_amd")
for _p in (ROOT, PKG_DIR):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK = 8.0e12          # B/s, MI355X HBM3E
MFMA_PEAK = {"wxa16": 2.5e15, "wxa8": 5.0e15, "wxfp8": 5.0e15, "wxfp4": 10.1e15}
DTYPE = {"wxa16": "f16", "wxa8": "i8", "wxfp8": "f8e4m3", "wxfp4": "f4e2m1"}
N_COPIES = 3


def layer_bytes(mod, counts):
    """Algorithmic HBM bytes of one forward: packed weights (indices + fp16 norms) of the
    distinct routed experts plus activations in and out."""
    h, i = mod.hidden_size, mod.intermediate_size
    total = 0
    per_pool = {}
    n_exp = mod.num_experts + mod.n_shared      # the shared expert counts as n_shared slices
    for bit_str, bw in mod.bit_weights.items():
        distinct = sum(1 for e in range(n_exp)
                       if counts[e] > 0 and bw.expert_offsets[e + 1] > bw.expert_offsets[e])
        rows = sum(int(counts[e]) for e in range(n_exp)
                   if bw.expert_offsets[e + 1] > bw.expert_offsets[e])
        per_pool[bit_str] = (distinct, rows, bw.bit)
        total += distinct * mod.weight_bytes_per_expert(bw.bit)
    return total, per_pool


PRELUDE_S = 0.5
MALL_BYTES = 256 << 20     # Infinity Cache of the MI355X
MAX_LOGIT_VARIANTS = 256


def settle_clocks(mods, x, logits, seconds):
    """Untimed load of fixed duration before a measurement: the GPU needs tens of milliseconds of
    sustained work to reach its working clocks (and drops them again while the host is busy), so
    without it a 20-step run reads 15 % slower than a 500-step run of the same thing."""
    import torch
    n, v = len(mods), len(logits)
    t0 = time.perf_counter()
    s = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            mods[s % n].forward(x, router_logits=logits[s % v])
            s += 1
        torch.cuda.synchronize()
    return time.perf_counter() - t0


def time_steps(mods, x, logits, steps, warmup):
    """Step s runs weight copy s % copies on router logits s % variants."""
    import torch
    n, v = len(mods), len(logits)
    settle_clocks(mods, x, logits, PRELUDE_S)
    for s in range(warmup):
        mods[s % n].forward(x, router_logits=logits[s % v])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        mods[s % n].forward(x, router_logits=logits[s % v])
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def pick_rotation(mods, x, base_logits):
    """Router logits for the timed steps such that no weight can stay in the Infinity Cache from
    one use to the next.  A small batch touches a few experts only, so three copies of them fit
    the cache; the steps therefore also cycle through variants of the logits with the expert axis
    rolled (the same distribution of routed rows under another expert numbering), as many as it
    takes for the distinct (copy, expert) weights of one cycle to exceed twice the cache.  Returns
    the logits, the routed-row counts of each variant and the description of the cycle."""
    import math
    import torch
    from dartmoq_hip.moe import forward_staged
    mod, copies = mods[0], len(mods)
    n_exp = mod.num_experts + mod.n_shared
    experts = base_logits.shape[1]
    counts_of = {}
    variants = 1
    while True:
        shifts = [v * (experts // variants) for v in range(variants)]
        for sh in shifts:
            if sh not in counts_of:
                lg = torch.roll(base_logits, shifts=sh, dims=1).contiguous()
                _o, _s, aux = forward_staged(mod, x, router_logits=lg, profile=False)
                counts_of[sh] = (lg, aux["counts"].cpu().tolist())
        cycle = math.lcm(copies, variants)
        weight_bytes = 0
        for c in range(copies):
            union = [0] * n_exp
            for s in range(c, cycle, copies):
                cnt = counts_of[shifts[s % variants]][1]
                union = [u or int(k > 0) for u, k in zip(union, cnt)]
            weight_bytes += layer_bytes(mod, union)[0]
        if weight_bytes >= 2 * MALL_BYTES or variants >= MAX_LOGIT_VARIANTS:
            break
        variants *= 2
    logits = [counts_of[sh][0] for sh in shifts]
    counts = [counts_of[sh][1] for sh in shifts]
    return logits, counts, {"weight_copies_rotated": copies, "logit_variants": variants,
                            "cycle_steps": cycle, "cycle_weight_bytes": weight_bytes,
                            "exceeds_twice_infinity_cache": weight_bytes >= 2 * MALL_BYTES}


def kernel_work(mod, counts, tokens, fused_pools):
    """Algorithmic work of one forward with these routed-row counts: the layer's bytes, and for
    the gate_up and the down launch the packed indices + fp16 norms of the distinct routed experts
    and the activation rows in and out (bytes) and the GEMM itself (flops).  What the gate_up
    launch does on top for the pools in `fused_pools` (it rotates its SiLU*up rows for the down
    projection: 2*I*128 flop per row, one 32 KiB matrix per distinct expert and down group) is
    kept apart as extra_*."""
    h, i = mod.hidden_size, mod.intermediate_size
    layer_total, per_pool = layer_bytes(mod, counts)
    w = {"layer_bytes": layer_total + 2 * tokens * h * 2, "gu_bytes": 0, "gu_flops": 0.0,
         "gu_extra_bytes": 0, "gu_extra_flops": 0.0, "dn_bytes": tokens * h * 2, "dn_flops": 0.0,
         "rows": 0, "distinct": 0}
    for p, (_key, (d_b, r_b, bit_b)) in enumerate(per_pool.items()):
        w["gu_bytes"] += d_b * (2 * h * i * bit_b // 8 + 4 * h * i // 128)
        w["gu_bytes"] += (tokens if r_b else 0) * h * 2 + r_b * i * 2
        w["gu_flops"] += 2.0 * r_b * h * 2 * i
        w["dn_bytes"] += d_b * (h * i * bit_b // 8 + 2 * h * i // 128) + r_b * i * 2
        w["dn_flops"] += 2.0 * r_b * i * h
        if fused_pools >> p & 1:
            w["gu_extra_flops"] += 2.0 * r_b * i * 128
            w["gu_extra_bytes"] += d_b * (i // 128) * 128 * 128 * 2
        w["rows"] += r_b
        w["distinct"] += d_b
    return w


def roofline_of(nbytes, flops, ms, mode):
    """The binding roofline of a launch of `nbytes` algorithmic bytes and `flops` algorithmic
    flops that took `ms`."""
    t_hbm, t_mfma = nbytes / HBM_PEAK, flops / MFMA_PEAK[mode]
    if t_hbm >= t_mfma:
        roof = {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9,
                "unit": "GB/s"}
    else:
        roof = {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12,
                "peak": MFMA_PEAK[mode] / 1e12, "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    return roof


def measure(mods, tokens, steps, warmup, seed, zipf, mode):
    """Throughput of the full layer plus the live timing of its two GEMM launches."""
    import torch
    from dartmoq_hip import synthetic
    from dartmoq_hip.moe import forward_staged
    mod = mods[0]
    x = torch.randn(tokens, mod.hidden_size, generator=torch.Generator().manual_seed(seed)).half().cuda()
    base = synthetic.zipf_logits(tokens, mod.num_experts, seed, skew=zipf).cuda()
    logits, counts, rotation = pick_rotation(mods, x, base)
    sec = time_steps(mods, x, logits, steps, warmup)

    # stage timing (events on the launch stream), copies and logits rotating like the timed loop,
    # every variant of the logits the same number of times
    n_var = len(logits)
    reps = n_var * -(-max(3, min(steps, 20)) // n_var)
    acc = {}
    aux = None
    for r in range(-1, reps):
        _out, stats, aux = forward_staged(mods[r % len(mods)], x, router_logits=logits[r % n_var])
        if r < 0:
            continue                                   # first pass warms the allocator
        for name, ms in stats.items():
            acc[name] = acc.get(name, 0.0) + ms
    stage_ms = {n: v / reps for n, v in acc.items()}
    fused = aux["fused_rot_pools"]
    work = [kernel_work(mod, c, tokens, fused) for c in counts]
    avg = {key: sum(w[key] for w in work) / len(work) for key in work[0]}
    flops = tokens * mod.flops_per_token()

    # dominant kernel: the merged gate_up dequant-GEMM (one launch over all bit pools)
    gu_ms = stage_ms["merged_gate_up"]
    roof = roofline_of(avg["gu_bytes"], avg["gu_flops"], gu_ms, mode)
    roof["traffic"] = None
    shared_k = f", K shared by {-aux['ks']} workgroups" if aux["ks"] < 0 else ""
    gemv = aux["tt"] == 0                        # at most four tokens: dot products on the vector ALU
    gu_kernel = (f"dmq_gemm_gf_kernel<tt={aux['tt']},ks={max(aux['ks'], 1)},"
                 f"{'SILU_ROT' if fused else 'SILU'}> merged gate_up"
                 f"{' + down rotation' if fused else ''}, nbl={min(aux['nbl'], 2)}{shared_k}")
    if gemv:
        gu_kernel = f"dmq_gemv_kernel<{mod.hidden_size // 512},SILU> merged gate_up"
    roof.update(kernel=gu_kernel, launch_ms=gu_ms,
                algorithmic_bytes=avg["gu_bytes"], algorithmic_flops=avg["gu_flops"],
                extra_bytes=avg["gu_extra_bytes"], extra_flops=avg["gu_extra_flops"],
                distinct_experts=avg["distinct"], routed_rows=avg["rows"])
    dn_ms = stage_ms["merged_down"]
    roof_down = roofline_of(avg["dn_bytes"], avg["dn_flops"], dn_ms, mode)
    dn_kernel = f"dmq_gemm_gf_kernel<tt={aux['down_tt']},SCATTER> merged down"
    if gemv:
        dn_kernel = f"dmq_gemv_kernel<{mod.intermediate_size // 512},SCATTER> merged down"
    roof_down.update(kernel=dn_kernel,
                     launch_ms=dn_ms, algorithmic_bytes=avg["dn_bytes"],
                     algorithmic_flops=avg["dn_flops"])
    return {
        "tokens": tokens, "ms_per_step": sec * 1e3, "tokens_per_s": tokens / sec,
        "eff_tflops": flops / sec / 1e12,
        "layer_hbm_frac": avg["layer_bytes"] / HBM_PEAK / sec,
        "layer_mfma_frac": flops / MFMA_PEAK[mode] / sec,
        "layer_algorithmic_bytes": avg["layer_bytes"],
        "gpu_stage_ms": {n: round(v, 4) for n, v in stage_ms.items()},
        "gpu_stage_sum_ms": round(sum(stage_ms.values()), 4),
        "tt": aux["tt"], "ks": aux["ks"], "nbl": aux["nbl"], "work_items": aux["n_items"],
        **rotation,
    }, roof, roof_down


def measure_prenorm(mods, tokens, steps, warmup, seed, variants=64):
    """A decode step that starts from the block's pre-norm hidden states: RMSNorm, router
    projection (randn * 0.02 gate weight: near-uniform routing) and top-k inside the layer's
    first launch (`forward_prenorm`) against the same step as three pieces (norm kernel, router
    GEMM by torch, `forward` from logits).  The steps cycle through the weight copies and through
    `variants` different hidden states, so consecutive uses of a weight are a full cycle apart."""
    import torch
    from dartmoq_hip import ops
    mod = mods[0]
    hdim, e = mod.hidden_size, mod.num_experts
    g = torch.Generator().manual_seed(seed + 31)
    wn = (torch.randn(hdim, generator=g) * 0.1).half().cuda()
    wg = (torch.randn(e, hdim, generator=g) * 0.02).half().cuda()
    hs = [(torch.randn(tokens, hdim, generator=g) * 2.0).half().cuda() for _ in range(variants)]
    for m in mods:
        m.gate_weight = wg
    n, v = len(mods), len(hs)

    def fused(s):
        return mods[s % n].forward_prenorm(hs[s % v], wn, 1e-6, fused=True)

    def separate(s):
        x = ops.rms_norm(hs[s % v], wn, 1e-6)
        return mods[s % n].forward(x, router_logits=torch.matmul(x, wg.t()))

    res = {"tokens": tokens, "hidden_state_variants": variants, "weight_copies_rotated": n}
    same = all(torch.equal(fused(s), separate(s)) for s in range(3))
    for name, fn in (("fused", fused), ("separate", separate)):
        t0 = time.perf_counter()
        s = 0
        while time.perf_counter() - t0 < PRELUDE_S / 2:
            for _ in range(20):
                fn(s)
                s += 1
            torch.cuda.synchronize()
        for s in range(warmup):
            fn(s)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(steps):
            fn(s)
        torch.cuda.synchronize()
        res[f"{name}_ms_per_step"] = (time.perf_counter() - t0) / steps * 1e3
    res["launches_fused"] = "norm + router + top-k (+ routing up to 4 tokens) + rotation, [routing], gate_up, down, combine"
    res["launches_separate"] = "norm, router GEMM (torch), top-k + rotation, [routing], gate_up, down, combine"
    res["outputs_equal_on_first_3_steps"] = bool(same)
    return res


def measured_traffic(config, mode, tokens):
    """HBM bytes per launch of the dominant kernel from the committed counter runs
    (profiles/gate_up_hbm_traffic.json: FETCH_SIZE + WRITE_SIZE, calibrated on a copy of known
    size), or None when no run covers this workload."""
    path = os.path.join(ROOT, "profiles", "gate_up_hbm_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    for r in rec.get("runs", []):
        if r.get("config") == config and r.get("mode") == mode and r.get("tokens") == tokens:
            return r.get("hbm_bytes_per_launch")
    return None


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(pools_cpu, spec, expert_bit, tokens, seed, zipf, shared_cpu=None, warm=2, timed=5,
                 budget_s=30.0):
    """The CPU oracle (dequantize-then-matmul, fp32 matmuls, all host threads) on the same seeded
    inputs as the GPU run at `tokens` tokens, the two variants of the reference's benchmark script
    (test_triton_mp_moe_e2e_bench.py:135-164): weights dequantized once before the timed calls
    ("cached") and dequantized inside every call ("per_call").  Each: `warm` untimed calls, then
    `timed` calls, median.  `value` is the cached variant (the faster one).  The per-call variant
    stops early (at least 3 timed calls) when its calls would pass `budget_s` seconds."""
    import statistics
    import torch
    from oracle import moe as omoe, routing
    layer = omoe.MoELayer(spec["hidden"], spec["inter"], spec["experts"], spec["top_k"], 128,
                          expert_bit=expert_bit)
    for b, p in pools_cpu.items():
        layer.pools[b] = omoe.BitPool(int(b), p["gate_up"], p["down"], p["expert_offsets"])
    layer.shared = shared_cpu
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    x = torch.randn(tokens, spec["hidden"], generator=torch.Generator().manual_seed(seed)).half()
    w, idx = routing.route_topk(routing.zipf_logits(tokens, spec["experts"], seed, skew=zipf),
                                spec["top_k"])

    def run(cache, n_warm, n_timed, budget):
        times = []
        t_start = time.perf_counter()
        for i in range(n_warm + n_timed):
            t0 = time.perf_counter()
            omoe.reference_forward(layer, x, idx, w, weight_cache=cache)
            dt = time.perf_counter() - t0
            if i >= n_warm:
                times.append(dt)
            if budget and len(times) >= 3 and time.perf_counter() - t_start + dt > budget:
                break
        return statistics.median(times), len(times)

    t0 = time.perf_counter()
    cache = omoe.build_weight_cache(layer)
    build_s = time.perf_counter() - t0
    cached_s, cached_n = run(cache, warm, timed, 0.0)
    del cache
    per_call_s, per_call_n = run(None, warm, timed, budget_s)
    return {"value": tokens / cached_s, "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "cpu_model": cpu_model_name(), "tokens": tokens,
            "cached": {"tokens_per_s": tokens / cached_s, "median_s": cached_s, "timed_calls": cached_n,
                       "warmup_calls": warm, "dequantize_once_s": build_s},
            "per_call": {"tokens_per_s": tokens / per_call_s, "median_s": per_call_s,
                         "timed_calls": per_call_n, "warmup_calls": warm},
            "sample": f"forwards of {tokens} tokens of the same layer and the same seeded inputs as the "
                      f"GPU sweep entry, fp32 dequantize-then-matmul oracle (reference_forward), "
                      f"{torch.get_num_threads()} threads; value = weights dequantized once (cached), "
                      f"per_call = dequantized inside every call; median of the timed calls"}


def bench_linear(spec, steps, warmup, seed):
    """Side leg (--linear "bit,mode,rows[,out_features,in_features]"): one quantized Linear
    (synthetic packed indices, the Lloyd-Max codebook of the width or the uniform 8-bit grid)
    through dmq_linear_forward; wall time per call and, from events around the timed loop, GPU time."""
    import torch
    import dartmoq_hip
    from dartmoq_hip import hostprep
    f = spec.split(",")
    bit, mode, rows = int(f[0]), f[1], int(f[2])
    n, k = (int(f[3]), int(f[4])) if len(f) >= 5 else (4096, 4096)
    g = torch.Generator().manual_seed(seed)
    if bit == 8:
        cb = ((torch.arange(256, dtype=torch.float32) - 128) * (3.5 / 128)).half()
    else:
        cb = hostprep.get_codebook(bit)[0].half()
    groups = k // 128
    idx = torch.randint(0, 256, (n, groups * 128 * bit // 8), dtype=torch.uint8, generator=g)
    norms = (torch.rand(n, groups, generator=g) * 0.02 + 0.01).half()
    lin = dartmoq_hip.WxA16Linear(k, n, bit, 128, idx, cb, norms, seed=seed)
    cls = {"wxa16": None, "wxa8": dartmoq_hip.WxA8Linear, "wxfp8": dartmoq_hip.WxFP8Linear}[mode]
    if cls is not None:
        lin = cls.from_wxa16(lin)
    x = torch.randn(rows, k, generator=g).half().cuda()
    for _ in range(warmup):
        lin(x)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        lin(x)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    packed = n * k * bit // 8 + n * groups * 2
    print(json.dumps({"metric": "linear_forward_us", "value": wall * 1e6, "unit": "us",
                      "higher_is_better": False, "steps": steps, "warmup": warmup, "n_gpus": 1,
                      "gpu_us_between_events": e0.elapsed_time(e1) * 1e3 / steps, "dtype": "f16",
                      "data": "synthetic",
                      "config": {"workload": f"one {mode} Linear, {bit}-bit weights [{n}, {k}], {rows} rows",
                                 "packed_weight_bytes": packed}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--tokens", type=int, default=2048)
    ap.add_argument("--sweep", type=str, default="1,16,64,256,4096")
    ap.add_argument("--config", type=int, default=1)
    ap.add_argument("--mode", type=str, default="wxa16", choices=list(MFMA_PEAK))
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--cpu-tokens", type=int, default=64)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--modes", type=str, default="2:wxa8:2048/64,4:wxfp8:2048/64,4:wxfp4:2048/64,3:wxa8:64/8/1",
                    help='extra entries of the "modes" array, "config:mode:tokens[/tokens...]" comma '
                         'separated ("" for none)')
    ap.add_argument("--prenorm", type=str, default="1,8",
                    help='token counts of the "prenorm" entries (decode steps that start from pre-norm '
                         'hidden states; "" for none)')
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch dmq_finalize_kernel on 64 Mi fp32 elements (256 MiB read, "
                         "128 MiB written): the known-size kernel that calibrates FETCH_SIZE / "
                         "WRITE_SIZE counter runs")
    ap.add_argument("--linear", type=str, default="",
                    help='side leg: time one quantized Linear instead of the layer, '
                         '"bit,mode,rows[,out_features,in_features]" (mode wxa16 / wxa8 / wxfp8)')
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    import dartmoq_hip
    from dartmoq_hip import synthetic
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(3)
    if args.linear:
        bench_linear(args.linear, args.steps, args.warmup, args.seed)
        return
    spec = synthetic.CONFIGS[args.config]
    layers = {}

    def build(cfg):
        """Packed pools (and shared expert) of a config; configs with the same layer share them."""
        sp = synthetic.CONFIGS[cfg]
        key = json.dumps({k: v for k, v in sp.items() if k != "zipf"}, sort_keys=True)
        if key not in layers:
            eb = synthetic.assign_bits(sp["experts"], sp["fractions"], args.seed)
            pl = synthetic.build_pools(sp["hidden"], sp["inter"], sp["experts"], eb, seed=args.seed,
                                       device="cuda")
            sh = None
            if sp.get("shared_inter"):
                sh = synthetic.build_shared_expert(sp["hidden"], sp["shared_inter"], args.seed,
                                                   sp.get("shared_bit", 4), device="cuda")
            layers[key] = (eb, pl, sh)
        return layers[key]

    def modules(cfg, mode):
        sp = synthetic.CONFIGS[cfg]
        _eb, pl, sh = build(cfg)
        out = []
        for _ in range(N_COPIES):
            m = dartmoq_hip.WxA16BitPartitionedGroupMoE.from_packed(
                pl, sp["experts"], sp["hidden"], sp["inter"], sp["top_k"], device="cuda",
                shared_expert=sh)
            out.append(dartmoq_hip.convert_moe(m, mode))
        return out

    expert_bit, pools, shared = build(args.config)
    mods = modules(args.config, args.mode)

    if args.traffic_probe:
        from dartmoq_hip import ops
        probe = torch.ones(64 << 20, dtype=torch.float32, device="cuda")
        for _ in range(3):
            ops.finalize_f16(probe)
        torch.cuda.synchronize()
        del probe

    main_res, roof, roof_down = measure(mods, args.tokens, args.steps, args.warmup, args.seed,
                                        spec["zipf"], args.mode)
    roof["traffic"] = measured_traffic(args.config, args.mode, args.tokens)
    sweep = []
    for t in [int(v) for v in args.sweep.split(",") if v]:
        if t == args.tokens:
            continue
        res, r, rd = measure(mods, t, args.steps, args.warmup, args.seed, spec["zipf"], args.mode)
        r["traffic"] = measured_traffic(args.config, args.mode, t)
        res["roofline"] = r
        res["roofline_down"] = rd
        sweep.append(res)
    prenorm = []
    for t in [int(v) for v in args.prenorm.split(",") if v]:
        prenorm.append(measure_prenorm(mods, t, args.steps, args.warmup, args.seed))
    del mods

    # the activation-quantized modes on the configurations BASELINE names for them
    mode_results = []
    for entry in [v for v in args.modes.split(",") if v]:
        cfg_s, mode_s, tok_s = entry.split(":")
        cfg_m = int(cfg_s)
        sp = synthetic.CONFIGS[cfg_m]
        mm = modules(cfg_m, mode_s)
        for t in [int(v) for v in tok_s.split("/")]:
            res, r, rd = measure(mm, t, args.steps, args.warmup, args.seed, sp["zipf"], mode_s)
            r["traffic"] = measured_traffic(cfg_m, mode_s, t)
            mode_results.append({"config": cfg_m, "mode": mode_s, "dtype": DTYPE[mode_s], "tokens": t,
                                 "value": res["tokens_per_s"], "unit": "tokens/s",
                                 "ms_per_step": res["ms_per_step"], "eff_tflops": res["eff_tflops"],
                                 "layer_hbm_frac": res["layer_hbm_frac"],
                                 "layer_mfma_frac": res["layer_mfma_frac"],
                                 "gpu_stage_ms": res["gpu_stage_ms"],
                                 "weight_copies_rotated": res["weight_copies_rotated"],
                                 "logit_variants": res["logit_variants"],
                                 "cycle_steps": res["cycle_steps"],
                                 "cycle_weight_bytes": res["cycle_weight_bytes"],
                                 "exceeds_twice_infinity_cache": res["exceeds_twice_infinity_cache"],
                                 "roofline": r, "roofline_down": rd})
        del mm
        torch.cuda.empty_cache()

    cpu = None
    if not args.no_cpu:
        pools_cpu = {b: {"gate_up": {k: (v.cpu() if torch.is_tensor(v) else v)
                                     for k, v in p["gate_up"].items()},
                         "down": {k: (v.cpu() if torch.is_tensor(v) else v)
                                  for k, v in p["down"].items()},
                         "expert_offsets": p["expert_offsets"]} for b, p in pools.items()}
        shared_cpu = None if shared is None else {
            k: ({kk: (vv.cpu() if torch.is_tensor(vv) else vv) for kk, vv in v.items()}
                if isinstance(v, dict) else v.cpu()) for k, v in shared.items()}
        cpu = cpu_baseline(pools_cpu, spec, expert_bit, args.cpu_tokens, args.seed, spec["zipf"],
                           shared_cpu)

    bits = {b: sum(1 for e in expert_bit if e == int(b)) for b in pools}
    line = {
        "metric": "moe_layer_tokens_per_s", "value": main_res["tokens_per_s"], "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DTYPE[args.mode], "data": "synthetic",
        "config": {
            "workload": f"configs[{args.config}]: single MoE FFN layer, {args.mode}, H={spec['hidden']} "
                        f"E={spec['experts']} top-{spec['top_k']} I={spec['inter']} SwiGLU, "
                        f"experts per bit {bits}, "
                        + (f"shared expert I_s={spec['shared_inter']} bit{spec.get('shared_bit', 4)}, "
                           if shared is not None else "") +
                        f"group 128, T={args.tokens} tokens, "
                        f"{'Zipf(1.1)-skewed' if spec['zipf'] else 'uniform'} randn router logits",
            "tokens": args.tokens, "mode": args.mode,
            "weight_copies_rotated": main_res["weight_copies_rotated"],
            "logit_variants": main_res["logit_variants"],
        },
        "eff_tflops": main_res["eff_tflops"],
        "layer": main_res,
        "roofline": roof,
        "roofline_down": roof_down,
        "cpu_baseline": cpu,
        "sweep": sweep,
        "prenorm": prenorm,
        "modes": mode_results,
        "clock_prelude_s": PRELUDE_S,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
