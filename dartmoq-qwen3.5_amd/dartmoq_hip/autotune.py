"""Offline search over the launch shapes of the layer forward.

The counterpart of the reference's tile tuner for its Triton kernels
(turboquant_utils/kernel_autotune.py: ``SEARCH_SPACE`` :56-62, ``search_best_config`` :252,
``run_full_autotune`` :405, ``generate_config_table`` :501), for the knobs the HIP kernels have:

* ``tt``   16-row tiles per wave of a work item (1, 2, 4: 16, 32 or 64 rows per item),
* ``ks``   how K of a gate_up block is shared: 1 = not, 4 = over the four waves of the workgroup,
           -2 / -4 = between that many workgroups,
* ``nbl``  feature blocks per workgroup of the GEMM launches,

each with 0 = the library's own choice (``csrc/api.hip``: ``pick_tt``, ``pick_ks``, ``pick_nbl`` and the
dot-product launches of one- and two-token steps).  Same principles as the reference's module: the
search runs offline, it times the whole layer forward (routing, rotation, both GEMMs, combine) on
weights that cannot stay in the Infinity Cache, medians of event-timed repeats, results as JSON
with the same keys (``params``, ``baseline``, ``best``, ``results``), and a table per token-count
bucket that a module applies with ``apply_config_table``.

    python -m dartmoq_hip.autotune --config 1 --mode wxa16 --tokens 1,8,64,2048 --output-dir results/autotune
"""

from __future__ import annotations

import itertools
import json
import math
import os
import statistics
import time

import torch

SEARCH_SPACE = {
    "tt": [1, 2, 4],
    "ks": [0, 1, 4, -2, -4],
    "nbl": [0, 1, 2, 4],
}
AUTO = {"tt": 0, "ks": 0, "nbl": 0}
SPLIT_MAX_ROWS = 1024            # routed rows up to which K may be shared between workgroups


def generate_configs() -> list[dict]:
    keys = list(SEARCH_SPACE)
    return [dict(zip(keys, combo)) for combo in itertools.product(*(SEARCH_SPACE[k] for k in keys))]


def is_config_valid(cfg: dict, tokens: int, top_k: int, hidden: int) -> bool:
    """What the library accepts (csrc/gemm_dispatch.h ``dmq_gemm_config_ok`` and the checks of the
    layer forward): K is split over waves or shared between workgroups with 16-row tiles only, the
    group count must divide, and the shared form is bounded by its scratch."""
    tt, ks = cfg["tt"], cfg["ks"]
    if tt not in (0, 1, 2, 4):
        return False
    if ks not in (0, 1, 4, -2, -4):
        return False
    if ks == 4 and tt != 1:
        return False
    if ks < 0:
        if tt != 1 or (hidden // 128) % -ks or tokens * top_k > SPLIT_MAX_ROWS:
            return False
    if cfg["nbl"] not in (0, 1, 2, 4):
        return False
    return True


def _rolled_logits(tokens: int, experts: int, seed: int, skew, variants: int, device):
    from . import synthetic
    base = synthetic.zipf_logits(tokens, experts, seed, skew=skew).to(device)
    return [torch.roll(base, shifts=v * (experts // variants), dims=1).contiguous() for v in range(variants)]


def benchmark_config(mods, x, logits, cfg: dict, n_warmup: int = 3, n_repeat: int = 10, inner: int = 12):
    """Median milliseconds per forward under ``cfg`` (None when the library refuses the shape).
    Step s runs module copy s mod len(mods) on logits variant s mod len(logits), so that a weight
    is not reused while it may still sit in a cache."""
    before = [(m.tt_override, m.ks_override, m.nbl_override, m.tile_table) for m in mods]
    for m in mods:
        m.tt_override, m.ks_override, m.nbl_override, m.tile_table = cfg["tt"], cfg["ks"], cfg["nbl"], None
    try:
        step = 0
        times = []
        for rep in range(n_warmup + n_repeat):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(inner):
                mods[step % len(mods)].forward(x, router_logits=logits[step % len(logits)])
                step += 1
            end.record()
            end.synchronize()
            if rep >= n_warmup:
                times.append(start.elapsed_time(end) / inner)
        return statistics.median(times), times
    except (ValueError, RuntimeError):
        torch.cuda.synchronize()
        return None
    finally:
        for m, b in zip(mods, before):
            m.tt_override, m.ks_override, m.nbl_override, m.tile_table = b


def search_best_config(mods, tokens: int, skew=True, seed: int = 42, n_warmup: int = 3, n_repeat: int = 10,
                       variants: int = 8, configs: list[dict] | None = None, prelude_s: float = 0.3) -> dict:
    """Grid search at one token count.  ``mods``: independent copies of the layer (three or more keep
    a 200 MB layer out of the Infinity Cache).  The baseline is the library's own choice."""
    mod = mods[0]
    dev = "cuda"
    x = torch.randn(tokens, mod.hidden_size, generator=torch.Generator().manual_seed(seed)).half().to(dev)
    logits = _rolled_logits(tokens, mod.num_experts, seed, skew, variants, dev)
    space = configs if configs is not None else generate_configs()
    valid = [c for c in space if is_config_valid(c, tokens, mod.top_k + mod.n_shared, mod.hidden_size)]
    flops = tokens * mod.flops_per_token()
    # the GPU reaches its working clocks after tens of milliseconds of load: an untimed prelude
    # first, and the baseline is timed before and after the candidates
    t_end = time.perf_counter() + prelude_s
    while time.perf_counter() < t_end:
        for i in range(32):
            mods[i % len(mods)].forward(x, router_logits=logits[i % len(logits)])
        torch.cuda.synchronize()
    base = benchmark_config(mods, x, logits, AUTO, n_warmup, n_repeat)
    if base is None:
        raise RuntimeError("the library refused its own launch shape")
    failed = 0
    timed = []
    for cfg in valid:
        r = benchmark_config(mods, x, logits, cfg, n_warmup, n_repeat)
        if r is None:
            failed += 1
            continue
        timed.append((cfg, r[0]))
    again = benchmark_config(mods, x, logits, AUTO, n_warmup, n_repeat)
    base_ms = statistics.median(base[1] + again[1])
    results = [{"config": dict(AUTO), "median_ms": base_ms, "tflops": flops / base_ms / 1e9, "speedup": 1.0,
                "is_baseline": True}]
    for cfg, ms in timed:
        results.append({"config": cfg, "median_ms": ms, "tflops": flops / ms / 1e9,
                        "speedup": base_ms / ms, "is_baseline": False})
    results.sort(key=lambda r: r["median_ms"])
    best = results[0]
    return {
        "params": {"tokens": tokens, "hidden": mod.hidden_size, "inter": mod.intermediate_size,
                   "experts": mod.num_experts, "top_k": mod.top_k, "n_shared": mod.n_shared,
                   "mode": type(mod).__name__, "copies": len(mods), "logit_variants": variants,
                   "n_warmup": n_warmup, "n_repeat": n_repeat, "seed": seed,
                   "total_configs": len(valid), "failed_count": failed},
        "baseline": {"config": dict(AUTO), "median_ms": base_ms, "tflops": flops / base_ms / 1e9},
        "best": {k: best[k] for k in ("config", "median_ms", "tflops", "speedup")},
        "results": results,
    }


def save_result(result: dict, path: str) -> None:
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        json.dump(result, f, indent=2)


def run_full_autotune(mods, token_counts, output_dir: str = "results/kernel_autotune", **kw) -> list[dict]:
    """One search per token count, one JSON file each (``tokens_<T>.json``)."""
    out = []
    for t in token_counts:
        res = search_best_config(mods, t, **kw)
        save_result(res, os.path.join(output_dir, f"tokens_{t}.json"))
        out.append(res)
    return out


def print_topk(result: dict, k: int = 10) -> None:
    p = result["params"]
    print(f"tokens={p['tokens']} H={p['hidden']} I={p['inter']} E={p['experts']} top-{p['top_k']}: "
          f"library's choice {result['baseline']['median_ms'] * 1e3:.1f} us")
    for r in result["results"][:k]:
        c = r["config"]
        print(f"  tt={c['tt']} ks={c['ks']:>2} nbl={c['nbl']}  {r['median_ms'] * 1e3:8.1f} us  x{r['speedup']:.3f}"
              f"{'  (baseline)' if r['is_baseline'] else ''}")


def generate_config_table(result_dir: str, min_gain: float = 0.03) -> dict:
    """Table of launch shapes by token count from the JSON files of ``run_full_autotune``.  A
    measured size keeps the library's own choice unless the best shape beat it by ``min_gain``
    (run-to-run noise of a timed forward is a few per cent).  A forward of T tokens uses the entry of
    the measured size nearest to T on a logarithmic scale (``lookup_config``)."""
    entries = []
    for name in sorted(os.listdir(result_dir)):
        if not (name.startswith("tokens_") and name.endswith(".json")):
            continue
        with open(os.path.join(result_dir, name)) as f:
            res = json.load(f)
        best, cfg = res["best"], dict(AUTO)
        if best["speedup"] >= 1.0 + min_gain:
            cfg = dict(best["config"])
        entries.append({"tokens": res["params"]["tokens"], **cfg, "speedup": best["speedup"] if cfg != AUTO else 1.0})
    entries.sort(key=lambda e: e["tokens"])
    return {"entries": entries}


def lookup_config(table: dict | None, tokens: int) -> dict:
    if not table or not table.get("entries"):
        return dict(AUTO)
    e = min(table["entries"], key=lambda e: abs(math.log(max(tokens, 1)) - math.log(max(e["tokens"], 1))))
    return {"tt": e["tt"], "ks": e["ks"], "nbl": e["nbl"]}


def apply_config_table(mod, table: dict | None) -> None:
    """Make ``mod.forward`` use the table (explicit ``tt_override`` etc. still win).  Shapes the
    library refuses for a given batch (K shared between workgroups beyond its row bound) fall back
    to the library's choice."""
    mod.tile_table = table


def main(argv=None) -> None:
    import argparse
    import dartmoq_hip
    from . import synthetic
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--config", type=int, default=1, help="index into dartmoq_hip.synthetic.CONFIGS")
    ap.add_argument("--mode", default="wxa16", choices=["wxa16", "wxa8", "wxfp8", "wxfp4"])
    ap.add_argument("--tokens", default="1,8,64,256,2048")
    ap.add_argument("--copies", type=int, default=3)
    ap.add_argument("--repeat", type=int, default=10)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--routing", default="config", choices=["config", "zipf", "uniform"],
                    help="router logits: the configuration's own, Zipf(1.1)-biased, or unbiased")
    ap.add_argument("--output-dir", default="results/kernel_autotune")
    args = ap.parse_args(argv)
    sp = synthetic.CONFIGS[args.config]
    eb = synthetic.assign_bits(sp["experts"], sp["fractions"], args.seed)
    pools = synthetic.build_pools(sp["hidden"], sp["inter"], sp["experts"], eb, seed=args.seed, device="cuda")
    shared = None
    if sp.get("shared_inter"):
        shared = synthetic.build_shared_expert(sp["hidden"], sp["shared_inter"], args.seed,
                                               sp.get("shared_bit", 4), device="cuda")
    mods = []
    for _ in range(args.copies):
        m = dartmoq_hip.WxA16BitPartitionedGroupMoE.from_packed(
            pools, sp["experts"], sp["hidden"], sp["inter"], sp["top_k"], device="cuda", shared_expert=shared)
        mods.append(dartmoq_hip.convert_moe(m, args.mode))
    results = run_full_autotune(mods, [int(t) for t in args.tokens.split(",") if t], args.output_dir,
                                skew=sp["zipf"] if args.routing == "config" else args.routing == "zipf",
                                seed=args.seed, n_repeat=args.repeat)
    for r in results:
        print_topk(r)
    table = generate_config_table(args.output_dir)
    with open(os.path.join(args.output_dir, "config_table.json"), "w") as f:
        json.dump(table, f, indent=2)
    print(json.dumps(table))


if __name__ == "__main__":
    main()
