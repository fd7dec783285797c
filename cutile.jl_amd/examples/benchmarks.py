"""Mirror of examples/benchmarks.jl: the generic benchmark runner of the examples.

It finds the example modules of this package, and for each calls ``prepare(benchmark=True)``, ``metric(data)``,
``run(data, nruns=NRUNS, warmup=WARMUP)`` and, where defined, ``run_others`` (benchmarks.jl:82-130), then
prints one table per example with the minimum and mean time of every implementation and the throughput
computed from the minimum (benchmarks.jl:26-62,136-183).

    python cutile.jl_amd/examples benchmarks               # every example
    python cutile.jl_amd/examples benchmarks matmul fmha
"""
from __future__ import annotations

import importlib
import pkgutil
import sys

NRUNS = 20      # benchmarks.jl:12
WARMUP = 5      # benchmarks.jl:13


def format_throughput(total, unit: str, time_ms: float) -> str:
    """benchmarks.jl:26-38."""
    if unit == "GB/s":
        return f"{round(total / (time_ms / 1000) / 1e9)} GB/s"
    if unit == "TFLOPS":
        return f"{total / (time_ms / 1000) / 1e12:.1f} TFLOPS"
    if unit in ("us", "\u03bcs"):
        return f"{round(time_ms * 1000)} \u03bcs"
    return ""


def print_table(title: str, results, file=sys.stdout) -> None:
    """benchmarks.jl:40-62; ``results``: list of (name, min_ms, mean_ms, throughput)."""
    print(file=file)
    print("=" * 72, file=file)
    print("  " + title, file=file)
    print("=" * 72, file=file)
    has_throughput = any(r[3] for r in results)
    head = "Implementation".ljust(28) + "Min (ms)".ljust(12) + "Mean (ms)".ljust(12)
    print(head + ("Throughput" if has_throughput else ""), file=file)
    print("-" * 72, file=file)
    for name, min_ms, mean_ms, tp in results:
        print(name.ljust(28) + f"{min_ms:.3f}".ljust(12) + f"{mean_ms:.3f}".ljust(12) + (tp if has_throughput else ""), file=file)
    print("-" * 72, file=file)


def discover_benchmarks(*names):
    """benchmarks.jl:68-80: every example module of the package (sorted), or the named ones."""
    import cutile_jl_amd.examples as pkg
    found = [m.name for m in pkgutil.iter_modules(pkg.__path__) if not m.name.startswith("_") and m.name != "benchmarks"]
    return sorted(n for n in found if not names or n in names)


def run_benchmark(name: str):
    """benchmarks.jl:82-130: returns ``(results, metric)`` or None when the module has no prepare / run;
    ``results`` maps an implementation name to its list of times in ms."""
    mod = importlib.import_module(f"cutile_jl_amd.examples.{name}")
    if not hasattr(mod, "prepare") or not hasattr(mod, "run"):
        return None
    data = mod.prepare(benchmark=True)
    metric_result = mod.metric(data) if hasattr(mod, "metric") else None
    result = mod.run(data, nruns=NRUNS, warmup=WARMUP)
    if hasattr(result, "times"):
        t = result.times
        results = dict(t) if isinstance(t, dict) else {"cuTile": list(t)}
    elif hasattr(result, "times_fwd"):
        results = {"cuTile Fwd": list(result.times_fwd), "cuTile Bwd": list(result.times_bwd)}
    else:
        return None
    if hasattr(mod, "run_others"):
        results.update(mod.run_others(data, nruns=NRUNS, warmup=WARMUP))
    return results, metric_result


def summarize(results, metric_result):
    """benchmarks.jl:158-177: rows (name, min, mean, throughput from the minimum), fastest first.  A metric that
    is one (total, unit) pair applies to every row, a dict only to the rows it names."""
    rows = []
    for impl, times in results.items():
        lo, mean = min(times), sum(times) / len(times)
        tp = ""
        if isinstance(metric_result, dict):
            if impl in metric_result:
                tp = format_throughput(*metric_result[impl], lo)
        elif isinstance(metric_result, tuple):
            tp = format_throughput(*metric_result, lo)
        rows.append((impl, lo, mean, tp))
    return sorted(rows, key=lambda r: r[1])


def main(*args, file=sys.stdout) -> None:
    """benchmarks.jl:136-183."""
    import torch
    print("=" * 72, file=file)
    print("  mi355tile benchmarks (the examples of cuTile.jl)", file=file)
    print("=" * 72, file=file)
    print(file=file)
    print("Configuration:", file=file)
    print(f"  Runs: {NRUNS} (+ {WARMUP} warmup)", file=file)
    print("  GPU: " + torch.cuda.get_device_name(0), file=file)
    for name in discover_benchmarks(*args):
        print(f"\nBenchmarking {name}...", file=file)
        ret = run_benchmark(name)
        if ret is None:
            print("  (skipped - no prepare/run functions)", file=file)
            continue
        print_table(name, summarize(*ret), file=file)
        torch.cuda.empty_cache()
    print(file=file)
    print("=" * 72, file=file)
    print("  Benchmark Complete", file=file)
    print("=" * 72, file=file)

