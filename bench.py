#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: the kernels of cuTile.jl's examples, through the
C ABI of libmi355tile.so.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--table]

Prints ONE JSON line on stdout.  A "step" is one pass of the headline workload over one
batch of synthetic, seeded input already resident in HBM:

    headline workload (default) = "layernorm_softmax": LayerNorm fwd + bwd and the column
    softmax on 4096x4096 fp32 (the second entry of BASELINE.json's configs);
    ``value`` = algorithmic bytes of the step / time per step, in GB/s.

Every other configuration of BASELINE.json (vadd, transpose, GEMM, batched GEMM, FMHA, MoE)
is measured in the same run with the reference's protocol (examples/benchmarks.jl:12-13:
5 warm-up launches, 20 timed launches, min and mean) and reported under ``"kernels"``, each
with absolute GB/s or TFLOP/s and its fraction of the MI355X roofline (HBM 8 TB/s; dense
MFMA f16 2.5 PFLOP/s, fp8 5.0 PFLOP/s, fp32 157.3 TFLOP/s).  ``roofline`` on the top level
is the dominant kernel of the headline workload.  ``cpu_baseline`` times the numpy/OpenBLAS
restatement of the reference's CPU path for the headline workload on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "fp8": 5000.0, "f32": 157.3}
NRUNS, WARMUP = 20, 5  # examples/benchmarks.jl:12-13


def _event_times(fn, nruns, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(nruns):
        e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
        e0.record(); fn(); e1.record(); e1.synchronize()
        out.append(e0.elapsed_time(e1))
    return out


def _entry(name, times_ms, work, unit, bound, peak, dtype, extra=None):
    tmin = min(times_ms); tmean = sum(times_ms) / len(times_ms)
    scale = 1e9 if unit == "GB/s" else 1e12
    ach_min = work / (tmin * 1e-3) / scale
    ach_mean = work / (tmean * 1e-3) / scale
    e = {"name": name, "min_ms": round(tmin, 5), "mean_ms": round(tmean, 5), "work": work,
         "achieved": round(ach_mean, 2), "achieved_at_min": round(ach_min, 2), "unit": unit if unit == "GB/s" else "TFLOP/s",
         "bound": bound, "peak": peak, "frac": round(ach_mean / peak, 4), "frac_at_min": round(ach_min / peak, 4),
         "dtype": dtype}
    if extra:
        e.update(extra)
    return e


def bench_kernels(ct, which, nruns=NRUNS, warmup=WARMUP):
    """Measure each configuration; returns {name: entry}."""
    import torch
    from cutile_jl_amd import examples  # noqa: F401
    import importlib
    res = {}

    def want(n):
        return which is None or n in which

    if want("vadd"):
        m = importlib.import_module("cutile_jl_amd.examples.vadd")
        d = m.prepare(benchmark=True)
        t = _event_times(lambda: ct.vec_add_kernel_1d(d.a, d.b, d.c, 1024), nruns, warmup)
        res["vadd"] = _entry("vadd 2^27 f32", t, m.metric(d)[0], "GB/s", "hbm", HBM_PEAK_GBS, "f32",
                             {"variant": ct.last_variant()})
        del d
    if want("transpose"):
        m = importlib.import_module("cutile_jl_amd.examples.transpose")
        d = m.prepare(benchmark=True)
        t = _event_times(lambda: ct.transpose_kernel(d.x, d.y, 64, 64), nruns, warmup)
        res["transpose"] = _entry("transpose 8192^2 f32", t, m.metric(d)[0], "GB/s", "hbm", HBM_PEAK_GBS, "f32",
                                  {"variant": ct.last_variant()})
        del d
    if want("layernorm"):
        m = importlib.import_module("cutile_jl_amd.examples.layernorm")
        d = m.prepare(benchmark=True)
        r = m.run(d, nruns=nruns, warmup=warmup)
        MN4 = d.M * d.N * 4
        fwd_bytes = 2 * MN4 + (2 * d.N + 2 * d.M) * 4
        bwd_bytes = 3 * MN4 + (d.N + 2 * d.M) * 4 + 4 * d.N * d.GROUP_SIZE_M * 4 + 2 * d.N * 4
        res["layernorm_fwd"] = _entry("LayerNorm fwd 4096^2 f32", r.times_fwd, fwd_bytes, "GB/s", "hbm", HBM_PEAK_GBS,
                                      "f32", {"reference_formula_bytes": 4 * MN4})
        res["layernorm_bwd"] = _entry("LayerNorm bwd 4096^2 f32 (3 fills + 2 kernels)", r.times_bwd, bwd_bytes, "GB/s",
                                      "hbm", HBM_PEAK_GBS, "f32", {"reference_formula_bytes": 5 * MN4})
        del d, r
    if want("softmax"):
        m = importlib.import_module("cutile_jl_amd.examples.softmax")
        d = m.prepare(benchmark=True)
        r = m.run(d, nruns=nruns, warmup=warmup)
        MN4 = d.M * d.N * 4
        res["softmax_tma"] = _entry("softmax (single tile) 4096^2 f32", r.times["cuTile TMA"], 2 * MN4, "GB/s", "hbm",
                                    HBM_PEAK_GBS, "f32")
        res["softmax_chunked"] = _entry("softmax (chunked) 4096^2 f32", r.times["cuTile Chunked"], 2 * MN4, "GB/s",
                                        "hbm", HBM_PEAK_GBS, "f32", {"reference_formula_bytes": 4 * MN4})
        del d, r
    for name in ("matmul", "batchmatmul", "fmha", "moe"):
        if not want(name):
            continue
        try:
            m = importlib.import_module(f"cutile_jl_amd.examples.{name}")
        except ModuleNotFoundError:
            continue
        res.update(m.bench(ct, _entry, _event_times, nruns, warmup))
    torch.cuda.synchronize()
    return res


def headline(ct, steps, warmup):
    """configs[1]: LayerNorm fwd+bwd and softmax on 4096x4096 fp32; returns timing + per-kernel
    durations measured with events on the launch stream inside the timed region."""
    import torch
    from cutile_jl_amd.examples import layernorm, softmax
    dl = layernorm.prepare(benchmark=True)
    ds = softmax.prepare(benchmark=True)

    def ln_fwd():
        ct.layer_norm_fwd(dl.X, dl.W, dl.B, dl.Y, dl.Mean, dl.Rstd, dl.eps, 1024)

    def ln_bwd_fill():
        dl.DW_partial.zero_(); dl.DB_partial.zero_(); dl.Locks.zero_()

    def ln_bwd_main():
        ct.layer_norm_bwd_dx_partial_dwdb(dl.DX, dl.DY, dl.DW_partial, dl.DB_partial, dl.X, dl.W, dl.Mean, dl.Rstd,
                                          dl.Locks, dl.GROUP_SIZE_M, 1024)

    def ln_bwd_final():
        ct.layer_norm_bwd_dwdb(dl.DW_partial, dl.DB_partial, dl.FINAL_DW, dl.FINAL_DB, 32, 1024)

    def sm():
        ct.softmax_tma_kernel(ds.output_tma, ds.input, 4096, num_programs=ds.M)

    stages = [("layer_norm_fwd", ln_fwd), ("fills", ln_bwd_fill), ("layer_norm_bwd_dx_partial_dwdb", ln_bwd_main),
              ("layer_norm_bwd_dwdb", ln_bwd_final), ("softmax_tma_kernel", sm)]
    for _ in range(warmup):
        for _, f in stages:
            f()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(stages) + 1)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        ev[s][0].record()
        for i, (_, f) in enumerate(stages):
            f()
            ev[s][i + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per_stage = {name: sum(ev[s][i].elapsed_time(ev[s][i + 1]) for s in range(steps)) / steps
                 for i, (name, _) in enumerate(stages)}
    MN4 = dl.M * dl.N * 4
    work = {
        "layer_norm_fwd": 2 * MN4 + (2 * dl.N + 2 * dl.M) * 4,
        "layer_norm_bwd_dx_partial_dwdb": 3 * MN4 + (dl.N + 2 * dl.M) * 4 + 2 * dl.N * dl.GROUP_SIZE_M * 4,
        "layer_norm_bwd_dwdb": 2 * dl.N * dl.GROUP_SIZE_M * 4 + 2 * dl.N * 4,
        "softmax_tma_kernel": 2 * MN4,
        "fills": 0,
    }
    return (t1 - t0) / steps, per_stage, work


def cpu_baseline_headline(sample_rows=512):
    """numpy restatement of the reference's CPU path (Julia Base broadcast + reductions,
    examples/layernorm.jl:284-313 and softmax.jl:175-188) on `sample_rows` of the 4096 rows,
    single-threaded as Julia's broadcasting is.  Returns GB/s on the same byte count."""
    import numpy as np
    from oracle import cutile_oracle as orc
    rng = np.random.default_rng(1)
    N, M = 4096, sample_rows
    X = np.asfortranarray(rng.standard_normal((N, M), dtype=np.float32))
    W = rng.standard_normal(N, dtype=np.float32); B = rng.standard_normal(N, dtype=np.float32)
    DY = np.asfortranarray(rng.standard_normal((N, M), dtype=np.float32))
    S = np.asfortranarray(rng.standard_normal((N, M), dtype=np.float32) * 2)
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        orc.layer_norm_fwd(X, W, B, 1e-5, dtype=np.float32)
        orc.layer_norm_bwd(X, W, DY, 1e-5, dtype=np.float32)
        orc.softmax(S, dtype=np.float32)
        best = min(best, time.perf_counter() - t0)
    MN4 = M * N * 4
    work = (2 * MN4) + (3 * MN4) + (2 * MN4)
    return {"value": round(work / best / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{sample_rows} of 4096 rows (N=4096 f32) of LayerNorm fwd+bwd and softmax, numpy single-threaded, min of 3"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--kernels", type=str, default="all", help="comma list for the per-kernel table, 'all' or 'none'")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--table", action="store_true", help="also print a human-readable table on stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X; multi-GPU runs are not part of this build (use --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import __graft_entry__ as entry
    ct = entry.load_package()
    ct.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    sec_per_step, per_stage, work = headline(ct, args.steps, args.warmup)
    total_work = sum(work.values())
    dom = max((k for k in work if work[k] > 0), key=lambda k: per_stage[k])
    ach = work[dom] / (per_stage[dom] * 1e-3) / 1e9
    out = {
        "metric": "LayerNorm fwd+bwd + softmax 4096x4096 f32, algorithmic GB/s (norm/softmax leg of: FMHA/MoE/GEMM TFLOPS + norm/softmax GB/s, % of MI355X roofline)",
        "value": round(total_work / sec_per_step / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: row LayerNorm fwd+bwd (y, dx, dgamma, dbeta) + row softmax on 4096x4096 Float32",
                   "M": 4096, "N": 4096, "eps": 1e-5, "GROUP_SIZE_M": 64, "bytes_per_step": total_work},
        "roofline": {"bound": "hbm", "achieved": round(ach, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "kernel": dom,
                     "avg_launch_ms": round(per_stage[dom], 5), "algorithmic_bytes": work[dom]},
        "stages_ms": {k: round(v, 5) for k, v in per_stage.items()},
    }
    if args.kernels != "none":
        which = None if args.kernels == "all" else set(args.kernels.split(","))
        out["kernels"] = bench_kernels(ct, which)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_headline()
    if args.table and "kernels" in out:
        for k, e in out["kernels"].items():
            print(f"{e['name']:<50} min {e['min_ms']:9.4f} ms  mean {e['mean_ms']:9.4f} ms  "
                  f"{e['achieved']:10.1f} {e['unit']:<8} {100 * e['frac']:6.2f}% of {e['bound']} peak", file=sys.stderr)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
