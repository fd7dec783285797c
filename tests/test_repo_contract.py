"""Checks on the repository itself that need no GPU: the command line of bench.py, and the separation between the
product (the package and what it loads) and the test infrastructure (the oracle, working files)."""
import ast
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cutile.jl_amd")


def _python_files(top):
    for base, dirs, files in os.walk(top):
        dirs[:] = [d for d in dirs if d not in ("__pycache__", "build")]
        for f in files:
            if f.endswith(".py"):
                yield os.path.join(base, f)


def _names_working_files(text):
    return any(t in text for t in ("_work/", "'_work'", '"_work"'))


def _imported_modules(path):
    tree = ast.parse(open(path).read(), filename=path)
    for node in ast.walk(tree):
        if isinstance(node, ast.Import):
            for a in node.names:
                yield a.name
        elif isinstance(node, ast.ImportFrom) and node.module:
            yield node.module


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one MI355X" in (r.stdout + r.stderr)


def test_bench_command_line_has_the_contract_flags():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in r.stdout


def test_the_package_never_imports_the_oracle_or_working_files():
    """The oracle is the checker: only the tests, the smoke check and bench.py's CPU baseline may load it."""
    for path in _python_files(PKG):
        text = open(path).read()
        mods = list(_imported_modules(path))
        assert not any(m == "oracle" or m.startswith("oracle.") or "cutile_oracle" in m for m in mods), path
        assert not _names_working_files(text), path
    for path in (os.path.join(ROOT, "bench.py"), os.path.join(ROOT, "__graft_entry__.py")):
        assert not _names_working_files(open(path).read()), path


def test_native_sources_do_not_reach_into_the_oracle_or_working_files():
    csrc = os.path.join(PKG, "csrc")
    for f in os.listdir(csrc):
        if f.endswith((".hip", ".h", ".cpp")) or f == "Makefile":
            text = open(os.path.join(csrc, f)).read()
            assert "oracle" not in text and not _names_working_files(text), f


def _canned_full_record():
    """A full bench record with every key the real run produces and figures of realistic width."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    kernels = {}
    for key, fig, _ in bench.TARGETS + [(k, f, None) for k, f in bench.REPORTED]:
        e = kernels.setdefault(key, {"name": key + " " + "x" * 150, "min_ms": 0.123456, "mean_ms": 0.134567, "avg_ms": 0.120123,
                                     "avg_ms_is": "y" * 200, "work": 137438953472.0, "achieved": 1144.17, "unit": "TFLOP/s",
                                     "bound": "mfma", "peak": 2500.0, "frac": 0.4577, "dtype": "f16", "flop": 6442450944.0,
                                     "variant": "v" * 60, "cpu_ms": 12345.6, "cpu_note": "z" * 120})
        e[fig] = 0.123456
    full = {
        "metric": "norm/softmax GB/s (LayerNorm fwd+bwd + softmax, 4096x4096 f32); FMHA/MoE/GEMM legs in summary",
        "value": 5312.77, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 0.08951, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: row LayerNorm fwd+bwd (y, dx, dgamma, dbeta) + row softmax on 4096x4096 Float32",
                   "M": 4096, "N": 4096, "eps": 1e-5, "GROUP_SIZE_M": 64, "bytes_per_step": 474546176},
        "roofline": {"bound": "hbm", "achieved": 5512.12, "peak": 8000.0, "unit": "GB/s", "frac": 0.689, "traffic": 210388516,
                     "kernel": "layer_norm_bwd_dx_partial_dwdb", "avg_launch_ms": 0.03691, "algorithmic_bytes": 203472896},
        "cpu_baseline": {"value": 1.234, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "s" * 200},
        "errors": {f"config {i} " + "e" * 50: {"max_abs": 1e-6, "max_rel_scale": 1e-7, "max_rel_elem": 1e-6, "tol": 1e-5, "pass": True,
                                               "sample": "all"} for i in range(11)},
        "stages_ms": {f"stage{i}": 0.02 for i in range(6)}, "kernels": kernels, "detail_file": "gpurun_out/bench_full.json",
    }
    full["summary"] = bench._summary(kernels)
    return bench, full


def test_bench_last_line_is_a_small_parseable_record():
    """The record a driver keeps is the last stdout line: it must hold the contract keys, the roofline and the CPU
    baseline, parse as strict JSON (no NaN / Infinity) and stay far below the size at which the end of stdout that a
    consumer keeps no longer contains the whole line."""
    import json
    bench, full = _canned_full_record()
    line = bench.headline_record(full)
    assert "\n" not in line and len(line) < 4096, len(line)
    rec = json.loads(line, parse_constant=lambda c: (_ for _ in ()).throw(ValueError(c)))
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "dtype", "config", "roofline", "cpu_baseline", "summary"):
        assert k in rec, k
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "avg_launch_ms", "algorithmic_bytes"):
        assert k in rec["roofline"], k
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in rec["cpu_baseline"], k
    assert "kernels" not in rec and "errors" not in rec and "stages_ms" not in rec
    for key, fig, target in bench.TARGETS:
        assert rec["summary"][f"{key}.{fig}"]["t"] == target
    assert rec["parity"] == {"configs": 11, "all_within_tolerance": True}


def test_bench_last_line_sheds_optional_parts_rather_than_outgrow_the_limit():
    import json
    bench, full = _canned_full_record()
    full["summary"] = {f"k{i}": {"frac": 0.5, "note": "n" * 100} for i in range(60)}
    line = bench.headline_record(full)
    assert len(line) < 4096
    rec = json.loads(line)
    assert "summary" not in rec and "roofline" in rec and "cpu_baseline" in rec


def test_bench_record_refuses_nan():
    import pytest
    bench, full = _canned_full_record()
    full["value"] = float("nan")
    with pytest.raises(ValueError):
        bench.headline_record(full)
