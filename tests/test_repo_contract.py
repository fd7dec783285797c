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
