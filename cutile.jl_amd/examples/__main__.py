"""``python cutile.jl_amd/examples <name> [...]`` runs ``main()`` of the named examples (all of them without a
name), the way ``julia examples/<name>.jl`` does; ``python cutile.jl_amd/examples benchmarks [names]`` is the
benchmark runner (examples/benchmarks.jl)."""
import importlib
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import __graft_entry__ as _g   # noqa: E402

_g.load_package()              # raises if libmi355tile.so has not been built
from cutile_jl_amd.examples import benchmarks   # noqa: E402

args = sys.argv[1:]
if args and args[0] == "benchmarks":
    benchmarks.main(*args[1:])
else:
    for name in benchmarks.discover_benchmarks(*args):
        importlib.import_module(f"cutile_jl_amd.examples.{name}").main()
        print()
