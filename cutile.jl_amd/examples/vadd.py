"""Mirror of examples/vadd.jl:52-136 (prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_uniform, time_launches


def prepare(*, benchmark: bool = False, shape=None, use_gather: bool = False,
            T: torch.dtype = torch.float32, seed: int = 0):
    """vadd.jl:52-63; a, b ~ U[0,1) from ``seed`` (the reference draws them with cuRAND)."""
    if shape is None:
        shape = (2 ** 27,) if benchmark else (1_024_000,)
    rng = np.random.default_rng(seed)
    a = rand_uniform(rng, shape, T)
    b = rand_uniform(rng, shape, T)
    return namespace(a=a, b=b, c=torch.empty_like(a), shape=tuple(shape), use_gather=use_gather)


def run(data, *, tile=1024, nruns: int = 1, warmup: int = 0):
    """vadd.jl:65-125."""
    a, b, c = data.a, data.b, data.c
    if len(data.shape) == 2:
        tile_x, tile_y = tile if isinstance(tile, tuple) else (tile, tile)
        launch = lambda: ct.vec_add_kernel_2d(a, b, c, tile_x, tile_y)
    else:
        tile_val = tile[0] if isinstance(tile, tuple) else tile
        if data.use_gather:
            launch = lambda: ct.vec_add_kernel_1d_gather(a, b, c, tile_val)
        else:
            launch = lambda: ct.vec_add_kernel_1d(a, b, c, tile_val)
    times = time_launches(launch, nruns, warmup)
    return namespace(c=c, times=times)



def run_others(data, *, nruns: int = 1, warmup: int = 0):
    """vadd.jl:141-195 compares with GPUArrays' broadcast (and a SIMT kernel); here the library behind
    ``torch`` plays that part: ``torch.add`` into a preallocated result."""
    c = torch.empty_like(data.a)
    return {"torch.add": time_launches(lambda: torch.add(data.a, data.b, out=c), nruns, warmup)}



def verify(data, result) -> None:
    """vadd.jl:127-129: ``Array(c) ~ Array(a) + Array(b)`` on the host."""
    assert isapprox(result.c.cpu(), data.a.cpu() + data.b.cpu())


def metric(data):
    """vadd.jl:131-136: 2 reads + 1 write."""
    n = int(np.prod(data.shape))
    return 3 * n * data.a.element_size(), "GB/s"


def test_vadd(shape, tile, *, use_gather: bool = False, T: torch.dtype = torch.float32, name: str | None = None) -> None:
    """vadd.jl:202-217."""
    tname = str(T).replace("torch.", "")
    if name is None:
        if len(shape) == 2:
            name = f"2D vec_add ({shape[0]} x {shape[1]}, {tname}, tile={tile})"
        elif use_gather:
            name = f"1D vec_add gather ({shape[0]} elements, {tname}, tile={tile})"
        else:
            name = f"1D vec_add ({shape[0]} elements, {tname}, tile={tile})"
    print(f"--- {name} ---")
    data = prepare(shape=shape, use_gather=use_gather, T=T)
    result = run(data, tile=tile)
    verify(data, result)
    print("  passed")


def main() -> None:
    """vadd.jl:219-248: the example's own list of shapes."""
    print("--- Vector/Matrix Addition Examples ---\n")
    test_vadd((1_024_000,), 1024)
    test_vadd((2 ** 20,), 512)
    test_vadd((2 ** 18,), 512, T=torch.float64)
    test_vadd((1_024_000,), 1024, T=torch.float16)
    test_vadd((2048, 1024), (32, 32))
    test_vadd((1024, 2048), (64, 64))
    test_vadd((1024, 512), (32, 32), T=torch.float64)
    test_vadd((1024, 1024), (64, 64), T=torch.float16)
    test_vadd((1_024_000,), 1024, use_gather=True)
    test_vadd((2 ** 20,), 512, use_gather=True)
    print("\n--- All addition examples completed ---")
