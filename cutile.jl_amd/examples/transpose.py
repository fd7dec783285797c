"""Mirror of examples/transpose.jl:25-66 (prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_uniform, time_launches


def prepare(*, benchmark: bool = False, m: int | None = None, n: int | None = None,
            T: torch.dtype = torch.float32, seed: int = 0):
    """transpose.jl:25-36: x (m, n) ~ U[0,1), y (n, m)."""
    m = (8192 if benchmark else 1024) if m is None else m
    n = (8192 if benchmark else 512) if n is None else n
    rng = np.random.default_rng(seed)
    x = rand_uniform(rng, (m, n), T)
    y = torch.empty((m, n), dtype=T, device=x.device)  # Julia (n, m)
    return namespace(x=x, y=y, m=m, n=n)


def run(data, *, tm: int = 64, tn: int = 64, nruns: int = 1, warmup: int = 0):
    """transpose.jl:38-56."""
    times = time_launches(lambda: ct.transpose_kernel(data.x, data.y, tm, tn), nruns, warmup)
    return namespace(y=data.y, times=times)



def run_others(data, *, nruns: int = 1, warmup: int = 0):
    """transpose.jl:72-123 compares with GPUArrays' ``permutedims!`` (and a naive SIMT kernel); here
    ``y.copy_(x.t())`` of the library behind ``torch``."""
    y = torch.empty_like(data.y)
    return {"torch copy_(x.t())": time_launches(lambda: y.copy_(data.x.t()), nruns, warmup)}



def verify(data, result) -> None:
    """transpose.jl:58-60: ``Array(y) ~ transpose(Array(x))``.  The Julia (m, n) array x is the torch (n, m)
    tensor, so torch sees the same relation: y == x.t()."""
    assert isapprox(result.y.cpu(), data.x.cpu().t().contiguous())


def metric(data):
    """transpose.jl:62-66: 1 read + 1 write."""
    return 2 * data.m * data.n * data.x.element_size(), "GB/s"


def test_transpose(T: torch.dtype, m: int, n: int, tm: int, tn: int, *, name: str | None = None) -> None:
    """transpose.jl:129-136."""
    name = name or f"transpose ({m} x {n}, {str(T).replace('torch.', '')}, tiles={tm} x {tn})"
    print(f"--- {name} ---")
    data = prepare(m=m, n=n, T=T)
    result = run(data, tm=tm, tn=tn)
    verify(data, result)
    print("  passed")


def main() -> None:
    """transpose.jl:138-147."""
    print("--- Matrix Transposition Examples ---\n")
    test_transpose(torch.float32, 256, 256, 32, 32)
    test_transpose(torch.float32, 512, 512, 64, 64)
    test_transpose(torch.float32, 256, 512, 32, 64)
    test_transpose(torch.float32, 1024, 1024, 64, 64)
    print("\n--- All transpose examples completed ---")
