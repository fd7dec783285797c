"""Shared pieces of the example harnesses: seeded synthetic inputs and the timing loop."""
from __future__ import annotations

from types import SimpleNamespace

import numpy as np
import torch

DEVICE = "cuda"

_NP = {torch.float32: np.float32, torch.float64: np.float64, torch.float16: np.float16}


def upload(jl_array: np.ndarray, dtype: torch.dtype | None = None) -> torch.Tensor:
    """Julia-shaped numpy array -> device tensor of the reversed shape (same memory order)."""
    t = torch.from_numpy(np.ascontiguousarray(jl_array.T))
    if dtype is not None and t.dtype != dtype:
        t = t.to(dtype)
    return t.to(DEVICE)


def rand_uniform(rng: np.random.Generator, jl_shape, dtype: torch.dtype, lo=0.0, hi=1.0) -> torch.Tensor:
    """U[lo, hi) in float32 then rounded to ``dtype``; Julia shape in, device tensor out."""
    a = rng.random(tuple(reversed(jl_shape)), dtype=np.float32)
    if lo != 0.0 or hi != 1.0:
        a = a * np.float32(hi - lo) + np.float32(lo)
    return torch.from_numpy(a).to(dtype).to(DEVICE)


def rand_normal(rng: np.random.Generator, jl_shape, dtype: torch.dtype, mean=0.0, std=1.0) -> torch.Tensor:
    a = rng.standard_normal(tuple(reversed(jl_shape)), dtype=np.float32)
    if std != 1.0:
        a *= np.float32(std)
    if mean != 0.0:
        a += np.float32(mean)
    return torch.from_numpy(a).to(dtype).to(DEVICE)


def time_launches(fn, nruns: int, warmup: int) -> list[float]:
    """The reference's protocol (examples/vadd.jl:73-86): ``warmup`` untimed calls followed by
    a sync, then ``nruns`` calls each bracketed by events on the launch stream; times in ms."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(nruns):
        t0 = torch.cuda.Event(enable_timing=True)
        t1 = torch.cuda.Event(enable_timing=True)
        t0.record()
        fn()
        t1.record()
        t1.synchronize()
        times.append(t0.elapsed_time(t1))
    return times


def isapprox(x: torch.Tensor, y: torch.Tensor, *, rtol: float | None = None, atol: float = 0.0) -> bool:
    """Julia's ``isapprox`` for arrays: ``norm(x - y) <= max(atol, rtol * max(norm(x), norm(y)))`` with the
    2-norm, and ``rtol = sqrt(eps)`` of the element type when neither tolerance is given."""
    if rtol is None:
        rtol = float(torch.finfo(x.dtype).eps) ** 0.5 if atol == 0.0 and x.dtype.is_floating_point else 0.0
    xd, yd = x.double().flatten(), y.double().flatten()
    return bool(torch.linalg.vector_norm(xd - yd) <= max(atol, rtol * max(torch.linalg.vector_norm(xd), torch.linalg.vector_norm(yd))))


def namespace(**kw) -> SimpleNamespace:
    return SimpleNamespace(**kw)
