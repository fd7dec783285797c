"""Host-level random fills: the Python mirror of ``cuTile.RNG`` and ``Random.rand!`` / ``randn!`` /
``randexp!`` on it (reference: src/language/random.jl:650-860) over ``mi_rng_fill``.

``RNG(seed)`` holds the reference's two UInt32 words (seed, counter).  Every fill writes the
reference's Philox2x32-7 stream on the device, value for value, then advances the counter by the
whole blocks of 512 it consumed, carrying into the seed on wrap-around, so consecutive fills of one
``RNG`` are disjoint and equal seeds reproduce.  Arrays are torch tensors on the GPU (any shape,
dense); they are filled in memory order.  Unsigned element types share the kernels of the signed
ones (the bits are the same).
"""
from __future__ import annotations

import ctypes
import os

from . import (MI_BF16, MI_F16, MI_F32, MI_F64, MI_I8, MI_I16, MI_I32, MI_I64, TileArray, _call, _stream)

RAND_FILL_TILE = 512      # src/language/random.jl:701
_RAND, _RANDN, _RANDEXP = 0, 1, 2


def _code(dtype) -> int:
    import torch
    table = {torch.float32: MI_F32, torch.float64: MI_F64, torch.float16: MI_F16, torch.bfloat16: MI_BF16,
             torch.int8: MI_I8, torch.uint8: MI_I8, torch.int16: MI_I16, torch.int32: MI_I32, torch.int64: MI_I64}
    for name, code in (("uint16", MI_I16), ("uint32", MI_I32), ("uint64", MI_I64)):
        if hasattr(torch, name):
            table[getattr(torch, name)] = code
    try:
        return table[dtype]
    except KeyError:
        raise TypeError(f"rand!: unsupported element type {dtype}") from None


class RNG:
    """``cuTile.RNG([seed])`` / ``cuTile.RNG(seed, counter)`` (src/language/random.jl:670-683)."""

    def __init__(self, seed: int | None = None, counter: int = 0):
        if seed is None:
            seed = int.from_bytes(os.urandom(4), "little")      # RandomDevice
        self.seed = int(seed) & 0xFFFFFFFF
        self.counter = int(counter) & 0xFFFFFFFF

    def copy(self):
        return RNG(self.seed, self.counter)

    def __eq__(self, other):
        return isinstance(other, RNG) and (self.seed, self.counter) == (other.seed, other.counter)

    def __hash__(self):
        return hash((self.seed, self.counter))

    def __repr__(self):
        return f"RNG(seed=0x{self.seed:08x}, counter={self.counter})"


def seed_(rng: RNG, seed: int | None = None) -> RNG:
    """``Random.seed!(rng, seed)``: new seed, counter back to 0 (src/language/random.jl:685-690)."""
    rng.seed = (int.from_bytes(os.urandom(4), "little") if seed is None else int(seed)) & 0xFFFFFFFF
    rng.counter = 0
    return rng


def advance_counter_(rng: RNG, n_elements: int) -> RNG:
    """``advance_counter!`` for a fill of ``n_elements`` (whole blocks of 512; the carry re-keys)."""
    s, c = ctypes.c_uint32(rng.seed), ctypes.c_uint32(rng.counter)
    _call("mi_rng_advance_counter", ctypes.byref(s), ctypes.byref(c), int(n_elements))
    rng.seed, rng.counter = s.value, c.value
    return rng


def _fill(rng: RNG, A, dist: int, stream=None):
    if not getattr(A, "is_cuda", False):
        raise ValueError("rand!: the array must live on the device")
    if A.numel() == 0:
        return A
    d = TileArray(A, dtype=_code(A.dtype))
    _call("mi_rng_fill", ctypes.byref(d), rng.seed, rng.counter, dist, _stream(stream))
    advance_counter_(rng, A.numel())
    return A


def rand_(rng: RNG, A, stream=None):
    """``Random.rand!(rng, A)`` (src/language/random.jl:765-781)."""
    return _fill(rng, A, _RAND, stream)


def randn_(rng: RNG, A, stream=None):
    """``Random.randn!(rng, A)`` (src/language/random.jl:793-800)."""
    return _fill(rng, A, _RANDN, stream)


def randexp_(rng: RNG, A, stream=None):
    """``Random.randexp!(rng, A)`` (src/language/random.jl:811-818)."""
    return _fill(rng, A, _RANDEXP, stream)


def _new(dtype, dims):
    import torch
    dims = tuple(dims[0]) if len(dims) == 1 and isinstance(dims[0], (tuple, list)) else tuple(dims)
    return torch.empty(tuple(reversed(dims)), dtype=torch.float32 if dtype is None else dtype, device="cuda")


def rand(rng: RNG, dtype, *dims, stream=None):
    """``Random.rand(rng, T, dims...)``: a new device array of Julia shape ``dims``."""
    return rand_(rng, _new(dtype, dims), stream)


def randn(rng: RNG, dtype, *dims, stream=None):
    return randn_(rng, _new(dtype, dims), stream)


def randexp(rng: RNG, dtype, *dims, stream=None):
    return randexp_(rng, _new(dtype, dims), stream)


# ``cuTile.rand`` / ``cuTile.rand!`` aliases on a lazily created global RNG (src/language/random.jl:744-757,820-860).
_global_rng: RNG | None = None


def get_global_rng() -> RNG:
    global _global_rng
    if _global_rng is None:
        _global_rng = RNG()
    return _global_rng


def seed(value: int | None = None) -> None:
    """``cuTile.seed!([seed])``."""
    seed_(get_global_rng(), value)
