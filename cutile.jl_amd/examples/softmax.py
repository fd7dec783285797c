"""Mirror of examples/softmax.jl:116-198 (prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import namespace, rand_normal, time_launches


def next_power_of_2(n: int) -> int:
    """softmax.jl:107-114"""
    if n <= 0:
        return 1
    p = 1
    while p < n:
        p <<= 1
    return p


def prepare(*, benchmark: bool = False, M: int | None = None, N: int | None = None,
            T: torch.dtype = torch.float32, seed: int = 2, std: float = 2.0):
    """softmax.jl:116-127: input Julia (N, M) = torch (M, N); measured configuration draws
    N(0, sigma^2 = 4)."""
    M = (4096 if benchmark else 256) if M is None else M
    N = (4096 if benchmark else 256) if N is None else N
    rng = np.random.default_rng(seed)
    inp = rand_normal(rng, (N, M), T, std=std)
    return namespace(input=inp, output_tma=torch.empty_like(inp),
                     output_chunked=torch.empty_like(inp), M=M, N=N)


def run(data, *, tile_tma: int | None = None, tile_chunked: int = 1024, nruns: int = 1,
        warmup: int = 0):
    """softmax.jl:129-173."""
    d = data
    if tile_tma is None:
        tile_tma = next_power_of_2(d.N)

    def run_tma():
        ct.softmax_tma_kernel(d.output_tma, d.input, tile_tma, num_programs=d.M)

    def run_chunked():
        ct.softmax_chunked_kernel(d.output_chunked, d.input, d.N, tile_chunked, num_programs=d.M)

    for _ in range(warmup):
        run_tma()
        run_chunked()
    torch.cuda.synchronize()
    times_tma = time_launches(run_tma, nruns, 0)
    times_chunked = time_launches(run_chunked, nruns, 0)
    return namespace(output_tma=d.output_tma, output_chunked=d.output_chunked,
                     times={"cuTile TMA": times_tma, "cuTile Chunked": times_chunked})



def run_others(data, *, nruns: int = 1, warmup: int = 0):
    """softmax.jl:205-232 compares with the unfused broadcast formulation on GPUArrays; the same three
    passes on ``torch``, and ``torch.softmax`` (one fused kernel of the vendor library) beside it."""
    x = data.input                      # torch (M, N): a Julia column is a torch row
    out = torch.empty_like(x)

    def broadcast():
        m = x.amax(dim=1, keepdim=True)
        e = torch.exp(x - m)
        torch.div(e, e.sum(dim=1, keepdim=True), out=out)

    return {"torch broadcast": time_launches(broadcast, nruns, warmup),
            "torch.softmax": time_launches(lambda: torch.softmax(x, dim=1), nruns, warmup)}



def verify(data, result) -> None:
    """softmax.jl:175-188: every column of both outputs against exp(x - max) / sum on the host, per column
    ``atol = 1e-5, rtol = 1e-4`` in the norm (a Julia column is a torch row)."""
    x = data.input.cpu()
    e = torch.exp(x - x.amax(dim=1, keepdim=True))
    expected = (e / e.sum(dim=1, keepdim=True)).double()
    for label in ("output_tma", "output_chunked"):
        out = getattr(result, label).cpu().double()
        err = torch.linalg.vector_norm(out - expected, dim=1)
        bound = torch.clamp(1e-4 * torch.maximum(torch.linalg.vector_norm(out, dim=1), torch.linalg.vector_norm(expected, dim=1)), min=1e-5)
        bad = torch.nonzero(err > bound)
        assert bad.numel() == 0, f"{label} column {int(bad[0]) + 1} mismatch"


def metric(data):
    """softmax.jl:190-198."""
    MN = data.M * data.N * 4
    return {"cuTile TMA": (2 * MN, "GB/s"), "cuTile Chunked": (4 * MN, "GB/s")}


def test_softmax(M: int, N: int, *, tile_tma: int | None = None, tile_chunked: int = 1024, name: str | None = None) -> None:
    """softmax.jl:238-245."""
    tile_tma = next_power_of_2(N) if tile_tma is None else tile_tma
    name = name or f"softmax ({M} x {N}), tma_tile={tile_tma}, chunked_tile={tile_chunked}"
    print(f"--- {name} ---")
    data = prepare(M=M, N=N)
    result = run(data, tile_tma=tile_tma, tile_chunked=tile_chunked)
    verify(data, result)
    print("  tma passed, chunked passed")


def main() -> None:
    """softmax.jl:247-256."""
    print("--- Softmax Examples ---\n")
    test_softmax(256, 256)
    test_softmax(1024, 1024)
    test_softmax(4096, 4096)
    print("\n--- All softmax examples completed ---")
