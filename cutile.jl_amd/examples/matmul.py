"""Mirror of examples/matmul.jl:66-106 (prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_normal, rand_uniform, time_launches


def prepare(*, benchmark: bool = False, M: int | None = None, N: int | None = None, K: int | None = None,
            T: torch.dtype = torch.float32, out_T: torch.dtype | None = None, seed: int = 3,
            dist: str = "uniform"):
    """matmul.jl:66-77.  A (M,K), B (K,N), C (M,N) Julia = torch (K,M), (N,K), (N,M).
    ``dist='uniform'`` is the reference's U[0,1); ``'normal64'`` is the measured
    configuration's N(0, 1/64).  ``out_T`` lets f16 inputs produce an f32 C."""
    M = (4096 if benchmark else 256) if M is None else M
    N = (4096 if benchmark else 256) if N is None else N
    K = (4096 if benchmark else 256) if K is None else K
    rng = np.random.default_rng(seed)
    gen = (lambda shp: rand_normal(rng, shp, T, std=0.125)) if dist == "normal64" else (lambda shp: rand_uniform(rng, shp, T))
    A = gen((M, K)); B = gen((K, N))
    C = torch.empty((N, M), dtype=out_T or T, device=A.device)
    return namespace(A=A, B=B, C=C, M=M, N=N, K=K)


def run(data, *, tm: int = 64, tn: int = 64, tk: int = 64, nruns: int = 1, warmup: int = 0):
    """matmul.jl:79-96: one untimed launch, then ``nruns`` timed ones."""
    launch = lambda: ct.matmul_kernel(data.A, data.B, data.C, tm, tn, tk)
    launch()
    times = time_launches(launch, nruns, warmup)
    return namespace(C=data.C, times=times)



def run_others(data, *, nruns: int = 1, warmup: int = 0):
    """matmul.jl:112-141 compares with cuBLAS through ``mul!``; here hipBLASLt / rocBLAS through
    ``torch.matmul`` (Julia C = A * B is torch C^T = B^T A^T on the same bytes; the result has the operands' type)."""
    C = torch.empty((data.N, data.M), dtype=data.A.dtype, device=data.A.device)
    return {"hipBLASLt (torch.matmul)": time_launches(lambda: torch.matmul(data.B, data.A, out=C), nruns, warmup)}



def verify(data, result) -> None:
    """matmul.jl:98-101: ``isapprox(C, A * B; rtol = 1e-2)`` against the host product (fp32 here for every
    operand type).  Julia's A * B on the arrays' bytes is torch's B @ A."""
    expected = data.B.cpu().float() @ data.A.cpu().float()
    got = result.C.cpu().float()
    assert isapprox(got, expected, rtol=1e-2), f"max diff: {float((got - expected).abs().max())}"


def metric(data):
    """matmul.jl:103-106."""
    return 2 * data.M * data.N * data.K, "TFLOPS"


def smoke(orc):
    d = prepare(M=192, N=128, K=160, T=torch.float16, out_T=torch.float32, dist="normal64")
    r = run(d)
    ref = orc.matmul(orc.to_julia(d.A), orc.to_julia(d.B))
    got = orc.to_julia(r.C).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 2e-2 * np.abs(ref) + 2e-2 * np.abs(ref).max() * 1e-2), np.abs(got - ref).max()


def test_matmul(T: torch.dtype, M: int, N: int, K: int, tm: int, tn: int, tk: int, *, name: str | None = None) -> None:
    """matmul.jl:147-154."""
    name = name or f"matmul ({M} x {K}) @ ({K} x {N}), {str(T).replace('torch.', '')}, tiles={tm} x {tn} x {tk}"
    print(f"--- {name} ---")
    data = prepare(M=M, N=N, K=K, T=T)
    result = run(data, tm=tm, tn=tn, tk=tk)
    verify(data, result)
    print("  passed")


def main() -> None:
    """matmul.jl:156-165."""
    print("--- Matrix Multiplication Examples ---\n")
    test_matmul(torch.float32, 256, 256, 256, 32, 32, 32)
    test_matmul(torch.float32, 512, 512, 512, 64, 64, 64)
    test_matmul(torch.float32, 256, 512, 128, 32, 32, 32)
    test_matmul(torch.float32, 1024, 1024, 1024, 64, 64, 64)
    print("\n--- All matmul examples completed ---")
