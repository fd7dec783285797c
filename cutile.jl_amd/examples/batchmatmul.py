"""Mirror of examples/batchmatmul.jl:62-111 (prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_uniform, time_launches


def prepare(*, benchmark: bool = False, M: int | None = None, K: int | None = None, N: int | None = None,
            Batch: int | None = None, T: torch.dtype = torch.float32, seed: int = 4, lo: float = -1.0, hi: float = 1.0):
    """batchmatmul.jl:62-73, batch-last: A (M,K,Batch) = torch (Batch,K,M) etc.  Inputs
    U(lo,hi); the measured configuration uses U(-1,1) (the reference U[0,1))."""
    M = (1024 if benchmark else 256) if M is None else M
    K = (512 if benchmark else 128) if K is None else K
    N = (2048 if benchmark else 256) if N is None else N
    Batch = (8 if benchmark else 4) if Batch is None else Batch
    rng = np.random.default_rng(seed)
    A = rand_uniform(rng, (M, K, Batch), T, lo, hi)
    B = rand_uniform(rng, (K, N, Batch), T, lo, hi)
    C = torch.empty((Batch, N, M), dtype=T, device=A.device)
    return namespace(A=A, B=B, C=C, M=M, K=K, N=N, Batch=Batch)


def run(data, *, tm: int = 128, tn: int = 128, tk: int = 64, nruns: int = 1, warmup: int = 0):
    """batchmatmul.jl:75-95."""
    times = time_launches(lambda: ct.batch_matmul_kernel(data.A, data.B, data.C, tm, tn, tk), nruns, warmup)
    return namespace(C=data.C, times=times)



def run_others(data, *, nruns: int = 1, warmup: int = 0):
    """batchmatmul.jl:117-146 compares with cuBLAS' strided-batched GEMM; here ``torch.bmm``."""
    C = torch.empty((data.Batch, data.N, data.M), dtype=data.A.dtype, device=data.A.device)
    return {"rocBLAS batched (torch.bmm)": time_launches(lambda: torch.bmm(data.B, data.A, out=C), nruns, warmup)}



def verify(data, result) -> None:
    """batchmatmul.jl:96-107: every batch entry against the host product, ``rtol = 1e-2`` over the whole array."""
    expected = torch.bmm(data.B.cpu().float(), data.A.cpu().float())
    got = result.C.cpu().float()
    assert isapprox(got, expected, rtol=1e-2), f"max diff: {float((got - expected).abs().max())}"


def metric(data):
    """batchmatmul.jl:108-111."""
    return 2 * data.M * data.K * data.N * data.Batch, "TFLOPS"


def smoke(orc):
    d = prepare(M=130, K=70, N=96, Batch=2)
    r = run(d)
    ref = orc.batch_matmul(orc.to_julia(d.A), orc.to_julia(d.B))
    got = orc.to_julia(r.C).astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()


def test_batch_matmul(T: torch.dtype, M: int, K: int, N: int, Batch: int, tm: int, tn: int, tk: int, *,
                      name: str | None = None) -> None:
    """batchmatmul.jl:152-159."""
    name = name or (f"batch_matmul ({M} x {K} x {Batch}) @ ({K} x {N} x {Batch}), {str(T).replace('torch.', '')}, "
                    f"tiles={tm} x {tn} x {tk}")
    print(f"--- {name} ---")
    data = prepare(M=M, K=K, N=N, Batch=Batch, T=T)
    result = run(data, tm=tm, tn=tn, tk=tk)
    verify(data, result)
    print("  passed")


def main() -> None:
    """batchmatmul.jl:161-169."""
    print("--- Batch Matrix Multiplication Examples ---\n")
    test_batch_matmul(torch.float32, 256, 128, 256, 4, 32, 32, 32)
    test_batch_matmul(torch.float32, 512, 256, 512, 4, 64, 64, 64)
    test_batch_matmul(torch.float16, 512, 256, 1024, 4, 128, 256, 64)
    print("\n--- All batch matmul examples completed ---")
