"""Mirror of examples/layernorm.jl:211-332 (prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_normal, time_launches


def prepare(*, benchmark: bool = False, M: int | None = None, N: int | None = None,
            eps: float = 1e-5, GROUP_SIZE_M: int = 64, seed: int = 1):
    """layernorm.jl:211-234.  Arrays are Julia (N, M) = torch (M, N).  Inputs follow the
    measured configuration: X ~ N(0,1), W ~ N(1,0.1), B ~ N(0,0.1), DY ~ N(0,1)."""
    M = (4096 if benchmark else 256) if M is None else M
    N = (4096 if benchmark else 256) if N is None else N
    rng = np.random.default_rng(seed)
    f32 = torch.float32
    X = rand_normal(rng, (N, M), f32)
    W = rand_normal(rng, (N,), f32, mean=1.0, std=0.1)
    B = rand_normal(rng, (N,), f32, mean=0.0, std=0.1)
    DY = rand_normal(rng, (N, M), f32)
    dev = X.device
    e = lambda *jl: torch.empty(tuple(reversed(jl)), dtype=f32, device=dev)
    # The two partial buffers share one allocation so that the zero-fill before every backward is
    # one launch instead of the reference's three (layernorm.jl:245-247; Locks is never touched
    # by this implementation and needs no fill).
    partials = e(N, GROUP_SIZE_M, 2)
    return namespace(
        X=X, W=W, B=B, Y=e(N, M), Mean=e(M), Rstd=e(M),
        DY=DY, DX=e(N, M), partials=partials, DW_partial=partials[0], DB_partial=partials[1],
        Locks=torch.zeros(GROUP_SIZE_M, dtype=torch.int64, device=dev),
        FINAL_DW=e(N), FINAL_DB=e(N), M=M, N=N, eps=eps, GROUP_SIZE_M=GROUP_SIZE_M)


def run(data, *, TILE_N: int = 1024, TILE_M: int = 32, nruns: int = 1, warmup: int = 0):
    """layernorm.jl:236-282: the backward timing includes the zero-fill of the partials and both kernels."""
    d = data

    def run_fwd():
        ct.layer_norm_fwd(d.X, d.W, d.B, d.Y, d.Mean, d.Rstd, d.eps, TILE_N)

    def run_bwd():
        d.partials.zero_()
        ct.layer_norm_bwd_dx_partial_dwdb(d.DX, d.DY, d.DW_partial, d.DB_partial, d.X, d.W, d.Mean,
                                          d.Rstd, d.Locks, d.GROUP_SIZE_M, TILE_N)
        ct.layer_norm_bwd_dwdb(d.DW_partial, d.DB_partial, d.FINAL_DW, d.FINAL_DB, TILE_M, TILE_N)

    def both():
        run_fwd()
        run_bwd()

    for _ in range(warmup):
        both()
    torch.cuda.synchronize()
    times_fwd = time_launches(run_fwd, nruns, 0)
    times_bwd = time_launches(run_bwd, nruns, 0)
    return namespace(Y=d.Y, Mean=d.Mean, Rstd=d.Rstd, DX=d.DX, FINAL_DW=d.FINAL_DW,
                     FINAL_DB=d.FINAL_DB, times_fwd=times_fwd, times_bwd=times_bwd)



def verify(data, result) -> None:
    """layernorm.jl:284-314: Y, dX, dW, dB against the host formulas in fp32, each ``rtol = 1e-2``.  The Julia
    arrays are (N, M) with the row along the first axis; the torch tensors are (M, N), the row along dim 1."""
    X, W, B, DY = data.X.cpu(), data.W.cpu(), data.B.cpu(), data.DY.cpu()
    N, eps = data.N, data.eps
    mean = X.sum(dim=1, keepdim=True) / N
    var = ((X - mean) ** 2).sum(dim=1, keepdim=True) / N
    rstd = 1.0 / torch.sqrt(var + eps)
    xhat = (X - mean) * rstd
    assert isapprox(xhat * W + B, result.Y.cpu(), rtol=1e-2), "Y mismatch"
    wdy = W * DY
    c1 = (xhat * wdy).sum(dim=1, keepdim=True) / N
    c2 = wdy.sum(dim=1, keepdim=True) / N
    assert isapprox((wdy - (xhat * c1 + c2)) * rstd, result.DX.cpu(), rtol=1e-2), "dX mismatch"
    assert isapprox((DY * xhat).sum(dim=0), result.FINAL_DW.cpu(), rtol=1e-2), "dW mismatch"
    assert isapprox(DY.sum(dim=0), result.FINAL_DB.cpu(), rtol=1e-2), "dB mismatch"


def metric(data):
    """layernorm.jl:324-332 (the reference's formula, which counts its L2-served re-reads)."""
    MN = data.M * data.N * 4
    return {"cuTile Fwd": (4 * MN, "GB/s"), "cuTile Bwd": (5 * MN, "GB/s")}


def test_layernorm(M: int, N: int, TILE_N: int, *, TILE_M: int = 32, eps: float = 1e-5, name: str | None = None) -> None:
    """layernorm.jl:316-322."""
    name = name or f"layernorm ({M} x {N}), tile_n={TILE_N}, tile_m={TILE_M}"
    print(f"--- {name} ---")
    data = prepare(M=M, N=N, eps=eps)
    result = run(data, TILE_N=TILE_N, TILE_M=TILE_M)
    verify(data, result)
    print("  fwd passed, bwd passed")


def main() -> None:
    """layernorm.jl:340-348."""
    print("=== LayerNorm Examples (fwd+bwd) ===\n")
    test_layernorm(256, 256, 256)
    test_layernorm(512, 512, 512)
    test_layernorm(1024, 1024, 1024)
    print("\n=== All layernorm examples completed ===")
