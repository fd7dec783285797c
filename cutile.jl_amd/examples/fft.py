"""Mirror of examples/fft.jl:130-260 (table generation, prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import namespace, time_launches, upload


def dft_matrix(size: int) -> np.ndarray:
    """fft.jl:130-140: (2, size, size) float32 in the Julia shape, W[i, j] = exp(-2 pi i * i*j / size)."""
    i, j = np.meshgrid(np.arange(size), np.arange(size), indexing="ij")
    W = np.exp(-2j * np.pi * i * j / size)
    return np.stack([W.real, W.imag]).astype(np.float32)


def make_twiddles(factors):
    """fft.jl:143-180: (W0, W1, W2, T0, T1) in the Julia shapes."""
    F0, F1, F2 = factors
    N, F1F2 = F0 * F1 * F2, F1 * F2
    j, i = np.meshgrid(np.arange(F1F2), np.arange(F0), indexing="ij")
    t0 = np.exp(-2j * np.pi * i * j / N)                       # T0[:, j, i]
    k, jj = np.meshgrid(np.arange(F2), np.arange(F1), indexing="ij")
    t1 = np.exp(-2j * np.pi * jj * k / F1F2)                   # T1[:, k, j]
    return (dft_matrix(F0), dft_matrix(F1), dft_matrix(F2),
            np.stack([t0.real, t0.imag]).astype(np.float32), np.stack([t1.real, t1.imag]).astype(np.float32))


def prepare(*, benchmark: bool = False, batch: int | None = None, factors=None, atom_packing_dim: int | None = None,
            seed: int = 42):
    """fft.jl:186-215: complex N(0,1) signals (N, batch) packed as float32 (D, 2N/D, batch)."""
    batch = (256 if benchmark else 2) if batch is None else batch
    factors = ((16, 16, 16) if benchmark else (2, 2, 2)) if factors is None else tuple(factors)
    N = factors[0] * factors[1] * factors[2]
    D = min(64, 2 * N) if atom_packing_dim is None else atom_packing_dim
    assert (2 * N) % D == 0, "2 * N must be divisible by atom_packing_dim"
    rng = np.random.default_rng(seed)
    # torch layout (batch, N) complex64 == Julia (N, batch) ComplexF32; randn(ComplexF32) has variance 1/2 per part
    inp = ((rng.standard_normal((batch, N), dtype=np.float32) + 1j * rng.standard_normal((batch, N), dtype=np.float32))
           * np.float32(np.sqrt(0.5))).astype(np.complex64)
    input_dev = torch.from_numpy(inp).to("cuda")
    x_packed = torch.view_as_real(input_dev).reshape(batch, 2 * N // D, D)     # Julia (D, 2N/D, batch)
    y_packed = torch.empty_like(x_packed)
    W0, W1, W2, T0, T1 = (upload(t) for t in make_twiddles(factors))
    return namespace(input=input_dev, x_packed=x_packed, y_packed=y_packed, W0=W0, W1=W1, W2=W2, T0=T0, T1=T1,
                     factors=factors, batch=batch, N=N, D=D)


def run(data, *, nruns: int = 1, warmup: int = 0):
    """fft.jl:217-246: one launch over the whole batch (BS = 1), then unpack to complex (N, batch)."""
    d = data
    F0, F1, F2 = d.factors
    times = time_launches(lambda: ct.fft_kernel(d.x_packed, d.y_packed, d.W0, d.W1, d.W2, d.T0, d.T1, d.N, F0, F1, F2,
                                                1, d.D), nruns, warmup)
    output = torch.view_as_complex(d.y_packed.reshape(d.batch, d.N, 2)).clone()
    return namespace(output=output, times=times)




def verify(data, result) -> None:
    """fft.jl:245-248: against the host FFT along the signal axis (FFTW there, numpy's pocketfft here),
    ``rtol = 1e-4`` in the norm."""
    reference = torch.from_numpy(np.fft.fft(data.input.cpu().numpy().astype(np.complex128), axis=1))
    got = result.output.cpu().to(torch.complex128)
    err = torch.linalg.vector_norm(torch.view_as_real(got - reference))
    assert float(err) <= 1e-4 * float(torch.linalg.vector_norm(torch.view_as_real(reference)))


def run_others(data, *, nruns: int = 1, warmup: int = 0):
    """fft.jl:262-279 compares with cuFFT; here rocFFT through ``torch.fft.fft`` over the batch."""
    return {"rocFFT (torch.fft.fft)": time_launches(lambda: torch.fft.fft(data.input, dim=1), nruns, warmup)}


def metric(data):
    """fft.jl:253-256: a latency benchmark, the time itself is the figure."""
    return 0, "us"


def test_fft(batch: int, factors, *, name: str | None = None) -> None:
    """fft.jl:285-293."""
    n = factors[0] * factors[1] * factors[2]
    name = name or f"fft batch={batch}, size={n}, factors={tuple(factors)}"
    print(f"--- {name} ---")
    data = prepare(batch=batch, factors=factors)
    result = run(data)
    verify(data, result)
    print("  passed")


def main() -> None:
    """fft.jl:295-303."""
    print("--- FFT Examples ---\n")
    test_fft(64, (8, 8, 8))
    test_fft(32, (8, 8, 8))
    print("\n--- All FFT examples completed ---")
