"""GPU parity tests for the batched FFT kernel through the C ABI.

Oracle: ``numpy.fft.fft`` in float64 on the complex64 inputs (what the reference's ``verify``
does with FFTW, examples/fft.jl:248-251), plus the numpy restatement of the kernel's three-stage
data flow with the same float32 tables.  Shapes: the reference's ``main()`` list (fft.jl:303-304),
its benchmark shape and its default, plus mixed radices.

Tolerance: the reference's norm criterion ``isapprox(rtol=1e-4)`` and, element-wise,
|err| <= 1e-5 * (|ref| + max|ref|).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd.examples import fft  # noqa: E402


@pytest.mark.parametrize("batch,factors", [(64, (8, 8, 8)), (32, (8, 8, 8)), (2, (2, 2, 2)), (256, (16, 16, 16)),
                                           (5, (4, 8, 2)), (3, (2, 4, 8)), (7, (16, 8, 8)), (1, (4, 4, 4))])
def test_fft_against_numpy(orc, batch, factors):
    d = fft.prepare(batch=batch, factors=factors)
    r = fft.run(d)
    x = d.input.cpu().numpy().T.astype(np.complex128)          # Julia (N, batch)
    got = r.output.cpu().numpy().T.astype(np.complex128)
    ref = np.fft.fft(x, axis=0)
    assert orc.isapprox(got, ref, rtol=1e-4)
    err = np.abs(got - ref)
    assert np.all(err <= 1e-5 * (np.abs(ref) + np.abs(ref).max())), f"max err {err.max():.3e}"
    # the restatement of the kernel's own data flow, with the same float32 tables
    tables = fft.make_twiddles(factors)
    flow = orc.fft_3stage(x, factors, tables=tables)
    assert np.all(np.abs(got - flow) <= 1e-5 * (np.abs(flow) + np.abs(flow).max()))


def test_fft_properties_full_size():
    """4096 points x 256 signals: a unit impulse at n0 gives the phase ramp exp(-2 pi i k n0 / N);
    linearity; Parseval."""
    d = fft.prepare(benchmark=True)
    N, B = d.N, d.batch
    x = torch.zeros(B, N, dtype=torch.complex64, device="cuda")
    n0 = torch.arange(B, device="cuda") * 13 % N
    x[torch.arange(B, device="cuda"), n0] = 1
    d.x_packed.copy_(torch.view_as_real(x).reshape(d.x_packed.shape))
    y = fft.run(d).output
    k = torch.arange(N, device="cuda", dtype=torch.float64)
    ref = torch.exp(-2j * np.pi * k[None, :] * n0[:, None].double() / N)
    assert torch.all((y.to(torch.complex128) - ref).abs() <= 1e-5)
    g = torch.Generator(device="cuda").manual_seed(1)
    a = torch.randn(B, N, 2, device="cuda", generator=g); b = torch.randn(B, N, 2, device="cuda", generator=g)

    def tf(v):
        d.x_packed.copy_(v.reshape(d.x_packed.shape))
        return fft.run(d).output
    ya, yb, yab = tf(a), tf(b), tf(2 * a - 3 * b)
    assert torch.all((yab - (2 * ya - 3 * yb)).abs() <= 2e-4 * yab.abs().max())
    ea = (torch.view_as_complex(a).abs() ** 2).sum(dim=1).double()
    assert torch.allclose((ya.abs() ** 2).sum(dim=1).double() / N, ea, rtol=1e-5)


def test_fft_argument_errors(ct):
    d = fft.prepare(batch=4, factors=(8, 8, 8))
    with pytest.raises(ct.MiError) as e:
        ct.fft_kernel(d.x_packed, d.y_packed, d.W0, d.W1, d.W2, d.T0, d.T1, d.N, 8, 8, 4, 1, d.D)   # N != F0*F1*F2
    assert e.value.code == ct.MI_E_ARG
    with pytest.raises(ct.MiError) as e:
        ct.fft_kernel(d.x_packed, d.y_packed, d.W0, d.W1, d.W2, d.T1, d.T0, d.N, 8, 8, 8, 1, d.D)   # tables swapped
    assert e.value.code == ct.MI_E_SHAPE
    with pytest.raises(ct.MiError) as e:
        ct.fft_kernel(d.x_packed, d.y_packed, d.W0, d.W1, d.W2, d.T0, d.T1, d.N, 8, 8, 8, 3, d.D)   # BS does not divide batch
    assert e.value.code == ct.MI_E_SHAPE
