"""GPU parity tests for the host-level RNG fills (through the C ABI): the device stream against the
numpy restatement of the reference's Philox2x32-7 fill (oracle/cutile_oracle.py: rng_fill), and the
properties the reference's own tests assert (test/device/random.jl:341-526).

Bars: `rand` of every element type is bit-exact (integer arithmetic plus exactly rounded float
conversions).  `randn` / `randexp` go through log / sin / cos / sqrt: |err| <= 1e-5 + 1e-5 |ref| for
Float32 (a few ulp of the transcendental functions, amplified by the 2 pi u angle), 1e-12 for
Float64, one ulp of the narrow type for Float16 / BFloat16.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd import random as R  # noqa: E402

N = 2048
INT_TYPES = [("u8", torch.uint8), ("i8", torch.int8), ("i16", torch.int16), ("i32", torch.int32), ("i64", torch.int64)]
FLOAT_TYPES = [("f16", torch.float16), ("bf16", torch.bfloat16), ("f32", torch.float32), ("f64", torch.float64)]


def host(t):
    return t.float().cpu().numpy() if t.dtype == torch.bfloat16 else t.cpu().numpy()


@pytest.mark.parametrize("kind,dtype", INT_TYPES + FLOAT_TYPES)
@pytest.mark.parametrize("n,seed,counter", [(N, 42, 0), (513, 0, 0), (100, 13, 7), (1, 5, 0), (70001, 0xDEADBEEF, 0xFFFFFF00)])
def test_rand_stream_is_the_references_bit_for_bit(orc, ct, kind, dtype, n, seed, counter):
    rng = R.RNG(seed, counter)
    A = torch.zeros(n, dtype=dtype, device="cuda")
    assert R.rand_(rng, A) is A
    assert ct.last_variant() == "rng_fill_philox2x32_7_rand"
    ref = orc.rng_fill(kind, n, seed, counter)
    assert np.array_equal(host(A), ref)
    s, c = orc.rng_advance_counter(seed & 0xFFFFFFFF, counter, -(-n // 512) * 512)
    assert (rng.seed, rng.counter) == (s, c)


@pytest.mark.parametrize("kind,dtype", FLOAT_TYPES)
@pytest.mark.parametrize("dist", ["randn", "randexp"])
def test_randn_randexp_against_the_restatement(orc, kind, dtype, dist):
    n = 5000
    A = torch.zeros(n, dtype=dtype, device="cuda")
    getattr(R, dist + "_")(R.RNG(7), A)
    ref = np.asarray(orc.rng_fill(kind, n, 7, 0, dist), np.float64)
    got = host(A).astype(np.float64)
    tol = {"f32": 1e-5, "f64": 1e-12, "f16": 2e-3, "bf16": 1.6e-2}[kind]
    assert np.all(np.abs(got - ref) <= tol + tol * np.abs(ref)), np.abs(got - ref).max()


def test_reference_host_rand_properties():
    """test/device/random.jl:421-526."""
    rng = R.RNG(42)
    A = torch.zeros(N, dtype=torch.int32, device="cuda")
    R.rand_(rng, A)
    assert len(np.unique(A.cpu().numpy())) == N and rng.counter == N           # basics + counter advance
    a = R.rand(R.RNG(123), torch.float32, N).cpu().numpy()
    b = R.rand(R.RNG(123), torch.float32, N).cpu().numpy()
    assert np.array_equal(a, b)                                                # determinism
    c = R.rand(R.RNG(42), torch.float32, N).cpu().numpy()
    d = R.rand(R.RNG(100), torch.float32, N).cpu().numpy()
    assert not any(np.array_equal(c[k:], d[:N - k]) for k in range(1, 65))      # re-keyed, not shifted
    cu = R.rand(R.RNG(42), torch.int32, N).cpu().numpy()
    du = R.rand(R.RNG(100), torch.int32, N).cpu().numpy()
    assert not set(cu.tolist()) & set(du.tolist())
    rng = R.RNG(7)
    a1 = R.rand(rng, torch.int32, N).cpu().numpy()
    a2 = R.rand(rng, torch.int32, N).cpu().numpy()
    assert not set(a1.tolist()) & set(a2.tolist())                              # consecutive fills disjoint
    R.seed_(rng, 7)
    assert rng.counter == 0
    v = R.rand(R.RNG(99), torch.int32, N).cpu().numpy().view(np.uint32).astype(np.float64)
    assert abs(v.mean() - (2**32 - 1) / 2) / ((2**32 - 1) / 2) < 0.05           # sample mean
    f = R.rand(R.get_global_rng(), torch.float32, N)
    assert bool(((f > 0) & (f <= 1)).all())
    rng = R.RNG(0)
    A = torch.zeros(513, dtype=torch.int32, device="cuda")                      # partial last tile
    R.rand_(rng, A)
    assert len(np.unique(A.cpu().numpy())) == 513 and rng.counter == 2 * R.RAND_FILL_TILE
    rng = R.RNG(7, 2**32 - 4)
    R.advance_counter_(rng, 1)                                                  # one block of 512 wraps the counter
    assert (rng.seed, rng.counter) == (8, 508)


@pytest.mark.parametrize("kind,dtype", FLOAT_TYPES)
def test_distribution_moments(kind, dtype):
    """test/device/random.jl:341-420: every float type, in range, four quartile bins populated; randn has
    mean 0 / variance 1, randexp mean 1."""
    n = 1 << 20
    u = R.rand(R.RNG(13), dtype, n).double()
    assert bool(((u >= 0) & (u <= 1)).all())
    counts = torch.histc(u.float(), bins=4, min=0, max=1)
    assert counts.min().item() > n / 4 * 0.97
    z = R.randn(R.RNG(13), dtype, n).double()
    assert abs(z.mean().item()) < 0.01 and abs(z.var().item() - 1) < 0.02
    e = R.randexp(R.RNG(13), dtype, n).double()
    assert bool((e >= 0).all()) and abs(e.mean().item() - 1) < 0.02


def test_multidimensional_and_argument_errors(ct, orc):
    A = R.rand(R.RNG(3), torch.float32, 33, 65)                                 # Julia (33, 65): memory order
    assert tuple(A.shape) == (65, 33)
    assert np.array_equal(A.cpu().numpy().reshape(-1), orc.rng_fill("f32", 33 * 65, 3, 0))
    E = torch.zeros(0, device="cuda")
    assert R.rand_(R.RNG(1), E) is E
    with pytest.raises(ct.MiError):
        R.randn_(R.RNG(1), torch.zeros(8, dtype=torch.int32, device="cuda"))     # randn needs a float type
    with pytest.raises(ct.MiError):
        R.rand_(R.RNG(1), torch.zeros(8, 8, device="cuda")[:, ::2])              # not dense
    with pytest.raises(ValueError):
        R.rand_(R.RNG(1), torch.zeros(8))


def test_large_fill_matches_restatement_at_the_far_end(orc):
    n = (1 << 27) + 5
    A = torch.empty(n, dtype=torch.float32, device="cuda")
    R.rand_(R.RNG(2024), A)
    ref = orc.rng_fill("f32", n, 2024, 0)
    got = A.cpu().numpy()
    assert np.array_equal(got[:4096], ref[:4096]) and np.array_equal(got[-4096:], ref[-4096:])
    assert np.array_equal(got[::65537], ref[::65537])
