"""GPU tests with arrays of more than 2^31 elements, through the C ABI.

The reference indexes such arrays with Int64 (test/device/int64_indexing.jl:10-34,
test/codegen/int64_indexing.jl); a device with 288 GB holds them easily, so every kernel on the path has to
form element offsets in 64 bits.  Each case places its data so that rows / tiles start on both sides of
element 2^31, and is checked on the device: element-wise kernels bit for bit against torch's own `+` /
transpose views over the whole array, the row kernels against a float64 evaluation of a few rows at the
start, across the 2^31 boundary and at the end (|err| <= 1e-5 * (|ref| + max|ref|), the bound of the
memory-bound parity tests).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd import tiled as T  # noqa: E402
from cutile_jl_amd.tiled import Tiled  # noqa: E402

WIDE = 2 ** 31


def _randn(shape, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, generator=g, device="cuda", dtype=dtype)


def _close(got, ref, tol=1e-5):
    got = got.double(); ref = ref.double()
    scale = ref.abs().max()
    err = (got - ref).abs()
    bound = tol * (ref.abs() + scale)
    assert bool((err <= bound).all()), f"max err {err.max().item():.3e}, worst ratio {(err / bound).max().item():.2f}"


@pytest.fixture(autouse=True)
def _release():
    yield
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def test_vadd_1d_beyond_2_31_elements(ct):
    n = WIDE + 4099
    a, b = _randn((n,), torch.float16, 1), _randn((n,), torch.float16, 2)
    c = torch.zeros(n, dtype=torch.float16, device="cuda")
    ct.vec_add_kernel_1d(a, b, c, 1024)
    assert torch.equal(c, a + b)
    # the element-wise (gather / scatter) form of the same kernel
    c.zero_()
    ct.vec_add_kernel_1d_gather(a, b, c, 512)
    assert torch.equal(c, a + b)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_transpose_beyond_2_31_elements(ct, dtype):
    m, n = 131_080, 16_392                       # Julia x is (m, n): m * n = 2^31 + 1.15e6
    assert m * n > WIDE
    x = _randn((n, m), dtype, 3)                 # torch layout: dimension 0 of the Julia array is the last one
    y = torch.zeros((m, n), dtype=dtype, device="cuda")
    ct.transpose_kernel(x, y, 64, 64)
    assert torch.equal(y, x.t())


def _rows_to_check(M, per_row):
    edge = WIDE // per_row                       # the row that starts at element 2^31
    return torch.tensor(sorted({0, 1, 2, edge - 2, edge - 1, edge, edge + 1, M - 2, M - 1}), device="cuda")


def test_softmax_beyond_2_31_elements(ct):
    N, M = 16_384, 131_080                       # Julia input is (N, M): columns of 16384, M of them
    assert N * M > WIDE
    x = _randn((M, N), torch.float32, 4)
    rows = _rows_to_check(M, N)
    ref = torch.softmax(x[rows].double(), dim=1)
    out = torch.zeros_like(x)
    ct.softmax_tma_kernel(out, x, N, num_programs=M)
    _close(out[rows], ref)
    assert abs(out.sum(dtype=torch.float64).item() / M - 1.0) < 1e-6      # every column sums to one
    out.zero_()
    ct.softmax_chunked_kernel(out, x, N, 1024, num_programs=M)
    _close(out[rows], ref)
    assert abs(out.sum(dtype=torch.float64).item() / M - 1.0) < 1e-6


def test_layernorm_beyond_2_31_elements(ct):
    N, M = 16_384, 131_080
    eps = 1e-5
    X = _randn((M, N), torch.float32, 5)
    DY = _randn((M, N), torch.float32, 6)
    W, B = _randn((N,), torch.float32, 7), _randn((N,), torch.float32, 8)
    Y, DX = torch.zeros_like(X), torch.zeros_like(X)
    Mean, Rstd = torch.zeros(M, device="cuda"), torch.zeros(M, device="cuda")
    G = 64
    DWp, DBp = torch.zeros((G, N), device="cuda"), torch.zeros((G, N), device="cuda")
    Locks = torch.zeros(G, dtype=torch.int64, device="cuda")
    FDW, FDB = torch.zeros(N, device="cuda"), torch.zeros(N, device="cuda")
    ct.layer_norm_fwd(X, W, B, Y, Mean, Rstd, eps, 1024)
    ct.layer_norm_bwd_dx_partial_dwdb(DX, DY, DWp, DBp, X, W, Mean, Rstd, Locks, G, 1024)
    ct.layer_norm_bwd_dwdb(DWp, DBp, FDW, FDB, 32, 1024)
    rows = _rows_to_check(M, N)
    x, dy, w, b = X[rows].double(), DY[rows].double(), W.double(), B.double()
    mean = x.mean(dim=1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=1, keepdim=True)
    rstd = 1.0 / torch.sqrt(var + eps)
    xhat = (x - mean) * rstd
    _close(Y[rows], xhat * w + b)
    _close(Mean[rows], mean[:, 0])
    _close(Rstd[rows], rstd[:, 0])
    wdy = w * dy
    c1 = (xhat * wdy).mean(dim=1, keepdim=True)
    c2 = wdy.mean(dim=1, keepdim=True)
    _close(DX[rows], (wdy - (xhat * c1 + c2)) * rstd)
    # dB = column sums of DY over every row, those past 2^31 elements included
    _close(FDB, DY.sum(dim=0, dtype=torch.float64))


def test_tiled_broadcast_and_reduction_beyond_2_31_elements(ct):
    n = WIDE + 4099
    a, b = _randn((n,), torch.float16, 9), _randn((n,), torch.float16, 10)
    c = torch.zeros(n, dtype=torch.float16, device="cuda")
    Tiled(c).assign(Tiled(a) + Tiled(b))
    assert torch.equal(c, a + b)
    # reductions of a vector that long: dimension 0 itself exceeds 31 bits
    assert T.maximum(Tiled(a)) == a.max().item()
    assert T.minimum(Tiled(b)) == b.min().item()
    mask = a > -5.0                                  # nearly all true: the count itself exceeds 2^31
    cnt = T.count(Tiled(mask))
    assert cnt == int(mask.sum().item()) and cnt > WIDE
    del a, b, c, mask
    torch.cuda.empty_cache()
    # a (16392, 131080) Float32 matrix: column sums (dims = 1) and the sum of everything
    n0, n1 = 16_392, 131_080
    A = torch.rand((n1, n0), device="cuda", generator=torch.Generator(device="cuda").manual_seed(11))
    R = T.sum(Tiled(A), dims=1)
    assert tuple(R.shape) == (n1, 1)
    _close(R[:, 0], A.sum(dim=1, dtype=torch.float64))
    total = T.sum(Tiled(A))
    ref = A.sum(dtype=torch.float64).item()
    assert abs(total - ref) <= 1e-5 * abs(ref)
    assert T.maximum(Tiled(A)) == A.max().item()


def test_matmul_operand_beyond_2_31_elements(ct):
    """A (65536 x 32776, Float16) has more than 2^31 elements; entries in {-1, 0, 1}, so every fp32 sum is exact
    and the product is compared bit for bit with torch's fp32 product of the same integers."""
    M, K, N = 65_536, 32_776, 128
    assert M * K > WIDE
    g = torch.Generator(device="cuda").manual_seed(12)
    A = torch.randint(-1, 2, (K, M), generator=g, device="cuda", dtype=torch.int8).to(torch.float16)    # Julia (M, K)
    B = torch.randint(-1, 2, (N, K), generator=g, device="cuda", dtype=torch.int8).to(torch.float16)    # Julia (K, N)
    C = torch.zeros((N, M), dtype=torch.float32, device="cuda")                                           # Julia (M, N)
    ct.matmul_kernel(A, B, C, 64, 64, 64)
    ref = torch.zeros_like(C)
    for k0 in range(0, K, 8194):                       # in slabs of K: the fp32 copy of A stays small
        ref += B[:, k0:k0 + 8194].float() @ A[k0:k0 + 8194].float()
    assert torch.equal(C, ref)


def test_fmha_beyond_2_31_elements(ct, orc):
    """Q, K, V, Out of 130 x 128 heads x 2048 x 64 Float16 (2^31 + 2^25 elements each), causal.  Checked against
    the oracle's float64 ref_fmha (examples/fmha.jl:175-220) on the first (batch, head) pair, the pair that starts
    at element 2^31 and the last one, with the bounds of the attention parity tests."""
    from cutile_jl_amd.examples import fmha
    B, H, S, D = 130, 128, 2048, 64
    assert B * H * S * D > WIDE
    Q, K, V = (_randn((B, H, S, D), torch.float16, 20 + i) for i in range(3))
    out = fmha.cutile_fmha(Q, K, V, causal=True)
    assert ct.last_variant().startswith("fmha_pipe")
    for b, h in [(0, 0), (WIDE // (H * S * D), 0), (B - 1, H - 1)]:
        q, k, v = (orc.to_julia(t[b:b + 1, h:h + 1].contiguous()) for t in (Q, K, V))
        ref = orc.ref_fmha(q, k, v, causal=True, dtype=np.float64)
        got = orc.to_julia(out[b:b + 1, h:h + 1].contiguous()).astype(np.float64)
        err = np.abs(got - ref)
        bound = 2e-2 * (np.abs(ref) + np.abs(ref).max())
        assert np.all(err <= bound), f"pair ({b}, {h}): max err {err.max():.3e}, worst ratio {np.max(err / bound):.3f}"
        assert orc.isapprox(got, ref, rtol=1e-2, atol=1e-3)


def test_moe_weights_beyond_2_31_elements(ct, orc):
    """66 experts of 4096 x 8192: w1 has 2^32 + 2^27 elements, w2 2^31 + 2^26, and expert 65 of w2 starts at
    element 2^31 exactly.  Every token is routed to the last two experts, so the result depends only on weights
    past that offset; the oracle's float64 ref_moe (examples/moe.jl:264-304) is evaluated on those two experts
    alone, with the bounds of the MoE parity tests."""
    from cutile_jl_amd.examples import moe
    E, H, I, tokens, topk = 66, 4096, 8192, 48, 2
    assert E * H * I > WIDE and (E - 2) * H * I == WIDE
    g = torch.Generator(device="cuda").manual_seed(30)
    w1 = torch.randn((E, 2 * I, H), generator=g, device="cuda", dtype=torch.float16) * 0.02
    w2 = torch.randn((E, H, I), generator=g, device="cuda", dtype=torch.float16) * 0.02
    hs = torch.randn((tokens, H), generator=g, device="cuda", dtype=torch.float16)
    tw = torch.rand((topk, tokens), generator=g, device="cuda", dtype=torch.float32).to(torch.float16)
    ids = torch.empty((topk, tokens), dtype=torch.int64, device="cuda")
    ids[0] = E - 1 + (torch.arange(tokens, device="cuda") % 2)        # 1-based: experts 65 and 66, alternating
    ids[1] = E - (torch.arange(tokens, device="cuda") % 2)
    out = moe.cutile_moe(hs, w1, w2, tw, ids, 128, 128, 64)
    J = orc.to_julia
    ref = orc.ref_moe(J(hs), J(w1[E - 2:].contiguous()), J(w2[E - 2:].contiguous()), J(tw), J(ids - (E - 2)), dtype=np.float64)
    got = J(out).astype(np.float64)
    err = np.abs(got - ref)
    bound = 2e-2 * (np.abs(ref) + np.abs(ref).max())
    assert np.all(err <= bound), f"max err {err.max():.3e}, worst ratio {np.max(err / bound):.3f}"
    assert orc.isapprox(got, ref, rtol=1e-2, atol=1e-2)
