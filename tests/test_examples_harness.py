"""The example mirrors keep the harness contract of the reference's example files: ``verify`` (the host check of
each example), ``test_<name>`` and ``main()`` (the example's own list of small shapes, which the reference's test
suite runs, test/runtests.jl:45-61)."""
import contextlib
import io
from types import SimpleNamespace

import pytest
import torch

EXAMPLES = ["vadd", "transpose", "matmul", "batchmatmul", "layernorm", "softmax", "fmha", "moe", "fft"]


def _mod(ct, name):
    import importlib
    return importlib.import_module(f"cutile_jl_amd.examples.{name}")


def test_isapprox_is_julias(ct):
    """Norm-wise comparison, rtol = sqrt(eps) of the element type by default, no default once atol is given."""
    from cutile_jl_amd.examples._harness import isapprox
    x = torch.ones(1000)
    assert isapprox(x, x + 3e-4)                      # sqrt(eps(Float32)) = 3.45e-4
    assert not isapprox(x, x + 4e-4)
    y = x.clone(); y[0] = 1.5                          # one large element error, small in the norm
    assert isapprox(x, y, rtol=2e-2) and not isapprox(x, y, rtol=1e-2)
    assert isapprox(torch.zeros(4), torch.full((4,), 1e-4), atol=1e-3) and not isapprox(torch.zeros(4), torch.full((4,), 1e-4))
    assert isapprox(torch.ones(8, dtype=torch.float16), torch.full((8,), 1.03, dtype=torch.float16))   # sqrt(eps(Float16)) = 0.031


def test_every_example_has_the_reference_entry_points(ct):
    for name in EXAMPLES:
        m = _mod(ct, name)
        for fn in ("prepare", "run", "verify", "metric", "main"):
            assert callable(getattr(m, fn, None)), (name, fn)
    for name in ("vadd", "transpose", "matmul", "batchmatmul", "softmax", "fft"):    # the ones the reference gives run_others
        assert callable(getattr(_mod(ct, name), "run_others", None)), name
    assert not hasattr(_mod(ct, "layernorm"), "run_others")                       # layernorm.jl:334 has none either


def test_verify_accepts_right_and_rejects_wrong_results_on_the_host(ct):
    """``verify`` is pure host code: feed it host tensors."""
    g = torch.Generator().manual_seed(0)
    vadd = _mod(ct, "vadd")
    a, b = torch.rand(1000, generator=g), torch.rand(1000, generator=g)
    vadd.verify(SimpleNamespace(a=a, b=b), SimpleNamespace(c=a + b))
    with pytest.raises(AssertionError):
        vadd.verify(SimpleNamespace(a=a, b=b), SimpleNamespace(c=a + b + 0.01))
    tr = _mod(ct, "transpose")
    x = torch.rand(8, 16, generator=g)
    tr.verify(SimpleNamespace(x=x), SimpleNamespace(y=x.t().contiguous()))
    with pytest.raises(AssertionError):
        tr.verify(SimpleNamespace(x=x), SimpleNamespace(y=x.t().contiguous().flip(0)))
    mm = _mod(ct, "matmul")
    A, B = torch.rand(32, 16, generator=g), torch.rand(24, 32, generator=g)        # Julia A (16, 32), B (32, 24)
    mm.verify(SimpleNamespace(A=A, B=B), SimpleNamespace(C=B @ A))
    with pytest.raises(AssertionError):
        mm.verify(SimpleNamespace(A=A, B=B), SimpleNamespace(C=(B @ A) * 1.05))
    sm = _mod(ct, "softmax")
    inp = torch.randn(6, 40, generator=g)
    good = torch.softmax(inp, dim=1)
    sm.verify(SimpleNamespace(input=inp, M=6, N=40), SimpleNamespace(output_tma=good, output_chunked=good.clone()))
    bad = good.clone(); bad[3] *= 1.001
    with pytest.raises(AssertionError, match="output_chunked column 4"):
        sm.verify(SimpleNamespace(input=inp, M=6, N=40), SimpleNamespace(output_tma=good, output_chunked=bad))
    ln = _mod(ct, "layernorm")
    M, N = 12, 32
    X = torch.randn(M, N, generator=g, requires_grad=True); W = torch.randn(N, generator=g, requires_grad=True)
    Bv = torch.randn(N, generator=g, requires_grad=True); DY = torch.randn(M, N, generator=g)
    Y = torch.nn.functional.layer_norm(X, (N,), W, Bv, 1e-5)
    Y.backward(DY)
    data = SimpleNamespace(X=X.detach(), W=W.detach(), B=Bv.detach(), DY=DY, N=N, eps=1e-5)
    res = SimpleNamespace(Y=Y.detach(), DX=X.grad, FINAL_DW=W.grad, FINAL_DB=Bv.grad)
    ln.verify(data, res)                                   # the host formulas agree with autograd
    with pytest.raises(AssertionError, match="dW mismatch"):
        ln.verify(data, SimpleNamespace(Y=Y.detach(), DX=X.grad, FINAL_DW=W.grad * 1.1, FINAL_DB=Bv.grad))
    fm = _mod(ct, "fmha")
    Q = torch.randn(1, 4, 16, 8, generator=g); K = torch.randn(1, 2, 16, 8, generator=g); V = torch.randn(1, 2, 16, 8, generator=g)
    ref = torch.nn.functional.scaled_dot_product_attention(Q, K.repeat_interleave(2, 1), V.repeat_interleave(2, 1), is_causal=True)
    fm.verify(SimpleNamespace(Q=Q, K=K, V=V, causal=True), SimpleNamespace(out=ref))        # ref_fmha agrees with the library
    with pytest.raises(AssertionError):
        fm.verify(SimpleNamespace(Q=Q, K=K, V=V, causal=False), SimpleNamespace(out=ref))


@pytest.mark.gpu
@pytest.mark.parametrize("name", EXAMPLES)
def test_example_main_runs_and_verifies(ct, name):
    """``main()`` of every example: the reference's list of shapes, each launched through the C ABI and checked
    by the example's own ``verify``."""
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        _mod(ct, name).main()
    text = out.getvalue()
    assert "passed" in text and "completed" in text
