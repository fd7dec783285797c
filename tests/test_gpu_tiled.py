"""GPU parity tests for the host-level Tiled broadcast / mapreduce entry points (through the C ABI,
via the Python mirror of the reference's API).

The cases follow the reference's own test files one by one -- test/host/broadcast.jl:3-235 and
test/host/mapreduce.jl:3-163 -- and add element types, strided views, large sizes and the two-pass
reductions.  Oracle: the numpy restatement in oracle/cutile_oracle.py (Julia element-type rules +
numpy arithmetic), torch CPU where numpy has no type (bfloat16).

Tolerances.  Element-wise + - * and comparisons, conversions, max / min, integer and Bool work:
bit-exact.  Transcendental functions: |err| <= 4 ulp-ish, written as rtol 2e-6 (float32; the
reference asserts rtol 1e-5) and 1e-14 (float64).  Float sums: rtol 1e-5 of the float64 sum (the
order of a reduction is not specified; the reference asserts `≈`, i.e. rtol sqrt(eps)).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd import tiled as T  # noqa: E402
from cutile_jl_amd.tiled import Tiled  # noqa: E402

F1 = np.float32(1.0)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rand(*julia_shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.rand(tuple(reversed(julia_shape)), generator=g).to(dtype).cuda()


def jl(t):
    """numpy array in the Julia shape."""
    return t.detach().cpu().numpy().T


# ================================================================================================
# broadcast: test/host/broadcast.jl
# ================================================================================================

def test_1d_elementwise(ct):
    A, B = rand(1024), rand(1024, seed=1)
    C = torch.zeros(1024, device="cuda")
    ret = Tiled(C).assign(Tiled(A) + Tiled(B))
    assert ret is C
    assert torch.equal(C, A + B)
    assert ct.last_variant().startswith("tiled_bc")


def test_fused_multi_op(orc):
    A = rand(1024) + 0.1
    C = torch.zeros(1024, device="cuda")
    Tiled(C).assign(Tiled(A) + Tiled(A) * T.sin(Tiled(A)))
    ref, _ = orc.tiled_eval("add(a0,mul(a0,sin(a0)))", (jl(A),))
    np.testing.assert_allclose(jl(C), ref, rtol=2e-6)


def test_scalar_broadcast():
    A = rand(1024)
    C = torch.zeros(1024, device="cuda")
    Tiled(C).assign(Tiled(A) + F1)
    assert torch.equal(C, A + 1.0)


@pytest.mark.parametrize("shape", [(128, 256), (64, 64, 4), (8, 4, 6, 10)])
def test_nd_elementwise(shape):
    A, B = rand(*shape), rand(*shape, seed=1)
    C = torch.zeros_like(A)
    Tiled(C).assign(Tiled(A) + Tiled(B))
    assert torch.equal(C, A + B)


def test_dot_macro_forms():
    """ct.@. in place, with a function, with a scalar, allocating; the in-place form returns the
    destination array itself (broadcast.jl:54-91,225-233)."""
    A, B = rand(1024) + 0.1, rand(1024, seed=1)
    C = torch.zeros(1024, device="cuda")
    ret = T.dot("C = A + B", C=C, A=A, B=B)
    assert ret is C and torch.equal(C, A + B)
    T.dot("C = A + sin(A)", C=C, A=A)
    np.testing.assert_allclose(jl(C), jl(A) + np.sin(jl(A)), rtol=2e-6)
    T.dot("C = A + 2.0", C=C, A=A)           # Float64 literal: computed in Float64, stored as Float32
    assert torch.equal(C, (A.double() + 2.0).float())
    D = T.dot("A + B", A=A, B=B)
    assert D.is_cuda and D.dtype == torch.float32 and torch.equal(D, A + B)


def test_allocating_copy():
    A, B = rand(1024), rand(1024, seed=1)
    C = (Tiled(A) + Tiled(B)).copy()
    assert C.is_cuda and C.shape == A.shape and torch.equal(C, A + B)


@pytest.mark.parametrize("shape", [(1, 1024), (1, 1, 512), (4, 1024)])
def test_leading_singleton_and_small_leading_dims(shape):
    A = rand(*shape)
    B = torch.zeros_like(A)
    Tiled(B).assign(Tiled(A) + F1)
    assert torch.equal(B, A + 1.0)
    Tiled(B).assign(Tiled(A) + Tiled(A))
    assert torch.equal(B, 2 * A)


@pytest.mark.parametrize("n", [1000, 1001, 1, 3, 4097])
def test_non_aligned_size(n):
    A, B = rand(n), rand(n, seed=1)
    C = torch.zeros(n, device="cuda")
    Tiled(C).assign(Tiled(A) + Tiled(B))
    assert torch.equal(C, A + B)


def test_shape_mismatch_throws():
    A = rand(11)
    C = torch.zeros(10, device="cuda")
    with pytest.raises(T.DimensionMismatch):
        Tiled(C).assign(Tiled(A))
    with pytest.raises(T.DimensionMismatch):
        Tiled(C).assign(Tiled(C) + Tiled(A))
    A2 = rand(8, 16)
    C2 = torch.zeros(8, 8, device="cuda")     # same memory shape either way
    with pytest.raises(T.DimensionMismatch):
        Tiled(C2).assign(Tiled(A2) * np.float32(2))


def test_c_abi_reports_shape_mismatch(ct):
    """The library itself refuses mismatching axes (the Python mirror checks first, so call it raw)."""
    import ctypes
    A, C = rand(11), torch.zeros(10, device="cuda")
    flat = T._Flat()
    flat.leaves = [A]
    d, a = T._descriptor(C), T._descriptor(A)
    ptrs = (ctypes.POINTER(ct.MiTileArray) * 1)(ctypes.pointer(a))
    rc = ct.lib().mi_tiled_broadcast(ctypes.byref(d), b"a0", ptrs, 1, flat.scalar_array(), 0, None)
    assert rc == ct.MI_E_SHAPE


def test_size1_expansion(orc):
    m, n = 64, 128
    row, col, full = rand(1, n), rand(m, 1, seed=1), rand(m, n, seed=2)
    C = torch.zeros(n, m, device="cuda")
    Tiled(C).assign(Tiled(row) + Tiled(full))
    assert np.array_equal(jl(C), jl(row) + jl(full))
    Tiled(C).assign(Tiled(col) * Tiled(full))
    assert np.array_equal(jl(C), jl(col) * jl(full))
    Tiled(C).assign(Tiled(row) + F1)                      # expansion only
    assert np.array_equal(jl(C), np.repeat(jl(row) + 1, m, axis=0))
    Tiled(C).assign(Tiled(full) + T.sin(Tiled(row)))      # nested
    ref, _ = orc.tiled_eval("add(a0,sin(a1))", (jl(full), jl(row)))
    np.testing.assert_allclose(jl(C), ref, rtol=2e-6)
    vec = rand(m, seed=3)                                 # rank expansion: vector + matrix
    Tiled(C).assign(Tiled(vec) + Tiled(full))
    assert np.array_equal(jl(C), jl(vec)[:, None] + jl(full))
    D = (Tiled(row) + Tiled(col)).copy()                  # allocating with expansion
    assert tuple(reversed(D.shape)) == (m, n)
    assert np.array_equal(jl(D), jl(row) + jl(col))


def test_scalar_rhs_fill():
    C = rand(1000)
    Tiled(C).assign(0)
    assert torch.all(C == 0)
    D = torch.zeros(65, 33, device="cuda")
    Tiled(D).assign(np.float32(2.5))
    assert torch.all(D == 2.5)


def test_empty_array_no_op(ct):
    C = torch.zeros(0, device="cuda")
    Tiled(C).assign(Tiled(C) + F1)
    D = torch.zeros(0, 4, device="cuda")
    Tiled(D).assign(F1)
    assert C.numel() == 0 and D.numel() == 0


def test_zero_dim_arrays():
    C = torch.zeros((), device="cuda")
    Tiled(C).assign(F1)
    assert C.item() == 1.0
    A = torch.full((), 2.0, device="cuda")
    Tiled(C).assign(Tiled(A) + F1)
    assert C.item() == 3.0


def test_host_side_leaves_rejected():
    C = torch.zeros(16, device="cuda")
    A_cpu = torch.rand(16)
    with pytest.raises(T.ArgumentError):
        Tiled(C).assign(Tiled(A_cpu) * np.float32(2))
    with pytest.raises(TypeError):
        Tiled(C).assign(Tiled(C) + range(1, 17))      # no device storage
    with pytest.raises(T.ArgumentError):
        Tiled(A_cpu).assign(0)


# ---- beyond the reference's cases ---------------------------------------------------------------

def _np_dtype(t):
    return {torch.float32: np.float32, torch.float64: np.float64, torch.float16: np.float16, torch.int32: np.int32,
            torch.int64: np.int64, torch.bool: np.bool_}[t]


TYPE_CASES = [
    ("add(a0,a1)", (torch.float16, torch.float32), "Float32"),
    ("add(a0,a1)", (torch.int32, torch.int64), "Int64"),
    ("add(a0,a1)", (torch.int64, torch.float32), "Float32"),
    ("add(a0,a1)", (torch.bool, torch.bool), "Int64"),
    ("mul(a0,a1)", (torch.bool, torch.float16), "Float16"),
    ("div(a0,a1)", (torch.int32, torch.int32), "Float64"),
    ("sub(a0,a1)", (torch.float64, torch.float32), "Float64"),
    ("fma(a0,a1,a0)", (torch.float16, torch.float16), "Float16"),
    ("lt(a0,a1)", (torch.int32, torch.float32), "Bool"),
    ("ifelse(gt(a0,a1),a0,a1)", (torch.float32, torch.float32), "Float32"),
    ("max(a0,a1)", (torch.int32, torch.int64), "Int64"),
    ("sqrt(abs(a0))", (torch.int32,), "Float64"),
    ("mod(a0,a1)", (torch.int64, torch.int32), "Int64"),
    ("pow(a0,abs(a1))", (torch.int32, torch.int64), "Int32"),        # ^ keeps the base's type and wraps in it
    ("pow(a0,abs(a1))", (torch.bool, torch.int32), "Bool"),
    ("mod(a0,a1)", (torch.float64, torch.float64), "Float64"),       # float quotients from the exact remainder
    ("fld(a0,a1)", (torch.float64, torch.float64), "Float64"),
    ("cld(a0,a1)", (torch.float64, torch.float64), "Float64"),
    ("div_int(a0,a1)", (torch.float64, torch.float64), "Float64"),
    ("mod(a0,trunc(a1))", (torch.float32, torch.float32), "Float32"),
    ("div_int(a0,a1)", (torch.int32, torch.int32), "Int32"),
    ("fld(a0,a1)", (torch.int32, torch.int32), "Int32"),
    ("cld(a0,a1)", (torch.int64, torch.int64), "Int64"),
    ("rem(a0,a1)", (torch.int32, torch.int64), "Int64"),
    ("xor(a0,a1)", (torch.int32, torch.int32), "Int32"),
    ("and(a0,not(a1))", (torch.bool, torch.bool), "Bool"),
    ("i32(trunc(mul(a0,a1)))", (torch.float32, torch.float32), "Int32"),
    ("f16(a0)", (torch.float64,), "Float16"),
    ("neg(a0)", (torch.bool,), "Int64"),
    ("abs2(a0)", (torch.float16,), "Float16"),
    ("copysign(a0,a1)", (torch.float32, torch.int32), "Float32"),
    ("clamp(a0,a1,a0)", (torch.int32, torch.int32), "Int32"),
    ("shl(a0,a1)", (torch.int32, torch.int64), "Int32"),      # counts -50 .. 49: both directions, >= 32 too
    ("shr(a0,a1)", (torch.int64, torch.int32), "Int64"),
    ("lshr(a0,a1)", (torch.int32, torch.int32), "Int32"),
    ("shl(a0,a1)", (torch.bool, torch.int32), "Int64"),
    ("mul_hi(shl(a0,a1),shl(a1,a0))", (torch.int32, torch.int32), "Int32"),      # operands of every magnitude and sign
    ("mul_hi(shl(a0,a1),shl(a1,a0))", (torch.int64, torch.int64), "Int64"),
]


def _leaf(dt, n, seed):
    rng = np.random.default_rng(seed)
    if dt == torch.bool:
        return rng.integers(0, 2, n).astype(np.bool_)
    if dt in (torch.int32, torch.int64):
        v = rng.integers(-50, 50, n).astype(_np_dtype(dt))
        v[v == 0] = 7          # divisors
        return v
    return (rng.standard_normal(n) * 4).astype(_np_dtype(dt))


@pytest.mark.parametrize("text,dtypes,jl_type", TYPE_CASES)
def test_element_types_follow_julia(orc, text, dtypes, jl_type):
    """Result element type (Base.Broadcast.combine_eltypes) and values, bit-exact against numpy in
    the same Julia type (none of these functions is transcendental except sqrt, which is exact)."""
    n = 1003
    leaves = [_leaf(dt, n, i) for i, dt in enumerate(dtypes)]
    ref, ref_type = orc.tiled_eval(text, leaves)
    assert ref_type == jl_type                          # the oracle's own rule, pinned in test_oracle
    tl = [dev(a) for a in leaves]
    flat = T._Flat()
    flat.leaves = tl
    code = T._eltype(flat, text)
    names = {T.MI_F32: "Float32", T.MI_F64: "Float64", T.MI_F16: "Float16", T.MI_I32: "Int32", T.MI_I64: "Int64",
             T.MI_BOOL: "Bool"}
    assert names[code] == jl_type
    dest = torch.empty(n, dtype=T._torch_dtype(code), device="cuda")
    T._launch_broadcast(dest, flat, text)
    got = dest.cpu().numpy()
    assert got.dtype == ref.dtype
    assert np.array_equal(got, np.broadcast_to(ref, got.shape), equal_nan=True), text


def test_bfloat16_against_torch():
    a = (torch.randn(4099) * 3).to(torch.bfloat16)
    b = (torch.randn(4099) * 3).to(torch.bfloat16)
    A, B = a.cuda(), b.cuda()
    C = torch.empty_like(A)
    Tiled(C).assign(Tiled(A) * Tiled(B) + Tiled(A))      # two roundings, like Julia's BFloat16 ops
    ref = ((a.float() * b.float()).to(torch.bfloat16).float() + a.float()).to(torch.bfloat16)
    assert torch.equal(C.cpu(), ref)
    D = (Tiled(A) + Tiled(B.to(torch.float16))).copy()      # BFloat16 + Float16 -> Float32
    assert D.dtype == torch.float32
    assert torch.equal(D.cpu(), a.float() + b.to(torch.float16).float())


MATH = "sqrt rsqrt cbrt inv exp exp2 exp10 expm1 log log2 log10 log1p sin cos tan asin acos atan sinh cosh tanh".split()


@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 2e-6), (torch.float64, 1e-14)])
def test_math_functions(orc, dtype, rtol):
    x = (torch.rand(2048, dtype=torch.float64) * 0.9 + 0.05).to(dtype)      # inside every domain
    X = x.cuda()
    Y = torch.empty_like(X)
    for name in MATH:
        Tiled(Y).assign(getattr(T, name)(Tiled(X)))
        ref, _ = orc.tiled_eval(f"{name}(a0)", (x.numpy(),))
        np.testing.assert_allclose(Y.cpu().numpy(), ref, rtol=rtol, atol=rtol * 1e-2, err_msg=name)
    Tiled(Y).assign(T.atan2(Tiled(X), F1 if dtype == torch.float32 else 1.0) + T.hypot(Tiled(X), Tiled(X)))
    ref = np.arctan2(x.numpy(), x.numpy().dtype.type(1)) + np.hypot(x.numpy(), x.numpy())
    np.testing.assert_allclose(Y.cpu().numpy(), ref, rtol=rtol)
    Tiled(Y).assign(Tiled(X) ** Tiled(X) + Tiled(X) ** 3)
    np.testing.assert_allclose(Y.cpu().numpy(), x.numpy() ** x.numpy() + x.numpy() ** 3, rtol=rtol * 2)


@pytest.mark.parametrize("npdt", [np.float32, np.float64, np.float16])
def test_max_min_follow_julia_for_nan_and_signed_zero(orc, npdt):
    a = np.array([1.0, np.nan, 2.0, -0.0, 0.0, np.nan, -np.inf, 5.0], npdt)
    b = np.array([np.nan, 1.0, 3.0, 0.0, -0.0, np.nan, np.inf, 5.0], npdt)
    A, B = dev(a), dev(b)
    for name in ("max", "min"):
        got = getattr(T, name)(Tiled(A), Tiled(B)).copy().cpu().numpy()
        ref, _ = orc.tiled_eval(f"{name}(a0,a1)", (a, b))
        assert np.array_equal(got, ref, equal_nan=True)
        assert np.array_equal(np.signbit(got), np.signbit(ref)), name


def test_strided_views_and_four_dims(orc):
    base = rand(12, 10, 6, 4)                            # Julia (12,10,6,4)
    A = base[1:4, ::2, 2:9, 3:11]                        # torch view == Julia base[4:11, 3:9, 1:2:5, 2:4]
    assert not A.is_contiguous()
    row = rand(1, A.shape[2], 1, A.shape[0], seed=3)
    C = torch.zeros(A.shape, device="cuda")
    Tiled(C).assign(Tiled(A) * np.float32(2) - Tiled(row))
    assert np.array_equal(jl(C), jl(A) * np.float32(2) - jl(row))
    Cv = torch.zeros(base.shape, device="cuda")
    Tiled(Cv[1:4, ::2, 2:9, 3:11]).assign(Tiled(A) + F1)          # strided destination
    ref = torch.zeros_like(base)
    ref[1:4, ::2, 2:9, 3:11] = A + 1
    assert torch.equal(Cv, ref)
    T_ = base[0, 0].t()                                   # dimension 0 not contiguous
    E = (Tiled(T_) + F1).copy()
    assert torch.equal(E, T_ + 1)


def test_large_broadcast_streams_and_matches_vadd(ct):
    n = 1 << 26
    A = torch.rand(n, device="cuda")
    B = torch.rand(n, device="cuda")
    C = torch.empty(n, device="cuda")
    Tiled(C).assign(Tiled(A) + Tiled(B))
    assert "stream" in ct.last_variant()
    assert torch.equal(C, A + B)


def test_kernels_are_cached():
    A, B = rand(777), rand(777, seed=1)
    C = torch.zeros(777, device="cuda")
    Tiled(C).assign(Tiled(A) - Tiled(B) * np.float32(3))
    n0 = T.compile_count()
    for k in range(3):
        Tiled(C).assign(Tiled(A) - Tiled(B) * np.float32(k))      # scalar values are run-time arguments
        assert torch.equal(C, A - B * float(k))
    assert T.compile_count() == n0


# ================================================================================================
# mapreduce: test/host/mapreduce.jl
# ================================================================================================

def close(got, ref):
    return abs(float(got) - float(ref)) <= 1e-5 * abs(float(ref))


def test_sum_1d():
    A = rand(1024)
    assert close(T.sum(Tiled(A)), jl(A).astype(np.float64).sum())
    R = T.sum(Tiled(A), dims=1)
    assert R.is_cuda and tuple(R.shape) == (1,)
    assert close(R.item(), jl(A).astype(np.float64).sum())


@pytest.mark.parametrize("shape,dims", [((128, 256), 1), ((128, 256), 2), ((128, 256), (2, 1, 2)), ((128, 256), range(1, 3)),
                                        ((128, 256), [2, 1]), ((64, 32), (2, 3)), ((100, 200), 1), ((100, 200), None),
                                        ((32, 16, 8), (1, 3)), ((32, 16, 8), 2), ((5, 7, 3, 11), (2, 4)),
                                        ((5, 7, 3, 11), (1, 2, 3)), ((4097, 3), 1), ((3, 4097), 2)])
def test_sum_dims(orc, shape, dims):
    A = rand(*shape)
    ref, _ = orc.tiled_mapreduce(None, "add_sum", jl(A), dims=dims)
    R = T.sum(Tiled(A), dims=dims)
    if dims is None:
        assert close(R, ref)
    else:
        assert tuple(reversed(R.shape)) == ref.shape
        np.testing.assert_allclose(jl(R), ref, rtol=1e-5)


def test_non_aligned_noop_dims():
    A = torch.full((17,), 2, dtype=torch.int32, device="cuda")
    assert torch.equal(T.prod(Tiled(A), dims=()), A.long())          # prod widens Int32 (mul_prod)
    assert torch.equal(T.maximum(Tiled(A), dims=()), A)
    assert torch.equal(T.prod(Tiled(A), dims=2), A.long())
    assert torch.equal(T.reduce("*", Tiled(A), dims=()), A)


def test_out_of_range_dims():
    A = rand(64, 32)
    with pytest.raises(T.InexactError):
        T.sum(Tiled(A), dims=2**63)
    with pytest.raises(T.ArgumentError):
        T.sum(Tiled(A), dims=0)
    with pytest.raises(T.ArgumentError, match="must be integers"):
        T.sum(Tiled(A), dims=(1.0,))


@pytest.mark.parametrize("fn,op,shape,dims", [("maximum", "max", (32, 16, 8), (1, 3)), ("maximum", "max", (1024,), None),
                                              ("minimum", "min", (1024,), None), ("maximum", "max", (64, 128), 1),
                                              ("minimum", "min", (64, 128), 2)])
def test_maximum_minimum(orc, fn, op, shape, dims):
    A = rand(*shape)
    ref, _ = orc.tiled_mapreduce(None, op, jl(A), dims=dims)
    R = getattr(T, fn)(Tiled(A), dims=dims)
    if dims is None:
        assert R == ref
    else:
        assert np.array_equal(jl(R), ref)


def test_prod_1d():
    A = 1 + rand(32) * 0.01
    assert abs(T.prod(Tiled(A)) - float(np.prod(jl(A).astype(np.float64)))) <= 1e-3


def test_max_min_with_oob_padding():
    """Non-aligned size: whatever stands in for out-of-range elements must be the identity."""
    A = torch.full((1000,), -5.0, device="cuda")
    assert T.maximum(Tiled(A)) == -5.0
    B = torch.full((1000,), 5.0, device="cuda")
    assert T.minimum(Tiled(B)) == 5.0


def test_non_aligned_sizes():
    A = rand(1000)
    assert close(T.sum(Tiled(A)), jl(A).astype(np.float64).sum())


def test_mapreduce_with_abs(orc):
    A = rand(1024) - 0.5
    ref, _ = orc.tiled_mapreduce("abs(a0)", "+", jl(A))
    assert close(T.mapreduce(abs, "+", Tiled(A)), ref)
    assert close(T.mapreduce(lambda x: x * x + F1, "+", Tiled(A)), (jl(A).astype(np.float64) ** 2 + 1).sum())


def test_large_array_multiple_blocks():
    A = rand(8192)
    assert close(T.sum(Tiled(A)), jl(A).astype(np.float64).sum())


def test_inplace_variants():
    A = rand(64, 128)
    R = torch.zeros(128, 1, device="cuda")               # Julia (1, 128)
    assert T.sum_(R, Tiled(A)) is R
    np.testing.assert_allclose(jl(R), jl(A).astype(np.float64).sum(axis=0, keepdims=True), rtol=1e-5)
    T.maximum_(R, Tiled(A))
    assert np.array_equal(jl(R), jl(A).max(axis=0, keepdims=True))
    T.minimum_(R, Tiled(A))
    assert np.array_equal(jl(R), jl(A).min(axis=0, keepdims=True))
    P = 1 + rand(16, 8) * 0.01
    R2 = torch.zeros(1, 16, device="cuda")               # Julia (16, 1)
    T.prod_(R2, Tiled(P))
    np.testing.assert_allclose(jl(R2), jl(P).astype(np.float64).prod(axis=1, keepdims=True), rtol=1e-5)
    with pytest.raises(T.DimensionMismatch):
        T.sum_(torch.zeros(7, device="cuda"), Tiled(A))


def test_any_all_count():
    A = torch.zeros(1024, dtype=torch.bool, device="cuda")
    assert T.any(Tiled(A)) is False
    B = A.clone()
    B[511] = True
    assert T.any(Tiled(B)) is True
    O = torch.ones(1024, dtype=torch.bool, device="cuda")
    assert T.all(Tiled(O)) is True
    O2 = O.clone()
    O2[511] = False
    assert T.all(Tiled(O2)) is False
    Cn = torch.zeros(1024, dtype=torch.bool, device="cuda")
    Cn[[0, 99, 499, 998]] = True
    assert T.count(Tiled(Cn)) == 4
    X = rand(3000)
    assert T.any(Tiled(X), f=lambda x: x > np.float32(2)) is False
    assert T.all(Tiled(X), f=lambda x: x < np.float32(2)) is True
    assert T.count(Tiled(X), f=lambda x: x > np.float32(0.5)) == int((X > 0.5).sum().item())
    M = rand(40, 30) > 0.5
    assert torch.equal(T.count(Tiled(M), dims=1), M.sum(dim=1, keepdim=True))


# ---- beyond the reference's cases ---------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.float64, torch.float16])
@pytest.mark.parametrize("op", ["add_sum", "+", "max", "min"])
def test_reduction_types(orc, dtype, op):
    rng = np.random.default_rng(5)
    a = rng.integers(-100, 100, (37, 53)).astype(_np_dtype(dtype))            # Julia (37, 53)
    if dtype == torch.float16:
        a = (a / 64).astype(np.float16)
    A = dev(np.ascontiguousarray(a.T))
    for dims in (None, 1, 2):
        ref, jt = orc.tiled_mapreduce(None, op, a, dims=dims)
        R = T.mapreduce(None, op, Tiled(A), dims=dims)
        if dims is None:
            got = np.asarray(R)
        else:
            assert str(R.dtype).endswith(jt.lower())
            got = jl(R)
        if dtype == torch.float16 and op in ("+", "add_sum"):
            np.testing.assert_allclose(got.astype(np.float64), np.asarray(ref, np.float64), rtol=2e-2, atol=0.5)
        else:
            assert np.array_equal(got, ref), (op, dims)


def test_init_is_applied_like_the_reference():
    A = rand(50, 20)
    R = T.sum(Tiled(A), dims=1, init=np.float32(10))
    np.testing.assert_allclose(jl(R), 10 + jl(A).astype(np.float64).sum(axis=0, keepdims=True), rtol=1e-5)
    assert close(T.sum(Tiled(A), init=100.0), 100 + jl(A).astype(np.float64).sum())
    assert T.maximum(Tiled(A), init=5.0) == 5.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
def test_nan_propagates_through_max(dtype):
    A = rand(5000, dtype=dtype)
    A[1234] = float("nan")
    assert np.isnan(T.maximum(Tiled(A)))
    assert np.isnan(T.minimum(Tiled(A)))
    M = rand(300, 40, dtype=dtype)                        # Julia (300, 40); NaN in column 7
    M[7, 123] = float("nan")
    for dims in (1, 2):
        R = T.maximum(Tiled(M), dims=dims)
        ref = M.double().cpu().numpy().max(axis=2 - dims, keepdims=True)      # numpy max propagates NaN too
        assert np.array_equal(R.double().cpu().numpy(), ref, equal_nan=True)


@pytest.mark.parametrize("shape,dims", [((1 << 24,), None), ((4096, 4096), None), ((4096, 4096), 1), ((4096, 4096), 2),
                                        ((64, 1 << 18), 2), ((1 << 18, 64), 1), ((8, 1 << 20), 1)])
def test_large_reductions_two_pass_and_reproducible(ct, shape, dims):
    A = rand(*shape, seed=3)
    a64 = A.double()
    R1 = T.sum(Tiled(A), dims=dims)
    variant = ct.last_variant()
    R2 = T.sum(Tiled(A), dims=dims)
    if dims is None:
        assert R1 == R2
        assert abs(R1 - a64.sum().item()) <= 1e-5 * a64.sum().item()
        assert "split" in variant
    else:
        assert torch.equal(R1, R2)                        # fixed order: bit-identical from run to run
        ref = a64.sum(dim=len(shape) - dims, keepdim=True)
        assert torch.allclose(R1.double(), ref, rtol=1e-5)
    M = T.maximum(Tiled(A), dims=dims)
    if dims is None:
        assert M == A.max().item()
    else:
        assert torch.equal(M, A.amax(dim=len(shape) - dims, keepdim=True))


def test_reduction_of_strided_view():
    base = rand(40, 30, 20)
    V = base[2:15, 5:25:2, 3:33]                         # Julia base[4:33, 6:2:24, 3:15]
    for dims in (1, 2, 3, (1, 3), None):
        R = T.sum(Tiled(V), dims=dims)
        if dims is None:
            assert close(R, V.double().sum().item())
            continue
        axes = tuple(3 - d for d in ((dims,) if isinstance(dims, int) else dims))
        assert torch.allclose(R.double(), V.double().sum(dim=axes, keepdim=True), rtol=1e-5)
