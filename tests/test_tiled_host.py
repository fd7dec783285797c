"""CPU tests of the host-level Tiled API: the expression text form, Julia's element-type rules as the
library applies them, argument validation of the Python mirror, and that every kernel shape the
generator can emit compiles for gfx950 (hiprtc needs no GPU; nothing is loaded or launched).

The element-type expectations are Julia facts (Base promotion.jl, float.jl, bool.jl, reduce.jl):
Int32 + Int64 -> Int64; Int64 + Float32 -> Float32; Float16 + Float32 -> Float32; Int / Int ->
Float64; true + true == 2 (Int64); Bool * Float16 -> Float16; sqrt(::Int32) -> Float64; comparisons
-> Bool; sum(::Array{Int32}) -> Int64 (add_sum) while reduce(+, ::Array{Int32}) stays Int32.
"""
import ctypes

import numpy as np
import pytest
import torch

from cutile_jl_amd import tiled as T
from cutile_jl_amd.tiled import Tiled

NAMES = {T.MI_F32: "Float32", T.MI_F64: "Float64", T.MI_F16: "Float16", T.MI_BF16: "BFloat16", T.MI_I32: "Int32",
         T.MI_I64: "Int64", T.MI_BOOL: "Bool"}
CODES = {v: k for k, v in NAMES.items()}


def eltype(ct, text, leaves=(), scalars=()):
    ld = (ctypes.c_int32 * max(1, len(leaves)))(*[CODES[x] for x in leaves])
    sd = (ctypes.c_int32 * max(1, len(scalars)))(*[CODES[x] for x in scalars])
    out = ctypes.c_int32(-1)
    rc = ct.lib().mi_tiled_broadcast_eltype(text.encode(), ld, len(leaves), sd, len(scalars), ctypes.byref(out))
    return rc, NAMES.get(out.value)


@pytest.mark.parametrize("text,leaves,scalars,want", [
    ("add(a0,a1)", ("Int32", "Int64"), (), "Int64"),
    ("add(a0,a1)", ("Int64", "Float32"), (), "Float32"),
    ("add(a0,a1)", ("Float16", "Float32"), (), "Float32"),
    ("add(a0,a1)", ("Float16", "BFloat16"), (), "Float32"),
    ("add(a0,a1)", ("Bool", "Bool"), (), "Int64"),
    ("mul(a0,a1)", ("Bool", "Bool"), (), "Bool"),
    ("mul(a0,a1)", ("Bool", "Float16"), (), "Float16"),
    ("div(a0,a1)", ("Int32", "Int32"), (), "Float64"),
    ("div(a0,a1)", ("Float32", "Int64"), (), "Float32"),
    ("add(a0,s0)", ("Float32",), ("Float64",), "Float64"),
    ("add(a0,s0)", ("Float32",), ("Float32",), "Float32"),
    ("add(a0,s0)", ("Float32",), ("Int64",), "Float32"),
    ("sqrt(a0)", ("Int32",), (), "Float64"),
    ("sin(a0)", ("Float16",), (), "Float16"),
    ("lt(a0,a1)", ("Float32", "Int32"), (), "Bool"),
    ("ifelse(lt(a0,a1),a0,a1)", ("Float32", "Float64"), (), "Float64"),
    ("pow(a0,a1)", ("Float32", "Int64"), (), "Float32"),
    ("pow(a0,a1)", ("Int32", "Int64"), (), "Int32"),           # Julia: ^(x::T, p::Integer) keeps the base type
    ("pow(a0,a1)", ("Bool", "Int64"), (), "Bool"),
    ("pow(a0,a1)", ("Float32", "Float64"), (), "Float64"),
    ("neg(a0)", ("Bool",), (), "Int64"),
    ("not(a0)", ("Bool",), (), "Bool"),
    ("i32(a0)", ("Float64",), (), "Int32"),
    ("copysign(a0,a1)", ("Float32", "Float64"), (), "Float32"),
    ("fma(a0,a1,s0)", ("Float16", "Float16"), ("Float32",), "Float32"),
    ("shl(a0,s0)", ("Int32",), ("Int64",), "Int32"),          # Julia: the shifted value's type
    ("shr(a0,a1)", ("Int64", "Int32"), (), "Int64"),
    ("lshr(a0,a1)", ("Bool", "Int32"), (), "Int64"),
    ("mul_hi(a0,a1)", ("Int32", "Int32"), (), "Int32"),
    ("rsqrt(a0)", ("Float16",), (), "Float16"),
])
def test_element_type_rules(ct, text, leaves, scalars, want):
    rc, got = eltype(ct, text, leaves, scalars)
    assert rc == 0 and got == want


def test_oracle_and_library_agree_on_promotion(ct, orc):
    names = ["Bool", "Int32", "Int64", "Float16", "Float32", "Float64"]
    for a in names:
        for b in names:
            rc, got = eltype(ct, "max(a0,a1)", (a, b))
            assert rc == 0 and got == orc.jl_promote(a, b), (a, b)


@pytest.mark.parametrize("text,code", [
    ("foo(a0)", "MI_E_UNSUPPORTED"), ("add(a0)", "MI_E_ARG"), ("add(a0,a1", "MI_E_ARG"), ("add(a0,a1))", "MI_E_ARG"),
    ("", "MI_E_ARG"), ("a", "MI_E_ARG"), ("a0 a1", "MI_E_ARG"), ("add(a0,a9)", "MI_E_UNSUPPORTED"), ("add(a0,a3)", "MI_E_ARG"),
    ("and(a0,a1)", "MI_E_DTYPE"), ("ifelse(a0,a0,a1)", "MI_E_DTYPE"), ("add(a0;a1)", "MI_E_ARG"),
    ("system(a0)", "MI_E_UNSUPPORTED"), ("add(a0,1.0)", "MI_E_ARG"), ("shl(a0,a1)", "MI_E_DTYPE"), ("mul_hi(a0,a1)", "MI_E_DTYPE"),
])
def test_malformed_or_unknown_expressions_are_refused(ct, text, code):
    rc, _ = eltype(ct, text, ("Float32", "Float32"))
    assert rc == getattr(ct, code)


def test_tree_to_text():
    A, B = torch.zeros(4), torch.zeros(4)
    flat = T._Flat()
    text = flat.text(Tiled(A) + Tiled(A) * T.sin(Tiled(B)) - np.float32(2) + abs(-Tiled(B)) / 3)
    assert text == "add(sub(add(a0,mul(a0,sin(a1))),s0),div(abs(neg(a1)),s1))"
    assert [t is x for t, x in zip(flat.leaves, (A, B))] == [True, True]
    assert [NAMES[s.dtype] for s in flat.scalars] == ["Float32", "Int64"]
    assert Tiled(3.5) == 3.5 and Tiled(Tiled(A)).parent is A           # numbers pass through (src/tiled.jl:11)
    assert flat.text((Tiled(A) < 1.0) & ~(Tiled(B) >= Tiled(A))) == "and(lt(a0,s2),not(ge(a1,a0)))"


def test_dot_wraps_every_leaf():
    """ct.@. C = A + sin(B) * 2 is Tiled(C) .= Tiled(A) .+ sin.(Tiled(B)) .* 2 (test/host/broadcast.jl:48-52)."""
    import ast
    A, B = torch.zeros(4), torch.zeros(4)
    tree = T._build(ast.parse("A + sin(B) * 2", mode="eval").body, {"A": A, "B": B})
    flat = T._Flat()
    assert flat.text(tree) == "add(a0,mul(sin(a1),s0))"
    assert flat.leaves[0] is A and flat.leaves[1] is B
    with pytest.raises(NameError):
        T._build(ast.parse("A + Z", mode="eval").body, {"A": A})
    with pytest.raises(NameError):
        T._build(ast.parse("__import__(A)", mode="eval").body, {"A": A})


def test_host_arrays_and_shapes_are_rejected_before_any_launch():
    C = torch.zeros(16)
    with pytest.raises(T.ArgumentError):
        Tiled(C).assign(0)
    with pytest.raises(T.ArgumentError):
        (Tiled(C) + 1.0).copy()
    with pytest.raises(T.ArgumentError):
        T.sum(Tiled(C))
    with pytest.raises(T.DimensionMismatch):
        T._broadcast_shape([(8, 16), (8, 8)])
    assert T._broadcast_shape([(1, 128), (64, 1), (64,)]) == (64, 128)
    assert T._broadcast_shape([(), (3,)]) == (3,)


def test_dims_normalisation():
    assert T._region(None, 3) == (1, 2, 3)
    assert T._region(2, 3) == (2,)
    assert T._region((2, 1, 2), 2) == (1, 2)
    assert T._region(range(1, 3), 2) == (1, 2)
    assert T._region((2, 3), 2) == (2,)            # out-of-range dimensions are ignored
    assert T._region((), 2) == ()
    with pytest.raises(T.ArgumentError):
        T._region(0, 2)
    with pytest.raises(T.ArgumentError, match="must be integers"):
        T._region((1.0,), 2)
    with pytest.raises(T.InexactError):
        T._region(2**63, 2)


@pytest.mark.parametrize("f,src,op,widen,want", [
    (None, "Int32", T.MI_OP_ADD, 1, "Int64"), (None, "Int32", T.MI_OP_ADD, 0, "Int32"),
    (None, "Bool", T.MI_OP_ADD, 0, "Int64"), (None, "Bool", T.MI_OP_OR, 0, "Bool"),
    (None, "Float16", T.MI_OP_ADD, 1, "Float16"), (None, "Int32", T.MI_OP_MAX, 0, "Int32"),
    ("abs(a0)", "Float32", T.MI_OP_ADD, 1, "Float32"), ("gt(a0,s0)", "Float32", T.MI_OP_OR, 0, "Bool"),
    ("sqrt(a0)", "Int64", T.MI_OP_MAX, 0, "Float64"), (None, "Bool", T.MI_OP_MUL, 1, "Int64"),
])
def test_mapreduce_result_types(ct, f, src, op, widen, want):
    sd = (ctypes.c_int32 * 1)(CODES["Float32"])
    out = ctypes.c_int32(-1)
    rc = ct.lib().mi_tiled_mapreduce_eltype(None if f is None else f.encode(), CODES[src], sd, 1, op, widen, ctypes.byref(out))
    assert rc == 0 and NAMES[out.value] == want
    rc = ct.lib().mi_tiled_mapreduce_eltype(None, CODES["Float32"], sd, 0, T.MI_OP_AND, 0, ctypes.byref(out))
    assert rc == ct.MI_E_DTYPE


@pytest.fixture
def dry_run():
    old = T.set_dry_run(True)
    yield
    T.set_dry_run(old)


def _bc(ct, dest, text, leaves, scalars=()):
    flat = T._Flat()
    flat.leaves = list(leaves)
    flat.scalars = [T._scalar(s) for s in scalars]
    descs = [T._descriptor(t) for t in flat.leaves]
    ptrs = (ctypes.POINTER(ct.MiTileArray) * max(1, len(descs)))(*[ctypes.pointer(d) for d in descs])
    d = T._descriptor(dest)
    return ct.lib().mi_tiled_broadcast(ctypes.byref(d), text.encode(), ptrs, len(descs), flat.scalar_array(),
                                       len(flat.scalars), None)


def test_generated_broadcast_kernels_compile(ct, dry_run):
    """One kernel per layout class and type family; the all-functions chains make sure every device
    function of the vocabulary instantiates for float32, float64, float16 and the integer types."""
    f32 = lambda *s: torch.zeros(*s)                                    # noqa: E731
    n0 = T.compile_count()
    assert _bc(ct, f32(1024), "add(a0,a1)", [f32(1024), f32(1024)]) == 0
    assert ct.last_variant() == "tiled_bc_v4_u1_tx256_nd1"
    assert _bc(ct, f32(1 << 20), "add(a0,s0)", [f32(1 << 20)], [np.float32(1)]) == 0
    assert "_u4_" in ct.last_variant()
    assert _bc(ct, f32(64, 128), "add(a0,a1)", [f32(64, 1), f32(1, 128)]) == 0
    assert ct.last_variant().endswith("nd2")
    assert _bc(ct, f32(4, 8, 16, 32), "add(a0,a1)", [f32(4, 1, 16, 1), f32(1, 8, 1, 32)]) == 0
    assert ct.last_variant().endswith("nd4")
    chain = "a0"
    for name in ("abs abs2 sign floor ceil round trunc sqrt rsqrt cbrt inv exp exp2 exp10 expm1 log log2 log10 log1p sin cos "
                 "tan asin acos atan sinh cosh tanh identity neg").split():
        chain = f"{name}({chain})"
    def total(terms):
        text = terms[0]
        for t in terms[1:]:
            text = f"add({text},{t})"
        return text
    two = total([f"{n}(a0,a1)" for n in "sub mul div pow max min copysign atan2 hypot div_int rem mod fld cld".split()]
                + ["fma(a0,a1,a0)", "muladd(a0,a1,a0)", "clamp(a0,a1,a0)"])
    for dt in (torch.float32, torch.float64, torch.float16, torch.bfloat16):
        x = torch.zeros(100, dtype=dt)
        assert _bc(ct, x, chain, [x]) == 0, dt
        assert _bc(ct, x, two, [x, x]) == 0, dt
    for dt in (torch.int32, torch.int64):
        x = torch.zeros(100, dtype=dt)
        ints = total([f"{n}(a0,a1)" for n in "sub mul pow max min copysign div_int rem mod fld cld and or xor shl shr lshr mul_hi".split()]
                     + ["fma(a0,a1,a0)", "clamp(a0,a1,a0)", "not(a0)", "abs(a0)", "abs2(a0)", "sign(a0)", "neg(a0)"])
        assert _bc(ct, x, ints, [x, x]) == 0, dt
    b = torch.zeros(100, dtype=torch.bool)
    assert _bc(ct, torch.zeros(100, dtype=torch.int64), "add(shl(a0,a1),mul_hi(a0,a0))", [b, torch.zeros(100, dtype=torch.int32)]) == 0
    preds = "xor(a0,not(a0))"
    for t in [f"{n}(a1,a1)" for n in "lt le gt ge eq ne".split()] + [f"{n}(a1)" for n in "isnan isinf isfinite signbit iszero bool".split()]:
        preds = f"and({preds},{t})"
    assert _bc(ct, b, preds, [b, f32(100)]) == 0
    assert _bc(ct, f32(100), "f32(i64(i32(f16(bf16(f64(bool(ifelse(a0,a1,a1))))))))", [b, f32(100)]) == 0
    assert T.compile_count() > n0
    again = T.compile_count()
    assert _bc(ct, f32(1024), "add(a0,a1)", [f32(1024), f32(1024)]) == 0          # cached
    assert T.compile_count() == again


def _mr(ct, dest, src, f, op, scalars=()):
    d, s = T._descriptor(dest), T._descriptor(src)
    need = ctypes.c_int64(-1)
    assert ct.lib().mi_tiled_mapreduce_workspace(ctypes.byref(d), ctypes.byref(s), op, ctypes.byref(need)) == 0
    flat = T._Flat()
    flat.scalars = [T._scalar(x) for x in scalars]
    rc = ct.lib().mi_tiled_mapreduce(ctypes.byref(d), ctypes.byref(s), f.encode() if f else None, flat.scalar_array(),
                                     len(flat.scalars), op, ctypes.c_void_p(4096 if need.value else 0), need.value, None)
    return rc, need.value


def test_generated_reduction_kernels_compile(ct, dry_run):
    z = torch.zeros
    rc, ws = _mr(ct, z(1), z(1024), None, T.MI_OP_ADD)
    assert rc == 0 and ws == 0 and ct.last_variant().startswith("tiled_mr_run_l256")
    rc, ws = _mr(ct, z(1), z(1 << 24), None, T.MI_OP_ADD)
    assert rc == 0 and ws > 0 and ws % 4 == 0 and "split" in ct.last_variant()
    rc, ws = _mr(ct, z(256, 1), z(256, 128), None, T.MI_OP_ADD)             # Julia dims=1
    assert rc == 0 and ws == 0 and "run" in ct.last_variant()
    rc, ws = _mr(ct, z(1, 4096), z(100000, 4096), None, T.MI_OP_MAX)         # Julia dims=2
    assert rc == 0 and ws > 0 and ws % (4096 * 4) == 0 and "column" in ct.last_variant()
    rc, _ = _mr(ct, z(1, 16, 1), z(8, 16, 32), "abs2(a0)", T.MI_OP_ADD)      # Julia dims=(1,3)
    assert rc == 0
    rc, ws = _mr(ct, z(1 << 20, 1), z(1 << 20, 8), None, T.MI_OP_ADD)        # short runs: one lane per output
    assert rc == 0 and ws == 0 and ct.last_variant().startswith("tiled_mr_run_l1_")
    rc, _ = _mr(ct, z(8, 1, 32), z(8, 16, 32), None, T.MI_OP_MIN)            # Julia dims=2
    assert rc == 0 and "column" in ct.last_variant()
    for dt, op in ((torch.int32, T.MI_OP_MUL), (torch.int64, T.MI_OP_AND), (torch.bool, T.MI_OP_OR), (torch.float64, T.MI_OP_MIN),
                   (torch.float16, T.MI_OP_ADD), (torch.bfloat16, T.MI_OP_MAX)):
        rc, _ = _mr(ct, z(1, dtype=dt), z(1 << 20, dtype=dt), None, op)
        assert rc == 0, dt
        rc, _ = _mr(ct, z(1, 64, dtype=dt), z(1 << 14, 64, dtype=dt), None, op)
        assert rc == 0, dt
    rc, _ = _mr(ct, z(1, dtype=torch.bool), z(3000), "gt(a0,s0)", T.MI_OP_OR, [np.float32(0.5)])
    assert rc == 0
    rc, _ = _mr(ct, z(17, dtype=torch.int32), z(17, dtype=torch.int32), None, T.MI_OP_MUL)      # no reduced dimension: map
    assert rc == 0
    d, s = T._descriptor(z(7)), T._descriptor(z(64, 128))
    need = ctypes.c_int64()
    assert ct.lib().mi_tiled_mapreduce_workspace(ctypes.byref(d), ctypes.byref(s), 0, ctypes.byref(need)) == ct.MI_E_SHAPE
    d, s = T._descriptor(z(1)), T._descriptor(z(1024))
    assert ct.lib().mi_tiled_mapreduce(ctypes.byref(d), ctypes.byref(s), None, None, 0, 17, None, 0, None) == ct.MI_E_ARG
