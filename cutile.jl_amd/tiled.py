"""Host-level ``Tiled`` broadcast and mapreduce: the Python mirror of cuTile.jl's array-level API
(reference: src/tiled.jl, src/broadcast.jl, src/mapreduce.jl) over ``mi_tiled_broadcast`` and
``mi_tiled_mapreduce``.

Julia writes ``ct.Tiled(C) .= ct.Tiled(A) .+ sin.(ct.Tiled(B))``; the dotted call builds a lazy
``Broadcasted`` tree and ``materialize!`` launches one fused kernel.  Python has no dot syntax, so
the operators of :class:`Tiled` / :class:`Broadcasted` build the same lazy tree and the three ways
to run it are spelled out::

    Tiled(C).assign(Tiled(A) + sin(Tiled(B)))      # Tiled(C) .= ...   -> returns C
    D = (Tiled(A) + Tiled(B)).copy()               # D = Tiled(A) .+ Tiled(B)  (allocates)
    dot("C = A + sin(B)", C=C, A=A, B=B)           # ct.@. C = A + sin(B)

Arrays follow the package convention: a Julia array of shape (d1, ..., dn) is a torch tensor of shape
(dn, ..., d1).  ``dims`` arguments are Julia's (1-based, dimension 1 contiguous).  Python numbers
map to Julia's defaults (``float`` -> Float64, ``int`` -> Int64, ``bool`` -> Bool); use
``numpy.float32(1)`` for ``1f0``.  Nothing here computes on the CPU: trees are handed to the shared
library as text and run as one generated gfx950 kernel.
"""
from __future__ import annotations

import ast
import builtins as _b
import ctypes
import numbers
import operator

import numpy as np

from . import (MI_BF16, MI_F16, MI_F32, MI_F64, MI_I32, MI_I64, MiError, MiTileArray, TileArray, _call, _stream,
               lib, MI_E_SHAPE)

MI_BOOL = 7
MI_OP_ADD, MI_OP_MUL, MI_OP_MAX, MI_OP_MIN, MI_OP_AND, MI_OP_OR = range(6)


class ArgumentError(ValueError):
    """Julia's ArgumentError."""


class DimensionMismatch(ValueError):
    """Julia's DimensionMismatch."""


class InexactError(OverflowError):
    """Julia's InexactError."""


class MiTileScalar(ctypes.Structure):
    """ctypes mirror of ``mi_tile_scalar``."""

    class _V(ctypes.Union):
        _fields_ = [("f", ctypes.c_double), ("i", ctypes.c_int64)]

    _fields_ = [("dtype", ctypes.c_int32), ("reserved", ctypes.c_int32), ("value", _V)]


def _torch_dtype(code: int):
    import torch
    return {MI_F32: torch.float32, MI_F64: torch.float64, MI_F16: torch.float16, MI_BF16: torch.bfloat16,
            MI_I32: torch.int32, MI_I64: torch.int64, MI_BOOL: torch.bool}[code]


def _array_dtype_code(t) -> int:
    import torch
    table = {torch.float32: MI_F32, torch.float64: MI_F64, torch.float16: MI_F16, torch.bfloat16: MI_BF16,
             torch.int32: MI_I32, torch.int64: MI_I64, torch.bool: MI_BOOL}
    try:
        return table[t.dtype]
    except KeyError:
        raise TypeError(f"Tiled: unsupported element type {t.dtype}") from None


def _scalar(x) -> MiTileScalar:
    s = MiTileScalar()
    if isinstance(x, (bool, np.bool_)):
        s.dtype, s.value.i = MI_BOOL, int(bool(x))
    elif isinstance(x, np.float32):
        s.dtype, s.value.f = MI_F32, float(x)
    elif isinstance(x, np.float16):
        s.dtype, s.value.f = MI_F16, float(x)
    elif isinstance(x, np.int32):
        s.dtype, s.value.i = MI_I32, int(x)
    elif isinstance(x, (int, np.int64)):
        if not -2**63 <= int(x) < 2**63:
            raise InexactError("integer scalar does not fit Int64")
        s.dtype, s.value.i = MI_I64, int(x)
    elif isinstance(x, (float, np.float64)):
        s.dtype, s.value.f = MI_F64, float(x)
    else:
        raise TypeError(f"Tiled broadcast: unsupported scalar {type(x).__name__}")
    return s


def _descriptor(t) -> MiTileArray:
    return TileArray(t, dtype=_array_dtype_code(t))


# ---- lazy tree ---------------------------------------------------------------------------------

class _Node:
    """Operators shared by Tiled and Broadcasted: every one builds a Broadcasted node."""

    def __add__(self, o): return Broadcasted("add", self, o)
    def __radd__(self, o): return Broadcasted("add", o, self)
    def __sub__(self, o): return Broadcasted("sub", self, o)
    def __rsub__(self, o): return Broadcasted("sub", o, self)
    def __mul__(self, o): return Broadcasted("mul", self, o)
    def __rmul__(self, o): return Broadcasted("mul", o, self)
    def __truediv__(self, o): return Broadcasted("div", self, o)
    def __rtruediv__(self, o): return Broadcasted("div", o, self)
    def __floordiv__(self, o): return Broadcasted("fld", self, o)
    def __rfloordiv__(self, o): return Broadcasted("fld", o, self)
    def __mod__(self, o): return Broadcasted("mod", self, o)
    def __rmod__(self, o): return Broadcasted("mod", o, self)
    def __pow__(self, o): return Broadcasted("pow", self, o)
    def __rpow__(self, o): return Broadcasted("pow", o, self)
    def __neg__(self): return Broadcasted("neg", self)
    def __pos__(self): return Broadcasted("identity", self)
    def __abs__(self): return Broadcasted("abs", self)
    def __invert__(self): return Broadcasted("not", self)
    def __and__(self, o): return Broadcasted("and", self, o)
    def __rand__(self, o): return Broadcasted("and", o, self)
    def __or__(self, o): return Broadcasted("or", self, o)
    def __ror__(self, o): return Broadcasted("or", o, self)
    def __xor__(self, o): return Broadcasted("xor", self, o)
    def __rxor__(self, o): return Broadcasted("xor", o, self)
    def __lshift__(self, o): return Broadcasted("shl", self, o)
    def __rlshift__(self, o): return Broadcasted("shl", o, self)
    def __rshift__(self, o): return Broadcasted("shr", self, o)      # arithmetic, like Julia's >> on signed integers
    def __rrshift__(self, o): return Broadcasted("shr", o, self)
    def __lt__(self, o): return Broadcasted("lt", self, o)
    def __le__(self, o): return Broadcasted("le", self, o)
    def __gt__(self, o): return Broadcasted("gt", self, o)
    def __ge__(self, o): return Broadcasted("ge", self, o)
    def __eq__(self, o): return Broadcasted("eq", self, o)      # element-wise, like Julia's .==
    def __ne__(self, o): return Broadcasted("ne", self, o)
    __hash__ = None


class Tiled(_Node):
    """``ct.Tiled(x)``: marks an array so that broadcasts and reductions over it run as generated
    kernels (reference: src/tiled.jl:8-17).  Numbers pass through unchanged."""

    def __new__(cls, x):
        if isinstance(x, (numbers.Number, np.generic)):
            return x
        if isinstance(x, Tiled):
            return x
        return super().__new__(cls)

    def __init__(self, x):
        if isinstance(x, Tiled):
            return
        self.parent = x

    @property
    def shape(self):
        """Julia shape (dimension 1 first)."""
        return tuple(reversed(self.parent.shape))

    def assign(self, rhs):
        """``Tiled(dest) .= rhs``; returns the destination array (src/broadcast.jl:20-24)."""
        return materialize(self, rhs)

    def copy(self):
        return Broadcasted("identity", self).copy()


class Broadcasted(_Node):
    """A lazy element-wise call, the analogue of Base.Broadcast.Broadcasted."""

    def __init__(self, fn: str, *args):
        self.fn = fn
        self.args = args

    def copy(self):
        """Allocating form: ``C = Tiled(A) .+ Tiled(B)`` (src/broadcast.jl:26-32)."""
        return copy(self)


class _Arg(_Node):
    """The element ``x`` a mapreduce function is applied to."""


def _fn(name, arity):
    def call(*args):
        if len(args) != arity:
            raise TypeError(f"{name} takes {arity} argument(s)")
        return Broadcasted(name, *args)
    call.__name__ = name
    call.__doc__ = f"Element-wise ``{name}`` node of a Tiled broadcast."
    return call


_UNARY = ("abs abs2 sign floor ceil round trunc sqrt rsqrt cbrt inv exp exp2 exp10 expm1 log log2 log10 log1p sin cos "
          "tan asin acos atan sinh cosh tanh isnan isinf isfinite signbit iszero identity").split()
_BINARY = "max min copysign atan2 hypot rem mod fld cld mul_hi lshr".split()   # lshr: Julia's >>>
for _n in _UNARY:
    globals()[_n] = _fn(_n, 1)
for _n in _BINARY:
    globals()[_n] = _fn(_n, 2)
fma = _fn("fma", 3)
muladd = _fn("muladd", 3)
clamp = _fn("clamp", 3)
ifelse = _fn("ifelse", 3)
div = _fn("div_int", 2)      # Julia's `div` / `÷`
Float16, BFloat16, Float32, Float64 = _fn("f16", 1), _fn("bf16", 1), _fn("f32", 1), _fn("f64", 1)
Int32, Int64, Bool = _fn("i32", 1), _fn("i64", 1), _fn("bool", 1)

_FUNCTIONS = {n: globals()[n] for n in _UNARY + _BINARY}
_FUNCTIONS.update(fma=fma, muladd=muladd, clamp=clamp, ifelse=ifelse, div=div, Float16=Float16, BFloat16=BFloat16,
                  Float32=Float32, Float64=Float64, Int32=Int32, Int64=Int64, Bool=Bool)


class _Flat:
    """Text form of a tree plus its leaves and scalars, in first-use order."""

    def __init__(self):
        self.leaves, self.scalars = [], []

    def text(self, node) -> str:
        if isinstance(node, Broadcasted):
            return node.fn + "(" + ",".join(self.text(a) for a in node.args) + ")"
        if isinstance(node, _Arg):
            return "a0"
        if isinstance(node, Tiled):
            for i, t in enumerate(self.leaves):
                if t is node.parent:
                    return f"a{i}"
            self.leaves.append(node.parent)
            return f"a{len(self.leaves) - 1}"
        if isinstance(node, (numbers.Number, np.generic)):
            self.scalars.append(_scalar(node))
            return f"s{len(self.scalars) - 1}"
        # A bare array inside a Tiled broadcast takes part like a Tiled one (TiledStyle wins,
        # src/broadcast.jl:10-14); anything without device storage is rejected below.
        if hasattr(node, "data_ptr"):
            return self.text(Tiled(node))
        raise TypeError(f"Tiled broadcast: leaf of type {type(node).__name__} has no device storage")

    def scalar_array(self):
        arr = (MiTileScalar * _b.max(1, len(self.scalars)))()
        for i, s in enumerate(self.scalars):
            arr[i] = s
        return arr


def _check_device(t, what: str):
    if not hasattr(t, "is_cuda") or not t.is_cuda:
        raise ArgumentError(f"Tiled broadcast: {what} must be a device array")


def _broadcast_shape(shapes):
    """Julia's Base.Broadcast.combine_axes on Julia-ordered shapes."""
    rank = _b.max((len(s) for s in shapes), default=0)
    out = []
    for d in range(rank):
        ext = 1
        for s in shapes:
            v = s[d] if d < len(s) else 1
            if v != 1:
                if ext != 1 and ext != v:
                    raise DimensionMismatch(f"arrays could not be broadcast to a common size: {ext} and {v} in dimension {d + 1}")
                ext = v
        out.append(ext)
    return tuple(out)


def _launch_broadcast(dest, flat: _Flat, text: str, stream=None):
    _check_device(dest, "the destination")
    for t in flat.leaves:
        _check_device(t, "every array leaf")
    dshape = tuple(reversed(dest.shape))
    for t in flat.leaves:   # Base.Broadcast.check_broadcast_axes
        ls = tuple(reversed(t.shape))
        for d in range(_b.max(len(ls), len(dshape))):
            v = ls[d] if d < len(ls) else 1
            w = dshape[d] if d < len(dshape) else 1
            if v != 1 and v != w:
                raise DimensionMismatch(f"destination axes {dshape} are not compatible with source axes {ls}")
    descs = [_descriptor(t) for t in flat.leaves]
    ptrs = (ctypes.POINTER(MiTileArray) * _b.max(1, len(descs)))(*[ctypes.pointer(d) for d in descs])
    d = _descriptor(dest)
    _call("mi_tiled_broadcast", ctypes.byref(d), text.encode(), ptrs, len(descs), flat.scalar_array(), len(flat.scalars),
          _stream(stream))


def materialize(dest, rhs, stream=None):
    """``Tiled(dest) .= rhs`` -- one fused kernel; returns the destination array."""
    arr = dest.parent if isinstance(dest, Tiled) else dest
    flat = _Flat()
    text = flat.text(rhs)
    _launch_broadcast(arr, flat, text, stream)
    return arr


def eltype(bc) -> int:
    """mi_dtype code of a tree's element type (Base.Broadcast.combine_eltypes)."""
    flat = _Flat()
    text = flat.text(bc)
    return _eltype(flat, text)


def _eltype(flat: _Flat, text: str) -> int:
    ld = (ctypes.c_int32 * _b.max(1, len(flat.leaves)))(*[_array_dtype_code(t) for t in flat.leaves])
    sd = (ctypes.c_int32 * _b.max(1, len(flat.scalars)))(*[s.dtype for s in flat.scalars])
    out = ctypes.c_int32()
    _call("mi_tiled_broadcast_eltype", text.encode(), ld, len(flat.leaves), sd, len(flat.scalars), ctypes.byref(out))
    return out.value


def copy(bc, stream=None):
    """Allocating broadcast: the result is `similar` to the first Tiled leaf (src/broadcast.jl:26-43)."""
    import torch
    flat = _Flat()
    text = flat.text(bc)
    if not flat.leaves:
        raise ArgumentError("tiled broadcast requires at least one Tiled() argument")
    for t in flat.leaves:
        _check_device(t, "every array leaf")
    shape = _broadcast_shape([tuple(reversed(t.shape)) for t in flat.leaves])
    dest = torch.empty(tuple(reversed(shape)), dtype=_torch_dtype(_eltype(flat, text)), device=flat.leaves[0].device)
    _launch_broadcast(dest, flat, text, stream)
    return dest


# ---- ct.@. ---------------------------------------------------------------------------------------

_BINOPS = {ast.Add: operator.add, ast.Sub: operator.sub, ast.Mult: operator.mul, ast.Div: operator.truediv,
           ast.Pow: operator.pow, ast.Mod: operator.mod, ast.FloorDiv: operator.floordiv, ast.BitAnd: operator.and_,
           ast.BitOr: operator.or_, ast.BitXor: operator.xor, ast.LShift: operator.lshift, ast.RShift: operator.rshift}
_CMPOPS = {ast.Lt: operator.lt, ast.LtE: operator.le, ast.Gt: operator.gt, ast.GtE: operator.ge, ast.Eq: operator.eq,
           ast.NotEq: operator.ne}


def _build(node, env):
    if isinstance(node, ast.BinOp) and type(node.op) in _BINOPS:
        return _BINOPS[type(node.op)](_build(node.left, env), _build(node.right, env))
    if isinstance(node, ast.UnaryOp):
        v = _build(node.operand, env)
        if isinstance(node.op, ast.USub):
            return -v
        if isinstance(node.op, ast.UAdd):
            return v
        if isinstance(node.op, ast.Invert):
            return ~v
    if isinstance(node, ast.Compare) and len(node.ops) == 1 and type(node.ops[0]) in _CMPOPS:
        return _CMPOPS[type(node.ops[0])](_build(node.left, env), _build(node.comparators[0], env))
    if isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and not node.keywords:
        f = _FUNCTIONS.get(node.func.id)
        if f is None:
            raise NameError(f"dot: unknown function {node.func.id}")
        return f(*[_build(a, env) for a in node.args])
    if isinstance(node, ast.Name):
        if node.id not in env:
            raise NameError(f"dot: {node.id} is not among the keyword arguments")
        return Tiled(env[node.id])        # every value-position leaf is wrapped (src/broadcast.jl:134-147)
    if isinstance(node, ast.Constant) and isinstance(node.value, (int, float, bool)):
        return node.value
    raise SyntaxError("dot: unsupported syntax " + ast.dump(node))


def dot(expr: str, stream=None, **arrays):
    """``ct.@. expr`` (src/broadcast.jl:149-165): every name in ``expr`` is looked up in the keyword
    arguments and wrapped in Tiled; ``"C = A + sin(B)"`` assigns in place and returns C, an
    expression without ``=`` allocates.  Function names are those of this module."""
    tree = ast.parse(expr.strip(), mode="exec").body
    if len(tree) != 1:
        raise SyntaxError("dot: one statement expected")
    st = tree[0]
    if isinstance(st, ast.Assign) and len(st.targets) == 1 and isinstance(st.targets[0], ast.Name):
        dest = arrays[st.targets[0].id]
        return materialize(Tiled(dest), _build(st.value, arrays), stream)
    if isinstance(st, ast.Expr):
        rhs = _build(st.value, arrays)
        return copy(rhs if isinstance(rhs, Broadcasted) else Broadcasted("identity", rhs), stream)
    raise SyntaxError("dot: `dest = expression` or an expression expected")


# ---- mapreduce -------------------------------------------------------------------------------------

def _op_code(op):
    """(operator code, widen flag, host function) for Julia's op."""
    table = {
        "+": (MI_OP_ADD, 0, operator.add), "add_sum": (MI_OP_ADD, 1, operator.add),
        "*": (MI_OP_MUL, 0, operator.mul), "mul_prod": (MI_OP_MUL, 1, operator.mul),
        "max": (MI_OP_MAX, 0, _b.max), "min": (MI_OP_MIN, 0, _b.min),
        "&": (MI_OP_AND, 0, operator.and_), "|": (MI_OP_OR, 0, operator.or_),
    }
    alias = {operator.add: "+", operator.mul: "*", _b.max: "max", _b.min: "min", operator.and_: "&",
             operator.or_: "|"}
    key = op if isinstance(op, str) else alias.get(op)
    if key not in table:
        raise ArgumentError(f"mapreduce: unsupported reduction operator {op!r}")
    return table[key]


_OP_NODE = {MI_OP_ADD: "add", MI_OP_MUL: "mul", MI_OP_MAX: "max", MI_OP_MIN: "min", MI_OP_AND: "and", MI_OP_OR: "or"}


def _f_text(f):
    flat = _Flat()
    if f is None or f is identity:
        return None, flat
    tree = f(_Arg())
    text = flat.text(tree)
    if flat.leaves:
        raise ArgumentError("mapreduce: the mapped function may only use its argument and numbers")
    return text, flat


def _region(dims, ndim):
    """Julia's normalisation of `dims` (src/mapreduce.jl:143-151)."""
    if dims is None:
        return tuple(range(1, ndim + 1))
    if isinstance(dims, (numbers.Integral, np.integer)) and not isinstance(dims, bool):
        region = (dims,)
    elif isinstance(dims, numbers.Number):
        raise ArgumentError("reduced dimension(s) must be integers")
    else:
        region = tuple(dims)
    for d in region:
        if isinstance(d, bool) or not isinstance(d, (numbers.Integral, np.integer)):
            raise ArgumentError("reduced dimension(s) must be integers")
        if int(d) >= 2**63:
            raise InexactError(f"dimension {d} does not fit Int")
        if int(d) < 1:
            raise ArgumentError(f"region dimension(s) must be ≥ 1, got {d}")
    return tuple(d for d in range(1, ndim + 1) if d in region)


def _run_mapreduce(R, A, f_text, flat, code, stream=None):
    import torch
    d, s = _descriptor(R), _descriptor(A)
    need = ctypes.c_int64()
    _call("mi_tiled_mapreduce_workspace", ctypes.byref(d), ctypes.byref(s), code, ctypes.byref(need))
    ws = torch.empty(need.value, dtype=torch.uint8, device=A.device) if need.value else None
    _call("mi_tiled_mapreduce", ctypes.byref(d), ctypes.byref(s), None if f_text is None else f_text.encode(),
          flat.scalar_array(), len(flat.scalars), code, ctypes.c_void_p(ws.data_ptr() if ws is not None else 0),
          need.value, _stream(stream))


def mapreduce(f, op, A, dims=None, init=None, stream=None):
    """``mapreduce(f, op, Tiled(A); dims, init)`` (src/mapreduce.jl:131-172).  ``f`` is None /
    ``identity`` or a function of one element built from this module's functions and operators;
    ``op`` one of "+", "*", "max", "min", "&", "|" (or "add_sum" / "mul_prod", which widen small
    integers as Julia's ``sum`` / ``prod`` do).  Returns a number for ``dims=None`` (Julia's ``:``),
    otherwise an array whose reduced dimensions have extent 1."""
    import torch
    arr = A.parent if isinstance(A, Tiled) else A
    _check_device(arr, "the reduced array")
    code, widen, host_op = _op_code(op)
    f_text, flat = _f_text(f)
    sd = (ctypes.c_int32 * _b.max(1, len(flat.scalars)))(*[s.dtype for s in flat.scalars])
    et = ctypes.c_int32()
    _call("mi_tiled_mapreduce_eltype", None if f_text is None else f_text.encode(), _array_dtype_code(arr), sd,
          len(flat.scalars), code, widen, ctypes.byref(et))
    jshape = tuple(reversed(arr.shape))
    red = _region(dims, len(jshape))
    out_shape = tuple(1 if (d + 1) in red else jshape[d] for d in range(len(jshape)))
    R = torch.empty(tuple(reversed(out_shape)), dtype=_torch_dtype(et.value), device=arr.device)
    _run_mapreduce(R, arr, f_text, flat, code, stream)
    if dims is None:
        value = R.reshape(-1)[0].item()
        if init is not None:
            value = host_op(type(value)(init), value)
        return value
    if init is not None:
        node = Broadcasted(_OP_NODE[code], _cast_scalar(init, et.value), Tiled(R))
        materialize(Tiled(R), node, stream)
    return R


def _cast_scalar(x, code):
    return {MI_F32: np.float32, MI_F64: float, MI_F16: np.float16, MI_BF16: np.float32, MI_I32: np.int32, MI_I64: int,
            MI_BOOL: bool}[code](x)


def reduce(op, A, dims=None, init=None, stream=None):
    """``reduce(op, Tiled(A); dims, init)`` (src/mapreduce.jl:177-178)."""
    return mapreduce(None, op, A, dims=dims, init=init, stream=stream)


def sum(A, dims=None, init=None, stream=None):          # noqa: A001 - mirrors Base.sum
    return mapreduce(None, "add_sum", A, dims=dims, init=init, stream=stream)


def prod(A, dims=None, init=None, stream=None):
    return mapreduce(None, "mul_prod", A, dims=dims, init=init, stream=stream)


def maximum(A, dims=None, init=None, stream=None):
    return mapreduce(None, "max", A, dims=dims, init=init, stream=stream)


def minimum(A, dims=None, init=None, stream=None):
    return mapreduce(None, "min", A, dims=dims, init=init, stream=stream)


def _require_bool(A, f):
    import torch
    arr = A.parent if isinstance(A, Tiled) else A
    if f is None and arr.dtype != torch.bool:
        raise TypeError("any / all without a predicate need a Bool array")


def any(A, f=None, dims=None, stream=None):             # noqa: A001 - mirrors Base.any
    """``any(Tiled(A))`` / ``any(f, Tiled(A))`` (src/mapreduce.jl:181-188)."""
    _require_bool(A, f)
    return mapreduce(f, "|", A, dims=dims, stream=stream)


def all(A, f=None, dims=None, stream=None):             # noqa: A001 - mirrors Base.all
    _require_bool(A, f)
    return mapreduce(f, "&", A, dims=dims, stream=stream)


def count(A, f=None, dims=None, stream=None):
    """``count(Tiled(A))``: number of true elements (Int64)."""
    _require_bool(A, f)
    return mapreduce(f, "add_sum", A, dims=dims, stream=stream)


def _inplace(code_name, R, A, stream=None):
    """``sum!(R, Tiled(A))`` and friends: the reduced dimensions are those where R has extent 1 and
    A has not (src/mapreduce.jl:191-203)."""
    arr = A.parent if isinstance(A, Tiled) else A
    _check_device(arr, "the reduced array")
    _check_device(R, "the destination")
    code, _, _ = _op_code(code_name)
    try:
        _run_mapreduce(R, arr, None, _Flat(), code, stream)
    except MiError as e:
        if e.code == MI_E_SHAPE:
            raise DimensionMismatch("destination and source sizes do not agree") from None
        raise
    return R


def sum_(R, A, stream=None):
    return _inplace("+", R, A, stream)


def prod_(R, A, stream=None):
    return _inplace("*", R, A, stream)


def maximum_(R, A, stream=None):
    return _inplace("max", R, A, stream)


def minimum_(R, A, stream=None):
    return _inplace("min", R, A, stream)


def set_dry_run(on: bool) -> bool:
    """Compile-only mode of the two entry points (no GPU needed); returns the previous setting."""
    return bool(lib().mi_tiled_set_dry_run(1 if on else 0))


def compile_count() -> int:
    return lib().mi_tiled_compile_count()
