"""Host side of libmi355tile: hand-written gfx950 (MI355X) HIP kernels behind a C ABI that
stand in for the kernels cuTile.jl's examples compile through Tile IR.

The directory name contains a dot, so the package is imported under the module name
``cutile_jl_amd`` (see ``__graft_entry__.load_package``).  Nothing here computes on the
CPU: every kernel wrapper calls the shared library and raises if it is missing.

Array convention.  The reference's arrays are Julia column-major arrays.  A Julia array of
shape ``(d1, d2, ..., dn)`` is held here as a ``torch`` tensor of shape ``(dn, ..., d2, d1)``
in row-major order, which is the same memory.  :func:`TileArray` turns such a tensor (or a
strided view of one) into the descriptor the C ABI takes, with sizes and strides listed in
the Julia order, mirroring ``ct.TileArray(arr)`` (reference: src/language/types.jl:350-357).
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI355TILE_LIB selects another build of the same library (e.g. an experimental variant).
LIB_PATH = os.environ.get("MI355TILE_LIB") or os.path.join(_HERE, "libmi355tile.so")

MI_F32, MI_F64, MI_F16, MI_BF16, MI_F8E4M3FN, MI_I32, MI_I64, MI_BOOL, MI_I8, MI_I16, MI_F8E5M2 = range(11)
MI_MAX_RANK = 4

# error codes of include/mi355tile.h
MI_OK = 0
MI_E_NULL, MI_E_DTYPE, MI_E_RANK, MI_E_SHAPE, MI_E_STRIDE = -1, -2, -3, -4, -5
MI_E_TILE, MI_E_GRID, MI_E_ALIGN, MI_E_ARG, MI_E_UNSUPPORTED, MI_E_SCRATCH = -6, -7, -8, -9, -10, -11


class MiTileArray(ctypes.Structure):
    """ctypes mirror of ``mi_tile_array`` (include/mi355tile.h)."""

    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("ndim", ctypes.c_int32),
        ("sizes", ctypes.c_int64 * MI_MAX_RANK),
        ("strides", ctypes.c_int64 * MI_MAX_RANK),
    ]


class MiError(RuntimeError):
    """A libmi355tile entry point returned a non-zero status."""

    def __init__(self, fn: str, code: int, msg: str):
        super().__init__(f"{fn} failed with status {code}: {msg}")
        self.code = code


_A = ctypes.POINTER(MiTileArray)
_i = ctypes.c_int
_vp = ctypes.c_void_p
_SIGNATURES = {
    "mi_version": ([], ctypes.c_int),
    "mi_strerror": ([_i], ctypes.c_char_p),
    "mi_last_variant": ([], ctypes.c_char_p),
    "mi_vec_add_kernel_1d": ([_A, _A, _A, _i, _vp], _i),
    "mi_vec_add_kernel_2d": ([_A, _A, _A, _i, _i, _vp], _i),
    "mi_vec_add_kernel_1d_gather": ([_A, _A, _A, _i, _vp], _i),
    "mi_transpose_kernel": ([_A, _A, _i, _i, _vp], _i),
    "mi_matmul_kernel": ([_A, _A, _A, _i, _i, _i, _vp], _i),
    "mi_batch_matmul_kernel": ([_A, _A, _A, _i, _i, _i, _vp], _i),
    "mi_swizzle_2d": ([ctypes.c_int32] * 6 + [ctypes.POINTER(ctypes.c_int32)] * 2, None),
    "mi_layer_norm_fwd": ([_A, _A, _A, _A, _A, _A, ctypes.c_float, _i, _vp], _i),
    "mi_layer_norm_bwd_dx_partial_dwdb": ([_A] * 9 + [_i, _i, _vp], _i),
    "mi_layer_norm_bwd_dwdb": ([_A, _A, _A, _A, _i, _i, _vp], _i),
    "mi_layer_norm_bwd_static": ([_A] * 8 + [_i, _i, _i, _vp], _i),
    "mi_softmax_tma_kernel": ([_A, _A, _i, _i, _vp], _i),
    "mi_softmax_chunked_kernel": ([_A, _A, _i, _i, _i, _vp], _i),
    "mi_fmha_kernel": ([_A, _A, _A, _A, ctypes.c_float, ctypes.c_int32, _i, _i, _i, _i, _i, _i, _i, _vp], _i),
    "mi_fft_kernel": ([_A, _A, _A, _A, _A, _A, _A, _i, _i, _i, _i, _i, _i, _vp], _i),
    "mi_moe_align_tile_size_device": ([_A, _i, _i, _A, _A, _vp], _i),
    "mi_moe_align_tile_size_device_clear": ([_A, _i, _i, _A, _A, _A, _vp], _i),
    "mi_moe_route_topk": ([_A, _A, _A, _vp], _i),
    "mi_moe_align_tile_size": (
        [ctypes.POINTER(ctypes.c_int64), ctypes.c_int64, ctypes.c_int64, _i, _i,
         ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32),
         ctypes.POINTER(ctypes.c_int64)], _i),
    "mi_fused_moe_kernel": ([_A] * 6 + [_i, _i, _i, _i, _i, _A, _vp], _i),
    "mi_fused_moe_silu_kernel": ([_A] * 6 + [_i, _i, _i, _i, _i, _A, _vp], _i),
    "mi_fused_moe_accumulate_kernel": ([_A] * 6 + [_i, _i, _i, _A, _vp], _i),
    "mi_silu_and_mul_kernel": ([_A, _A, _A, _i, _vp], _i),
    "mi_moe_sum_topk": ([_A, _A, _vp], _i),
    "mi_scratch_under_capture": ([_i], _i),
    "mi_quantize_e4m3fn": ([_A, _A, _A, _A, _vp], _i),
    "mi_quantize_e4m3fn_fold": ([_A, _A, _A, _A, _A, _A, _vp], _i),
    "mi_tiled_broadcast": ([_A, ctypes.c_char_p, ctypes.POINTER(_A), _i, _vp, _i, _vp], _i),
    "mi_tiled_broadcast_eltype": ([ctypes.c_char_p, ctypes.POINTER(ctypes.c_int32), _i,
                                   ctypes.POINTER(ctypes.c_int32), _i, ctypes.POINTER(ctypes.c_int32)], _i),
    "mi_tiled_mapreduce": ([_A, _A, ctypes.c_char_p, _vp, _i, _i, _vp, ctypes.c_int64, _vp], _i),
    "mi_tiled_mapreduce_workspace": ([_A, _A, _i, ctypes.POINTER(ctypes.c_int64)], _i),
    "mi_tiled_mapreduce_eltype": ([ctypes.c_char_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_int32), _i, _i, _i,
                                   ctypes.POINTER(ctypes.c_int32)], _i),
    "mi_rng_fill": ([_A, ctypes.c_uint32, ctypes.c_uint32, _i, _vp], _i),
    "mi_rng_advance_counter": ([ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32), ctypes.c_int64], _i),
    "mi_tiled_set_dry_run": ([_i], _i),
    "mi_tiled_compile_count": ([], _i),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def lib() -> ctypes.CDLL:
    """Load libmi355tile.so (built in-tree by ``__graft_entry__.build``).  Raises if absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(or python -c 'import __graft_entry__ as g; g.build()'). There is no CPU fallback.")
        # torch ships its own HIP runtime with the same soname; importing it first makes the
        # kernels and torch's allocator share one runtime (and therefore streams).
        import torch  # noqa: F401
        cdll = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(cdll, name)  # AttributeError if the library lacks a declared symbol
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = cdll
    return _lib


def strerror(code: int) -> str:
    return lib().mi_strerror(code).decode()


def scratch_under_capture(allow: bool) -> bool:
    """Hand the library's shared static arrays to capturing streams as well (see ``mi_scratch_under_capture``): the
    caller keeps replays of such graphs apart from one another and from other launches that use the arrays.  Returns
    the previous setting."""
    return bool(lib().mi_scratch_under_capture(1 if allow else 0))


def last_variant() -> str:
    return lib().mi_last_variant().decode()


_DTYPE_CODES = None   # torch dtype -> MI_* code, filled on first use (torch is imported lazily)


def _dtype_code(t) -> int:
    global _DTYPE_CODES
    if _DTYPE_CODES is None:
        import torch
        _DTYPE_CODES = {
            torch.float32: MI_F32, torch.float64: MI_F64, torch.float16: MI_F16,
            torch.bfloat16: MI_BF16, torch.int32: MI_I32, torch.int64: MI_I64,
            torch.float8_e4m3fn: MI_F8E4M3FN, torch.float8_e5m2: MI_F8E5M2,
        }
    try:
        return _DTYPE_CODES[t]
    except KeyError:
        raise TypeError(f"unsupported dtype {t}") from None


_I64x4 = ctypes.c_int64 * MI_MAX_RANK


def TileArray(t, dtype: int | None = None) -> MiTileArray:
    """Descriptor for a torch tensor holding a Julia array in reversed-shape row-major form."""
    n = t.dim()
    if n > MI_MAX_RANK:
        raise ValueError("rank > 4")
    # (one constructor call with ready-made arrays: a third of the time of field-by-field assignment, which matters
    # for a launch of a few microseconds that takes four descriptors)
    return MiTileArray(t.data_ptr(), _dtype_code(t.dtype) if dtype is None else dtype, n,
                       _I64x4(*t.shape[::-1]), _I64x4(*t.stride()[::-1]))


def _stream(stream=None):
    import torch
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _ref(x):
    return None if x is None else ctypes.byref(x if isinstance(x, MiTileArray) else TileArray(x))


def _call(name: str, *args):
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise MiError(name, rc, strerror(rc))


def fft_kernel(x_packed_in, y_packed_out, W0, W1, W2, T0, T1, N: int, F0: int, F1: int, F2: int, BS: int,
               D: int, stream=None):
    """examples/fft.jl:22-126"""
    _call("mi_fft_kernel", _ref(x_packed_in), _ref(y_packed_out), _ref(W0), _ref(W1), _ref(W2), _ref(T0),
          _ref(T1), N, F0, F1, F2, BS, D, _stream(stream))


def bind(name: str, *args, stream=None):
    """Pre-bound launch: converts the arguments of entry point ``name`` once (arrays to descriptors,
    the stream handle) and returns a zero-argument callable that only makes the C call.  For
    launch loops where Python's per-call argument handling would otherwise outweigh a 20 us
    kernel.  ``args`` are the entry point's arguments without the trailing stream."""
    fn = getattr(lib(), name)
    keep = [a if isinstance(a, MiTileArray) or not hasattr(a, "data_ptr") else TileArray(a) for a in args]
    cargs = tuple(ctypes.byref(a) if isinstance(a, MiTileArray) else (int(a) if isinstance(a, bool) else a)
                  for a in keep) + (_stream(stream),)

    def call():
        rc = fn(*cargs)
        if rc != 0:
            raise MiError(name, rc, strerror(rc))
    call._keep = keep
    return call


# ---- kernel wrappers: one per entry point, argument order of the reference kernels --------

def vec_add_kernel_1d(a, b, c, tile: int, stream=None):
    """examples/vadd.jl:10-17"""
    _call("mi_vec_add_kernel_1d", _ref(a), _ref(b), _ref(c), tile, _stream(stream))


def vec_add_kernel_2d(a, b, c, tile_x: int, tile_y: int, stream=None):
    """examples/vadd.jl:20-28"""
    _call("mi_vec_add_kernel_2d", _ref(a), _ref(b), _ref(c), tile_x, tile_y, _stream(stream))


def vec_add_kernel_1d_gather(a, b, c, tile: int, stream=None):
    """examples/vadd.jl:31-45"""
    _call("mi_vec_add_kernel_1d_gather", _ref(a), _ref(b), _ref(c), tile, _stream(stream))


def transpose_kernel(x, y, tm: int, tn: int, stream=None):
    """examples/transpose.jl:11-19"""
    _call("mi_transpose_kernel", _ref(x), _ref(y), tm, tn, _stream(stream))


def matmul_kernel(A, B, C, tm: int, tn: int, tk: int, stream=None):
    """examples/matmul.jl:28-60"""
    _call("mi_matmul_kernel", _ref(A), _ref(B), _ref(C), tm, tn, tk, _stream(stream))


def batch_matmul_kernel(A, B, C, tm: int, tn: int, tk: int, stream=None):
    """examples/batchmatmul.jl:15-56"""
    _call("mi_batch_matmul_kernel", _ref(A), _ref(B), _ref(C), tm, tn, tk, _stream(stream))


def swizzle_2d(M, N, tm, tn, GROUP_SIZE_M, bid):
    """examples/matmul.jl:13-24 — 1-based bid -> 1-based (bid_m, bid_n)."""
    bm, bn = ctypes.c_int32(), ctypes.c_int32()
    lib().mi_swizzle_2d(M, N, tm, tn, GROUP_SIZE_M, bid, ctypes.byref(bm), ctypes.byref(bn))
    return bm.value, bn.value


def layer_norm_fwd(X, W, B, Y, Mean, Rstd, eps: float, TILE_N: int, stream=None):
    """examples/layernorm.jl:27-68"""
    _call("mi_layer_norm_fwd", _ref(X), _ref(W), _ref(B), _ref(Y), _ref(Mean), _ref(Rstd),
          ctypes.c_float(eps), TILE_N, _stream(stream))


def layer_norm_bwd_dx_partial_dwdb(DX, DY, DW, DB, X, W, Mean, Rstd, Locks, GROUP_SIZE_M: int,
                                   TILE_N: int, stream=None):
    """examples/layernorm.jl:118-171"""
    _call("mi_layer_norm_bwd_dx_partial_dwdb", _ref(DX), _ref(DY), _ref(DW), _ref(DB), _ref(X),
          _ref(W), _ref(Mean), _ref(Rstd), _ref(Locks), GROUP_SIZE_M, TILE_N, _stream(stream))


def layer_norm_bwd_dwdb(DW, DB, FINAL_DW, FINAL_DB, TILE_M: int, TILE_N: int, stream=None):
    """examples/layernorm.jl:186-205"""
    _call("mi_layer_norm_bwd_dwdb", _ref(DW), _ref(DB), _ref(FINAL_DW), _ref(FINAL_DB), TILE_M,
          TILE_N, _stream(stream))


def layer_norm_bwd_static(DX, DY, X, W, Mean, Rstd, FINAL_DW, FINAL_DB, GROUP_SIZE_M: int, TILE_M: int,
                          TILE_N: int, stream=None):
    """The whole backward of examples/layernorm.jl:245-251 in one call that allocates nothing: the
    partial slots live in the library's static scratch (MiError with MI_E_SCRATCH beyond its size)."""
    _call("mi_layer_norm_bwd_static", _ref(DX), _ref(DY), _ref(X), _ref(W), _ref(Mean), _ref(Rstd),
          _ref(FINAL_DW), _ref(FINAL_DB), GROUP_SIZE_M, TILE_M, TILE_N, _stream(stream))


def softmax_tma_kernel(output, input, TILE_SIZE: int, num_programs: int | None = None, stream=None):
    """examples/softmax.jl:18-42"""
    if num_programs is None:
        num_programs = max(1, min(input.shape[0] if input.dim() == 2 else 1, (1 << 24) - 1))
    _call("mi_softmax_tma_kernel", _ref(output), _ref(input), TILE_SIZE, num_programs, _stream(stream))


def softmax_chunked_kernel(output, input, n_elems: int, TILE_SIZE: int,
                           num_programs: int | None = None, stream=None):
    """examples/softmax.jl:48-100"""
    if num_programs is None:
        num_programs = max(1, min(input.shape[0] if input.dim() == 2 else 1, (1 << 24) - 1))
    _call("mi_softmax_chunked_kernel", _ref(output), _ref(input), n_elems, TILE_SIZE, num_programs,
          _stream(stream))


def fmha_kernel(Q, K, V, Out, qk_scale: float, input_pos: int, TILE_D: int, H: int, TILE_M: int,
                TILE_N: int, QUERY_GROUP_SIZE: int, CAUSAL: bool, EVEN_K: bool, stream=None):
    """examples/fmha.jl:20-139"""
    _call("mi_fmha_kernel", _ref(Q), _ref(K), _ref(V), _ref(Out), ctypes.c_float(qk_scale),
          ctypes.c_int32(input_pos), TILE_D, H, TILE_M, TILE_N, QUERY_GROUP_SIZE, int(bool(CAUSAL)),
          int(bool(EVEN_K)), _stream(stream))


def moe_align_tile_size(topk_ids, tile_m: int, num_experts: int):
    """examples/moe.jl:142-183.  ``topk_ids``: CPU int64 tensor holding the Julia
    (num_tokens, topk) matrix, i.e. torch shape (topk, num_tokens).  Returns CPU int32
    tensors (sorted_token_ids, sorted_expert_ids), both 1-based."""
    import torch
    assert topk_ids.device.type == "cpu" and topk_ids.dtype == torch.int64 and topk_ids.dim() == 2
    ids = topk_ids.contiguous()
    topk, num_tokens = ids.shape
    p = ctypes.cast(ids.data_ptr(), ctypes.POINTER(ctypes.c_int64))
    nblk = ctypes.c_int64()
    _call("mi_moe_align_tile_size", p, num_tokens, topk, tile_m, num_experts, None, None,
          ctypes.byref(nblk))
    tok = torch.empty(nblk.value * tile_m, dtype=torch.int32)
    exp = torch.empty(nblk.value, dtype=torch.int32)
    _call("mi_moe_align_tile_size", p, num_tokens, topk, tile_m, num_experts,
          ctypes.cast(tok.data_ptr(), ctypes.POINTER(ctypes.c_int32)),
          ctypes.cast(exp.data_ptr(), ctypes.POINTER(ctypes.c_int32)), ctypes.byref(nblk))
    return tok, exp


def moe_align_capacity(num_tokens: int, topk: int, tile_m: int, num_experts: int):
    """(blocks, slots) that always hold the result of ``moe_align_tile_size`` for these sizes."""
    total = num_tokens * topk
    blocks = -(-(total + min(total, num_experts) * (tile_m - 1)) // tile_m)
    return blocks, blocks * tile_m


def moe_align_tile_size_device(topk_ids, tile_m: int, num_experts: int, sorted_token_ids=None,
                               sorted_expert_ids=None, stream=None, clear=None):
    """On-device ``moe_align_tile_size`` (no host round trip).  ``topk_ids``: device int64 tensor
    of torch shape (topk, num_tokens).  Returns device int32 tensors of fixed capacity
    (``moe_align_capacity``); unused slots hold the sentinel, unused blocks expert 0.
    ``clear``: a dense device tensor of whole 16-byte units that the same launch fills with zeros
    (the output that ``fused_moe_accumulate_kernel`` adds into)."""
    import torch
    topk, num_tokens = topk_ids.shape
    blocks, slots = moe_align_capacity(num_tokens, topk, tile_m, num_experts)
    if sorted_token_ids is None:
        sorted_token_ids = torch.empty(slots, dtype=torch.int32, device=topk_ids.device)
    if sorted_expert_ids is None:
        sorted_expert_ids = torch.empty(blocks, dtype=torch.int32, device=topk_ids.device)
    if clear is None:
        _call("mi_moe_align_tile_size_device", _ref(topk_ids), tile_m, num_experts, _ref(sorted_token_ids),
              _ref(sorted_expert_ids), _stream(stream))
    else:
        _call("mi_moe_align_tile_size_device_clear", _ref(topk_ids), tile_m, num_experts, _ref(sorted_token_ids),
              _ref(sorted_expert_ids), _ref(clear), _stream(stream))
    return sorted_token_ids, sorted_expert_ids


def moe_route_topk(logits, topk: int, weight_dtype=None, topk_weights=None, topk_ids=None, stream=None):
    """Router on the device: the ``topk`` largest logits of every token (ties to the lower expert
    id) and the softmax over them.  ``logits``: device tensor of torch shape (num_experts,
    num_tokens), i.e. Julia (num_tokens, num_experts).  Returns (topk_weights, topk_ids) of torch
    shape (topk, num_tokens), the layout ``cutile_moe`` takes; ids are int64 and 1-based."""
    import torch
    num_experts, num_tokens = logits.shape
    if topk_weights is None:
        topk_weights = torch.empty((topk, num_tokens), dtype=weight_dtype or logits.dtype, device=logits.device)
    if topk_ids is None:
        topk_ids = torch.empty((topk, num_tokens), dtype=torch.int64, device=logits.device)
    _call("mi_moe_route_topk", _ref(logits), _ref(topk_weights), _ref(topk_ids), _stream(stream))
    return topk_weights, topk_ids


def fused_moe_kernel(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids,
                     num_token_replicas: int, mul_routed_weight: bool, TILE_M: int, TILE_N: int,
                     TILE_K: int, b_scale=None, stream=None):
    """examples/moe.jl:45-105 (``b_scale``: per-(n, expert) fp32 scales of fp8 weights)."""
    _call("mi_fused_moe_kernel", _ref(A), _ref(B), _ref(C), _ref(topk_weights),
          _ref(sorted_token_ids), _ref(sorted_expert_ids), num_token_replicas,
          int(bool(mul_routed_weight)), TILE_M, TILE_N, TILE_K, _ref(b_scale), _stream(stream))


def fused_moe_accumulate_kernel(A, B, Out, topk_weights, sorted_token_ids, sorted_expert_ids, TILE_M: int, TILE_N: int,
                                TILE_K: int, b_scale=None, stream=None):
    """The down projection of cutile_moe (fused_moe_kernel with mul_routed_weight, moe.jl:245-251) and the sum over
    the top-k slots (moe.jl:256) in one launch: ``Out`` (torch (num_tokens, N), zeroed beforehand) receives every
    replica's weighted row, rounded to the storage type as cache3 would hold it, by memory-side packed atomic adds.
    top-k of 1 or 2 only (two terms add up the same in either order), ``topk_weights`` as the (num_tokens, topk)
    matrix, N even."""
    _call("mi_fused_moe_accumulate_kernel", _ref(A), _ref(B), _ref(Out), _ref(topk_weights), _ref(sorted_token_ids),
          _ref(sorted_expert_ids), TILE_M, TILE_N, TILE_K, _ref(b_scale), _stream(stream))


def fused_moe_silu_kernel(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids,
                          num_token_replicas: int, mul_routed_weight: bool, TILE_M: int, TILE_N: int,
                          TILE_K: int, b_scale=None, stream=None):
    """fused_moe_kernel (moe.jl:45-105) on the gate / up projection with silu_and_mul_kernel
    (moe.jl:110-128) as its epilogue: ``C`` is (N/2, total_tokens)."""
    _call("mi_fused_moe_silu_kernel", _ref(A), _ref(B), _ref(C), _ref(topk_weights),
          _ref(sorted_token_ids), _ref(sorted_expert_ids), num_token_replicas,
          int(bool(mul_routed_weight)), TILE_M, TILE_N, TILE_K, _ref(b_scale), _stream(stream))


def silu_and_mul_kernel(A, B, C, TILE_N: int, stream=None):
    """examples/moe.jl:110-128"""
    _call("mi_silu_and_mul_kernel", _ref(A), _ref(B), _ref(C), TILE_N, _stream(stream))


def quantize_e4m3fn(x, codes=None, scale=None, workspace=None, stream=None, fold=None, fold_out=None):
    """Per-tensor E4M3FN codes of a 16-bit activation matrix (torch (columns, K)) and their scale (a 1-element fp32
    device tensor): the fp8 operand of ``fused_moe_kernel`` with fp8 weights.  Returns (codes, scale), or with
    ``fold`` (a dense fp32 tensor, e.g. the weights' scales) (codes, scale, fold * scale) from the same two launches."""
    import torch
    if codes is None:
        codes = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    if scale is None:
        scale = torch.empty(1, dtype=torch.float32, device=x.device)
    if workspace is None:
        workspace = torch.empty(1024, dtype=torch.float32, device=x.device)
    if fold is not None:
        if fold_out is None:
            fold_out = torch.empty_like(fold)
        _call("mi_quantize_e4m3fn_fold", _ref(x), _ref(codes), _ref(scale), _ref(workspace), _ref(fold), _ref(fold_out),
              _stream(stream))
        return codes, scale, fold_out
    _call("mi_quantize_e4m3fn", _ref(x), _ref(codes), _ref(scale), _ref(workspace), _stream(stream))
    return codes, scale


def moe_sum_topk(inp, out, stream=None):
    """The ``sum(cache3; dims=2)`` of examples/moe.jl:256."""
    _call("mi_moe_sum_topk", _ref(inp), _ref(out), _stream(stream))
