"""The C-ABI library loads, exports every symbol include/mi355tile.h declares, and rejects bad
arguments on the host with the documented error codes.  No kernel is launched (no GPU)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi355tile.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(ct):
    lib = ctypes.CDLL(ct.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), name
    assert set(declared) == set(ct.EXPORTED_SYMBOLS)
    assert ct.lib().mi_version() == 100
    assert ct.strerror(0) == "success" and "power of two" in ct.strerror(ct.MI_E_TILE)


def _desc(ct, shape_jl, dtype=None, ptr=0x1000, strides=None):
    d = ct.MiTileArray()
    d.ptr = ptr
    d.dtype = ct.MI_F32 if dtype is None else dtype
    d.ndim = len(shape_jl)
    st = 1
    for i, s in enumerate(shape_jl):
        d.sizes[i] = s
        d.strides[i] = st if strides is None else strides[i]
        st *= s
    return d


def test_argument_errors_are_reported_without_launching(ct):
    L = ct.lib()
    a = _desc(ct, (1024,)); b = _desc(ct, (1024,)); c = _desc(ct, (1024,))
    r = ctypes.byref
    assert L.mi_vec_add_kernel_1d(None, r(b), r(c), 1024, None) == ct.MI_E_NULL
    assert L.mi_vec_add_kernel_1d(r(a), r(b), r(c), 1000, None) == ct.MI_E_TILE
    assert L.mi_vec_add_kernel_1d(r(a), r(b), r(_desc(ct, (512,))), 1024, None) == ct.MI_E_SHAPE
    assert L.mi_vec_add_kernel_1d(r(a), r(b), r(_desc(ct, (1024,), ct.MI_F16)), 1024, None) == ct.MI_E_DTYPE
    assert L.mi_vec_add_kernel_1d(r(a), r(b), r(_desc(ct, (32, 32))), 1024, None) == ct.MI_E_RANK
    assert L.mi_vec_add_kernel_1d(r(a), r(b), r(_desc(ct, (1024,), ptr=0x1002)), 1024, None) == ct.MI_E_ALIGN
    # 24-bit grid limit of the reference launch path (src/launch.jl:743,801-807)
    big = _desc(ct, (2 ** 25,))
    assert L.mi_vec_add_kernel_1d(r(big), r(big), r(big), 1, None) == ct.MI_E_GRID
    x = _desc(ct, (64, 32)); y = _desc(ct, (64, 32))
    assert L.mi_transpose_kernel(r(x), r(y), 64, 64, None) == ct.MI_E_SHAPE
    xs = _desc(ct, (64, 32), strides=(2, 128))
    assert L.mi_transpose_kernel(r(xs), r(_desc(ct, (32, 64))), 64, 64, None) == ct.MI_E_STRIDE
    inp = _desc(ct, (256, 8))
    assert L.mi_softmax_tma_kernel(r(inp), r(inp), 100, 8, None) == ct.MI_E_TILE
    assert L.mi_softmax_tma_kernel(r(inp), r(inp), 256, 0, None) == ct.MI_E_GRID
    X = _desc(ct, (256, 8)); W = _desc(ct, (128,)); v = _desc(ct, (8,))
    assert L.mi_layer_norm_fwd(r(X), r(W), r(W), r(X), r(v), r(v), ctypes.c_float(1e-5), 256, None) == ct.MI_E_SHAPE
    # device router: topk within 1..num_experts, at most 512 experts, i64 ids
    lg = _desc(ct, (16, 32)); tw = _desc(ct, (16, 2)); ti = _desc(ct, (16, 2), ct.MI_I64)
    assert L.mi_moe_route_topk(r(lg), r(tw), r(_desc(ct, (16, 2), ct.MI_I32)), None) == ct.MI_E_DTYPE
    assert L.mi_moe_route_topk(r(lg), r(_desc(ct, (16, 3))), r(ti), None) == ct.MI_E_SHAPE
    assert L.mi_moe_route_topk(r(lg), r(_desc(ct, (16, 33))), r(_desc(ct, (16, 33), ct.MI_I64)), None) == ct.MI_E_ARG
    assert L.mi_moe_route_topk(r(_desc(ct, (16, 513))), r(tw), r(ti), None) == ct.MI_E_UNSUPPORTED
    assert L.mi_moe_route_topk(r(_desc(ct, (0, 32), ptr=0)), r(_desc(ct, (0, 2), ptr=0)),
                               r(_desc(ct, (0, 2), ct.MI_I64, ptr=0)), None) == 0
    # empty arrays are a successful no-op
    e = _desc(ct, (0,), ptr=0)
    assert L.mi_vec_add_kernel_1d(r(e), r(e), r(e), 1024, None) == 0


def test_tilearray_descriptor_follows_julia_order(ct):
    t = torch.zeros(3, 5, 7)  # Julia (7, 5, 3)
    d = ct.TileArray(t)
    assert d.ndim == 3 and list(d.sizes)[:3] == [7, 5, 3] and list(d.strides)[:3] == [1, 7, 35]
    v = t[:, :, 2:6]          # Julia view(t, 3:6, :, :)
    dv = ct.TileArray(v)
    assert list(dv.sizes)[:3] == [4, 5, 3] and list(dv.strides)[:3] == [1, 7, 35]
    assert dv.ptr == t.data_ptr() + 2 * 4


def test_descriptor_struct_layout_matches_header(ct):
    # struct mi_tile_array: void* ptr; int32 dtype; int32 ndim; int64 sizes[4]; int64 strides[4]
    M = ct.MiTileArray
    assert ctypes.sizeof(M) == 80
    assert (M.ptr.offset, M.dtype.offset, M.ndim.offset, M.sizes.offset, M.strides.offset) == (0, 8, 12, 16, 48)


def test_host_swizzle_matches_oracle(ct, orc):
    for (M, N, tm, tn) in [(4096, 4096, 64, 64), (200, 100, 64, 64), (1000, 130, 32, 64), (4096, 512, 128, 128)]:
        for bid in range(1, orc.cld(M, tm) * orc.cld(N, tn) + 1):
            assert ct.swizzle_2d(M, N, tm, tn, 8, bid) == orc.swizzle_2d(M, N, tm, tn, 8, bid)


@pytest.mark.parametrize("num_tokens,topk,E,tile_m", [(48, 8, 64, 128), (256, 2, 32, 128), (128, 4, 32, 128),
                                                       (7, 2, 4, 4), (1, 1, 1, 1), (33, 3, 5, 16)])
def test_host_moe_align_matches_oracle(ct, orc, num_tokens, topk, E, tile_m):
    rng = np.random.default_rng(num_tokens)
    ids = np.stack([rng.permutation(E)[:topk] + 1 for _ in range(num_tokens)]).astype(np.int64)
    tok_ref, exp_ref = orc.moe_align_tile_size(ids, tile_m, E)
    tok, exp = ct.moe_align_tile_size(orc.from_julia(ids), tile_m, E)
    assert np.array_equal(tok.numpy(), tok_ref) and np.array_equal(exp.numpy(), exp_ref)


def test_host_moe_align_rejects_bad_ids(ct):
    L = ct.lib()
    ids = (ctypes.c_int64 * 4)(1, 2, 9, 1)
    n = ctypes.c_int64()
    assert L.mi_moe_align_tile_size(ids, 2, 2, 4, 4, None, None, ctypes.byref(n)) == ct.MI_E_ARG
    assert L.mi_moe_align_tile_size(ids, 2, 2, 3, 16, None, None, ctypes.byref(n)) == ct.MI_E_TILE
