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


def _no_gpu_here():
    return not torch.cuda.is_available()


@pytest.mark.skipif(not _no_gpu_here(), reason="launches with placeholder pointers: only where no GPU can take them")
def test_dimensions_beyond_65535_pass_the_host_checks(ct):
    """The reference's grids are flattened and take up to 2^24 - 1 blocks per dimension
    (src/launch.jl:743,801-807).  Dimensions that this library maps to the second or third grid
    dimension (at most 65535 workgroups) must not be rejected on the host: tokens * topk columns of
    silu_and_mul, tokens of the top-k sum, dimension 2 of a strided 2-D vadd, the batch of a batched
    GEMM, batch * heads of attention.  Without a GPU the launch itself fails with a (positive) HIP
    status, which is how the test tells "accepted" from a host-side MI_E_* rejection."""
    L = ct.lib()
    r = ctypes.byref
    n = 70_000
    h16 = ct.MI_F16
    a = _desc(ct, (64, n), h16); c = _desc(ct, (64, n), h16)
    assert L.mi_silu_and_mul_kernel(r(a), r(a), r(c), 64, None) > 0
    assert L.mi_moe_sum_topk(r(_desc(ct, (64, 2, n), h16)), r(_desc(ct, (64, n), h16)), None) > 0
    v = _desc(ct, (16, n), strides=(2, 32))
    assert L.mi_vec_add_kernel_2d(r(v), r(v), r(v), 16, 16, None) > 0
    A = _desc(ct, (8, 8, n), h16)
    assert L.mi_batch_matmul_kernel(r(A), r(A), r(A), 8, 8, 8, None) > 0
    q = _desc(ct, (64, 16, 7000, 10), h16)
    assert L.mi_fmha_kernel(r(q), r(q), r(q), r(q), ctypes.c_float(0.125), 0, 64, 7000, 16, 16, 1, 1, 1, None) > 0
    # the 24-bit limits of the reference still hold
    A2 = _desc(ct, (8, 8, 2 ** 24), h16)
    assert L.mi_batch_matmul_kernel(r(A2), r(A2), r(A2), 8, 8, 8, None) == ct.MI_E_GRID
    # ... and so does the launch's own: (tile, batch entry) pairs, or (query block, head) pairs, share one grid
    # dimension, which takes fewer than 2^32 lanes; a product past that is a host-side MI_E_GRID, not a HIP error
    A3 = _desc(ct, (128, 128, 2 ** 23), h16)         # 4 tiles of 64 x 64 per entry: 2^25 workgroups of 256 lanes
    assert L.mi_batch_matmul_kernel(r(A3), r(A3), r(A3), 64, 64, 64, None) == ct.MI_E_GRID
    A4 = _desc(ct, (128, 128, 2 ** 21), h16)         # 2^23 workgroups: accepted
    assert L.mi_batch_matmul_kernel(r(A4), r(A4), r(A4), 64, 64, 64, None) > 0
    q2 = _desc(ct, (64, 128 * 4096, 8192, 1), h16)   # 4096 query blocks x 8192 heads
    assert L.mi_fmha_kernel(r(q2), r(q2), r(q2), r(q2), ctypes.c_float(0.125), 0, 64, 8192, 128, 128, 1, 1, 1, None) == ct.MI_E_GRID


@pytest.mark.skipif(not _no_gpu_here(), reason="launches with placeholder pointers: only where no GPU can take them")
def test_direct_to_lds_gemms_are_not_chosen_for_descending_or_overlapping_rows(ct):
    """The direct-to-LDS GEMM kernels compute lane offsets in 32 bits and assume leading dimensions
    that are at least the row length and positive; a reversed view (negative stride) or overlapping
    rows must fall to the kernels that index with 64-bit offsets."""
    L = ct.lib()
    r = ctypes.byref
    for dt, bigname in ((ct.MI_F16, "gemm16_big"), (ct.MI_F32, "gemm32_big"), (ct.MI_F8E4M3FN, "gemm8_big")):
        M = N = K = 2048
        good = _desc(ct, (M, K), dt); goodB = _desc(ct, (K, N), dt); C = _desc(ct, (M, N), ct.MI_F32)
        assert L.mi_matmul_kernel(r(good), r(goodB), r(C), 64, 64, 64, None) > 0
        assert ct.last_variant().startswith(bigname)
        for bad in (_desc(ct, (M, K), dt, ptr=0x10000000, strides=(1, -M)), _desc(ct, (M, K), dt, strides=(1, M - 16))):
            assert L.mi_matmul_kernel(r(bad), r(goodB), r(C), 64, 64, 64, None) > 0
            assert not ct.last_variant().startswith(bigname), ct.last_variant()
        badC = _desc(ct, (M, N), ct.MI_F32, ptr=0x10000000, strides=(1, -M))
        assert L.mi_matmul_kernel(r(good), r(goodB), r(badC), 64, 64, 64, None) > 0
        assert not ct.last_variant().startswith(bigname), ct.last_variant()


def test_static_scratch_entry_point_rejects_oversized_problems_on_the_host(ct):
    """mi_layer_norm_bwd_static: cld(N, 4) * 4 * GROUP_SIZE_M floats must fit the 524288-float static array."""
    L = ct.lib()
    r = ctypes.byref
    X = _desc(ct, (16384, 4)); W = _desc(ct, (16384,)); v = _desc(ct, (4,))
    assert L.mi_layer_norm_bwd_static(r(X), r(X), r(X), r(W), r(v), r(v), r(W), r(W), 64, 32, 1024, None) == ct.MI_E_SCRATCH
    assert "scratch" in ct.strerror(ct.MI_E_SCRATCH)


def test_fused_moe_routed_weight_layouts_are_validated_on_the_host(ct):
    """The routed weights may be the flattened vector of moe.jl:193 or the (num_tokens, topk) matrix itself; other
    ranks, a matrix of the wrong extent or element type are refused before anything is launched."""
    L = ct.lib(); r = ctypes.byref
    K, N, E, tokens, topk, tile_m = 64, 128, 4, 6, 2, 16
    total = tokens * topk
    A = _desc(ct, (K, tokens), ct.MI_F16); B = _desc(ct, (K, N, E), ct.MI_F16); C = _desc(ct, (N, total), ct.MI_F16)
    tok = _desc(ct, (4 * tile_m,), ct.MI_I32); exp = _desc(ct, (4,), ct.MI_I32)
    call = lambda w, mul=1: L.mi_fused_moe_kernel(r(A), r(B), r(C), w, r(tok), r(exp), 1, mul, tile_m, 128, 64, None, None)
    assert call(None) == ct.MI_E_NULL
    assert call(r(_desc(ct, (tokens, topk, 1), ct.MI_F16))) == ct.MI_E_RANK
    assert call(r(_desc(ct, (tokens, topk), ct.MI_F32))) == ct.MI_E_DTYPE
    assert call(r(_desc(ct, (tokens - 1, topk), ct.MI_F16))) == ct.MI_E_SHAPE
    assert call(r(_desc(ct, (tokens, topk + 1), ct.MI_F16))) == ct.MI_E_SHAPE
    assert call(r(_desc(ct, (total - 1,), ct.MI_F16))) == ct.MI_E_SHAPE
    assert call(r(_desc(ct, (total,), ct.MI_F16, strides=(2,)))) == ct.MI_E_STRIDE
    # weights that are not used (mul_routed_weight = 0) need no particular extent; an empty problem is a no-op
    C0 = _desc(ct, (0, total), ct.MI_F16, ptr=0); B0 = _desc(ct, (K, 0, E), ct.MI_F16, ptr=0)
    assert L.mi_fused_moe_kernel(r(A), r(B0), r(C0), r(_desc(ct, (3,), ct.MI_F16)), r(tok), r(exp), 1, 0, tile_m, 128, 64, None, None) == 0


def test_accumulating_down_projection_and_clearing_sort_validate_on_the_host(ct):
    L = ct.lib(); r = ctypes.byref
    K, N, E, tokens, topk, tile_m = 64, 128, 4, 6, 2, 16
    A = _desc(ct, (K, tokens * topk), ct.MI_F16); B = _desc(ct, (K, N, E), ct.MI_F16); Out = _desc(ct, (N, tokens), ct.MI_F16)
    tok = _desc(ct, (4 * tile_m,), ct.MI_I32); exp = _desc(ct, (4,), ct.MI_I32); w = _desc(ct, (tokens, topk), ct.MI_F16)
    call = lambda a=A, b=B, o=Out, ww=w: L.mi_fused_moe_accumulate_kernel(r(a), r(b), r(o), r(ww), r(tok), r(exp), tile_m, 128, 64, None, None)
    assert call(ww=_desc(ct, (tokens * topk,), ct.MI_F16)) == ct.MI_E_ARG                 # needs the matrix: top-k is read from it
    assert call(ww=_desc(ct, (tokens, 3), ct.MI_F16), a=_desc(ct, (K, tokens * 3), ct.MI_F16)) == ct.MI_E_UNSUPPORTED
    assert call(o=_desc(ct, (N, tokens + 1), ct.MI_F16)) == ct.MI_E_SHAPE
    assert call(b=_desc(ct, (K, N - 1, E), ct.MI_F16), o=_desc(ct, (N - 1, tokens), ct.MI_F16)) == ct.MI_E_ALIGN   # odd channel count
    assert call(o=_desc(ct, (N, tokens), ct.MI_F16, ptr=0x1002)) == ct.MI_E_ALIGN
    assert call(o=_desc(ct, (N, tokens), ct.MI_F16, strides=(1, N + 1))) == ct.MI_E_ALIGN
    ids = _desc(ct, (tokens, topk), ct.MI_I64)
    cap_t = _desc(ct, (12 * tile_m,), ct.MI_I32); cap_e = _desc(ct, (12,), ct.MI_I32)
    clr = lambda c: L.mi_moe_align_tile_size_device_clear(r(ids), tile_m, E, r(cap_t), r(cap_e), c, None)
    assert clr(None) == ct.MI_E_NULL
    assert clr(r(_desc(ct, (N - 1, tokens), ct.MI_F16))) == ct.MI_E_ALIGN                 # not whole 16-byte units
    assert clr(r(_desc(ct, (N, tokens), ct.MI_F16, ptr=0x1008))) == ct.MI_E_ALIGN
    assert clr(r(_desc(ct, (N, tokens), ct.MI_F16, strides=(1, N + 8)))) == ct.MI_E_STRIDE
