"""GPU parity tests for the memory-bound kernels (vadd, transpose, softmax, LayerNorm),
through the C ABI, against the CPU oracle.  The shape lists are those of the reference
examples' ``main()`` (vadd.jl:219-248, transpose.jl:137-146, layernorm.jl:340-348,
softmax.jl:248-256) plus ragged / strided / empty edge cases.

Tolerances.  vadd and transpose: bit-exact.  fp32 kernels: |got - ref| <= 1e-5 * (|ref| +
max|ref|) element-wise against a float64 evaluation of the reference's formulas (that is,
relative 1e-5 for elements near the array's scale, and 1e-5 of that scale in absolute
terms for elements near zero).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd.examples import vadd, transpose, layernorm, softmax  # noqa: E402


def close_f32(got, ref, tol=1e-5):
    got = np.asarray(got, dtype=np.float64); ref = np.asarray(ref, dtype=np.float64)
    scale = np.abs(ref).max()
    err = np.abs(got - ref)
    bound = tol * (np.abs(ref) + scale)
    assert np.all(err <= bound), f"max err {err.max():.3e} (scale {scale:.3e}), worst ratio {np.max(err / bound):.2f}"


# ---- vadd ---------------------------------------------------------------------------------

@pytest.mark.parametrize("shape,tile,T,gather", [
    ((1_024_000,), 1024, torch.float32, False), ((2 ** 20,), 512, torch.float32, False),
    ((2 ** 18,), 512, torch.float64, False), ((1_024_000,), 1024, torch.float16, False),
    ((2048, 1024), (32, 32), torch.float32, False), ((1024, 2048), (64, 64), torch.float32, False),
    ((1024, 512), (32, 32), torch.float64, False), ((1024, 1024), (64, 64), torch.float16, False),
    ((1_024_000,), 1024, torch.float32, True), ((2 ** 20,), 512, torch.float32, True),
    ((1_000_003,), 1024, torch.float32, False), ((1001,), 256, torch.float16, False), ((3,), 1, torch.float64, False),
    ((1000, 37), (32, 32), torch.float32, False), ((70_001,), 1024, torch.bfloat16, False),
])
def test_vadd_bit_exact(orc, shape, tile, T, gather):
    d = vadd.prepare(shape=shape, use_gather=gather, T=T)
    r = vadd.run(d, tile=tile)
    ref = orc.from_julia(orc.vadd(orc.to_julia(d.a), orc.to_julia(d.b))) if T != torch.bfloat16 else (d.a.cpu().float() + d.b.cpu().float()).to(T)
    assert torch.equal(r.c.cpu(), ref.to(T))


def test_vadd_strided_views_and_misaligned(ct, orc):
    rng = np.random.default_rng(0)
    base = torch.from_numpy(rng.random(4099 * 3, dtype=np.float32)).cuda()
    a, b = base[1::3], base[2::3]         # stride 3, misaligned start
    c = torch.zeros(a.shape[0] * 2, device="cuda")[::2]
    ct.vec_add_kernel_1d(a, b, c, 1024)
    assert torch.equal(c, a + b)
    a2 = base[1:4098]; b2 = base[5000:5000 + 4097]; c2 = torch.empty(4097 + 1, device="cuda")[1:]
    ct.vec_add_kernel_1d(a2, b2, c2, 256)  # dense but only 4-byte aligned
    assert torch.equal(c2, a2 + b2)
    # 2-D column-strided view: Julia view(A, 1:100, :) of a (128, 50) array
    A = torch.from_numpy(rng.random((50, 128), dtype=np.float32)).cuda()
    B = torch.from_numpy(rng.random((50, 128), dtype=np.float32)).cuda()
    C = torch.zeros(50, 128, device="cuda")
    ct.vec_add_kernel_2d(A[:, :100], B[:, :100], C[:, :100], 32, 32)
    assert torch.equal(C[:, :100], A[:, :100] + B[:, :100]) and torch.all(C[:, 100:] == 0)


@pytest.mark.parametrize("T", [torch.float32, torch.float16, torch.bfloat16, torch.float64, torch.int32, torch.int64])
def test_vadd_views_off_a_16_byte_boundary_and_integers(ct, T):
    """Views that start 1, 2, 3 or 5 elements past a 16-byte boundary: a head up to the boundary, 16-byte vectors and
    a tail when all three arrays sit at the same offset, element by element when they do not; the gather kernel with
    three different lengths; 2-D views of a padded parent.  Integers wrap like Julia's +.  What lies around every
    destination view stays as it was."""
    g = torch.Generator(device="cuda"); g.manual_seed(9)

    def rnd(*shape):
        if T.is_floating_point:
            return torch.randn(*shape, device="cuda", generator=g).to(T)
        return (torch.randint(-2 ** 31, 2 ** 31 - 1, shape, device="cuda", generator=g).to(T) * (3 if T == torch.int64 else 1))

    for nn in (1, 3, 4, 5, 17, 1000, 4099, 70001):
        for off in (0, 1, 2, 3, 5):
            x, y = rnd(nn + 8), rnd(nn + 8)
            z = torch.zeros(nn + 8, device="cuda", dtype=T)
            ct.vec_add_kernel_1d(x[off:off + nn], y[off:off + nn], z[off:off + nn], 1024)
            assert torch.equal(z[off:off + nn], x[off:off + nn] + y[off:off + nn]), (nn, off, ct.last_variant())
            assert bool((z[:off] == 0).all()) and bool((z[off + nn:] == 0).all())
            if nn >= 64:
                assert ct.last_variant().startswith("vadd_vec16")
            z.zero_()
            ct.vec_add_kernel_1d(x[off:off + nn], y[1:1 + nn], z[2:2 + nn], 1024)       # offsets that do not agree
            assert torch.equal(z[2:2 + nn], x[off:off + nn] + y[1:1 + nn]) and bool((z[:2] == 0).all()) and bool((z[2 + nn:] == 0).all())
            na, nb = max(1, nn - 3), nn + 5
            zz = torch.full((nn + 8,), 7, device="cuda", dtype=T)
            ct.vec_add_kernel_1d_gather(x[off:off + na], y[off:off + nb], zz[off:off + nn], 256)
            ref = torch.zeros(nn, device="cuda", dtype=T)
            ref[:na] += x[off:off + na]
            ref += y[off:off + nb][:nn]
            assert torch.equal(zz[off:off + nn], ref), (nn, off, ct.last_variant())
            assert bool((zz[:off] == 7).all()) and bool((zz[off + nn:] == 7).all())
    v = 16 // torch.empty(0, dtype=T).element_size()
    for r, cfull, ccols, coff, vec in [(33, 64, 40, 0, True), (100, 1000, 1000 - 2 * v, v, True), (7, 520, 513, 0, True),
                                       (5, 16, 3, 0, v <= 3), (300, 128, 128, 0, True), (9, 100, 50, 1, False)]:
        X, Y = rnd(r, cfull), rnd(r, cfull)
        Z = torch.zeros(r, cfull, device="cuda", dtype=T)
        ct.vec_add_kernel_2d(X[:, coff:coff + ccols], Y[:, coff:coff + ccols], Z[:, coff:coff + ccols], 32, 32)
        assert torch.equal(Z[:, coff:coff + ccols], X[:, coff:coff + ccols] + Y[:, coff:coff + ccols]), (r, cfull, ccols, coff)
        assert bool((Z[:, :coff] == 0).all()) and bool((Z[:, coff + ccols:] == 0).all())
        if cfull % v == 0:
            assert (ct.last_variant() != "vadd_2d_strided") == vec, (r, cfull, ccols, coff, ct.last_variant())


def test_vadd_gather_out_of_bounds_semantics(ct, orc):
    """test/device/gather_scatter.jl:75-113: an out-of-bounds gather lane reads 0, an
    out-of-bounds scatter lane is dropped."""
    a = torch.ones(16, device="cuda"); b = torch.full((32,), 2.0, device="cuda")
    c = torch.zeros(32, device="cuda")
    ct.vec_add_kernel_1d_gather(a, b, c, 32)
    assert torch.all(c[:16] == 3.0) and torch.all(c[16:] == 2.0)
    rng = np.random.default_rng(8)
    for na, nb, nc, tile in [(1000, 700, 1500, 256), (33, 1025, 1024, 1024), (5000, 5000, 4097, 512)]:
        x = torch.from_numpy(rng.random(na, dtype=np.float32)).cuda(); y = torch.from_numpy(rng.random(nb, dtype=np.float32)).cuda()
        z = torch.full((nc,), -1.0, device="cuda")
        ct.vec_add_kernel_1d_gather(x, y, z, tile)
        assert np.array_equal(z.cpu().numpy(), orc.vadd_gather(x.cpu().numpy(), y.cpu().numpy(), nc))
    guard = torch.zeros(48, device="cuda")
    c_small = guard[:16]
    ct.vec_add_kernel_1d_gather(b, b, c_small, 32)
    assert torch.all(guard[:16] == 4.0) and torch.all(guard[16:] == 0.0)


def test_vadd_full_size_linearity():
    """Benchmark size (2^27 f32): bit-exact against torch's own IEEE add on the device, and
    (a+b)-b == a wherever that identity holds on the CPU for a sample."""
    d = vadd.prepare(benchmark=True)
    r = vadd.run(d)
    assert torch.equal(r.c, d.a + d.b)
    idx = torch.arange(0, 2 ** 27, 4099, device="cuda")
    ref = d.a[idx].cpu().numpy() + d.b[idx].cpu().numpy()
    assert np.array_equal(r.c[idx].cpu().numpy(), ref)


# ---- transpose ----------------------------------------------------------------------------

@pytest.mark.parametrize("m,n,tm,tn,T", [
    (256, 256, 32, 32, torch.float32), (512, 512, 64, 64, torch.float32), (256, 512, 32, 64, torch.float32),
    (1024, 1024, 64, 64, torch.float32), (1024, 512, 64, 64, torch.float32),
    (100, 37, 32, 32, torch.float32), (1, 1, 64, 64, torch.float32), (65, 129, 64, 64, torch.float16),
    (384, 200, 64, 64, torch.float16), (130, 66, 16, 16, torch.float64), (4, 1000, 64, 64, torch.float32),
])
def test_transpose_bit_exact(orc, m, n, tm, tn, T):
    d = transpose.prepare(m=m, n=n, T=T)
    r = transpose.run(d, tm=tm, tn=tn)
    assert np.array_equal(orc.to_julia(r.y), orc.transpose(orc.to_julia(d.x)))


def test_transpose_order_load_known_answer(ct):
    """test/device/tile.jl:657-698: src = reshape(1:n^2, n, n), dst == transpose(src)."""
    n = 64
    src = torch.arange(1, n * n + 1, dtype=torch.float32, device="cuda").reshape(n, n)
    dst = torch.zeros(n, n, device="cuda")
    ct.transpose_kernel(src, dst, 16, 16)
    assert torch.equal(dst, src.T.contiguous())


def test_transpose_padded_leading_dimension(ct):
    rng = np.random.default_rng(1)
    big = torch.from_numpy(rng.random((40, 96), dtype=np.float32)).cuda()
    x = big[:, :70]                     # Julia (70, 40) with column stride 96
    ybig = torch.full((70, 48), -1.0, device="cuda")
    y = ybig[:, :40]                    # Julia (40, 70) with column stride 48
    ct.transpose_kernel(x, y, 64, 64)
    assert torch.equal(y, x.T) and torch.all(ybig[:, 40:] == -1.0)


@pytest.mark.parametrize("T,isz", [(torch.float8_e4m3fn, 1), (torch.float16, 2), (torch.bfloat16, 2),
                                   (torch.float32, 4), (torch.float64, 8), (torch.int64, 8)])
def test_transpose_every_element_size_takes_the_register_path(ct, T, isz):
    """Random bit patterns (NaN payloads and denormals included) of 1-, 2-, 4- and 8-byte elements
    through the 16-byte path: whole tiles, ragged edges, skinny matrices, a matrix large enough for
    the big tiles, and padded leading dimensions on both sides with the padding left untouched."""
    v = 16 // isz
    iv = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[isz]
    g = torch.Generator(device="cuda"); g.manual_seed(100 + isz)

    def bits(r, c):
        return torch.randint(0, 256, (r, c * isz), device="cuda", generator=g).to(torch.uint8).view(iv)

    for r, c in [(v, v), (8 * v, 24 * v), (256, 512), (1008 // v * v, 528), (2064, 1040), (v, 4096), (4096, v),
                 (8192, 2048 * v)]:
        x = bits(r, c)
        y = torch.zeros(c, r, dtype=iv, device="cuda")
        ct.transpose_kernel(x.view(T), y.view(T), 64, 64)
        assert "regmicro" in ct.last_variant(), ct.last_variant()
        assert torch.equal(y, x.t()), (r, c)
        xb = bits(r, c + 2 * v); x2 = xb[:, v:v + c]
        yb = torch.full((c, r + v), 85, dtype=iv, device="cuda"); y2 = yb[:, :r]
        ct.transpose_kernel(x2.view(T), y2.view(T), 32, 32)
        assert "regmicro" in ct.last_variant(), ct.last_variant()
        assert torch.equal(y2, x2.t()) and bool((yb[:, r:] == 85).all()), (r, c)
    # one element short of a whole vector on either side: the element-wise kernel
    x = bits(3 * v + 1, 5 * v); y = torch.zeros(5 * v, 3 * v + 1, dtype=iv, device="cuda")
    ct.transpose_kernel(x.view(T), y.view(T), 64, 64)
    assert "regmicro" not in ct.last_variant() and torch.equal(y, x.t())


@pytest.mark.parametrize("T,isz", [(torch.float8_e4m3fn, 1), (torch.float16, 2), (torch.float32, 4), (torch.float64, 8)])
def test_transpose_views_of_a_padded_parent_with_ragged_sizes(ct, T, isz):
    """Sizes that are not multiples of a 16-byte vector inside parents whose leading dimensions are: the register path
    with edge tiles that move the vectors crossing the edge element by element.  Small and large tile variants; what
    lies around the destination view stays as it was.  A dense matrix with such sizes has misaligned columns and takes
    the element-wise kernel (several bands of tile rows, short last band, ragged last tiles)."""
    v = 16 // isz
    iv = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[isz]
    g = torch.Generator(device="cuda"); g.manual_seed(200 + isz)
    big = {1: (4100, 4099), 2: (4090, 4093), 4: (4095, 4090), 8: (2051, 2049)}[isz]
    for r, c in [(1, 1), (3, 5), (v + 1, v + 1), (100, 37), (257, 129), (1000, 999), (130, 4097), big]:
        R, C = (r + v - 1) // v * v + v, (c + v - 1) // v * v + v
        xb = torch.randint(0, 256, (R, C * isz), device="cuda", generator=g).to(torch.uint8).view(iv)
        yb = torch.full((C, R), 85, dtype=iv, device="cuda")
        x, y = xb[:r, :c], yb[:c, :r]
        ct.transpose_kernel(x.view(T), y.view(T), 64, 64)
        assert ct.last_variant().endswith("_regmicro_ragged"), ct.last_variant()
        assert torch.equal(y, x.t()), (r, c)
        assert bool((yb[c:, :] == 85).all()) and bool((yb[:, r:] == 85).all()), (r, c)
    for r, c in [(1001, 999), (3, 2049), (2049, 3), (577, 1), (1, 577), (4097, 67)]:   # torch (r, c) = Julia (c, r)
        x = torch.randint(0, 256, (r, c * isz), device="cuda", generator=g).to(torch.uint8).view(iv)
        yb = torch.full((c + 1, r + 2), 85, dtype=iv, device="cuda")
        y = yb[:c, :r]
        if c % v == 0 or r == 1:
            continue   # (aligned columns: not this kernel's case)
        ct.transpose_kernel(x.view(T), y.view(T), 64, 64)
        assert ct.last_variant().startswith("transpose_elem_"), ct.last_variant()
        assert torch.equal(y, x.t()), (r, c)
        assert bool((yb[c:, :] == 85).all()) and bool((yb[:, r:] == 85).all()), (r, c)


def test_transpose_full_size_involution():
    d = transpose.prepare(benchmark=True)
    r = transpose.run(d)
    assert torch.equal(r.y, d.x.T.contiguous())
    import cutile_jl_amd as ct
    back = torch.empty_like(d.x)
    ct.transpose_kernel(r.y, back, 64, 64)
    assert torch.equal(back, d.x)


# ---- softmax ------------------------------------------------------------------------------

@pytest.mark.parametrize("M,N,T", [(256, 256, torch.float32), (64, 1000, torch.float32), (33, 4096, torch.float32),
                                   (17, 5000, torch.float32), (8, 16384, torch.float32), (4, 20000, torch.float32),
                                   (5, 1, torch.float32), (3, 7, torch.float32), (128, 1024, torch.float16)])
def test_softmax_both_kernels(orc, M, N, T):
    d = softmax.prepare(M=M, N=N, T=T)
    r = softmax.run(d)
    ref = orc.softmax(orc.to_julia(d.input))
    for got in (r.output_tma, r.output_chunked):
        g = orc.to_julia(got).astype(np.float64)
        if T == torch.float32:
            close_f32(g, ref)
            assert np.all(np.abs(g - ref) <= 1e-5 * ref + 1e-12)  # relative 1e-5 on every element
        else:
            assert np.all(np.abs(g - ref) <= 2e-2 * ref + 1e-7)
        np.testing.assert_allclose(g.sum(axis=0), 1.0, rtol=1e-5 if T == torch.float32 else 2e-3)


@pytest.mark.parametrize("M,N,T,variant", [
    (7, 100003, torch.float32, "softmax_3pass_b1024"),     # few long columns, odd length: scalar head, vectors, scalar tail
    (3, 131075, torch.bfloat16, "softmax_3pass_b1024"), (1100, 65540, torch.float16, "softmax_3pass_b256"),
    # up to 65536 elements: the registers of 1024 lanes, 32 or 64 elements per lane, unaligned vectors where the
    # columns start off 16-byte boundaries
    (40, 50257, torch.float16, "softmax_regs_b1024_e64"), (50, 50257, torch.float32, "softmax_regs_b1024_e64"),
    (1100, 16388, torch.float32, "softmax_regs_b1024_e32"), (1030, 16391, torch.float32, "softmax_regs_b1024_e32"),
    (300, 40000, torch.float32, "softmax_regs_b1024_e64"), (600, 65536, torch.bfloat16, "softmax_regs_b1024_e64"),
    (9, 32768, torch.float32, "softmax_regs_b1024_e32"),
])
def test_softmax_columns_too_long_for_registers(ct, orc, M, N, T, variant):
    """Columns beyond the 256-lane register kernels (16384 four-byte, 32768 two-byte elements): up to 65536 elements
    the registers of 1024 lanes hold a column (one pass; more columns than workgroup slots are walked by persistent
    workgroups), beyond that three passes; a column that does not start on a 16-byte boundary moves in unaligned vectors
    (register kernels) or as head, vectors and tail (three passes)."""
    d = softmax.prepare(M=M, N=N, T=T)
    out = torch.full_like(d.input, float("nan"))
    ct.softmax_tma_kernel(out, d.input, 1 << (N - 1).bit_length())
    assert ct.last_variant() == variant
    ref = orc.softmax(orc.to_julia(d.input))
    g = orc.to_julia(out).astype(np.float64)
    if T == torch.float32:
        assert np.all(np.abs(g - ref) <= 1e-5 * ref + 1e-12)
    else:
        assert np.all(np.abs(g - ref) <= 2e-2 * ref + 1e-7)
    # views: input and output at the same / at different offsets from a 16-byte boundary
    if T == torch.float32 and M < 100:
        xb = torch.randn(M, N + 10, device="cuda"); ob = torch.zeros(M, N + 12, device="cuda")
        for xo, oo in ((3, 3), (1, 2)):
            ob.zero_()
            x, o = xb[:, xo:xo + N], ob[:, oo:oo + N]
            ct.softmax_tma_kernel(o, x, 1 << (N - 1).bit_length())
            got = orc.to_julia(o).astype(np.float64)
            r2 = orc.softmax(orc.to_julia(x))
            assert np.all(np.abs(got - r2) <= 1e-5 * r2 + 1e-12)
            assert bool((ob[:, :oo] == 0).all()) and bool((ob[:, oo + N:] == 0).all())


def test_softmax_tile_smaller_than_column_and_padding(ct, orc):
    """A TILE_SIZE below N covers rows 1..TILE_SIZE only (softmax.jl:29-38); the chunked
    kernel walks cld(n_elems, TILE)*TILE rows, clipped to the array."""
    d = softmax.prepare(M=9, N=1000)
    out = torch.full_like(d.input, -7.0)
    ct.softmax_tma_kernel(out, d.input, 512)
    close_f32(orc.to_julia(out)[:512], orc.softmax(orc.to_julia(d.input), rows=512))
    assert torch.all(out[:, 512:] == -7.0)
    out.fill_(-7.0)
    ct.softmax_chunked_kernel(out, d.input, 300, 256)      # 2 chunks -> rows 1..512
    close_f32(orc.to_julia(out)[:512], orc.softmax(orc.to_julia(d.input), rows=512))
    assert torch.all(out[:, 512:] == -7.0)
    # strided columns (padded leading dimension) and a different program count
    big = torch.randn(9, 1100, device="cuda")
    obig = torch.zeros(9, 1100, device="cuda")
    ct.softmax_tma_kernel(obig[:, :1000], big[:, :1000], 1024, num_programs=4)
    close_f32(orc.to_julia(obig[:, :1000]), orc.softmax(orc.to_julia(big[:, :1000])))
    assert torch.all(obig[:, 1000:] == 0)


def test_softmax_full_size_properties(orc):
    d = softmax.prepare(benchmark=True)
    r = softmax.run(d)
    for out in (r.output_tma, r.output_chunked):
        s = out.double().sum(dim=1)
        assert torch.all((s - 1).abs() < 1e-5)
        cols = [0, 1, 2047, 4095]
        ref = orc.softmax(orc.to_julia(d.input[cols]))
        close_f32(orc.to_julia(out[cols]), ref)
    # shift invariance at full size
    shifted = torch.empty_like(d.input)
    import cutile_jl_amd as ct
    ct.softmax_tma_kernel(shifted, d.input + 3.0, 4096)
    assert torch.allclose(shifted, r.output_tma, rtol=2e-5, atol=1e-9)


# ---- LayerNorm ----------------------------------------------------------------------------

@pytest.mark.parametrize("M,N,TILE_N,G", [(256, 256, 256, 64), (512, 512, 512, 64), (1024, 1024, 1024, 64),
                                          (100, 300, 128, 64), (7, 4096, 1024, 64), (130, 1000, 256, 16),
                                          (64, 8192, 1024, 64), (5, 16384, 1024, 4), (3, 20000, 1024, 2),
                                          (1000, 64, 64, 512), (1, 5, 8, 1)])
def test_layernorm_fwd_bwd(orc, M, N, TILE_N, G):
    d = layernorm.prepare(M=M, N=N, GROUP_SIZE_M=G)
    r = layernorm.run(d, TILE_N=TILE_N)
    X, W, B, DY = (orc.to_julia(t) for t in (d.X, d.W, d.B, d.DY))
    Y, mean, rstd = orc.layer_norm_fwd(X, W, B, d.eps)
    DX, DW, DB = orc.layer_norm_bwd(X, W, DY, d.eps)
    close_f32(orc.to_julia(r.Y), Y)
    close_f32(orc.to_julia(r.Mean), mean, tol=1e-5 if N > 1 else 1e-5)
    close_f32(orc.to_julia(r.Rstd), rstd)
    close_f32(orc.to_julia(r.DX), DX)
    close_f32(orc.to_julia(r.FINAL_DW), DW)
    close_f32(orc.to_julia(r.FINAL_DB), DB)
    # the reference's own criterion (layernorm.jl:299,311-313)
    for got, ref in ((r.Y, Y), (r.DX, DX), (r.FINAL_DW, DW), (r.FINAL_DB, DB)):
        assert orc.isapprox(ref, orc.to_julia(got), rtol=1e-2)


@pytest.mark.parametrize("M,N,G", [(300, 12288, 64), (37, 8196, 8), (70, 10240, 256), (3, 16380, 2), (1, 16384, 1), (513, 16384, 64)])
def test_layernorm_bwd_wide_rows(ct, orc, M, N, G):
    """Rows of 8192 to 16384 elements: the backward kernel whose row in flight lands in LDS (one, several and more
    workgroups than rows per partial slot; rows that fill 1024 lanes x 4 vectors and rows that leave lanes idle)."""
    d = layernorm.prepare(M=M, N=N, GROUP_SIZE_M=G)
    ct.layer_norm_fwd(d.X, d.W, d.B, d.Y, d.Mean, d.Rstd, d.eps, 1024)
    d.partials.zero_()
    ct.layer_norm_bwd_dx_partial_dwdb(d.DX, d.DY, d.DW_partial, d.DB_partial, d.X, d.W, d.Mean, d.Rstd, d.Locks, G, 1024)
    assert ct.last_variant() == "ln_bwd_wide_b1024_v4_lds_lookahead"
    ct.layer_norm_bwd_dwdb(d.DW_partial, d.DB_partial, d.FINAL_DW, d.FINAL_DB, 32, 1024)
    X, W, DY = (orc.to_julia(t) for t in (d.X, d.W, d.DY))
    DX, DW, DB = orc.layer_norm_bwd(X, W, DY, d.eps)
    close_f32(orc.to_julia(d.DX), DX)
    close_f32(orc.to_julia(d.FINAL_DW), DW)
    close_f32(orc.to_julia(d.FINAL_DB), DB)


@pytest.mark.parametrize("M,N,G,variant", [(130, 32768, 64, "ln_bwd_two_pass_b512_v16"), (37, 16388, 8, "ln_bwd_two_pass_b512_v16"),
                                           (300, 20000, 256, "ln_bwd_two_pass_b512_v16"), (5, 24580, 1, "ln_bwd_two_pass_b512_v16"),
                                           (9, 32772, 4, "ln_bwd_long_b256"), (6, 20001, 4, "ln_bwd_long_b256")])
def test_layernorm_bwd_rows_beyond_the_register_kernels(ct, orc, M, N, G, variant):
    """Rows of 16385 to 32768 aligned elements: dW / dB of a lane's columns in registers, the row walked twice (vectors
    that lie past the end of the row for every lane are skipped, the last partly used one is clamped); longer or
    misaligned rows: the kernel that adds every element to the partial slots."""
    d = layernorm.prepare(M=M, N=N, GROUP_SIZE_M=G)
    ct.layer_norm_fwd(d.X, d.W, d.B, d.Y, d.Mean, d.Rstd, d.eps, 1024)
    d.partials.zero_()
    d.DX.fill_(float("nan"))
    ct.layer_norm_bwd_dx_partial_dwdb(d.DX, d.DY, d.DW_partial, d.DB_partial, d.X, d.W, d.Mean, d.Rstd, d.Locks, G, 1024)
    assert ct.last_variant() == variant
    ct.layer_norm_bwd_dwdb(d.DW_partial, d.DB_partial, d.FINAL_DW, d.FINAL_DB, 32, 1024)
    X, W, DY = (orc.to_julia(t) for t in (d.X, d.W, d.DY))
    DX, DW, DB = orc.layer_norm_bwd(X, W, DY, d.eps)
    close_f32(orc.to_julia(d.DX), DX)
    close_f32(orc.to_julia(d.FINAL_DW), DW)
    close_f32(orc.to_julia(d.FINAL_DB), DB)


@pytest.mark.parametrize("M,N,variant", [(9, 65536, "ln_fwd_3pass_b1024_v4"), (5, 100003, "ln_fwd_3pass_b1024"),
                                         (1030, 32772, "ln_fwd_3pass_b256_v4"), (1025, 32771, "ln_fwd_3pass_b256"),
                                         (1030, 16388, "ln_fwd_regs_b1024_v8"), (1025, 16387, "ln_fwd_regs_b1024_v8"),
                                         (300, 32768, "ln_fwd_regs_b1024_v8"), (7, 20001, "ln_fwd_regs_b1024_v8")])
def test_layernorm_fwd_rows_too_long_for_registers(ct, orc, M, N, variant):
    """Rows beyond 16384 elements: up to 32768 in the registers of 1024 lanes (eight vectors per lane, W and B asked
    for after the reductions), beyond that three passes, 16-byte accesses when every row allows them, 1024 lanes per
    row when there are fewer than 1024 rows."""
    rng = np.random.default_rng(3)
    X = torch.from_numpy(rng.standard_normal((M, N), dtype=np.float32)).cuda()
    W = torch.from_numpy(rng.standard_normal(N, dtype=np.float32)).cuda(); B = torch.from_numpy(rng.standard_normal(N, dtype=np.float32)).cuda()
    Y = torch.full_like(X, float("nan")); Mean = torch.empty(M, device="cuda"); Rstd = torch.empty(M, device="cuda")
    ct.layer_norm_fwd(X, W, B, Y, Mean, Rstd, 1e-5, 1024)
    assert ct.last_variant() == variant
    x = X.cpu().numpy().astype(np.float64)
    mean = x.mean(axis=1); var = x.var(axis=1); rstd = 1.0 / np.sqrt(var + 1e-5)
    ref = (x - mean[:, None]) * rstd[:, None] * W.cpu().numpy().astype(np.float64) + B.cpu().numpy().astype(np.float64)
    np.testing.assert_allclose(Mean.cpu().numpy(), mean, rtol=0, atol=2e-6)
    np.testing.assert_allclose(Rstd.cpu().numpy(), rstd, rtol=2e-5)
    np.testing.assert_allclose(Y.cpu().numpy(), ref, rtol=0, atol=2e-4)


def test_layernorm_partials_accumulate_into_caller_buffers(ct, orc):
    """The partial kernel ADDS into DW/DB (the reference's critical section loads, adds and
    stores, layernorm.jl:159-163): pre-loading the slots shifts the final sums by exactly
    that amount; slot g only receives rows m = g mod GROUP_SIZE_M."""
    d = layernorm.prepare(M=40, N=256, GROUP_SIZE_M=8)
    ct.layer_norm_fwd(d.X, d.W, d.B, d.Y, d.Mean, d.Rstd, d.eps, 256)
    d.DW_partial.zero_(); d.DB_partial.zero_()
    ct.layer_norm_bwd_dx_partial_dwdb(d.DX, d.DY, d.DW_partial, d.DB_partial, d.X, d.W, d.Mean, d.Rstd, None, 8, 256)
    DY = orc.to_julia(d.DY).astype(np.float64)
    db_slots = orc.to_julia(d.DB_partial)
    for g in range(8):
        close_f32(db_slots[:, g], DY[:, g::8].sum(axis=1))
    d.DW_partial.fill_(1.0); d.DB_partial.fill_(2.0)
    ct.layer_norm_bwd_dx_partial_dwdb(d.DX, d.DY, d.DW_partial, d.DB_partial, d.X, d.W, d.Mean, d.Rstd, d.Locks, 8, 256)
    ct.layer_norm_bwd_dwdb(d.DW_partial, d.DB_partial, d.FINAL_DW, d.FINAL_DB, 32, 256)
    _, DW, DB = orc.layer_norm_bwd(orc.to_julia(d.X), orc.to_julia(d.W), DY, d.eps)
    close_f32(orc.to_julia(d.FINAL_DW), DW + 8.0)
    close_f32(orc.to_julia(d.FINAL_DB), DB + 16.0)


def test_layernorm_full_size(orc):
    d = layernorm.prepare(benchmark=True)
    r = layernorm.run(d)
    X, W, B, DY = (orc.to_julia(t) for t in (d.X, d.W, d.B, d.DY))
    Y, mean, rstd = orc.layer_norm_fwd(X, W, B, d.eps)
    DX, DW, DB = orc.layer_norm_bwd(X, W, DY, d.eps)
    close_f32(orc.to_julia(r.Y), Y)
    close_f32(orc.to_julia(r.Rstd), rstd)
    close_f32(orc.to_julia(r.DX), DX)
    close_f32(orc.to_julia(r.FINAL_DW), DW)
    close_f32(orc.to_julia(r.FINAL_DB), DB)


def test_second_dimension_beyond_65535(ct):
    """A strided 2-D vadd and a transpose whose second dimension exceeds the 65535 workgroups one grid
    dimension holds here (the reference's grids take 2^24 - 1 blocks per dimension)."""
    rng = np.random.default_rng(12)
    n = 70_003
    A = torch.from_numpy(rng.random((n, 40), dtype=np.float32)).cuda()
    B = torch.from_numpy(rng.random((n, 40), dtype=np.float32)).cuda()
    C = torch.zeros(n, 40, device="cuda")
    ct.vec_add_kernel_2d(A[:, ::2], B[:, ::2], C[:, ::2], 16, 16)     # dimension 0 strided: the element-wise 2-D kernel
    assert ct.last_variant() == "vadd_2d_strided"
    assert torch.equal(C[:, ::2], A[:, ::2] + B[:, ::2]) and bool((C[:, 1::2] == 0).all())
    # one-byte elements take the generic transpose; 64-row tiles along n: 65536 * 64 < n
    m, nn = 8, 65_540 * 64 + 5
    x = torch.from_numpy(rng.integers(0, 255, (nn, m), dtype=np.uint8)).cuda().view(torch.float8_e4m3fn)
    y = torch.empty((m, nn), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    ct.transpose_kernel(x, y, 64, 64)
    assert torch.equal(y.view(torch.uint8), x.view(torch.uint8).t())
