"""GPU parity tests for matmul / batch matmul through the C ABI against the float64 oracle.
Shapes: the reference examples' ``main()`` lists (matmul.jl:156-165, batchmatmul.jl:161-169),
the ragged 200x100x300 case of docs/src/tutorials/matmul.md:225-256, the 64x16x64 case of
test/device/tile.jl:1036-1066, plus strided / misaligned / degenerate cases.

Tolerances (stated against a float64 evaluation of ``A*B`` on the same inputs):
  fp32 inputs : |err| <= 1e-5 * (|ref| + max|ref|)       (true fp32 MFMA, fp32 accumulate)
  f16 / bf16  : |err| <= 2e-2 * (|ref| + max|ref|) when C is f32; the same plus one output
                rounding (2^-11 / 2^-8 relative) when C is stored in the input type.
  fp8 (E4M3FN / E5M2 operands, ext/DLFP8TypesExt.jl:15-19): the reference compares with ``==``
                against ``Float32.(a) * Float32.(b)`` on exactly representable operands
                (test/extensions/DLFP8Types.jl:143-152), and so do the tests here (products and fp32
                sums are exact); random operands: 2e-2 as above against float64 on the decoded values.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd.examples import matmul, batchmatmul  # noqa: E402


def check(got, ref, tol):
    got = np.asarray(got, dtype=np.float64)
    err = np.abs(got - ref)
    bound = tol * (np.abs(ref) + np.abs(ref).max())
    assert np.all(err <= bound), f"max err {err.max():.3e}, worst ratio {np.max(err / np.maximum(bound, 1e-300)):.3f}"


@pytest.mark.parametrize("M,N,K,tm,tn,tk", [(256, 256, 256, 32, 32, 32), (512, 512, 512, 64, 64, 64),
                                            (256, 512, 128, 32, 32, 32), (1024, 1024, 1024, 64, 64, 64),
                                            (200, 100, 300, 64, 64, 64), (64, 64, 16, 32, 32, 16),
                                            (1, 1, 1, 64, 64, 64), (129, 65, 33, 64, 64, 64), (5, 700, 9, 64, 64, 64)])
def test_matmul_f32(orc, M, N, K, tm, tn, tk):
    d = matmul.prepare(M=M, N=N, K=K)
    r = matmul.run(d, tm=tm, tn=tn, tk=tk)
    ref = orc.matmul(orc.to_julia(d.A), orc.to_julia(d.B))
    check(orc.to_julia(r.C), ref, 1e-5)
    assert orc.isapprox(orc.to_julia(r.C), ref, rtol=1e-2)  # matmul.jl:98-101


@pytest.mark.parametrize("T", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (512, 256, 1024), (200, 100, 300), (64, 64, 16), (33, 17, 41),
                                   (1024, 768, 512), (256, 256, 64), (512, 1024, 192), (8, 8, 8)])
@pytest.mark.parametrize("out32", [True, False])
def test_matmul_16bit(orc, T, M, N, K, out32):
    d = matmul.prepare(M=M, N=N, K=K, T=T, out_T=torch.float32 if out32 else None, dist="normal64")
    r = matmul.run(d)
    ref = orc.matmul(orc.to_julia(d.A), orc.to_julia(d.B))
    extra = 0.0 if out32 else (2.0 ** -11 if T == torch.float16 else 2.0 ** -8)
    check(orc.to_julia(r.C), ref, 2e-2 + extra)
    # far tighter in practice: fp32 accumulation of exactly-representable products
    assert np.abs(orc.to_julia(r.C).astype(np.float64) - ref).max() <= (1e-4 + 2 * extra) * np.abs(ref).max() + 1e-6


def test_matmul_integer_valued_inputs_are_exact(ct, orc):
    """Small-integer f16 operands: every product and partial sum is exact in fp32, so the
    result must equal the integer matrix product bit for bit (catches any operand
    permutation inside the MFMA / transpose-read path)."""
    rng = np.random.default_rng(0)
    for (M, N, K) in [(256, 256, 256), (96, 160, 80), (512, 512, 1024)]:
        A = rng.integers(-4, 5, (M, K)).astype(np.float32); B = rng.integers(-4, 5, (K, N)).astype(np.float32)
        At = orc.from_julia(A).to(torch.float16).cuda(); Bt = orc.from_julia(B).to(torch.float16).cuda()
        C = torch.empty((N, M), dtype=torch.float32, device="cuda")
        ct.matmul_kernel(At, Bt, C, 64, 64, 64)
        assert np.array_equal(orc.to_julia(C), A @ B)


@pytest.mark.parametrize("M,N,K,T,out32", [(1504, 1544, 200, torch.float16, True), (1500, 1540, 233, torch.float16, False),
                                           (2048, 1100, 96, torch.bfloat16, True), (1536, 1536, 32, torch.float16, True)])
def test_matmul_mid_tile_kernel_exact(ct, orc, M, N, K, T, out32):
    """The register-staged 128x128 kernel (shapes the direct-to-LDS kernel does not take: K below 256; enough
    tiles to fill half the chip):
    aligned interior tiles without predicates, ragged edges in M, N and K, rows that are not 16-byte
    aligned (M = 1500), one and many K steps.  Integer-valued operands make every sum exact, so any
    mistake in the tile mapping, the register look-ahead or the fragment reads changes the result."""
    rng = np.random.default_rng(M + K)
    A = rng.integers(-3, 4, (M, K)).astype(np.float32); B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    At = orc.from_julia(A).to(T).cuda(); Bt = orc.from_julia(B).to(T).cuda()
    C = torch.empty((N, M), dtype=torch.float32 if out32 else T, device="cuda")
    ct.matmul_kernel(At, Bt, C, 128, 128, 32)
    assert ct.last_variant() == "gemm16_mid_128x128x32"
    assert np.array_equal(orc.to_julia(C.float()), A @ B)      # (random sums of 233 terms stay far below 2048: exact in f16 too)


@pytest.mark.parametrize("M,N,K,T,out32,tile", [(2048, 2048, 256, torch.float16, True, "128x128"), (2048, 2048, 384, torch.float16, False, "128x128"),
                                                 (4096, 1024, 512, torch.bfloat16, True, "128x128"), (1024, 4096, 640, torch.bfloat16, False, "128x128"),
                                                 (512, 512, 768, torch.float16, True, "128x128"),
                                                 (4096, 4096, 256, torch.float16, False, "256x256"), (3072, 3072, 384, torch.bfloat16, True, "256x256"),
                                                 (8192, 2048, 640, torch.bfloat16, False, "256x256"),
                                                 (4096, 2048, 512, torch.float16, True, "256x128"), (2560, 2560, 256, torch.bfloat16, False, "256x128"),
                                                 (2048, 4096, 384, torch.float16, False, "256x128")])
def test_matmul_large_tile_kernel_exact(ct, orc, M, N, K, T, out32, tile):
    """Shapes that take the direct-to-LDS kernel (K >= 256) in each of its three tile sizes (chosen by
    the number of workgroups the problem gives the 256 CUs), with small-integer operands so the
    expected result is exact: checks the swizzled LDS layouts, the ring of stages (K/32 = 8, 12, 16, 20
    steps) and the tile -> workgroup mapping."""
    rng = np.random.default_rng(7)
    A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-2, 3, (K, N)).astype(np.float32)
    At = orc.from_julia(A).to(T).cuda(); Bt = orc.from_julia(B).to(T).cuda()
    C = torch.empty((N, M), dtype=torch.float32 if out32 else T, device="cuda")
    ct.matmul_kernel(At, Bt, C, 64, 64, 64)
    assert ct.last_variant() == f"gemm16_big_{tile}x32_ring4"
    ref = A @ B
    assert out32 or np.abs(ref).max() <= 256  # integers up to 256 are exact in bf16's 8 bits as well
    assert np.array_equal(orc.to_julia(C).astype(np.float32), ref)


@pytest.mark.parametrize("M,N,K,T,out32,pad", [
    (1500, 1540, 333, torch.float16, False, (0, 0)),     # dense, everything ragged: rows of A 4-byte, of B 2-byte aligned
    (4095, 520, 271, torch.float16, True, (0, 0)),       # odd M: the straddling chunk of A; K - Kd = 7
    (1501, 1536, 512, torch.bfloat16, True, (0, 0)),     # K a multiple of 8 with odd M: the last 8 rows of A go by registers
    (1536, 1500, 517, torch.float16, False, (0, 0)),     # M a multiple of 8, K not: B rows misaligned, K - Kd = 5
    (2048, 2048, 264, torch.float16, True, (3, 5)),      # aligned sizes inside parents with odd leading dimensions
    (1001, 1003, 1025, torch.bfloat16, False, (1, 2)),
    (4100, 4097, 265, torch.float16, True, (0, 0)),      # 256 x 128 tiles
])
def test_matmul_large_tile_kernel_takes_misaligned_rows_and_ragged_sizes(ct, orc, M, N, K, T, out32, pad):
    """The direct-to-LDS kernel on rows that are not 16-byte aligned and on M / K that are not multiples of 8 (the K
    tail and, with a ragged M, the last rows of A are one register-fed MFMA step).  Exact integer sums.  The operands
    are views: the cells right behind every row of A and B and behind the arrays hold NaN, so a value taken from
    past an edge shows; C is a view of a buffer filled with a sentinel."""
    rng = np.random.default_rng(M + K)
    A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-2, 3, (K, N)).astype(np.float32)
    lda, ldb = M + pad[0], K + pad[1]
    Aflat = torch.full((K * lda + 16,), float("nan"), dtype=T, device="cuda")
    Bflat = torch.full((N * ldb + 16,), float("nan"), dtype=T, device="cuda")
    Av = Aflat[:K * lda].view(K, lda)[:, :M]; Bv = Bflat[:N * ldb].view(N, ldb)[:, :K]
    Av.copy_(orc.from_julia(A).to(T)); Bv.copy_(orc.from_julia(B).to(T))
    buf = torch.full((N + 2, M + 9), -77.0, dtype=torch.float32 if out32 else T, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Av, Bv, C, 64, 64, 64)
    assert ct.last_variant().startswith("gemm16_big_") and "splitk" not in ct.last_variant(), ct.last_variant()
    ref = A @ B
    assert out32 or np.abs(ref).max() <= (2048 if T == torch.float16 else 256)
    assert np.array_equal(orc.to_julia(C.contiguous()).astype(np.float32), ref)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


@pytest.mark.parametrize("M,N,K,T,out32,pad", [
    (4097, 4096, 1024, torch.float16, True, (0, 0)),      # one row more than 16 x 16 tiles: the strip starts inside the main part
    (4096, 4100, 1032, torch.float16, False, (0, 0)),     # four columns more
    (4100, 4130, 2048, torch.bfloat16, True, (3, 1)),     # both, in parents with odd leading dimensions
    (4160, 4096, 1027, torch.float16, True, (0, 0)),      # 64 rows more, K off the chunks of 8
    (4097, 4096, 1024, torch.float32, True, (0, 0)),      # fp32 operands: a strip of four rows, three of them written twice
    (4096, 4352, 1030, torch.float32, True, (1, 3)),      # a whole last column of tiles
])
def test_matmul_whole_rounds_plus_a_thin_strip_are_launched_apart(ct, orc, M, N, K, T, out32, pad):
    """A product whose 256 x 256 tiles are whole rounds of the 256 CUs plus a last row or column of tiles goes out as the
    product without that strip (or both) and the strip(s) as small products of their own, where the estimates say that
    saves a round.  Exact integer sums; operands and C are views with NaN / a sentinel behind every row, as in the
    test above."""
    rng = np.random.default_rng(M + N)
    A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-2, 3, (K, N)).astype(np.float32)
    lda, ldb = M + pad[0], K + pad[1]
    Aflat = torch.full((K * lda + 16,), float("nan"), dtype=T, device="cuda")
    Bflat = torch.full((N * ldb + 16,), float("nan"), dtype=T, device="cuda")
    Av = Aflat[:K * lda].view(K, lda)[:, :M]; Bv = Bflat[:N * ldb].view(N, ldb)[:, :K]
    Av.copy_(orc.from_julia(A).to(T)); Bv.copy_(orc.from_julia(B).to(T))
    buf = torch.full((N + 2, M + 9), -77.0, dtype=torch.float32 if out32 else T, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Av, Bv, C, 64, 64, 64)
    assert ct.last_variant() == ("gemm32_big_256x256x16_ring4" if T == torch.float32 else "gemm16_big_256x256x32_ring4") + "+edge_strips", ct.last_variant()
    ref = A @ B
    assert out32 or np.abs(ref).max() <= 2048
    assert np.array_equal(orc.to_julia(C.contiguous()).astype(np.float32), ref)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


def test_batch_matmul_large_tile_kernel_ragged(ct, orc):
    """The same through mi_batch_matmul_kernel: three dense 1023 x 1030 x 515 products."""
    rng = np.random.default_rng(11)
    M, N, K, nb = 1023, 1030, 515, 3
    A = rng.integers(-1, 2, (M, K, nb)).astype(np.float32); B = rng.integers(-2, 3, (K, N, nb)).astype(np.float32)
    At = orc.from_julia(A).to(torch.float16).cuda(); Bt = orc.from_julia(B).to(torch.float16).cuda()
    C = torch.empty((nb, N, M), dtype=torch.float32, device="cuda")
    ct.batch_matmul_kernel(At, Bt, C, 64, 64, 64)
    assert ct.last_variant().startswith("gemm16_big_"), ct.last_variant()
    assert np.array_equal(orc.to_julia(C), np.einsum("mkb,knb->mnb", A, B))


@pytest.mark.parametrize("M,N,K,T,out32", [(512, 512, 4096, torch.float16, True), (512, 512, 4096, torch.bfloat16, False),
                                            (1024, 1024, 8192, torch.float16, False), (256, 256, 4096, torch.float16, True),
                                            (520, 500, 4000, torch.float16, True), (264, 1001, 3080, torch.bfloat16, False)])
def test_matmul_split_over_k_exact(ct, orc, M, N, K, T, out32):
    """Few tiles and a long K: the 128 x 128 direct-to-LDS kernel runs in several parts along K that write fp32
    partial sums into the library's static scratch, and a second kernel adds the parts in fixed order.  Exact
    integer sums (K off the part grid, M and N off the tile grid included); A and B are views of buffers whose
    cells past K hold NaN and C is a view of a larger buffer filled with a sentinel."""
    rng = np.random.default_rng(M + K)
    A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-1, 2, (K, N)).astype(np.float32)
    Abuf = torch.full((K + 128, M), float("nan"), dtype=T, device="cuda"); Bbuf = torch.full((N, K + 128), float("nan"), dtype=T, device="cuda")
    Abuf[:K] = orc.from_julia(A).to(T).cuda(); Bbuf[:, :K] = orc.from_julia(B).to(T).cuda()
    buf = torch.full((N + 3, M + 24), -77.0, dtype=torch.float32 if out32 else T, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Abuf[:K], Bbuf[:, :K], C, 64, 64, 64)
    assert ct.last_variant().startswith("gemm16_big_128x128x32_ring4_splitk")
    ref = A @ B
    assert out32 or np.abs(ref).max() <= (2048 if T == torch.float16 else 256)   # integers the output type holds exactly
    assert np.array_equal(orc.to_julia(C.contiguous()).astype(np.float32), ref)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


@pytest.mark.parametrize("M,N,K,pad", [(512, 512, 4096, (1, 3)), (264, 1001, 3080, (5, 1)), (520, 500, 4000, (2, 2))])
def test_matmul_split_over_k_on_misaligned_rows(ct, orc, M, N, K, pad):
    """The split over K with operands whose rows are not 16-byte aligned (views with odd leading dimensions; M and K
    multiples of 8, as the split wants them): the parts' transfers take the misaligned rows like the plain kernel's.
    Exact integer sums, NaN around the operands."""
    rng = np.random.default_rng(M + K + 1)
    A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-1, 2, (K, N)).astype(np.float32)
    lda, ldb = M + pad[0], K + pad[1]
    Aflat = torch.full((K * lda + 16,), float("nan"), dtype=torch.float16, device="cuda")
    Bflat = torch.full((N * ldb + 16,), float("nan"), dtype=torch.float16, device="cuda")
    Av = Aflat[:K * lda].view(K, lda)[:, :M]; Bv = Bflat[:N * ldb].view(N, ldb)[:, :K]
    Av.copy_(orc.from_julia(A).to(torch.float16)); Bv.copy_(orc.from_julia(B).to(torch.float16))
    C = torch.full((N, M), -77.0, device="cuda")
    ct.matmul_kernel(Av, Bv, C, 64, 64, 64)
    assert ct.last_variant().startswith("gemm16_big_128x128x32_ring4_splitk"), ct.last_variant()
    assert np.array_equal(orc.to_julia(C), A @ B)


def test_matmul_split_over_k_is_reproducible_and_ordered_across_streams(ct, orc):
    """The parts are added in a fixed order, so two runs give the same bits; launches from two streams share the
    scratch and are ordered by the library, so alternating between streams still gives every product its own
    result.  Random f16 data against the float64 product."""
    rng = np.random.default_rng(21)
    M = N = 512; K = 4096
    mats = []
    for i in range(3):
        a = (rng.standard_normal((M, K)) / 8).astype(np.float32); b = (rng.standard_normal((K, N)) / 8).astype(np.float32)
        mats.append((orc.from_julia(a).to(torch.float16).cuda(), orc.from_julia(b).to(torch.float16).cuda()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.empty((N, M), dtype=torch.float32, device="cuda") for _ in range(6)]
    for i in range(6):
        At, Bt = mats[i % 3]
        ct.matmul_kernel(At, Bt, outs[i], 64, 64, 64, stream=streams[i % 2])
    assert ct.last_variant().startswith("gemm16_big_128x128x32_ring4_splitk")
    torch.cuda.synchronize()
    for i in range(3):
        assert torch.equal(outs[i], outs[i + 3])
        At, Bt = mats[i]
        ref = orc.to_julia(At).astype(np.float64) @ orc.to_julia(Bt).astype(np.float64)
        got = orc.to_julia(outs[i]).astype(np.float64)
        assert np.abs(got - ref).max() <= 1e-5 * (np.abs(ref).max() + 1.0) * 4


def test_batch_matmul_split_over_k_exact(ct, orc):
    """Two entries of 512 x 512 x 8192: 32 tiles, split over K as well."""
    rng = np.random.default_rng(5)
    Bn, M, N, K = 2, 512, 512, 8192
    A = rng.integers(-1, 2, (Bn, M, K)).astype(np.float32); B = rng.integers(-1, 2, (Bn, K, N)).astype(np.float32)
    At = torch.from_numpy(np.ascontiguousarray(A.transpose(0, 2, 1))).to(torch.float16).cuda()   # Julia (M, K, Bn)
    Bt = torch.from_numpy(np.ascontiguousarray(B.transpose(0, 2, 1))).to(torch.float16).cuda()   # Julia (K, N, Bn)
    C = torch.empty((Bn, N, M), dtype=torch.float32, device="cuda")
    ct.batch_matmul_kernel(At, Bt, C, 64, 64, 64)
    assert ct.last_variant().startswith("gemm16_big_128x128x32_ring4_splitk")
    got = C.cpu().numpy().transpose(0, 2, 1)
    assert np.array_equal(got, A @ B)


@pytest.mark.parametrize("M,N,K,T,out32,tile", [(2040, 2000, 256, torch.float16, True, "128x128"), (2056, 2311, 384, torch.bfloat16, False, "256x128"),
                                                 (4000, 4001, 256, torch.float16, False, "256x256"), (8, 16385, 256, torch.float16, True, "128x128"),
                                                 (2048, 2048, 264, torch.float16, True, "128x128"), (2040, 2000, 1000, torch.float16, False, "128x128"),
                                                 (2048, 2304, 376, torch.bfloat16, True, "256x128"), (4096, 4096, 4000, torch.float16, True, "256x256"),
                                                 (3072, 3081, 328, torch.bfloat16, False, "256x256"), (1096, 1001, 1064, torch.bfloat16, False, "128x128")])
def test_matmul_large_tile_kernel_ragged_edges(ct, orc, M, N, K, T, out32, tile):
    """M (a multiple of 8) and N off the tile grid on the direct-to-LDS kernel: edge tiles re-read the last
    valid rows on the way in and clip their stores.  K (a multiple of 8) off the 128 grid: the last
    group of four steps takes zeros for k >= K (remainders of 8, 104, 120 and 32 here; A and B are
    views of buffers whose cells past K hold NaN, which must not reach the result).  Exact integer
    sums; C is a view of a wider, taller buffer filled with a sentinel, which must come back
    untouched (remainders of 8 rows of m and of 7 / 1 columns of n included)."""
    rng = np.random.default_rng(M ^ N)
    A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-2, 3, (K, N)).astype(np.float32)
    # A is (M, K) column-major = torch (K, M): rows past K hold NaN; B is (K, N) = torch (N, K): columns past K hold NaN
    Abuf = torch.full((K + 128, M), float("nan"), dtype=T, device="cuda"); Bbuf = torch.full((N, K + 128), float("nan"), dtype=T, device="cuda")
    Abuf[:K] = orc.from_julia(A).to(T).cuda(); Bbuf[:, :K] = orc.from_julia(B).to(T).cuda()
    At, Bt = Abuf[:K], Bbuf[:, :K]
    buf = torch.full((N + 3, M + 24), -77.0, dtype=torch.float32 if out32 else T, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(At, Bt, C, 64, 64, 64)
    assert ct.last_variant() == f"gemm16_big_{tile}x32_ring4"       # every tile size of the kernel sees ragged M, N and K
    assert np.array_equal(orc.to_julia(C.contiguous()).astype(np.float32), A @ B)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


def test_matmul_direct_to_lds_kernel_shape_sweep(ct, orc):
    """Thirty seeded shapes with M, K multiples of 8 (K >= 256) and any N, so that every tile size of the
    direct-to-LDS kernel meets edges in M, N and K at many remainders; small-integer operands, exact sums."""
    rng = np.random.default_rng(2024)
    seen = set()
    for case in range(30):
        M = 8 * int(rng.integers(16, 420)); N = int(rng.integers(100, 3400)); K = 8 * int(rng.integers(32, 160))
        T = torch.float16 if case % 2 == 0 else torch.bfloat16
        out32 = case % 3 != 0
        A = rng.integers(-1, 2, (M, K)).astype(np.float32); B = rng.integers(-2, 3, (K, N)).astype(np.float32)
        At = orc.from_julia(A).to(T).cuda(); Bt = orc.from_julia(B).to(T).cuda()
        C = torch.full((N, M), -77.0, dtype=torch.float32 if out32 else T, device="cuda")
        ct.matmul_kernel(At, Bt, C, 64, 64, 64)
        v = ct.last_variant()
        if (-(-M // 128)) * (-(-N // 128)) >= 16:
            assert v.startswith("gemm16_big_"), (M, N, K, v)
        seen.add(v)
        assert np.array_equal(orc.to_julia(C).astype(np.float32), A @ B), (M, N, K, v)
    assert {"gemm16_big_128x128x32_ring4", "gemm16_big_256x128x32_ring4", "gemm16_big_256x256x32_ring4"} <= seen


@pytest.mark.parametrize("M,N,K,tile", [(2040, 2000, 256, "128x128"), (2056, 2311, 388, "256x128"), (4000, 4001, 132, "256x256"),
                                         (4, 16385, 128, "64x64"), (3072, 3081, 196, "128x128"), (1096, 1001, 1060, "64x64"),
                                         (2048, 2304, 376, "256x128"), (512, 512, 128, "64x64"), (4096, 4096, 320, "256x256"),
                                         (260, 250, 132, "64x64")])
def test_matmul_f32_direct_to_lds_kernel_exact(ct, orc, M, N, K, tile):
    """The fp32 direct-to-LDS kernel in each tile size: M and K multiples of 4 off the tile / 64 grid, any
    N.  Small-integer operands make every fp32 sum exact; A and B are views of buffers whose cells past K
    hold NaN, C a view of a wider, taller buffer of sentinels that must come back untouched."""
    rng = np.random.default_rng(M ^ N)
    A = rng.integers(-3, 4, (M, K)).astype(np.float32); B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    Abuf = torch.full((K + 64, M), float("nan"), device="cuda"); Bbuf = torch.full((N, K + 64), float("nan"), device="cuda")
    Abuf[:K] = orc.from_julia(A).cuda(); Bbuf[:, :K] = orc.from_julia(B).cuda()
    buf = torch.full((N + 3, M + 12), -77.0, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Abuf[:K], Bbuf[:, :K], C, 64, 64, 64)
    assert ct.last_variant() == f"gemm32_big_{tile}x16_ring4"
    assert np.array_equal(orc.to_julia(C.contiguous()), A @ B)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


@pytest.mark.parametrize("M,N,K,pad", [(2041, 2000, 259, (0, 0)), (1001, 1003, 1025, (1, 2)), (2048, 2050, 133, (3, 1)),
                                        (4095, 519, 132, (0, 0)), (1023, 1030, 515, (0, 0)), (2052, 2049, 128, (5, 5))])
def test_matmul_f32_direct_to_lds_kernel_takes_misaligned_rows_and_ragged_sizes(ct, orc, M, N, K, pad):
    """The fp32 direct-to-LDS kernel on rows that are not 16-byte aligned and on M / K that are not multiples of 4 (the K
    tail and, with a ragged M, the last row of A go through registers).  Exact integer sums; every cell around the
    operands holds NaN, C is a view of a buffer of sentinels."""
    rng = np.random.default_rng(M * 5 + K)
    A = rng.integers(-3, 4, (M, K)).astype(np.float32); B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    lda, ldb = M + pad[0], K + pad[1]
    Aflat = torch.full((K * lda + 8,), float("nan"), device="cuda"); Bflat = torch.full((N * ldb + 8,), float("nan"), device="cuda")
    Av = Aflat[:K * lda].view(K, lda)[:, :M]; Bv = Bflat[:N * ldb].view(N, ldb)[:, :K]
    Av.copy_(orc.from_julia(A)); Bv.copy_(orc.from_julia(B))
    buf = torch.full((N + 2, M + 7), -77.0, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Av, Bv, C, 64, 64, 64)
    assert ct.last_variant().startswith("gemm32_big_"), ct.last_variant()
    assert np.array_equal(orc.to_julia(C.contiguous()), A @ B)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


def test_batch_matmul_large_tile_kernel(ct, orc):
    rng = np.random.default_rng(8)
    M, K, N, Bn = 1024, 256, 1024, 4
    A = rng.integers(-2, 3, (M, K, Bn)).astype(np.float32); B = rng.integers(-2, 3, (K, N, Bn)).astype(np.float32)
    At = orc.from_julia(A).to(torch.float16).cuda(); Bt = orc.from_julia(B).to(torch.float16).cuda()
    C = torch.empty((Bn, N, M), dtype=torch.float16, device="cuda")
    ct.batch_matmul_kernel(At, Bt, C, 128, 128, 64)
    assert "big" in ct.last_variant()
    assert np.array_equal(orc.to_julia(C).astype(np.float32), np.einsum("mkb,knb->mnb", A, B))
    # the same through padded leading dimensions (views of wider buffers)
    Aw = torch.zeros((Bn, K, M + 64), dtype=torch.float16, device="cuda"); Aw[:, :, :M] = At
    Bw = torch.zeros((Bn, N, K + 8), dtype=torch.float16, device="cuda"); Bw[:, :, :K] = Bt
    C2 = torch.empty_like(C)
    ct.batch_matmul_kernel(Aw[:, :, :M], Bw[:, :, :K], C2, 128, 128, 64)
    assert "big" in ct.last_variant() and torch.equal(C, C2)


@pytest.mark.parametrize("T", [torch.float16, torch.float32])
@pytest.mark.parametrize("M,K,N,Bn", [(1024, 512, 2048, 8), (520, 264, 1001, 3), (2048, 320, 2040, 5), (256, 256, 384, 16)])
def test_batch_matmul_direct_to_lds_kernels_exact(ct, orc, T, M, K, N, Bn):
    """Batched problems on the direct-to-LDS kernels (16-bit and fp32): the (tile, batch entry) -> workgroup
    mapping with batch counts that are and are not multiples of 8, ragged tiles inside every entry, and
    padded leading dimensions / batch strides (views of wider buffers).  Small-integer operands: exact."""
    rng = np.random.default_rng(M + Bn)
    A = rng.integers(-2, 3, (M, K, Bn)).astype(np.float32); B = rng.integers(-2, 3, (K, N, Bn)).astype(np.float32)
    # (contiguous copies: numpy multiplies strided slices without BLAS, minutes at these sizes)
    ref = np.stack([np.ascontiguousarray(A[:, :, b]) @ np.ascontiguousarray(B[:, :, b]) for b in range(Bn)], axis=2)
    Aw = torch.zeros((Bn, K + 3, M + 16), dtype=T, device="cuda"); Aw[:, :K, :M] = orc.from_julia(A).to(T).cuda()
    Bw = torch.zeros((Bn, N + 2, K + 8), dtype=T, device="cuda"); Bw[:, :N, :K] = orc.from_julia(B).to(T).cuda()
    Cw = torch.full((Bn, N + 1, M + 4), -77.0, dtype=torch.float32, device="cuda")
    C = Cw[:, :N, :M]
    ct.batch_matmul_kernel(Aw[:, :K, :M], Bw[:, :N, :K], C, 128, 128, 64)
    assert ct.last_variant().startswith("gemm32_big_" if T == torch.float32 else "gemm16_big_")
    assert np.array_equal(orc.to_julia(C.contiguous()), ref)
    assert bool((Cw[:, N:] == -77.0).all()) and bool((Cw[:, :, M:] == -77.0).all())


def test_matmul_padded_leading_dims_and_misaligned(ct, orc):
    rng = np.random.default_rng(1)
    M, N, K = 100, 90, 70
    Abig = torch.from_numpy(rng.standard_normal((K, 128), dtype=np.float32)).to(torch.float16).cuda()
    Bbig = torch.from_numpy(rng.standard_normal((N, 77), dtype=np.float32)).to(torch.float16).cuda()
    Cbig = torch.full((N, 111), -5.0, dtype=torch.float32, device="cuda")
    A = Abig[:, 3:3 + M]      # Julia view(Abig, 4:103, :)  -> misaligned start, lda = 128
    B = Bbig[:, 1:1 + K]      # ldb = 77 (odd)
    C = Cbig[:, :M]
    ct.matmul_kernel(A, B, C, 64, 64, 64)
    ref = orc.matmul(orc.to_julia(A), orc.to_julia(B))
    check(orc.to_julia(C), ref, 2e-2)
    assert np.abs(orc.to_julia(C) - ref).max() < 1e-3
    assert torch.all(Cbig[:, M:] == -5.0)


@pytest.mark.parametrize("M,K,N,Batch,T", [(256, 128, 256, 4, torch.float32), (512, 256, 1024, 4, torch.float16),
                                           (130, 70, 96, 3, torch.float32), (64, 32, 48, 1, torch.float16),
                                           (100, 50, 60, 2, torch.bfloat16)])
def test_batch_matmul(orc, M, K, N, Batch, T):
    d = batchmatmul.prepare(M=M, K=K, N=N, Batch=Batch, T=T)
    r = batchmatmul.run(d)
    ref = orc.batch_matmul(orc.to_julia(d.A), orc.to_julia(d.B))
    tol = 1e-5 if T == torch.float32 else 2e-2 + (2.0 ** -11 if T == torch.float16 else 2.0 ** -8)
    check(orc.to_julia(r.C), ref, tol)
    assert orc.isapprox(orc.to_julia(r.C), ref, rtol=1e-2)  # batchmatmul.jl:97-106


def test_matmul_full_size_f16(orc):
    """4096^3 f16 -> f32 (the measured configuration): sampled rows/columns against float64,
    and linearity C(A, B1+B2) == C(A,B1) + C(A,B2) on integer-valued inputs (exact)."""
    d = matmul.prepare(benchmark=True, T=torch.float16, out_T=torch.float32, dist="normal64")
    r = matmul.run(d)
    A = orc.to_julia(d.A).astype(np.float64); B = orc.to_julia(d.B).astype(np.float64)
    C = orc.to_julia(r.C)
    rows = [0, 1, 255, 256, 2049, 4095]; cols = [0, 31, 32, 1000, 4095]
    ref_rows = A[rows] @ B
    check(C[rows], ref_rows, 2e-2)
    assert np.abs(C[rows] - ref_rows).max() <= 1e-4 * np.abs(ref_rows).max()
    ref_cols = A @ B[:, cols]
    assert np.abs(C[:, cols] - ref_cols).max() <= 1e-4 * np.abs(ref_cols).max()
    # checksum of checksums: sum over all of C equals (column sums of A) . (row sums of B)
    total = torch.sum(r.C.double()).item()
    expect = float(A.sum(axis=0) @ B.sum(axis=1))
    assert abs(total - expect) <= 1e-4 * np.abs(A).sum(axis=0) @ np.abs(B).sum(axis=1)


def test_batch_matmul_full_size_f32(orc):
    d = batchmatmul.prepare(benchmark=True)
    r = batchmatmul.run(d)
    A = orc.to_julia(d.A); B = orc.to_julia(d.B); C = orc.to_julia(r.C)
    for b in (0, 7):
        ref = A[:, :, b].astype(np.float64) @ B[:, :, b].astype(np.float64)
        check(C[:, :, b], ref, 1e-5)


# ---- fp8 operands ---------------------------------------------------------------------------------

FP8 = {"e4m3fn": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}


def fp8_tensor(orc, vals, fmt):
    """Exactly representable values (numpy, Julia shape) -> (device tensor of the fp8 type, codes)."""
    codes = (orc.e4m3fn_encode if fmt == "e4m3fn" else orc.e5m2_encode)(vals)
    dec = (orc.e4m3fn_decode if fmt == "e4m3fn" else orc.e5m2_decode)(codes)
    assert np.array_equal(dec, vals.astype(np.float32))
    return orc.from_julia(codes).view(FP8[fmt]).cuda(), codes


@pytest.mark.parametrize("fmt", ["e4m3fn", "e5m2"])
@pytest.mark.parametrize("acc", [torch.float32, torch.float16])
def test_matmul_fp8_reference_exact_case(ct, orc, fmt, acc):
    """test/extensions/DLFP8Types.jl:143-152: 16 x 16 operands drawn from {0, 0.5, 1}, result compared
    with ``==``, for both accumulator / result types the reference allows."""
    rng = np.random.default_rng(3)
    A = rng.integers(0, 3, (16, 16)) / 2.0; B = rng.integers(0, 3, (16, 16)) / 2.0
    At, Ac = fp8_tensor(orc, A, fmt); Bt, Bc = fp8_tensor(orc, B, fmt)
    C = torch.full((16, 16), -1.0, dtype=acc, device="cuda")
    ct.matmul_kernel(At, Bt, C, 16, 16, 16)
    assert ct.last_variant() == "gemm8_generic_64x64x64"
    assert np.array_equal(orc.to_julia(C).astype(np.float64), orc.fp8_matmul(Ac, Bc, fmt))


@pytest.mark.parametrize("fmt", ["e4m3fn", "e5m2"])
@pytest.mark.parametrize("M,N,K", [(200, 100, 300), (33, 17, 41), (64, 64, 16), (1, 1, 1), (129, 65, 33), (5, 700, 9),
                                   (512, 256, 1024), (256, 256, 64)])
def test_matmul_fp8_generic_kernel_exact(ct, orc, fmt, M, N, K):
    """Any shape on the register-staged fp8 kernel: ragged M, N, K, rows that are not 16-byte aligned
    (views of wider buffers whose cells past the edges hold NaN codes), C inside a buffer of sentinels.
    Operands are multiples of 1/2 up to 2 in magnitude: exact in both fp8 types, exact sums."""
    rng = np.random.default_rng(M * 7 + K)
    A = rng.integers(-4, 5, (M, K)) / 2.0; B = rng.integers(-4, 5, (K, N)) / 2.0
    At, Ac = fp8_tensor(orc, A, fmt); Bt, Bc = fp8_tensor(orc, B, fmt)
    nan = torch.full((1,), float("nan")).to(FP8[fmt]).view(torch.uint8).item()
    Abuf = torch.full((K + 3, M + 5), nan, dtype=torch.uint8, device="cuda").view(FP8[fmt])
    Bbuf = torch.full((N + 2, K + 7), nan, dtype=torch.uint8, device="cuda").view(FP8[fmt])
    Abuf.view(torch.uint8)[:K, 1:1 + M] = At.view(torch.uint8); Bbuf.view(torch.uint8)[:N, 3:3 + K] = Bt.view(torch.uint8)
    buf = torch.full((N + 3, M + 9), -77.0, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Abuf[:K, 1:1 + M], Bbuf[:N, 3:3 + K], C, 64, 64, 64)
    assert ct.last_variant() == "gemm8_generic_64x64x64"
    assert np.array_equal(orc.to_julia(C.contiguous()).astype(np.float64), orc.fp8_matmul(Ac, Bc, fmt))
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())
    # 16-byte aligned operands of the same problem take the vector loads of the same kernel
    C2 = torch.empty((N, M), device="cuda")
    ct.matmul_kernel(At, Bt, C2, 64, 64, 64)
    assert torch.equal(C2, C)


@pytest.mark.parametrize("M,N,K,fmt,out", [(4096, 4096, 512, "e4m3fn", torch.float32), (2048, 2304, 1040, "e5m2", torch.float16),
                                           (4000, 4001, 528, "e4m3fn", torch.float16), (1024, 512, 2048, "e5m2", torch.float32),
                                           (3072, 3081, 784, "e4m3fn", torch.bfloat16), (16, 16385, 512, "e5m2", torch.float32),
                                           (2064, 2000, 1296, "e4m3fn", torch.float32)])
def test_matmul_fp8_direct_to_lds_kernel_exact(ct, orc, M, N, K, fmt, out):
    """The fp8 direct-to-LDS kernel (256 x 256 tiles of 32x32x64 MFMAs, ring of four stages): M and K
    multiples of 16 off the tile / 256 grid, any N, K/64 = 8 ... 32 steps with remainders of 16, 48 and
    16 bytes of K in the last group.  Operands in {-1, -1/2, 0, 1/2, 1}: every sum is exact, so any slip
    in the byte-transposing LDS reads, the swizzles, the ring or the tile mapping changes the result.
    Cells past K hold NaN codes; C is a view of a buffer of sentinels that must come back untouched."""
    rng = np.random.default_rng(M ^ N ^ K)
    A = rng.integers(-2, 3, (M, K)) / 2.0; B = rng.integers(-2, 3, (K, N)) / 2.0
    At, Ac = fp8_tensor(orc, A, fmt); Bt, Bc = fp8_tensor(orc, B, fmt)
    nan = torch.full((1,), float("nan")).to(FP8[fmt]).view(torch.uint8).item()
    Abuf = torch.full((K + 128, M), nan, dtype=torch.uint8, device="cuda"); Bbuf = torch.full((N, K + 128), nan, dtype=torch.uint8, device="cuda")
    Abuf[:K] = At.view(torch.uint8); Bbuf[:, :K] = Bt.view(torch.uint8)
    buf = torch.full((N + 3, M + 48), -77.0, dtype=out, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Abuf.view(FP8[fmt])[:K], Bbuf.view(FP8[fmt])[:, :K], C, 64, 64, 64)
    assert ct.last_variant() == "gemm8_big_256x256x64_ring4"
    ref = orc.fp8_matmul(Ac, Bc, fmt)
    want = orc.to_julia(orc.from_julia(ref.astype(np.float32)).to(out).float())   # the exact fp32 sum, rounded once on the store
    assert np.array_equal(orc.to_julia(C.contiguous().float()), want)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


@pytest.mark.parametrize("M,N,K,fmt,out", [(4095, 2100, 529, "e4m3fn", torch.float32), (2049, 2049, 1031, "e5m2", torch.float16),
                                           (2051, 2048, 1024, "e4m3fn", torch.bfloat16), (2048, 2047, 1025, "e5m2", torch.float32),
                                           (2048, 2048, 528, "e4m3fn", torch.float32)])
def test_matmul_fp8_direct_to_lds_kernel_takes_misaligned_rows_and_ragged_sizes(ct, orc, M, N, K, fmt, out):
    """The fp8 direct-to-LDS kernel on rows that start at odd byte offsets (views at offsets 1 and 3 inside wider buffers) and
    on M / K that are not multiples of 16: the K tail and, with a ragged M, the last rows of A are one register-fed
    MFMA step.  Every cell outside the operands holds a NaN code; exact sums; C inside a buffer of sentinels."""
    rng = np.random.default_rng(M * 3 + K)
    A = rng.integers(-2, 3, (M, K)) / 2.0; B = rng.integers(-2, 3, (K, N)) / 2.0
    At, Ac = fp8_tensor(orc, A, fmt); Bt, Bc = fp8_tensor(orc, B, fmt)
    nan = torch.full((1,), float("nan")).to(FP8[fmt]).view(torch.uint8).item()
    Abuf = torch.full((K + 3, M + 5), nan, dtype=torch.uint8, device="cuda")
    Bbuf = torch.full((N + 2, K + 7), nan, dtype=torch.uint8, device="cuda")
    Abuf[:K, 1:1 + M] = At.view(torch.uint8); Bbuf[:N, 3:3 + K] = Bt.view(torch.uint8)
    buf = torch.full((N + 3, M + 9), -77.0, dtype=out, device="cuda")
    C = buf[:N, :M]
    ct.matmul_kernel(Abuf.view(FP8[fmt])[:K, 1:1 + M], Bbuf.view(FP8[fmt])[:N, 3:3 + K], C, 64, 64, 64)
    assert ct.last_variant() == "gemm8_big_256x256x64_ring4"
    ref = orc.fp8_matmul(Ac, Bc, fmt)
    want = orc.to_julia(orc.from_julia(ref.astype(np.float32)).to(out).float())
    assert np.array_equal(orc.to_julia(C.contiguous().float()), want)
    assert bool((buf[N:] == -77.0).all()) and bool((buf[:, M:] == -77.0).all())


def test_matmul_fp8_direct_to_lds_kernel_shape_sweep(ct, orc):
    """Sixteen seeded shapes with M, K multiples of 16 (K >= 512) and any N on the fp8 direct-to-LDS
    kernel; exact sums."""
    rng = np.random.default_rng(808)
    for case in range(16):
        M = 16 * int(rng.integers(32, 200)); N = int(rng.integers(600, 3000)); K = 16 * int(rng.integers(32, 120))
        fmt = "e4m3fn" if case % 2 == 0 else "e5m2"
        A = rng.integers(-2, 3, (M, K)) / 2.0; B = rng.integers(-2, 3, (K, N)) / 2.0
        At, Ac = fp8_tensor(orc, A, fmt); Bt, Bc = fp8_tensor(orc, B, fmt)
        C = torch.full((N, M), -77.0, device="cuda")
        ct.matmul_kernel(At, Bt, C, 64, 64, 64)
        v = ct.last_variant()
        if (-(-M // 256)) * (-(-N // 256)) >= 8:
            assert v == "gemm8_big_256x256x64_ring4", (M, N, K, v)
        assert np.array_equal(orc.to_julia(C).astype(np.float64), orc.fp8_matmul(Ac, Bc, fmt)), (M, N, K, v)


@pytest.mark.parametrize("M,K,N,Bn,big", [(512, 512, 512, 8, True), (528, 784, 1001, 3, True), (100, 70, 90, 5, False)])
def test_batch_matmul_fp8_exact(ct, orc, M, K, N, Bn, big):
    """batch_matmul_kernel on fp8 operands: both kernels, padded leading dimensions and batch strides."""
    rng = np.random.default_rng(M + Bn)
    A = rng.integers(-2, 3, (M, K, Bn)) / 2.0; B = rng.integers(-2, 3, (K, N, Bn)) / 2.0
    At, Ac = fp8_tensor(orc, A, "e4m3fn"); Bt, Bc = fp8_tensor(orc, B, "e4m3fn")
    ref = np.stack([orc.fp8_matmul(np.ascontiguousarray(Ac[:, :, b]), np.ascontiguousarray(Bc[:, :, b])) for b in range(Bn)], axis=2)
    Aw = torch.zeros((Bn, K + 3, M + 16), dtype=torch.uint8, device="cuda"); Aw[:, :K, :M] = At.view(torch.uint8)
    Bw = torch.zeros((Bn, N + 2, K + 16), dtype=torch.uint8, device="cuda"); Bw[:, :N, :K] = Bt.view(torch.uint8)
    Cw = torch.full((Bn, N + 1, M + 4), -77.0, device="cuda")
    C = Cw[:, :N, :M]
    ct.batch_matmul_kernel(Aw.view(FP8["e4m3fn"])[:, :K, :M], Bw.view(FP8["e4m3fn"])[:, :N, :K], C, 128, 128, 64)
    assert ct.last_variant() == ("gemm8_big_256x256x64_ring4" if big else "gemm8_generic_64x64x64")
    assert np.array_equal(orc.to_julia(C.contiguous()).astype(np.float64), ref)
    assert bool((Cw[:, N:] == -77.0).all()) and bool((Cw[:, :, M:] == -77.0).all())


def test_matmul_fp8_rejects_mixed_operand_types(ct):
    """lhs and rhs must share the type (src/compiler/intrinsics/core.jl:589-590); C may not be fp8."""
    a = torch.zeros((64, 64), dtype=torch.uint8, device="cuda")
    C = torch.empty((64, 64), device="cuda")
    with pytest.raises(ct.MiError) as e:
        ct.matmul_kernel(a.view(torch.float8_e4m3fn), a.view(torch.float8_e5m2), C, 64, 64, 64)
    assert e.value.code == ct.MI_E_DTYPE
    with pytest.raises(ct.MiError) as e:
        ct.matmul_kernel(a.view(torch.float8_e4m3fn), a.view(torch.float8_e4m3fn), a.view(torch.float8_e4m3fn), 64, 64, 64)
    assert e.value.code == ct.MI_E_DTYPE


@pytest.mark.parametrize("fmt", ["e4m3fn", "e5m2"])
def test_matmul_full_size_fp8(ct, orc, fmt):
    """4096^3 fp8 -> f32: operands ~ N(0, 1) rounded to the fp8 type; sampled rows / columns against float64
    on the decoded operands, and the checksum of checksums over all of C."""
    rng = np.random.default_rng(9)
    enc, dec = (orc.e4m3fn_encode, orc.e4m3fn_decode) if fmt == "e4m3fn" else (orc.e5m2_encode, orc.e5m2_decode)
    Ac = enc(rng.standard_normal((4096, 4096), dtype=np.float32)); Bc = enc(rng.standard_normal((4096, 4096), dtype=np.float32))
    At = orc.from_julia(Ac).view(FP8[fmt]).cuda(); Bt = orc.from_julia(Bc).view(FP8[fmt]).cuda()
    Ct = torch.empty((4096, 4096), device="cuda")
    ct.matmul_kernel(At, Bt, Ct, 64, 64, 64)
    assert ct.last_variant() == "gemm8_big_256x256x64_ring4"
    A = dec(Ac).astype(np.float64); B = dec(Bc).astype(np.float64); C = orc.to_julia(Ct)
    rows = [0, 1, 255, 256, 2049, 4095]; cols = [0, 31, 32, 1000, 4095]
    ref_rows = A[rows] @ B
    check(C[rows], ref_rows, 2e-2)
    assert np.abs(C[rows] - ref_rows).max() <= 1e-4 * np.abs(ref_rows).max()      # exact products, fp32 sums of 4096 terms
    ref_cols = A @ B[:, cols]
    assert np.abs(C[:, cols] - ref_cols).max() <= 1e-4 * np.abs(ref_cols).max()
    total = torch.sum(Ct.double()).item()
    expect = float(A.sum(axis=0) @ B.sum(axis=1))
    assert abs(total - expect) <= 1e-4 * np.abs(A).sum(axis=0) @ np.abs(B).sum(axis=1)


@pytest.mark.parametrize("T", [torch.float16, torch.float32, torch.float8_e4m3fn])
def test_batch_matmul_more_than_65535_entries(ct, orc, T):
    """batch_matmul_kernel's grid is (cld(M,tm), cld(N,tn), Batch) with up to 2^24 - 1 blocks per dimension
    (batchmatmul.jl:78-80, src/launch.jl:743): 70 000 small entries, integer operands, exact."""
    rng = np.random.default_rng(21)
    Bn, M, K, N = 70_000, 16, 16, 8
    A = rng.integers(-2, 3, (Bn, K, M)).astype(np.float32); B = rng.integers(-2, 3, (Bn, N, K)).astype(np.float32)
    At = torch.from_numpy(A).to(T).cuda(); Bt = torch.from_numpy(B).to(T).cuda()
    C = torch.empty((Bn, N, M), dtype=torch.float32, device="cuda")
    ct.batch_matmul_kernel(At, Bt, C, 16, 8, 16)
    ref = torch.bmm(torch.from_numpy(B), torch.from_numpy(A))       # torch (N,K) x (K,M) = Julia (A * B)^T
    assert torch.equal(C.cpu(), ref)
