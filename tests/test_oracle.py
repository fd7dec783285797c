"""Pins the CPU oracle (oracle/cutile_oracle.py, oracle/oracle_int.c) without a GPU.

The reference ships no golden files (every reference test draws its inputs in-process), so
the oracle is pinned by (a) the literal known-answer data the reference's tests do hold,
(b) independent library routines already in this image (torch CPU, scipy), (c) invariants
and brute-force loops chosen so that a dropped term, a wrong sign / index or a transposed
operand fails.  None of these tests retypes the oracle's own formula.
"""
import ctypes
import itertools
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import cutile_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


@pytest.fixture(scope="module")
def corc():
    path = os.path.join(ROOT, "oracle", "liboracle_int.so")
    if not os.path.exists(path):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(path)
    lib.oracle_e4m3fn_decode.restype = ctypes.c_float
    lib.oracle_e4m3fn_decode.argtypes = [ctypes.c_uint8]
    lib.oracle_e4m3fn_encode.restype = ctypes.c_uint8
    lib.oracle_e4m3fn_encode.argtypes = [ctypes.c_float]
    lib.oracle_moe_align_tile_size.restype = ctypes.c_int64
    return lib


# ---- swizzle_2d ---------------------------------------------------------------------------

@pytest.mark.parametrize("M,N,tm,tn,G", [(4096, 4096, 64, 64, 8), (200, 100, 64, 64, 8),
                                          (1000, 130, 32, 64, 8), (64, 64, 64, 64, 8),
                                          (9 * 16, 5 * 16, 16, 16, 4), (17 * 8, 3 * 8, 8, 8, 8)])
def test_swizzle_is_a_bijection_with_grouped_order(M, N, tm, tn, G):
    nm, nn = orc.cld(M, tm), orc.cld(N, tn)
    seen = [orc.swizzle_2d(M, N, tm, tn, G, bid) for bid in range(1, nm * nn + 1)]
    assert sorted(seen) == sorted(itertools.product(range(1, nm + 1), range(1, nn + 1)))
    # grouped ordering: within the first group the m index cycles fastest over min(G, nm) rows
    g = min(G, nm)
    assert [s[0] for s in seen[:g]] == list(range(1, g + 1))
    assert all(s[1] == 1 for s in seen[:g])
    # all blocks of group k come before any block of group k+1
    groups = [(bm - 1) // G for bm, _ in seen]
    assert groups == sorted(groups)


def test_swizzle_c_restatement_agrees(corc):
    bm, bn = ctypes.c_int32(), ctypes.c_int32()
    for (M, N, tm, tn, G) in [(4096, 4096, 64, 64, 8), (200, 100, 64, 64, 8), (1000, 130, 32, 64, 8)]:
        for bid in range(1, orc.cld(M, tm) * orc.cld(N, tn) + 1):
            corc.oracle_swizzle_2d(M, N, tm, tn, G, bid, ctypes.byref(bm), ctypes.byref(bn))
            assert (bm.value, bn.value) == orc.swizzle_2d(M, N, tm, tn, G, bid)


# ---- matmul -------------------------------------------------------------------------------

def test_matmul_known_case_by_loops():
    """Shape of test/device/tile.jl:1036-1066 (M,K,N = 64,16,64), checked against scalar loops."""
    rng = np.random.default_rng(0)
    A = rng.random((64, 16), dtype=np.float32)
    B = rng.random((16, 64), dtype=np.float32)
    C = orc.matmul(A, B)
    ref = np.zeros((64, 64))
    for i in range(64):
        for j in range(64):
            ref[i, j] = sum(float(A[i, k]) * float(B[k, j]) for k in range(16))
    np.testing.assert_allclose(C, ref, rtol=1e-12)
    # not symmetric in its operands: a transposed-operand mistake fails
    assert not np.allclose(orc.matmul(A, B), orc.matmul(B.T, A.T))


def test_batch_matmul_batch_last():
    rng = np.random.default_rng(1)
    A = rng.standard_normal((5, 7, 3)); B = rng.standard_normal((7, 4, 3))
    C = orc.batch_matmul(A, B)
    assert C.shape == (5, 4, 3)
    np.testing.assert_allclose(C, np.einsum("mkb,knb->mnb", A, B), rtol=1e-12)


# ---- layernorm ----------------------------------------------------------------------------

def test_layernorm_against_torch_autograd():
    rng = np.random.default_rng(2)
    N, M, eps = 48, 10, 1e-5
    X = rng.standard_normal((N, M)); W = rng.standard_normal(N); B = rng.standard_normal(N)
    DY = rng.standard_normal((N, M))
    Y, mean, rstd = orc.layer_norm_fwd(X, W, B, eps)
    DX, DW, DB = orc.layer_norm_bwd(X, W, DY, eps)
    xt = torch.tensor(X.T.copy(), dtype=torch.float64, requires_grad=True)  # (M, N)
    wt = torch.tensor(W, dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(B, dtype=torch.float64, requires_grad=True)
    yt = torch.nn.functional.layer_norm(xt, (N,), wt, bt, eps)
    yt.backward(torch.tensor(DY.T.copy()))
    np.testing.assert_allclose(Y, yt.detach().numpy().T, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(DX, xt.grad.numpy().T, rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(DW, wt.grad.numpy(), rtol=1e-10)
    np.testing.assert_allclose(DB, bt.grad.numpy(), rtol=1e-10)
    np.testing.assert_allclose(mean, X.mean(axis=0), rtol=1e-12)
    np.testing.assert_allclose(rstd, 1 / np.sqrt(X.var(axis=0) + eps), rtol=1e-12)  # biased var


def test_layernorm_invariants():
    rng = np.random.default_rng(3)
    N, M = 64, 6
    X = rng.standard_normal((N, M)); DY = rng.standard_normal((N, M))
    ones = np.ones(N)
    DX, _, _ = orc.layer_norm_bwd(X, ones, DY, 0.0)
    _, mean, rstd = orc.layer_norm_fwd(X, ones, np.zeros(N), 0.0)
    xhat = (X - mean) * rstd
    np.testing.assert_allclose(DX.sum(axis=0), 0, atol=1e-10)           # dx ⟂ 1
    np.testing.assert_allclose((DX * xhat).sum(axis=0), 0, atol=1e-10)  # dx ⟂ xhat
    # constant row: var = 0 -> rstd = 1/sqrt(eps), y = b
    Xc = np.full((N, 2), 3.25)
    Y, m, r = orc.layer_norm_fwd(Xc, ones, np.full(N, 0.5), 1e-5)
    np.testing.assert_allclose(r, 1 / math.sqrt(1e-5))
    np.testing.assert_allclose(Y, 0.5)


# ---- softmax ------------------------------------------------------------------------------

def test_softmax_against_scipy_and_invariants():
    from scipy.special import softmax as sp_softmax
    rng = np.random.default_rng(4)
    x = rng.standard_normal((37, 9)) * 2
    s = orc.softmax(x)
    np.testing.assert_allclose(s, sp_softmax(x, axis=0), rtol=1e-12)
    np.testing.assert_allclose(s.sum(axis=0), 1, rtol=1e-12)
    np.testing.assert_allclose(orc.softmax(x + 5.0), s, rtol=1e-10)
    part = orc.softmax(x, rows=16)
    assert part.shape == (16, 9)
    np.testing.assert_allclose(part, sp_softmax(x[:16], axis=0), rtol=1e-12)


# ---- FMHA ---------------------------------------------------------------------------------

def _fmha_loops(Q, K, V, scale, causal, input_pos=0):
    D, M, H, B = Q.shape
    N, KH = K.shape[1], K.shape[2]
    out = np.zeros((V.shape[0], M, H, B))
    for b in range(B):
        for h in range(H):
            kh = h // (H // KH)
            for i in range(M):
                s = np.array([sum(Q[d, i, h, b] * K[d, j, kh, b] for d in range(D)) * scale for j in range(N)])
                if causal:
                    s[np.arange(N) > i + input_pos] = -np.inf
                p = np.exp(s - s.max()); p /= p.sum()
                for j in range(N):
                    out[:, i, h, b] += p[j] * V[:, j, kh, b]
    return out


@pytest.mark.parametrize("causal", [False, True])
def test_ref_fmha_brute_force_tiny_gqa(causal):
    rng = np.random.default_rng(5)
    D, M, N, H, KH, B = 16, 8, 8, 4, 2, 1
    Q = rng.standard_normal((D, M, H, B)); K = rng.standard_normal((D, N, KH, B)); V = rng.standard_normal((D, N, KH, B))
    out = orc.ref_fmha(Q, K, V, causal=causal, dtype=np.float64)
    np.testing.assert_allclose(out, _fmha_loops(Q, K, V, 1 / math.sqrt(D), causal), rtol=1e-10)
    if causal:
        np.testing.assert_allclose(out[:, 0, :, 0], V[:, 0, [0, 0, 1, 1], 0], rtol=1e-12)  # row 1 sees key 1 only


def test_ref_fmha_against_torch_sdpa():
    rng = np.random.default_rng(6)
    D, M, H, B = 32, 24, 3, 2
    Q = rng.standard_normal((D, M, H, B)); K = rng.standard_normal((D, M, H, B)); V = rng.standard_normal((D, M, H, B))
    t = lambda a: torch.tensor(np.ascontiguousarray(a.T))  # (B,H,M,D)
    for causal in (False, True):
        ref = torch.nn.functional.scaled_dot_product_attention(t(Q), t(K), t(V), is_causal=causal)
        np.testing.assert_allclose(orc.ref_fmha(Q, K, V, causal=causal, dtype=np.float64), ref.numpy().T, rtol=1e-9, atol=1e-12)


def test_fmha_general_matches_ref_and_offset_limit():
    rng = np.random.default_rng(7)
    D, M, N, H, B = 16, 8, 24, 2, 1
    Q = rng.standard_normal((D, M, H, B)); K = rng.standard_normal((D, N, H, B)); V = rng.standard_normal((D, N, H, B))
    np.testing.assert_allclose(orc.fmha_general(Q, K, V, causal=True), orc.ref_fmha(Q, K, V, causal=True, dtype=np.float64), rtol=1e-12)
    # decode offset: brute force, and with input_pos >= N every key is visible == non-causal
    np.testing.assert_allclose(orc.fmha_general(Q, K, V, causal=True, input_pos=16),
                               _fmha_loops(Q, K, V, 1 / math.sqrt(D), True, input_pos=16), rtol=1e-10)
    np.testing.assert_allclose(orc.fmha_general(Q, K, V, causal=True, input_pos=N),
                               orc.ref_fmha(Q, K, V, causal=False, dtype=np.float64), rtol=1e-12)


# ---- MoE ----------------------------------------------------------------------------------

def _random_topk_ids(rng, num_tokens, topk, E):
    return np.stack([rng.permutation(E)[:topk] + 1 for _ in range(num_tokens)]).astype(np.int64)


@pytest.mark.parametrize("num_tokens,topk,E,tile_m", [(48, 8, 64, 128), (7, 2, 4, 4), (256, 2, 32, 128), (5, 3, 3, 2)])
def test_moe_align_invariants(num_tokens, topk, E, tile_m, corc):
    rng = np.random.default_rng(8)
    ids = _random_topk_ids(rng, num_tokens, topk, E)
    tok, exp = orc.moe_align_tile_size(ids, tile_m, E)
    total = num_tokens * topk
    flat = ids.reshape(-1)
    real = tok[tok != total + 1]
    assert sorted(real.tolist()) == list(range(1, total + 1))          # each replica exactly once
    counts = np.bincount(flat - 1, minlength=E)
    assert len(tok) == tile_m * int(np.sum(-(-counts // tile_m))) and len(exp) * tile_m == len(tok)
    for blk in range(len(exp)):
        seg = tok[blk * tile_m:(blk + 1) * tile_m]
        segr = seg[seg != total + 1]
        assert np.all(flat[segr - 1] == exp[blk])                      # block holds one expert
        assert np.all(np.diff(segr) > 0)                               # stable: ascending replica id
        assert np.all(seg[len(segr):] == total + 1)                    # padding only at the tail
    assert np.all(np.diff(exp) >= 0)
    # C restatement (literal stable selection) agrees
    ids_f = np.asfortranarray(ids)
    tok_c = np.empty_like(tok); exp_c = np.empty_like(exp)
    nb = corc.oracle_moe_align_tile_size(ids_f.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(num_tokens),
                                         ctypes.c_int64(topk), ctypes.c_int32(tile_m), ctypes.c_int32(E),
                                         tok_c.ctypes.data_as(ctypes.c_void_p), exp_c.ctypes.data_as(ctypes.c_void_p))
    assert nb == len(exp)
    assert np.array_equal(tok_c, tok) and np.array_equal(exp_c, exp)


def test_ref_moe_per_token_dense_loop():
    rng = np.random.default_rng(9)
    hidden, inter, E, T, topk = 8, 6, 5, 7, 2
    hs = rng.standard_normal((hidden, T)); w1 = rng.standard_normal((hidden, 2 * inter, E)) * 0.3
    w2 = rng.standard_normal((inter, hidden, E)) * 0.3
    ids = _random_topk_ids(rng, T, topk, E); tw = rng.random((T, topk))
    ref = np.zeros((hidden, T))
    for t in range(T):
        for s in range(topk):
            e = ids[t, s] - 1
            gu = w1[:, :, e].T @ hs[:, t]
            g, u = gu[:inter], gu[inter:]
            act = g * (1 / (1 + np.exp(-g))) * u
            ref[:, t] += tw[t, s] * (w2[:, :, e].T @ act)
    np.testing.assert_allclose(orc.ref_moe(hs, w1, w2, tw, ids, dtype=np.float64), ref, rtol=1e-10)
    np.testing.assert_allclose(orc.silu_and_mul(np.array([0.0, 1.0, -2.0]), np.array([3.0, 2.0, 1.0])),
                               [0.0, 2 / (1 + math.exp(-1)), -2 / (1 + math.exp(2))], rtol=1e-12)


def test_route_top2():
    logits = np.array([[0.1, 2.0, -1.0, 1.0], [3.0, 3.0, 0.0, -5.0]])
    w, ids = orc.route_top2(logits)
    assert ids.tolist() == [[2, 4], [1, 2]]
    np.testing.assert_allclose(w[0], np.exp([2.0, 1.0]) / np.exp([2.0, 1.0]).sum(), rtol=1e-6)
    np.testing.assert_allclose(w[1], [0.5, 0.5])


# ---- FP8 E4M3FN ---------------------------------------------------------------------------

GOLDEN = json.load(open(os.path.join(HERE, "golden", "dlfp8_vectors.json")))


def test_e4m3fn_reference_known_answers(corc):
    """test/extensions/DLFP8Types.jl:126-141: 16 representable values round-trip bit for bit;
    the fma vectors are exact in e4m3."""
    rep = np.array(GOLDEN["representable"], dtype=np.float32)
    assert np.array_equal(orc.e4m3fn_decode(orc.e4m3fn_encode(rep)), rep)
    assert [corc.oracle_e4m3fn_decode(corc.oracle_e4m3fn_encode(float(v))) for v in rep] == rep.tolist()
    a, b, c = (np.array(GOLDEN["fma"][k], dtype=np.float32) for k in ("a", "b", "c"))
    q = lambda v: orc.e4m3fn_decode(orc.e4m3fn_encode(v))
    assert np.array_equal(q(q(a) * q(b) + q(c)), a * b + c)


def test_e4m3fn_all_codes_against_torch(corc):
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    dec = orc.e4m3fn_decode(codes)
    assert np.array_equal(np.isnan(dec), np.isnan(ref))
    assert np.array_equal(dec[~np.isnan(ref)], ref[~np.isnan(ref)])
    cdec = np.array([corc.oracle_e4m3fn_decode(int(c)) for c in codes], dtype=np.float32)
    assert np.array_equal(cdec[~np.isnan(ref)], ref[~np.isnan(ref)])
    assert dec[0x7E] == 448.0 and dec[0x08] == 2.0 ** -6 and dec[0x01] == 2.0 ** -9
    finite = codes[~np.isnan(ref)]
    assert np.array_equal(orc.e4m3fn_encode(dec[finite]), finite)  # encode∘decode = id (incl. -0)


def test_e5m2_codec_against_torch_and_reference_vectors():
    """Every E5M2 code decodes as torch.float8_e5m2 does; encoding is round-to-nearest-even with
    overflow to Inf (torch's conversion is an independent implementation); the reference's 16
    exactly representable values round-trip (test/extensions/DLFP8Types.jl:126-134)."""
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e5m2).to(torch.float32).numpy()
    dec = orc.e5m2_decode(codes)
    assert np.array_equal(np.isnan(dec), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(dec[ok], ref[ok]) and np.array_equal(np.signbit(dec[ok]), np.signbit(ref[ok]))
    assert np.array_equal(orc.e5m2_encode(dec[ok]), codes[ok])          # encode . decode = id, -0 and Inf included
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(s) for s in (1e-5, 1e-3, 1.0, 300.0, 4e4)]
                       + [dec[ok], (dec[ok][:-1] + dec[ok][1:])[np.isfinite(dec[ok][:-1] + dec[ok][1:])] / 2])   # ties
    got = orc.e5m2_encode(x)
    want = torch.from_numpy(x.astype(np.float32)).to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    with open(os.path.join(os.path.dirname(__file__), "golden", "dlfp8_vectors.json")) as f:
        rep = np.array(json.load(f)["representable"], dtype=np.float32)
    assert np.array_equal(orc.e5m2_decode(orc.e5m2_encode(rep)), rep)


def test_fp8_matmul_reference_exact_case():
    """The reference's own mma check (test/extensions/DLFP8Types.jl:143-152): operands drawn from
    {0, 0.5, 1}, so twice every operand is an integer and 4 * (A * B) is an integer matrix product."""
    rng = np.random.default_rng(11)
    for fmt, enc in (("e4m3fn", orc.e4m3fn_encode), ("e5m2", orc.e5m2_encode)):
        a2 = rng.integers(0, 3, (16, 16)); b2 = rng.integers(0, 3, (16, 16))
        got = orc.fp8_matmul(enc(a2 / 2.0), enc(b2 / 2.0), fmt)
        want = np.zeros((16, 16), dtype=np.int64)
        for i in range(16):
            for j in range(16):
                want[i, j] = sum(int(a2[i, k]) * int(b2[k, j]) for k in range(16))
        assert np.array_equal(got * 4, want)


def test_e4m3fn_encode_rne_against_torch_and_c(corc):
    rng = np.random.default_rng(10)
    x = np.concatenate([rng.standard_normal(4000) * 3, rng.standard_normal(2000) * 200,
                        rng.standard_normal(2000) * 0.01,
                        # exact midpoints between neighbours: ties must go to even
                        np.array([0.5625 * 2, 1.0625, 1.1875, 2.0 ** -10, 3 * 2.0 ** -10, 17.0, 19.0, 464.0, 463.9, 448.0])]).astype(np.float32)
    x = x[np.abs(x) < 480]
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = orc.e4m3fn_encode(x)
    assert np.array_equal(got & 0x7F, ref & 0x7F)
    nz = got & 0x7F != 0
    assert np.array_equal(got[nz], ref[nz])
    sub = x[:: 37]
    assert [corc.oracle_e4m3fn_encode(float(v)) for v in sub] == orc.e4m3fn_encode(sub).tolist()


def test_quantize_per_channel_bound():
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((64, 12, 3)) * 0.02).astype(np.float32)
    codes, scale = orc.quantize_e4m3fn_per_channel(w)
    deq = orc.e4m3fn_decode(codes) * scale[None]
    assert np.all(np.abs(deq - w) <= np.abs(w) * 2.0 ** -4 + scale[None] * 2.0 ** -10)  # half-ulp of 3 mantissa bits
    assert np.all(np.abs(orc.e4m3fn_decode(codes)).max(axis=0) == 448.0)


def test_isapprox_is_normwise():
    x = np.array([1.0, 0.0]); y = np.array([1.0, 0.005])
    assert orc.isapprox(x, y, rtol=1e-2) and not orc.isapprox(x, y, rtol=1e-3)


# ---- FFT (examples/fft.jl) ---------------------------------------------------------------------

@pytest.mark.parametrize("factors", [(2, 2, 2), (8, 8, 8), (16, 16, 16), (4, 8, 2), (2, 4, 8)])
def test_fft_3stage_matches_numpy_fft(factors):
    """The three-stage data flow restated from fft.jl:45-121 equals the library FFT (an index or
    permutation slip in any stage scrambles the spectrum)."""
    rng = np.random.default_rng(3)
    N = factors[0] * factors[1] * factors[2]
    x = rng.standard_normal((N, 3)) + 1j * rng.standard_normal((N, 3))
    y = orc.fft_3stage(x, factors)
    ref = np.fft.fft(x, axis=0)
    assert np.abs(y - ref).max() <= 1e-6 * np.abs(ref).max()      # float32 tables


def test_fft_tables_and_brute_force_dft():
    W = orc.dft_matrix(8)
    assert W.shape == (2, 8, 8) and W.dtype == np.float32
    assert np.allclose(W[0] + 1j * W[1], np.fft.fft(np.eye(8)), atol=1e-6)
    W0, W1, W2, T0, T1 = orc.make_twiddles((2, 4, 8))
    assert T0.shape == (2, 32, 2) and T1.shape == (2, 8, 4)
    assert np.allclose(T0[0, 5, 1] + 1j * T0[1, 5, 1], np.exp(-2j * np.pi * 5 / 64), atol=1e-7)   # fft.jl:146-150
    assert np.allclose(T1[0, 3, 2] + 1j * T1[1, 3, 2], np.exp(-2j * np.pi * 6 / 32), atol=1e-7)   # fft.jl:158-162
    x = np.arange(8, dtype=np.float64)[:, None] * (1 + 0.5j)
    brute = np.array([sum(x[n, 0] * np.exp(-2j * np.pi * k * n / 8) for n in range(8)) for k in range(8)])
    assert np.allclose(orc.fft_3stage(x, (2, 2, 2))[:, 0], brute, atol=1e-5)


# ---- host-level Tiled broadcast / mapreduce ---------------------------------------------------------

def test_jl_promote_known_julia_facts(orc):
    """Facts of Julia's promotion (Base promotion.jl / bool.jl / float.jl), written out."""
    facts = {("Int32", "Int64"): "Int64", ("Int64", "Float32"): "Float32", ("Int32", "Float16"): "Float16",
             ("Float16", "Float32"): "Float32", ("Float32", "Float64"): "Float64", ("Bool", "Int32"): "Int32",
             ("Bool", "Float16"): "Float16", ("Bool", "Bool"): "Bool", ("Int64", "Int64"): "Int64"}
    for (a, b), want in facts.items():
        assert orc.jl_promote(a, b) == want and orc.jl_promote(b, a) == want


def test_tiled_eval_types_and_values_by_hand(orc):
    a = np.array([1, -2, 3], np.int32)
    b = np.array([2, 2, 2], np.int64)
    v, t = orc.tiled_eval("div(a0,a1)", (a, b))
    assert t == "Float64" and np.array_equal(v, [0.5, -1.0, 1.5])          # Int / Int is Float64
    v, t = orc.tiled_eval("add(a0,a0)", (np.array([True, False]),))
    assert t == "Int64" and np.array_equal(v, [2, 0])                      # true + true == 2
    v, t = orc.tiled_eval("mul(a0,a1)", (np.array([True, False]), np.array([1.5, 2.5], np.float16)))
    assert t == "Float16" and np.array_equal(v, np.array([1.5, 0], np.float16))
    v, t = orc.tiled_eval("add(a0,s0)", (np.array([0.1], np.float32),), (1.0,))
    assert t == "Float64" and v[0] == np.float64(np.float32(0.1)) + 1.0    # Float32 .+ 1.0 is Float64
    v, t = orc.tiled_eval("add(a0,s0)", (np.array([0.1], np.float32),), (np.float32(1),))
    assert t == "Float32" and v[0] == np.float32(0.1) + np.float32(1)
    # Julia: div rounds toward zero, fld down, cld up, rem takes the dividend's sign, mod the divisor's
    x, y = np.array([7, -7, 7, -7], np.int64), np.array([2, 2, -2, -2], np.int64)
    for name, want in (("div_int", [3, -3, -3, 3]), ("fld", [3, -4, -4, 3]), ("cld", [4, -3, -3, 4]),
                       ("rem", [1, -1, 1, -1]), ("mod", [1, 1, -1, -1])):
        v, t = orc.tiled_eval(f"{name}(a0,a1)", (x, y))
        assert t == "Int64" and np.array_equal(v, want), name
    # the same on floats, answers worked out by hand from Julia's definitions (Base div.jl, float.jl): the quotients
    # come from the exact remainder, so div(1.0, 0.1) == fld(1.0, 0.1) == 9.0 although 1.0 / 0.1 == 10.0 (rem is
    # 0.09999999999999995), cld(1.0, 0.1) == 10.0; mod of an exact multiple takes the divisor's sign: mod(4.0, -2.0)
    # is -0.0, mod(-4.0, 2.0) is 0.0; mod(-1.0, 3.0) == 2.0, mod(1.0, -3.0) == -2.0
    fx, fy = np.array([1.0, 4.0, -4.0, -1.0, 1.0, 7.5]), np.array([0.1, -2.0, 2.0, 3.0, -3.0, 2.0])
    for name, want in (("div_int", [9.0, -2.0, -2.0, 0.0, 0.0, 3.0]), ("fld", [9.0, -2.0, -2.0, -1.0, -1.0, 3.0]),
                       ("cld", [10.0, -2.0, -2.0, 0.0, 0.0, 4.0]), ("mod", [0.09999999999999995, -0.0, 0.0, 2.0, -2.0, 1.5])):
        v, t = orc.tiled_eval(f"{name}(a0,a1)", (fx, fy))
        assert t == "Float64" and np.array_equal(v, want), (name, v)
        assert name != "mod" or np.array_equal(np.signbit(v), np.signbit(want))      # the sign of a zero remainder
    # ^ keeps the type of the base for integer and Bool exponents (^(x::T, p::Integer), power_by_squaring):
    # Int32(3)^Int64(4) isa Int32 (and wraps: Int32(2)^40 == 0), true^0 == true^5 == false^0 == true, false^2 == false,
    # Float32(2)^3 isa Float32; a float exponent promotes: Int32(2)^0.5 isa Float64
    v, t = orc.tiled_eval("pow(a0,a1)", (np.array([3, 2, -2], np.int32), np.array([4, 40, 3], np.int64)))
    assert t == "Int32" and np.array_equal(v, [81, 0, -8])
    v, t = orc.tiled_eval("pow(a0,a1)", (np.array([True, True, False, False]), np.array([0, 5, 0, 2], np.int64)))
    assert t == "Bool" and np.array_equal(v, [True, True, True, False])
    v, t = orc.tiled_eval("pow(a0,a1)", (np.array([True, False]), np.array([False, True])))
    assert t == "Bool" and np.array_equal(v, [True, False])
    v, t = orc.tiled_eval("pow(a0,a1)", (np.array([2.0], np.float32), np.array([3], np.int32)))
    assert t == "Float32" and v[0] == 8.0
    v, t = orc.tiled_eval("pow(a0,a1)", (np.array([2], np.int32), np.array([0.5])))
    assert t == "Float64" and v[0] == 2.0 ** 0.5
    # Julia's shifts (answers worked out by hand): the value keeps its type; Int32 wraps; a count of the word size
    # or more empties the word (>> keeps the sign); >>> is logical; a negative count shifts the other way
    w = np.array([1, -8, 5, -1, 2 ** 30], np.int32)
    for text, cnt, want in (("shl", 2, [4, -32, 20, -4, 0]), ("shr", 1, [0, -4, 2, -1, 2 ** 29]),
                            ("lshr", 28, [0, 15, 0, 15, 4]), ("shl", 40, [0, 0, 0, 0, 0]), ("shr", 40, [0, -1, 0, -1, 0]),
                            ("shl", -1, [0, -4, 2, -1, 2 ** 29]), ("lshr", -2, [4, -32, 20, -4, 0])):
        v, t = orc.tiled_eval(f"{text}(a0,s0)", (w,), (np.int64(cnt),))
        assert t == "Int32" and np.array_equal(v, want), (text, cnt)
    v, t = orc.tiled_eval("shl(a0,s0)", (np.array([True, False]),), (3,))
    assert t == "Int64" and np.array_equal(v, [8, 0])                      # true << 3 == 8
    # mul_hi: high word of the exact product
    v, t = orc.tiled_eval("mul_hi(a0,a1)", (w, np.array([7, -8, 2 ** 30, -1, 2 ** 30], np.int32)))
    assert t == "Int32" and np.array_equal(v, [0, 0, 1, 0, 2 ** 28])       # 5 * 2^30 >> 32 == 1
    big = np.array([2 ** 62, -2 ** 62, 3], np.int64)
    v, t = orc.tiled_eval("mul_hi(a0,a1)", (big, np.array([4, 4, -1], np.int64)))
    assert t == "Int64" and np.array_equal(v, [1, -1, -1])                 # 2^64 >> 64, -2^64 >> 64, -3 >> 64
    v, t = orc.tiled_eval("rsqrt(a0)", (np.array([4.0, 0.25], np.float32),))
    assert t == "Float32" and np.array_equal(v, [0.5, 2.0])
    # max / min: NaN wins, +0.0 > -0.0
    v, _ = orc.tiled_eval("max(a0,a1)", (np.array([np.nan, 1, -0.0], np.float32), np.array([1, np.nan, 0.0], np.float32)))
    assert np.isnan(v[0]) and np.isnan(v[1]) and not np.signbit(v[2])
    v, _ = orc.tiled_eval("min(a0,a1)", (np.array([-0.0], np.float32), np.array([0.0], np.float32)))
    assert np.signbit(v[0])
    # Float16 arithmetic rounds after every operation: (2048 + 1) + 1 stays 2048, 2048 + (1 + 1) is 2050
    h = np.array([2048], np.float16)
    one = np.array([1], np.float16)
    assert orc.tiled_eval("add(add(a0,a1),a1)", (h, one))[0][0] == 2048
    assert orc.tiled_eval("add(a0,add(a1,a1))", (h, one))[0][0] == 2050


def test_tiled_broadcast_reference_cases(orc):
    """Known answers of test/host/broadcast.jl: scalar fills (:175-183), 0-dim (:194-203), size-1
    expansion only (:138-144), allocating with expansion (:166-173), shape mismatch (:112-122)."""
    assert np.all(orc.tiled_broadcast((1000,), "Float32", "s0", (), (0,)) == 0)
    assert np.all(orc.tiled_broadcast((33, 65), "Float32", "s0", (), (np.float32(2.5),)) == 2.5)
    assert orc.tiled_broadcast((), "Float32", "add(a0,s0)", (np.array(2.0, np.float32),), (np.float32(1),))[()] == 3.0
    A = np.arange(512, dtype=np.float32).reshape(1, 512)
    got = orc.tiled_broadcast((32, 512), "Float32", "add(a0,s0)", (A,), (np.float32(1),))
    assert np.array_equal(got, np.repeat(A + 1, 32, axis=0))
    row, col = np.arange(128, dtype=np.float32).reshape(1, 128), np.arange(64, dtype=np.float32).reshape(64, 1)
    v, _ = orc.tiled_eval("add(a0,a1)", (row, col))
    assert v.shape == (64, 128) and v[5, 7] == 12
    vec, mat = np.arange(64, dtype=np.float32), np.ones((64, 128), np.float32)
    v, _ = orc.tiled_eval("add(a0,a1)", (vec, mat))                       # rank expansion along trailing dims
    assert v.shape == (64, 128) and v[9, 100] == 10
    for bad_dest, leaf in (((10,), np.zeros(11, np.float32)), ((8, 8), np.zeros((8, 16), np.float32))):
        with pytest.raises(ValueError):
            orc.tiled_broadcast(bad_dest, "Float32", "a0", (leaf,))


def test_tiled_mapreduce_reference_cases_and_brute_force(orc):
    """Known answers of test/host/mapreduce.jl (count == 4 :153-160, any / all :131-151, max of
    fill(-5) == -5 :97-104, out-of-range dims ignored :47-57) and brute-force loops on a tiny array."""
    c = np.zeros(1024, bool)
    c[[0, 99, 499, 998]] = True
    assert orc.tiled_mapreduce(None, "add_sum", c) == (4, "Int64")
    assert orc.tiled_mapreduce(None, "|", np.zeros(1024, bool))[0] == False          # noqa: E712
    assert orc.tiled_mapreduce(None, "|", c)[0] == True                             # noqa: E712
    assert orc.tiled_mapreduce(None, "&", ~c)[0] == False                           # noqa: E712
    assert orc.tiled_mapreduce(None, "max", np.full(1000, -5, np.float32)) == (-5.0, "Float32")
    rng = np.random.default_rng(0)
    A = rng.standard_normal((3, 4, 5)).astype(np.float32)
    r, t = orc.tiled_mapreduce(None, "add_sum", A, dims=(2, 7))
    assert t == "Float32" and r.shape == (3, 1, 5)
    for i in range(3):
        for k in range(5):
            assert abs(r[i, 0, k] - sum(float(A[i, j, k]) for j in range(4))) < 1e-5
    r, _ = orc.tiled_mapreduce("abs(a0)", "max", A, dims=(1, 3))
    for j in range(4):
        assert r[0, j, 0] == max(abs(A[i, j, k]) for i in range(3) for k in range(5))
    assert orc.tiled_mapreduce(None, "add_sum", np.array([2**31 - 1, 1], np.int32)) == (2**31, "Int64")   # sum widens
    assert orc.tiled_mapreduce(None, "+", np.array([3, 4], np.int32))[1] == "Int32"                       # reduce(+) does not
    r, _ = orc.tiled_mapreduce(None, "mul_prod", np.full(17, 2, np.int32), dims=())
    assert r.shape == (17,) and np.all(r == 2)                                      # no reduced dimension: map
    assert orc.tiled_mapreduce(None, "add_sum", A, init=100.0)[0] == pytest.approx(100 + A.astype(np.float64).sum(), rel=1e-6)


def test_vadd_gather_out_of_bounds_by_brute_force():
    """vec_add_kernel_1d_gather with arrays of different lengths: an out-of-bounds gather lane reads 0
    and an out-of-bounds scatter lane is dropped (test/device/gather_scatter.jl:75-113: the lanes past
    the end of the source come back as 0.0).  Element by element with scalar loops."""
    assert orc.vadd_gather(np.ones(16, np.float32), np.full(32, 2.0, np.float32), 32).tolist() == [3.0] * 16 + [2.0] * 16
    rng = np.random.default_rng(3)
    for na, nb, nc in [(5, 9, 7), (9, 5, 12), (0, 3, 4), (6, 6, 6), (10, 2, 1)]:
        a = rng.random(na).astype(np.float32); b = rng.random(nb).astype(np.float32)
        want = [(a[i] if i < na else np.float32(0)) + (b[i] if i < nb else np.float32(0)) for i in range(nc)]
        assert orc.vadd_gather(a, b, nc).tolist() == [float(w) for w in want]


# ---- Philox2x32-7 RNG fills -----------------------------------------------------------------------

def test_philox2x32_random123_known_answers(orc):
    """Random123's published known-answer vectors for philox2x32 at 7 and 10 rounds
    (tests/golden/philox2x32_kat.json)."""
    import json
    import os
    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "philox2x32_kat.json")))["vectors"]
    assert len(kat) == 6
    for v in kat:
        a, b = orc.philox2x32([int(v["ctr"][0], 16)], [int(v["ctr"][1], 16)], [int(v["key"], 16)], v["rounds"])
        assert (int(a[0]), int(b[0])) == (int(v["out"][0], 16), int(v["out"][1], 16)), v


def test_rng_fill_layout_by_brute_force(orc):
    """Slot placement of a block's Philox outputs for every width, element by element with scalar
    loops (src/language/random.jl:262-338), on two blocks with a partial second one."""
    seed, counter, n = 0x1234ABCD, 0xFFFFFFF0, 700          # the counter wraps inside the block

    def call(b, i):
        key = ((b * orc.PHILOX_W) & 0xFFFFFFFF) ^ seed
        a, c = orc.philox2x32([(counter + i) & 0xFFFFFFFF], [0], [key])
        return int(a[0]), int(c[0])
    want32, want64, want16, want8 = [0] * 1024, [0] * 1024, [0] * 1024, [0] * 1024
    for b in range(2):
        for i in range(256):
            c1, c2 = call(b, i)
            want32[512 * b + i], want32[512 * b + 256 + i] = c1, c2
        for i in range(512):
            c1, c2 = call(b, i)
            want64[512 * b + i] = c1 | (c2 << 32)
        raw = [0] * 256
        for i in range(128):
            raw[i], raw[128 + i] = call(b, i)
        for m in range(256):
            want16[512 * b + m], want16[512 * b + 256 + m] = raw[m] & 0xFFFF, raw[m] >> 16
        raw = [0] * 128
        for i in range(64):
            raw[i], raw[64 + i] = call(b, i)
        for q in range(4):
            for m in range(128):
                want8[512 * b + 128 * q + m] = (raw[m] >> (8 * q)) & 0xFF
    assert orc.rng_fill("u32", n, seed, counter).tolist() == want32[:n]
    assert orc.rng_fill("u64", n, seed, counter).tolist() == want64[:n]
    assert orc.rng_fill("u16", n, seed, counter).tolist() == want16[:n]
    assert orc.rng_fill("u8", n, seed, counter).tolist() == want8[:n]
    assert np.array_equal(orc.rng_fill("i32", n, seed, counter).view(np.uint32), orc.rng_fill("u32", n, seed, counter))


def test_randn_randexp_layout_by_brute_force(orc):
    """Which Philox word feeds what in randn! / randexp!, element by element with scalar loops and
    ``math`` in double precision.  32-bit class (src/language/random.jl:369-380,420-441): call i of a
    block gives (c1, c2); the radius comes from c2, r = sqrt(-2 log u01(c2)), the angle from c1,
    2 pi u01(c1); slot i takes r sin, slot 256 + i takes r cos.  Float64 (:386-398,449-480): u1 packs
    the two words of counter i, u2 those of counter 256 + i; the radius comes from u1 and the angle
    from u2.  randexp (:500-501) is -log of the rand! value of the same slot.  Swapping the two words,
    the sine and cosine slots or the counter pairing changes every value; the oracle computes the 32-bit
    class in Float32, hence the tolerance."""
    seed, counter, n = 0xCAFEF00D, 0xFFFFFF80, 600          # two blocks, the second partial; the counter wraps

    def call(b, i):
        key = ((b * orc.PHILOX_W) & 0xFFFFFFFF) ^ seed
        a, c = orc.philox2x32([(counter + i) & 0xFFFFFFFF], [0], [key])
        return int(a[0]), int(c[0])
    u32 = lambda w: w * 2.0 ** -32 + 2.0 ** -33                                   # u01(Float32, ::UInt32), :136-142
    u64 = lambda w: ((w >> 12) | 1) * 2.0 ** -52                                  # u01(Float64, ::UInt64), :169-174
    want32, want64 = [0.0] * 1024, [0.0] * 1024
    for b in range(2):
        for i in range(256):
            c1, c2 = call(b, i)
            r, ang = math.sqrt(-2.0 * math.log(u32(c2))), 2.0 * math.pi * u32(c1)
            want32[512 * b + i], want32[512 * b + 256 + i] = r * math.sin(ang), r * math.cos(ang)
            a1, a2 = call(b, i)
            b1, b2 = call(b, 256 + i)
            r, ang = math.sqrt(-2.0 * math.log(u64(a1 | (a2 << 32)))), 2.0 * math.pi * u64(b1 | (b2 << 32))
            want64[512 * b + i], want64[512 * b + 256 + i] = r * math.sin(ang), r * math.cos(ang)
    got32 = orc.rng_fill("f32", n, seed, counter, "randn").astype(np.float64)
    np.testing.assert_allclose(got32, want32[:n], rtol=0, atol=2e-5)            # Float32 evaluation of values up to 6.8
    np.testing.assert_allclose(orc.rng_fill("f64", n, seed, counter, "randn"), want64[:n], rtol=0, atol=1e-12)
    np.testing.assert_allclose(orc.rng_fill("f16", n, seed, counter, "randn").astype(np.float64), want32[:n], rtol=2e-3, atol=1e-3)
    # randexp: minus the logarithm of the uniform value in the same slot
    uni32 = orc.rng_fill("f32", n, seed, counter).astype(np.float64)
    np.testing.assert_allclose(orc.rng_fill("f32", n, seed, counter, "randexp"), [-math.log(u) for u in uni32], rtol=1e-6, atol=1e-7)
    uni64 = orc.rng_fill("f64", n, seed, counter)
    np.testing.assert_allclose(orc.rng_fill("f64", n, seed, counter, "randexp"), [-math.log(u) for u in uni64], rtol=1e-14)
    # and the uniform floats themselves sit where the raw words do (slot layout of rand!, :262-305)
    raw = orc.rng_fill("u32", n, seed, counter)
    np.testing.assert_allclose(uni32, [u32(int(w)) for w in raw], rtol=1e-7)


def test_rng_float_conversions_and_reference_properties(orc):
    """u01 end points (src/language/random.jl:129-174) and the properties the reference's tests assert
    for the host RNG (test/device/random.jl:421-526)."""
    assert orc._u01_f32(np.array([0, 0xFFFFFFFF], np.uint32)).tolist() == [2.0 ** -33, 1.0]
    f64 = orc._u01_f64(np.array([0, 0xFFFFFFFFFFFFFFFF], np.uint64))
    assert f64[0] == 2.0 ** -52 and f64[1] == 1.0 - 2.0 ** -52
    f16 = orc.rng_fill("f16", 4096, 1, 0)
    assert f16.min() > 0 and f16.max() < 1 and f16.dtype == np.float16
    bf = orc.rng_fill("bf16", 4096, 1, 0)
    assert bf.min() > 0 and bf.max() < 1 and np.array_equal(bf, orc.bf16_round(bf))
    v = orc.rng_fill("u32", 2048, 42, 0)
    assert len(np.unique(v)) == 2048
    assert not set(v.tolist()) & set(orc.rng_fill("u32", 2048, 100, 0).tolist())
    assert not set(v.tolist()) & set(orc.rng_fill("u32", 2048, 42, 2048).tolist())      # the next fill of the same RNG
    assert orc.rng_advance_counter(7, 2 ** 32 - 4, 10) == (8, 6)                          # random.jl test :520-525
    z = orc.rng_fill("f32", 1 << 16, 5, 0, "randn").astype(np.float64)
    assert abs(z.mean()) < 0.02 and abs(z.var() - 1) < 0.03
    e = orc.rng_fill("f64", 1 << 16, 5, 0, "randexp")
    assert abs(e.mean() - 1) < 0.02 and e.min() > 0
