"""Randomised differential tests on the GPU (fixed seeds): many shapes, element types, strides and paddings per
entry point, outputs pre-filled with NaN, each result compared on the device with an independent evaluation --
torch's float64 / float32 routines, not the oracle, whose own cases are in the per-kernel test files.  These runs
walk through every kernel variant the dispatchers choose between (`last_variant`) rather than the handful of shapes
the reference's examples name.

Bounds: GEMMs multiply small integers, so every fp32 sum is exact and the comparison is bit for bit (16-bit outputs:
exact while the integers fit the type, else rtol 1e-2).  Attention: |err| <= 2e-2 (f16) / 3e-2 (bf16) * (|ref| +
max|ref|).  Softmax / LayerNorm: 1e-5 / 2e-5 * (|ref| + max|ref|).  Host-level broadcast / reductions: 1e-6 / 1e-5.
"""
import random

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

from cutile_jl_amd import tiled as T  # noqa: E402
from cutile_jl_amd.tiled import Tiled  # noqa: E402
from cutile_jl_amd.examples import fmha, moe  # noqa: E402

NAN = float("nan")


def close(got, ref, tol):
    got = got.double(); ref = ref.double()
    return bool(((got - ref).abs() <= tol * (ref.abs() + ref.abs().max())).all())


def test_gemm_random_shapes_exact(ct):
    rnd = random.Random(3)
    dims = [1, 2, 7, 8, 16, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 200, 255, 256, 257, 384, 500, 512, 513, 777, 1000, 1024, 1100, 2048]
    seen = set()
    for it in range(120):
        M, N, K = (rnd.choice(dims) for _ in range(3))
        if rnd.random() < 0.25:
            K = rnd.choice([2048, 4096, 8192, 5000])
        batch = rnd.choice([0, 0, 0, 1, 3, 8])
        dt = rnd.choice([torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn, torch.float8_e5m2])
        odt = torch.float32 if dt in (torch.float32, torch.float8_e4m3fn, torch.float8_e5m2) else rnd.choice([dt, torch.float32])
        pad = rnd.choice([0, 0, 8, 3])
        g = torch.Generator(device="cuda").manual_seed(it)
        bs = (batch,) if batch else ()
        # torch layout of the Julia arrays A (M, K[, batch]), B (K, N[, batch]), C (M, N[, batch]); views of padded buffers
        A = torch.randint(-2, 3, bs + (K, M + pad), generator=g, device="cuda", dtype=torch.int8).to(torch.float32).to(dt)[..., :M]
        B = torch.randint(-2, 3, bs + (N, K + pad), generator=g, device="cuda", dtype=torch.int8).to(torch.float32).to(dt)[..., :K]
        Cfull = torch.full(bs + (N, M + pad), NAN, dtype=odt, device="cuda")
        C = Cfull[..., :M]
        (ct.batch_matmul_kernel if batch else ct.matmul_kernel)(A, B, C, 64, 64, 64)
        seen.add(ct.last_variant())
        ref = torch.matmul(B.double(), A.double())
        exact = odt == torch.float32 or ref.abs().max().item() <= (2048 if odt == torch.float16 else 256)
        what = f"M={M} N={N} K={K} batch={batch} {dt} -> {odt} pad={pad} {ct.last_variant()}"
        assert torch.equal(C.double(), ref) if exact else torch.allclose(C.double(), ref, rtol=1e-2, atol=1.0), what
        assert not pad or bool(torch.isnan(Cfull[..., M:].float()).all()), what
    assert len(seen) >= 8, seen      # generic, register-staged, direct-to-LDS, split-K, fp32 and fp8 kernels all took part


def test_fmha_random_shapes(ct):
    rnd = random.Random(1)
    for it in range(30):
        S = 128 * rnd.randint(1, 20)
        qg = rnd.choice([1, 1, 2, 4])
        H = rnd.choice([1, 2, 3, 4, 8]) * qg
        B = rnd.choice([1, 2, 3, 4, 8, 16])
        causal = rnd.choice([True, True, False])
        dt = rnd.choice([torch.float16, torch.bfloat16])
        d = fmha.prepare(batch=B, heads=H, seq_q=S, seq_kv=S, query_group_size=qg, causal=causal, T=dt, seed=S + B)
        out = torch.full_like(d.Q, NAN)
        fmha.cutile_fmha(d.Q, d.K, d.V, causal=causal, query_group_size=qg, out=out)
        K = d.K.repeat_interleave(qg, dim=1).float(); V = d.V.repeat_interleave(qg, dim=1).float()
        ref = F.scaled_dot_product_attention(d.Q.float(), K, V, is_causal=causal)
        assert close(out, ref, 3e-2 if dt == torch.bfloat16 else 2e-2), f"B={B} H={H} S={S} group={qg} causal={causal} {dt} {ct.last_variant()}"


def test_fmha_random_ragged_shapes(ct):
    """Sequence lengths off every tile grid, D = 64 and 128, grouped queries: the general kernels (EVEN_K = false).
    Causal here is the reference's mask with input_pos = 0 (query i sees keys <= i), which is torch's is_causal."""
    rnd = random.Random(2)
    for it in range(40):
        Sq = rnd.choice([1, 2, 17, 63, 64, 65, 100, 128, 130, 200, 257, 300, 511, 700])
        Skv = rnd.choice([1, 5, 64, 77, 128, 129, 255, 256, 300, 512, 513, 900])
        causal = rnd.choice([True, False])
        if causal and Skv < Sq:
            Skv = Sq
        D = rnd.choice([64, 128]); qg = rnd.choice([1, 2, 4]); H = rnd.choice([1, 2, 3]) * qg; B = rnd.choice([1, 2, 5])
        dt = rnd.choice([torch.float16, torch.bfloat16])
        d = fmha.prepare(batch=B, heads=H, seq_q=Sq, seq_kv=Skv, d_k=D, d_v=D, query_group_size=qg, causal=causal, T=dt, seed=it)
        out = torch.full_like(d.Q, NAN)
        fmha.cutile_fmha(d.Q, d.K, d.V, causal=causal, query_group_size=qg, out=out)
        K = d.K.repeat_interleave(qg, dim=1).float(); V = d.V.repeat_interleave(qg, dim=1).float()
        ref = F.scaled_dot_product_attention(d.Q.float(), K, V, is_causal=causal)
        assert close(out, ref, 3e-2 if dt == torch.bfloat16 else 2e-2), f"B={B} H={H} Sq={Sq} Skv={Skv} D={D} group={qg} causal={causal} {dt} {ct.last_variant()}"


def test_fmha_random_decode_and_chunked_prefill_shapes(ct):
    """Few queries at the end of a long cache (input_pos > 0), grouped heads, ragged caches: the kernels that split the
    keys over several workgroups and stack a head group in one query tile, and the unsplit ones where the cache is short.
    The mask is the kernel's rule -- query i sits at input_pos + i and sees the keys up to there."""
    rnd = random.Random(7)
    seen = set()
    for it in range(60):
        Sq = rnd.choice([1, 1, 1, 2, 5, 16, 33, 64, 65, 128, 200, 384])
        Skv = rnd.choice([64, 100, 257, 1000, 2048, 3001, 4096, 6000])
        causal = rnd.choice([True, True, False])
        Skv = max(Skv, Sq)
        pos = rnd.choice([Skv - Sq, Skv - Sq, 0, (Skv - Sq) // 2]) if causal else 0
        D = rnd.choice([64, 64, 128]); qg = rnd.choice([1, 2, 4, 8]); H = rnd.choice([1, 2, 4]) * qg; B = rnd.choice([1, 2, 8])
        dt = rnd.choice([torch.float16, torch.bfloat16])
        d = fmha.prepare(batch=B, heads=H, seq_q=Sq, seq_kv=Skv, d_k=D, d_v=D, query_group_size=qg, causal=causal, T=dt, seed=100 + it)
        out = torch.full_like(d.Q, NAN)
        fmha.cutile_fmha(d.Q, d.K, d.V, causal=causal, input_pos=pos, query_group_size=qg, out=out)
        seen.add(ct.last_variant())
        K = d.K.repeat_interleave(qg, dim=1).float(); V = d.V.repeat_interleave(qg, dim=1).float()
        mask = None
        if causal:
            mask = torch.arange(Skv, device="cuda")[None, :] <= (torch.arange(Sq, device="cuda")[:, None] + pos)
        ref = F.scaled_dot_product_attention(d.Q.float(), K, V, attn_mask=mask)
        assert close(out, ref, 3e-2 if dt == torch.bfloat16 else 2e-2), \
            f"B={B} H={H} Sq={Sq} Skv={Skv} pos={pos} D={D} group={qg} causal={causal} {dt} {ct.last_variant()}"
    split = ("_splitkv", "_splitkv_fused")
    assert any("_grouped_splitkv" in v for v in seen) and any(v.endswith(tuple("w64q" + e for e in split) + tuple("w32q" + e for e in split)) for v in seen)
    assert any(v.endswith("_fused") for v in seen) and any(v.endswith("_splitkv") for v in seen), seen
    assert any(v.endswith("_grouped") for v in seen), seen


def test_row_kernels_random_shapes(ct):
    rnd = random.Random(5)
    ns = [1, 3, 7, 64, 100, 255, 256, 257, 1000, 1024, 1500, 4096, 5000, 8192, 12000, 20000]
    for it in range(50):
        M = rnd.choice([1, 2, 5, 33, 100, 257, 1000]); N = rnd.choice(ns)
        g = torch.Generator(device="cuda").manual_seed(it)
        x = torch.randn((M, N), generator=g, device="cuda") * 3
        what = f"M={M} N={N}"
        out = torch.full_like(x, NAN)
        ct.softmax_tma_kernel(out, x, 1 << (N - 1).bit_length(), num_programs=M)
        ref = torch.softmax(x.double(), dim=1)
        assert close(out, ref, 1e-5), what + " softmax " + ct.last_variant()
        out.fill_(NAN)
        ct.softmax_chunked_kernel(out, x, N, rnd.choice([256, 1024]), num_programs=M)
        assert close(out, ref, 1e-5), what + " chunked softmax " + ct.last_variant()
        W = torch.randn(N, generator=g, device="cuda"); B = torch.randn(N, generator=g, device="cuda")
        DY = torch.randn((M, N), generator=g, device="cuda")
        Y, DX = torch.full_like(x, NAN), torch.full_like(x, NAN)
        Mean, Rstd = torch.full((M,), NAN, device="cuda"), torch.full((M,), NAN, device="cuda")
        G = rnd.choice([1, 4, 64, 256]); TN = rnd.choice([256, 1024])
        DWp, DBp = torch.zeros((G, N), device="cuda"), torch.zeros((G, N), device="cuda")
        Locks = torch.zeros(G, dtype=torch.int64, device="cuda")
        FDW, FDB = torch.full((N,), NAN, device="cuda"), torch.full((N,), NAN, device="cuda")
        ct.layer_norm_fwd(x, W, B, Y, Mean, Rstd, 1e-5, TN)
        ct.layer_norm_bwd_dx_partial_dwdb(DX, DY, DWp, DBp, x, W, Mean, Rstd, Locks, G, TN)
        ct.layer_norm_bwd_dwdb(DWp, DBp, FDW, FDB, 32, TN)
        xd = x.double(); mean = xd.mean(1, keepdim=True); var = ((xd - mean) ** 2).mean(1, keepdim=True)
        rstd = 1 / torch.sqrt(var + 1e-5); xh = (xd - mean) * rstd
        wdy = W.double() * DY.double(); c1 = (xh * wdy).mean(1, keepdim=True); c2 = wdy.mean(1, keepdim=True)
        for name, got, want in [("Y", Y, xh * W.double() + B.double()), ("dX", DX, (wdy - (xh * c1 + c2)) * rstd),
                                ("dW", FDW, (DY.double() * xh).sum(0)), ("dB", FDB, DY.double().sum(0)),
                                ("Mean", Mean, mean[:, 0]), ("Rstd", Rstd, rstd[:, 0])]:
            assert close(got, want, 2e-5), f"{what} G={G} TILE_N={TN} LayerNorm {name}"


def test_moe_random_configurations(ct):
    rnd = random.Random(5)
    for it in range(24):
        tokens = rnd.choice([1, 5, 33, 100, 256, 700]); hidden = rnd.choice([64, 128, 192, 512, 1024])
        E = rnd.choice([1, 2, 3, 8, 32, 60]); inter = rnd.choice([64, 96, 256, 512, 1024])
        topk = rnd.choice([k for k in (1, 2, 4, 8) if k <= E]); dt = rnd.choice([torch.float16, torch.float16, torch.bfloat16])
        d = moe.prepare(num_tokens=tokens, hidden_size=hidden, num_experts=E, intermediate_size=inter, topk=topk, T=dt, seed=it)
        out = moe.cutile_moe(d.hidden_states, d.w1, d.w2, d.topk_weights, d.topk_ids, 128, 128, 64)
        ref = moe.ref_moe(d.hidden_states, d.w1, d.w2, d.topk_weights, d.topk_ids).cuda()
        assert close(out.float(), ref, 2e-2 if dt == torch.float16 else 5e-2), f"tokens={tokens} hidden={hidden} E={E} inter={inter} topk={topk} {dt}"


def _jl(t):
    return t.detach().cpu().numpy().T


def test_tiled_random_shapes(ct):
    rnd = random.Random(7); rng = np.random.default_rng(7)
    sizes = [1, 1, 2, 3, 4, 5, 7, 8, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 1000, 1023, 1025, 4097]

    def rshape():
        nd = rnd.randint(1, 4)
        shp = [rnd.choice(sizes) for _ in range(nd)]
        while np.prod(shp) > 2_000_000:
            shp[rnd.randrange(nd)] = rnd.choice(sizes[:12])
        return tuple(shp)

    for it in range(150):      # reductions over random subsets of the dimensions, whole arrays and strided views
        shp = rshape(); nd = len(shp)
        dims = rnd.choice([None] + [tuple(sorted(rnd.sample(range(1, nd + 1), k))) for k in range(1, nd + 1)])
        kind = rnd.choice(["sum_f32", "max_f32", "min_i32", "sum_i32", "sum_f16", "max_f64"])
        if kind.endswith("f32"): a = rng.standard_normal(shp).astype(np.float32)
        elif kind.endswith("f64"): a = rng.standard_normal(shp)
        elif kind.endswith("f16"): a = (rng.random(shp) * 0.01).astype(np.float16)
        else: a = rng.integers(-1000, 1000, shp).astype(np.int32)
        A = torch.from_numpy(np.ascontiguousarray(a.T)).cuda()
        if rnd.random() < 0.3 and A.shape[-1] > 4:
            A = A[..., 1:-1]; a = a[1:-1]
        op = kind.split("_")[0]
        R = {"sum": T.sum, "max": T.maximum, "min": T.minimum}[op](Tiled(A), dims=dims)
        ax = None if dims is None else tuple(x - 1 for x in dims)
        ref = {"sum": np.sum, "max": np.max, "min": np.min}[op](a.astype(np.float64) if a.dtype.kind == "f" else a.astype(np.int64),
                                                               axis=ax, keepdims=dims is not None)
        got = np.float64(R) if dims is None else _jl(R).astype(np.float64)
        tol = 2e-3 if kind == "sum_f16" else 1e-5
        what = f"{kind} shape={shp} dims={dims} {ct.last_variant()}"
        assert np.shape(got) == np.shape(ref), what
        assert np.allclose(got, ref, rtol=tol, atol=tol * (np.abs(ref).max() + 1e-30)), what
    for it in range(150):      # a (op) b with size-1 expansion, lower-rank operands and mixed element types
        shp = rshape(); nd = len(shp)
        sa = tuple(s if rnd.random() < 0.7 else 1 for s in shp); sb = tuple(s if rnd.random() < 0.7 else 1 for s in shp)
        if rnd.random() < 0.2:
            sb = sb[:rnd.randint(1, nd)]
        ta, tb = rnd.choice([(np.float32, np.float32), (np.float32, np.int32), (np.int32, np.int32), (np.float16, np.float16), (np.float64, np.float32)])
        a = (rng.standard_normal(sa) * 10).astype(ta); b = (rng.standard_normal(sb) * 10).astype(tb)
        A = torch.from_numpy(np.ascontiguousarray(a.T)).cuda(); B = torch.from_numpy(np.ascontiguousarray(b.T)).cuda()
        opn = rnd.choice(["add", "mul", "sub", "max"])
        C = T.copy({"add": Tiled(A) + Tiled(B), "mul": Tiled(A) * Tiled(B), "sub": Tiled(A) - Tiled(B), "max": T.max(Tiled(A), Tiled(B))}[opn])
        af, bf = a.astype(np.float64), b.reshape(b.shape + (1,) * (len(sa) - len(sb))).astype(np.float64)
        ref = {"add": af + bf, "mul": af * bf, "sub": af - bf, "max": np.maximum(af, bf)}[opn]
        got = _jl(C).astype(np.float64)
        tol = 2e-3 if ta == np.float16 else 1e-6
        what = f"{opn} {sa} {sb} {ta.__name__} {tb.__name__} {ct.last_variant()}"
        assert got.shape == ref.shape, what
        assert np.allclose(got, ref, rtol=tol, atol=tol), what
