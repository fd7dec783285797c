"""GPU parity tests for the fused attention kernel through the C ABI.

Oracle: the numpy restatement of ``ref_fmha`` (examples/fmha.jl:175-220), evaluated in float64
on the f16/bf16 inputs (the "fp32 reference" of the tolerance, at higher precision).  Shapes:
the reference example's ``main()`` list (fmha.jl:314-325) plus GQA, decode offset
(``input_pos``), ragged sequence lengths (EVEN_K = false), D = 128 and strided views.

Tolerance: |err| <= 2e-2 * (|ref| + max|ref|) element-wise, and the reference's own
``isapprox(rtol=1e-2, atol=1e-3)`` (fmha.jl:277-282).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd.examples import fmha  # noqa: E402


def attend(Q, K, V, **kw):
    """cutile_fmha into an output buffer filled with NaN beforehand: an element the kernel never writes fails the check."""
    out = torch.full((Q.shape[0], Q.shape[1], Q.shape[2], V.shape[3]), float("nan"), dtype=Q.dtype, device=Q.device)
    ret = fmha.cutile_fmha(Q, K, V, out=out, **kw)
    assert ret is out
    return out


class _Result:
    def __init__(self, out):
        self.out = out


def run(data):
    return _Result(attend(data.Q, data.K, data.V, tile_m=data.tile_m, tile_n=data.tile_n,
                          query_group_size=data.query_group_size, causal=data.causal))


def check(orc, out, ref, tol=2e-2):
    got = orc.to_julia(out).astype(np.float64)
    err = np.abs(got - ref)
    bound = tol * (np.abs(ref) + np.abs(ref).max())
    assert np.all(err <= bound), f"max err {err.max():.3e}, worst ratio {np.max(err / bound):.3f}"
    assert orc.isapprox(got, ref, rtol=1e-2, atol=1e-3)
    return err.max()


@pytest.mark.parametrize("batch,heads,sq,skv,d,causal,qg,T", [
    (2, 8, 128, 128, 64, False, 1, torch.float16), (2, 8, 128, 128, 64, True, 1, torch.float16),
    (4, 16, 256, 256, 64, True, 1, torch.float16),
    (1, 4, 384, 384, 64, True, 2, torch.float16), (1, 8, 256, 512, 64, False, 4, torch.float16),
    (2, 2, 200, 200, 64, True, 1, torch.float16), (1, 2, 77, 130, 64, False, 1, torch.float16),
    (1, 2, 1, 1, 64, True, 1, torch.float16), (1, 2, 130, 64, 64, False, 1, torch.float16),
    (2, 4, 256, 256, 128, True, 1, torch.float16), (1, 2, 100, 300, 128, False, 2, torch.float16),
    (2, 4, 256, 256, 64, True, 1, torch.bfloat16), (1, 2, 192, 192, 128, False, 1, torch.bfloat16),
    (16, 8, 384, 384, 64, True, 1, torch.float16), (8, 8, 640, 640, 64, True, 1, torch.float16), (4, 4, 896, 896, 64, True, 2, torch.bfloat16),
    (8, 8, 384, 384, 64, False, 1, torch.float16), (24, 8, 128, 128, 64, True, 1, torch.float16), (8, 16, 1536, 1536, 64, True, 4, torch.float16),
])
def test_fmha_against_ref(orc, batch, heads, sq, skv, d, causal, qg, T):
    data = fmha.prepare(batch=batch, heads=heads, seq_q=sq, seq_kv=skv, d_k=d, d_v=d, query_group_size=qg,
                        causal=causal, T=T)
    r = run(data)
    Q, K, V = (orc.to_julia(t) for t in (data.Q, data.K, data.V))
    if causal and sq != skv:
        pytest.skip("ref_fmha's causal mask assumes aligned positions")
    ref = orc.ref_fmha(Q, K, V, causal=causal, dtype=np.float64)
    check(orc, r.out, ref, 2e-2 if T == torch.float16 else 3e-2)


def test_fmha_reference_input_distribution(orc):
    """The reference's own inputs, U(-0.5, 0.5) (fmha.jl:240-242)."""
    data = fmha.prepare(batch=2, heads=8, seq_q=256, seq_kv=256, dist="uniform")
    r = run(data)
    ref = orc.ref_fmha(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=True, dtype=np.float64)
    check(orc, r.out, ref)


@pytest.mark.parametrize("sq,skv,pos", [(64, 256, 192), (1, 200, 199), (128, 300, 100), (130, 512, 300)])
def test_fmha_decode_offset(orc, sq, skv, pos):
    """input_pos shifts the query positions (fmha.jl:45-46,66): query i sees keys <= pos + i."""
    data = fmha.prepare(batch=1, heads=4, seq_q=sq, seq_kv=skv, query_group_size=2)
    out = attend(data.Q, data.K, data.V, input_pos=pos, causal=True, query_group_size=2)
    ref = orc.fmha_general(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=True, input_pos=pos)
    check(orc, out, ref)


def test_fmha_causal_first_row_and_noncausal_limit(orc):
    data = fmha.prepare(batch=1, heads=2, seq_q=256, seq_kv=256)
    out = attend(data.Q, data.K, data.V, causal=True)
    # query 1 attends to key 1 only: output row equals V[:, 1] exactly (softmax weight 1.0)
    assert torch.equal(out[:, :, 0, :], data.V[:, :, 0, :])
    # with input_pos >= Skv the causal kernel sees every key: equals the non-causal kernel bit for bit
    a = attend(data.Q, data.K, data.V, causal=True, input_pos=256)
    b = attend(data.Q, data.K, data.V, causal=False)
    assert torch.equal(a, b)


def test_fmha_strided_views_and_scale(orc):
    """Q/K/V as views of a packed (B, S, 3, H, D) buffer, and an explicit qk_scale."""
    rng = np.random.default_rng(0)
    B, S, H, D = 2, 192, 4, 64
    packed = torch.from_numpy(rng.standard_normal((B, S, 3, H, D), dtype=np.float32)).to(torch.float16).cuda()
    Q, K, V = (packed[:, :, i].permute(0, 2, 1, 3) for i in range(3))  # torch (B,H,S,D) views, D contiguous
    out = attend(Q, K, V, causal=True, qk_scale=0.2)
    ref = orc.ref_fmha(orc.to_julia(Q), orc.to_julia(K), orc.to_julia(V), qk_scale=0.2, causal=True, dtype=np.float64)
    check(orc, out, ref)


@pytest.mark.parametrize("batch,heads,s,causal,qg,T", [
    (1, 4, 512, True, 2, torch.float16), (1, 2, 640, True, 1, torch.float16), (1, 2, 640, False, 1, torch.float16),
    (1, 2, 512, True, 1, torch.bfloat16), (3, 3, 256, True, 1, torch.float16), (1, 8, 1024, False, 8, torch.float16),
    (1, 2, 128, True, 1, torch.float16), (1, 1, 384, True, 1, torch.float16), (1, 2, 2048, True, 2, torch.bfloat16),
])
def test_fmha_pipelined_kernel_shapes(ct, orc, batch, heads, s, causal, qg, T):
    """Shapes served by the software-pipelined D = 64 kernel (Sq == Skv, multiple of 128): odd numbers
    of 128-query blocks, (batch*heads) not a multiple of 8, GQA, bf16, and both mask settings.  With the
    causal mask a wave walks its long tile two key halves per trip once its early tile is done: 128 keys give
    one such trip, 384 up to five, 2048 up to thirty-one."""
    data = fmha.prepare(batch=batch, heads=heads, seq_q=s, seq_kv=s, query_group_size=qg, causal=causal, T=T)
    r = run(data)
    assert ct.last_variant().startswith("fmha_pipe")
    ref = orc.ref_fmha(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=causal, dtype=np.float64)
    check(orc, r.out, ref, 2e-2 if T == torch.float16 else 3e-2)


@pytest.mark.parametrize("batch,heads,s,qg,T", [
    (1, 8, 129, 1, torch.float16), (2, 3, 160, 1, torch.float16), (1, 8, 191, 4, torch.bfloat16), (1, 2, 193, 1, torch.float16),
    (1, 4, 255, 2, torch.float16), (1, 8, 257, 1, torch.bfloat16), (1, 2, 333, 1, torch.float16), (1, 16, 500, 1, torch.float16),
    (2, 8, 647, 2, torch.float16), (1, 2, 1000, 1, torch.float16), (1, 1, 1023, 1, torch.bfloat16), (1, 2, 1025, 1, torch.float16),
])
def test_fmha_pipelined_kernel_ragged_causal(ct, orc, batch, heads, s, qg, T):
    """Causal attention over a sequence that is not a multiple of 128 runs on the pipelined kernel as well: the last
    key half that exists is partial (its missing rows re-read the last row and fall to the causal mask), halves past
    it are never fetched, query rows past the end are not stored.  Lengths one past / one short of a half, of a
    workgroup's 128 queries and of a pair of them; the output sits in a wider buffer whose rows past the end must
    stay as they were."""
    data = fmha.prepare(batch=batch, heads=heads, seq_q=s, seq_kv=s, query_group_size=qg, causal=True, T=T)
    big = torch.full((batch, heads, s + 40, 64), 777.0, dtype=T, device="cuda")
    out = big[:, :, :s, :]
    out.fill_(float("nan"))
    fmha.cutile_fmha(data.Q, data.K, data.V, query_group_size=qg, causal=True, out=out)
    assert ct.last_variant() == "fmha_pipe_d64_q128_kv32_ring4_ragged"
    assert bool((big[:, :, s:, :] == 777.0).all())
    ref = orc.ref_fmha(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=True, dtype=np.float64)
    check(orc, out, ref, 2e-2 if T == torch.float16 else 3e-2)


@pytest.mark.parametrize("batch,heads,s,qg,T", [
    (1, 8, 129, 1, torch.float16), (2, 3, 161, 1, torch.bfloat16), (1, 8, 192, 4, torch.float16), (1, 2, 197, 1, torch.float16),
    (1, 4, 225, 2, torch.bfloat16), (1, 8, 257, 1, torch.float16), (1, 2, 577, 1, torch.float16), (1, 2, 1000, 2, torch.float16),
    (1, 1, 1023, 1, torch.float16), (1, 2, 1025, 1, torch.bfloat16),
])
def test_fmha_pipelined_kernel_ragged_without_the_causal_mask(ct, orc, batch, heads, s, qg, T):
    """Without the causal mask nothing hides the keys past the end: the walk stops with the pair of key halves that
    holds the last key and masks their scores against the sequence length (an odd number of halves ends with one
    that is masked as a whole)."""
    data = fmha.prepare(batch=batch, heads=heads, seq_q=s, seq_kv=s, query_group_size=qg, causal=False, T=T)
    big = torch.full((batch, heads, s + 40, 64), 777.0, dtype=T, device="cuda")
    out = big[:, :, :s, :]
    out.fill_(float("nan"))
    fmha.cutile_fmha(data.Q, data.K, data.V, query_group_size=qg, causal=False, out=out)
    assert ct.last_variant() == "fmha_pipe_d64_q128_kv32_ring4_ragged"
    assert bool((big[:, :, s:, :] == 777.0).all())
    ref = orc.ref_fmha(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=False, dtype=np.float64)
    check(orc, out, ref, 2e-2 if T == torch.float16 else 3e-2)


def test_fmha_more_keys_than_queries_takes_the_general_kernel(ct, orc):
    data = fmha.prepare(batch=1, heads=2, seq_q=200, seq_kv=333, causal=False)
    r = run(data)
    assert ct.last_variant().startswith("fmha_dma") or ct.last_variant().startswith("fmha_regstage")
    ref = orc.ref_fmha(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=False, dtype=np.float64)
    check(orc, r.out, ref)


@pytest.mark.parametrize("batch,heads,sq,skv,qg,causal,pos,d,T", [
    (2, 4, 1, 1000, 1, True, 999, 64, torch.float16),        # one query at the end of the cache
    (1, 8, 1, 4096, 4, True, 4095, 64, torch.bfloat16),      # grouped heads
    (1, 2, 7, 777, 1, True, 770, 64, torch.float16),         # a few queries, ragged cache
    (1, 4, 130, 2000, 2, True, 1870, 64, torch.float16),     # two query blocks
    (1, 2, 200, 3000, 1, False, 0, 64, torch.bfloat16),      # no mask
    (1, 1, 64, 5000, 1, True, 4000, 64, torch.float16),      # the cache ends above every diagonal
    (1, 2, 512, 600, 1, True, 88, 64, torch.float16),        # the second part starts above the diagonals of the early rows:
    (1, 2, 512, 512, 1, True, 0, 128, torch.float16),        # they go through it without a visible key
    (1, 2, 256, 4096, 1, True, 1000, 128, torch.float16),    # D = 128
    (1, 3, 33, 2049, 1, False, 0, 128, torch.bfloat16),
    (1, 8, 1, 2048, 2, True, 2047, 128, torch.float16),
    # grouped heads with few queries: the heads of a group are stacked as rows of one query tile
    (2, 8, 1, 1300, 8, True, 1299, 64, torch.float16), (1, 16, 64, 640, 4, True, 576, 64, torch.bfloat16),
    (1, 12, 17, 555, 3, False, 0, 64, torch.float16), (2, 8, 40, 4000, 4, True, 3900, 128, torch.float16),
    (4, 32, 1, 2048, 4, True, 2047, 64, torch.float16),
])
def test_fmha_few_queries_many_keys_split_over_the_keys(ct, orc, batch, heads, sq, skv, qg, causal, pos, d, T):
    """Decode and chunked-prefill shapes: too few (query block, head) pairs to fill the chip, so the key range of each is
    dealt to several workgroups and a second kernel adds their parts.  Against the float64 restatement of the kernel's
    masking rule, into an output inside a wider buffer."""
    data = fmha.prepare(batch=batch, heads=heads, seq_q=sq, seq_kv=skv, d_k=d, d_v=d, query_group_size=qg, causal=causal, T=T)
    big = torch.full((batch, heads, sq + 8, d), 777.0, dtype=T, device="cuda")
    out = big[:, :, :sq, :]
    out.fill_(float("nan"))
    fmha.cutile_fmha(data.Q, data.K, data.V, query_group_size=qg, causal=causal, input_pos=pos, out=out)
    assert ct.last_variant().endswith(("_splitkv", "_splitkv_fused")), ct.last_variant()
    # few rows per (batch, head) and few parts: the part that arrives last adds the parts, no second launch
    if sq * (qg if sq <= 64 else 1) <= 64 and ct.last_variant().endswith("_fused"):
        again = torch.full_like(big, 555.0)[:, :, :sq, :]
        fmha.cutile_fmha(data.Q, data.K, data.V, query_group_size=qg, causal=causal, input_pos=pos, out=again)
        assert torch.equal(again, out), "a second launch found the arrival counters of the first in another state"
    assert ("_grouped" in ct.last_variant()) == (qg > 1 and sq <= 64)
    assert bool((big[:, :, sq:, :] == 777.0).all())
    ref = orc.fmha_general(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=causal, input_pos=pos)
    check(orc, out, ref, 2e-2 if T == torch.float16 else 3e-2)


@pytest.mark.parametrize("batch,heads,sq,skv,qg,causal,pos,d", [
    (2, 8, 1, 200, 8, True, 199, 64), (1, 8, 33, 100, 8, True, 10, 64), (3, 6, 5, 130, 2, False, 0, 128), (1, 4, 64, 64, 4, True, 0, 64),
])
def test_fmha_grouped_heads_stacked_short_cache(ct, orc, batch, heads, sq, skv, qg, causal, pos, d):
    """Grouped heads with few queries and too few keys to split: the group's heads as rows of one query tile, one
    workgroup per (batch, K / V head)."""
    data = fmha.prepare(batch=batch, heads=heads, seq_q=sq, seq_kv=skv, d_k=d, d_v=d, query_group_size=qg, causal=causal)
    out = attend(data.Q, data.K, data.V, query_group_size=qg, causal=causal, input_pos=pos)
    assert ct.last_variant().endswith("_grouped"), ct.last_variant()
    ref = orc.fmha_general(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=causal, input_pos=pos)
    check(orc, out, ref)


@pytest.mark.parametrize("batch,heads,sq,skv,qg,pos,d,T", [
    (2, 4, 1, 1000, 1, 999, 64, torch.float16),        # split over the keys, parts added by the last one to arrive
    (1, 8, 1, 4096, 4, 4095, 64, torch.bfloat16),      # grouped heads stacked in one query tile
    (1, 2, 7, 777, 1, 770, 64, torch.float16),         # ragged cache: the last tile's clamped transfers
    (1, 8, 1, 2048, 2, 2047, 128, torch.float16),      # D = 128
    (2, 8, 33, 100, 8, 10, 64, torch.float16),         # too few keys to split: one workgroup per (batch, K / V head)
])
def test_fmha_key_cache_streamed_with_non_temporal_transfers(ct, orc, monkeypatch, batch, heads, sq, skv, qg, pos, d, T):
    """A cache that one query block walks alone and that is larger than the memory-side cache is requested with
    non-temporal transfers; the choice is forced both ways here (MI_FMHA_KV_STREAM), on small caches: the same
    arithmetic, so the same bits, and the oracle's values."""
    data = fmha.prepare(batch=batch, heads=heads, seq_q=sq, seq_kv=skv, d_k=d, d_v=d, query_group_size=qg, causal=True, T=T)
    outs = []
    for knob in ("0", "1"):
        monkeypatch.setenv("MI_FMHA_KV_STREAM", knob)
        outs.append(attend(data.Q, data.K, data.V, query_group_size=qg, causal=True, input_pos=pos))
        assert ct.last_variant().startswith("fmha_dma_"), ct.last_variant()
    assert torch.equal(outs[0], outs[1])
    ref = orc.fmha_general(*(orc.to_julia(t) for t in (data.Q, data.K, data.V)), causal=True, input_pos=pos)
    check(orc, outs[1], ref, 2e-2 if T == torch.float16 else 3e-2)


def test_fmha_split_launches_from_two_streams_are_ordered(ct, orc):
    """The parts live in one array per GPU: launches that alternate between two streams each get their own result."""
    datas = [fmha.prepare(batch=1, heads=4, seq_q=1, seq_kv=3000 + 64 * i, causal=True, seed=20 + i) for i in range(3)]
    refs = [orc.fmha_general(*(orc.to_julia(t) for t in (d.Q, d.K, d.V)), causal=True, input_pos=d.seq_kv - 1) for d in datas]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = []
    for i in range(12):
        d = datas[i % 3]
        with torch.cuda.stream(streams[i % 2]):
            outs.append(fmha.cutile_fmha(d.Q, d.K, d.V, causal=True, input_pos=d.seq_kv - 1))
            assert ct.last_variant().endswith(("_splitkv", "_splitkv_fused"))
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        check(orc, o, refs[i % 3])
        assert torch.equal(o, outs[i % 3])


@pytest.mark.parametrize("causal", [True, False])
def test_fmha_pipelined_kernel_strided_views(ct, orc, causal):
    """Q/K/V as views of one packed (B, S, 3, H, D) buffer and Out as a view of a wider buffer: row,
    head and batch strides all differ from the dense ones."""
    rng = np.random.default_rng(4)
    B, S, H, D = 2, 256, 4, 64
    packed = torch.from_numpy(rng.standard_normal((B, S, 3, H, D), dtype=np.float32)).to(torch.float16).cuda()
    Q, K, V = (packed[:, :, i].permute(0, 2, 1, 3) for i in range(3))        # torch (B, H, S, D) views
    out_buf = torch.zeros((B, H, S, 2 * D), dtype=torch.float16, device="cuda")
    out = out_buf[..., D:]                                                     # rows 2*D apart, offset D
    fmha.cutile_fmha(Q, K, V, causal=causal, out=out)
    assert ct.last_variant().startswith("fmha_pipe")
    ref = orc.ref_fmha(orc.to_julia(Q), orc.to_julia(K), orc.to_julia(V), causal=causal, dtype=np.float64)
    check(orc, out, ref)
    assert torch.all(out_buf[..., :D] == 0)


@pytest.mark.parametrize("causal", [True, False])
def test_fmha_running_maximum_keeps_rising(ct, orc, causal):
    """Scores that grow with the key index by far more than the kernel's lazy-rescale threshold:
    the running maximum has to be raised again and again, and early keys end up with weights
    far below the smallest f16 subnormal."""
    rng = np.random.default_rng(11)
    D, S, H, B = 64, 512, 2, 1
    q = rng.standard_normal((D, S, H, B)).astype(np.float32) * 0.25 + 1.0
    ramp = (1.0 + 6.0 * np.arange(S) / S)[None, :, None, None]
    k = (rng.standard_normal((D, S, H, B)).astype(np.float32) * 0.25 + 1.0) * ramp
    v = rng.standard_normal((D, S, H, B)).astype(np.float32)
    Q, K, V = (orc.from_julia(x).to(torch.float16).cuda() for x in (q, k, v))
    out = attend(Q, K, V, causal=causal)
    assert ct.last_variant().startswith("fmha_pipe")
    ref = orc.ref_fmha(*(orc.to_julia(t) for t in (Q, K, V)), causal=causal, dtype=np.float64)
    check(orc, out, ref)


def test_fmha_argument_errors(ct):
    data = fmha.prepare(batch=1, heads=2, seq_q=128, seq_kv=128)
    out = torch.empty_like(data.Q)
    with pytest.raises(ct.MiError) as e:
        ct.fmha_kernel(data.Q, data.K, data.V, out, 0.125, 0, 64, 2, 128, 128, 1, True, False)  # EVEN_K mismatch
    assert e.value.code == ct.MI_E_ARG
    with pytest.raises(ct.MiError) as e:
        ct.fmha_kernel(data.Q, data.K, data.V, out, 0.125, 0, 32, 2, 128, 128, 1, True, True)   # TILE_D != D
    assert e.value.code == ct.MI_E_SHAPE


def test_fmha_full_size(orc):
    """Benchmark shape 8x16x1024x64 causal: a sample of (batch, head) pairs against float64 and
    the softmax-weights-sum-to-one property via V = ones."""
    data = fmha.prepare(benchmark=True)
    r = run(data)
    Q, K, V = (orc.to_julia(t) for t in (data.Q, data.K, data.V))
    got = orc.to_julia(r.out).astype(np.float64)
    for (h, b) in [(0, 0), (15, 7), (7, 3)]:
        ref = orc.ref_fmha(Q[:, :, h:h + 1, b:b + 1], K[:, :, h:h + 1, b:b + 1], V[:, :, h:h + 1, b:b + 1],
                           causal=True, dtype=np.float64)
        err = np.abs(got[:, :, h, b] - ref[:, :, 0, 0])
        assert np.all(err <= 2e-2 * (np.abs(ref[:, :, 0, 0]) + np.abs(ref).max()))
    ones = torch.ones_like(data.V)
    out1 = attend(data.Q, data.K, ones, causal=True)
    assert torch.all((out1.float() - 1).abs() <= 2e-3)


def test_fmha_more_than_65535_batch_heads(ct, orc):
    """The reference's grid is (cld(Sq, TILE_M), B * H) with up to 2^24 - 1 blocks per dimension
    (fmha.jl:163-165, src/launch.jl:743): 70 000 (batch, head) pairs of a short sequence."""
    data = fmha.prepare(batch=10, heads=7000, seq_q=16, seq_kv=16, causal=True)
    r = run(data)
    Q, K, V = (orc.to_julia(t) for t in (data.Q, data.K, data.V))
    got = orc.to_julia(r.out).astype(np.float64)
    for b, hs in ((0, slice(0, 3)), (9, slice(6997, 7000)), (9, slice(3552, 3555))):    # pairs 0.., 69997.., 66552..
        ref = orc.ref_fmha(Q[:, :, hs, b:b + 1], K[:, :, hs, b:b + 1], V[:, :, hs, b:b + 1], causal=True, dtype=np.float64)
        g = got[:, :, hs, b:b + 1]
        assert np.all(np.abs(g - ref) <= 2e-2 * (np.abs(ref) + np.abs(ref).max()))
