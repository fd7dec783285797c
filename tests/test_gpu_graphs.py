"""HIP graphs.  A caller with a launch-bound loop captures the library's launches into a graph and replays it.
Each case here captures one entry point (or one of the examples' orchestrations) over static buffers, then
replays the graph three times: before every replay the static inputs receive new data and the same work runs
eagerly on that data (so the program's own launches and synchronisations sit between the replays), and the
replay has to reproduce the eager result -- bit for bit, except where the eager call may pick another summation
order than the captured one (the matmul that is split over K uses a scratch array of the library, which a
capturing stream is not given; stated at that case)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd import tiled as T  # noqa: E402
from cutile_jl_amd.tiled import Tiled  # noqa: E402
from cutile_jl_amd.examples import fft, fmha, moe  # noqa: E402


def replay_check(make_inputs, op, rounds=3, compare=None):
    """``make_inputs(seed)`` -> tuple of tensors; ``op(*inputs)`` launches on the current stream and returns a tuple of
    output tensors."""
    compare = compare or (lambda got, ref, name: torch.equal(got, ref))
    static = make_inputs(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        op(*static)                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = op(*static)
    for r in range(1, rounds + 1):
        fresh = make_inputs(r)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        eager = [o.clone() for o in op(*fresh)]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert len(outs) == len(eager)
        for i, (got, ref) in enumerate(zip(outs, eager)):
            assert not torch.isnan(ref.float()).any() if ref.is_floating_point() else True
            assert compare(got, ref, i), f"replay {r}: output {i} differs from the eager result"


def gen(seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(7000 + seed)
    return g


def test_graph_vadd_and_transpose(ct):
    def inputs(seed):
        g = gen(seed)
        return (torch.rand((1 << 20) + 3, device="cuda", generator=g), torch.rand((1 << 20) + 3, device="cuda", generator=g),
                torch.rand(1024, 512, device="cuda", generator=g), torch.rand(264, 520, device="cuda", generator=g).half())

    def op(a, b, x, xh):
        c = torch.empty_like(a); ct.vec_add_kernel_1d(a, b, c, 1024)
        y = torch.empty(512, 1024, device="cuda"); ct.transpose_kernel(x, y, 64, 64)
        yh = torch.empty(520, 264, device="cuda", dtype=torch.float16); ct.transpose_kernel(xh, yh, 32, 32)
        return c, y, yh

    replay_check(inputs, op)


def test_graph_softmax_and_layernorm(ct):
    M, N = 300, 2048

    def inputs(seed):
        g = gen(seed)
        return (torch.randn(M, N, device="cuda", generator=g), torch.randn(N, device="cuda", generator=g) * 0.1 + 1.0,
                torch.randn(N, device="cuda", generator=g) * 0.1, torch.randn(M, N, device="cuda", generator=g))

    def op(X, W, B, DY):
        e = lambda *s: torch.empty(*s, device="cuda")
        S1, S2 = e(M, N), e(M, N)
        ct.softmax_tma_kernel(S1, X, 2048)
        ct.softmax_chunked_kernel(S2, X, N, 1024)
        Y, Mean, Rstd, DX, FDW, FDB = e(M, N), e(M), e(M), e(M, N), e(N), e(N)
        partials = e(2, 64, N)
        locks = torch.zeros(64, dtype=torch.int64, device="cuda")
        ct.layer_norm_fwd(X, W, B, Y, Mean, Rstd, 1e-5, 1024)
        partials.zero_()
        ct.layer_norm_bwd_dx_partial_dwdb(DX, DY, partials[0], partials[1], X, W, Mean, Rstd, locks, 64, 1024)
        ct.layer_norm_bwd_dwdb(partials[0], partials[1], FDW, FDB, 32, 1024)
        return S1, S2, Y, Mean, Rstd, DX, FDW, FDB

    replay_check(inputs, op)


def test_graph_layernorm_backward_without_allocation(ct):
    """The one entry point made for capturing callers: the warm-up call outside the capture is also what makes the
    address of the library's static array known (the lookup is not allowed inside a capture)."""
    M, N, G = 257, 1536, 32

    def inputs(seed):
        g = gen(seed)
        return (torch.randn(M, N, device="cuda", generator=g), torch.randn(N, device="cuda", generator=g) * 0.1 + 1.0,
                torch.randn(N, device="cuda", generator=g) * 0.1, torch.randn(M, N, device="cuda", generator=g))

    def op(X, W, B, DY):
        e = lambda *s: torch.empty(*s, device="cuda")
        Y, Mean, Rstd, DX, FDW, FDB = e(M, N), e(M), e(M), e(M, N), e(N), e(N)
        ct.layer_norm_fwd(X, W, B, Y, Mean, Rstd, 1e-5, 1024)
        ct.layer_norm_bwd_static(DX, DY, X, W, Mean, Rstd, FDW, FDB, G, 32, 1024)
        return DX, FDW, FDB

    def compare(got, ref, i):
        # dW / dB are sums of float atomics, whose order differs from launch to launch
        if i == 0:
            return torch.equal(got, ref)
        return bool(((got - ref).abs() <= 1e-5 * (ref.abs() + ref.abs().max())).all())

    replay_check(inputs, op, compare=compare)


def test_graph_matmul(ct):
    def inputs(seed):
        g = gen(seed)
        h = lambda *s: (torch.randn(*s, device="cuda", generator=g) / 8).half()
        return (h(512, 2048), h(2048, 512),            # Julia A (2048, 512), B (512, 2048): the 256 x 256 ring kernel
                h(4096, 512), h(512, 4096),            # Julia A (512, 4096), B (4096, 512): split over K when eager
                torch.randn(3, 96, 200, device="cuda", generator=g), torch.randn(3, 72, 96, device="cuda", generator=g))

    def op(A, B, A2, B2, A3, B3):
        C = torch.empty(2048, 2048, device="cuda"); ct.matmul_kernel(A, B, C, 64, 64, 64)
        C2 = torch.empty(512, 512, device="cuda"); ct.matmul_kernel(A2, B2, C2, 64, 64, 64)
        C3 = torch.empty(3, 72, 200, device="cuda"); ct.batch_matmul_kernel(A3, B3, C3, 32, 32, 32)
        return C, C2, C3

    def compare(got, ref, i):
        # output 1: eager splits K into parts and adds them in a fixed order, the captured launch walks K in one
        # piece: the same products in fp32, another order of the additions
        return torch.allclose(got, ref, rtol=1e-4, atol=1e-4) if i == 1 else torch.equal(got, ref)

    replay_check(inputs, op, compare=compare)


def test_graph_attention(ct):
    def inputs(seed):
        g = gen(seed)
        h = lambda *s: torch.randn(*s, device="cuda", generator=g).half()
        return (h(2, 8, 512, 64), h(2, 8, 512, 64), h(2, 8, 512, 64), h(1, 4, 200, 64), h(1, 2, 333, 64), h(1, 2, 333, 64),
                h(2, 8, 1, 64), h(2, 2, 3000, 64), h(2, 2, 3000, 64))

    def op(Q, K, V, Q2, K2, V2, Q3, K3, V3):
        return (fmha.cutile_fmha(Q, K, V, causal=True), fmha.cutile_fmha(Q, K, V, causal=False),
                fmha.cutile_fmha(Q2, K2, V2, causal=False, query_group_size=2, tile_m=64, tile_n=64),
                fmha.cutile_fmha(Q3, K3, V3, causal=True, input_pos=2999, query_group_size=4))

    def compare(got, ref, i):
        # output 3, one new token against 3000 cached keys: eager deals the keys to several workgroups and adds their
        # parts, the captured launch walks them in one piece (the library's scratch is not handed to a capturing stream)
        return torch.allclose(got.float(), ref.float(), rtol=2e-3, atol=2e-3) if i == 3 else torch.equal(got, ref)

    replay_check(inputs, op, compare=compare)


def test_graph_with_the_shared_arrays_handed_to_the_capture(ct):
    """mi_scratch_under_capture(1): the caller keeps its replays apart, and a capturing stream gets what an eager one
    gets -- attention split over the keys (with the last part adding the parts), the matmul split over K, the token
    sort of several workgroups.  The recorded variants are the eager ones and every replay equals the eager result
    bit for bit (split sums are added in a fixed order).  Off again, the one-piece kernels are recorded."""
    seen = []

    def inputs(seed):
        g = gen(seed)
        h = lambda *s: (torch.randn(*s, device="cuda", generator=g) / 4).half()
        ids = torch.randint(1, 41, (3, 5000), device="cuda", generator=g)
        return (h(2, 8, 1, 64), h(2, 2, 3000, 64), h(2, 2, 3000, 64), h(4096, 512), h(512, 4096), ids)

    def op(Q, K, V, A, B, ids):
        o = fmha.cutile_fmha(Q, K, V, causal=True, input_pos=2999, query_group_size=4)
        seen.append(ct.last_variant())
        C = torch.empty(512, 512, device="cuda"); ct.matmul_kernel(A, B, C, 64, 64, 64)
        seen.append(ct.last_variant())
        tok, exp = ct.moe_align_tile_size_device(ids, 64, 40)
        seen.append(ct.last_variant())
        return o, C, tok, exp

    was = ct.scratch_under_capture(True)
    try:
        replay_check(inputs, op)
        # calls in order: warm-up, capture, then one eager call per round
        assert all("splitkv" in v for v in seen[0::3]) and all("splitk" in v for v in seen[1::3]), seen
        assert all(v == "moe_align_device_count_place" for v in seen[2::3]), seen
        ct.scratch_under_capture(False)
        del seen[:]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        static = inputs(9)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                op(*static)
        assert "splitkv" not in seen[0] and "splitk" not in seen[1] and seen[2] == "moe_align_device_1wg", seen
    finally:
        ct.scratch_under_capture(was)


@pytest.mark.parametrize("topk", [2, 8])
def test_graph_moe_with_its_defaults(ct, topk):
    """Token sort on the device, both grouped GEMMs, and for top-2 the down projection that adds into an output the
    sort launch has cleared: everything a replay needs is part of the graph."""
    def inputs(seed):
        d = moe.prepare(num_tokens=70, hidden_size=256, num_experts=16, intermediate_size=512, topk=topk, seed=seed)
        return d.hidden_states, d.w1, d.w2, d.topk_weights, d.topk_ids

    def op(h, w1, w2, tw, ids):
        return (moe.cutile_moe(h, w1, w2, tw, ids, 32, 128, 128),)

    replay_check(inputs, op)


def test_graph_tiled_and_fft(ct):
    d0 = fft.prepare(batch=8, factors=(8, 8, 8))
    F0, F1, F2 = d0.factors

    def inputs(seed):
        g = gen(seed)
        return torch.randn(257, 1000, device="cuda", generator=g), torch.randn(d0.x_packed.shape, device="cuda", generator=g)

    def op(x, xp):
        e = torch.empty_like(x)
        X = Tiled(x)
        Tiled(e).assign(T.sin(X) * 2.0 + X)
        yp = torch.empty_like(xp)
        ct.fft_kernel(xp, yp, d0.W0, d0.W1, d0.W2, d0.T0, d0.T1, d0.N, F0, F1, F2, 1, d0.D)
        # (a reduction over every dimension with dims=None returns a host number: a synchronisation, not capturable)
        return e, T.sum(X, dims=1), T.sum(X, dims=2), T.maximum(X, dims=(1, 2)), yp

    replay_check(inputs, op)
