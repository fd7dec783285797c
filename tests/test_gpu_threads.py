"""Host threads.  The library keeps a little state of its own -- the record of the last kernel variant (per thread),
the compiled plans of the host-level Tiled entry points (behind a lock), the partial sums of the matmul that is
split over K (one array per GPU, users ordered by an event) -- and callers such as a Julia or Python server call
it from several threads at once, each on its own stream (ctypes releases the interpreter lock during a call).
Every thread repeats a fixed mix of kernels on its own stream and inputs and must get, bit for bit, what the same
mix gave when it ran alone."""
import threading

import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd import tiled as T  # noqa: E402
from cutile_jl_amd.tiled import Tiled  # noqa: E402
from cutile_jl_amd.examples import fmha, moe  # noqa: E402

NTHREADS, REPEATS = 4, 6


def _inputs(seed):
    g = torch.Generator(device="cuda"); g.manual_seed(1000 + seed)
    n = 1 << 18
    d = {}
    d["a"], d["b"] = torch.rand(n + seed, device="cuda", generator=g), torch.rand(n + seed, device="cuda", generator=g)
    d["x"] = torch.randn(300 + seed, 1024, device="cuda", generator=g)
    d["A"] = (torch.randn(4096, 512, device="cuda", generator=g) / 8).to(torch.float16)     # Julia (M, K) = (512, 4096)
    d["B"] = (torch.randn(512, 4096, device="cuda", generator=g) / 8).to(torch.float16)     # Julia (K, N)
    d["Q"] = torch.randn(2, 4, 256 + 128 * seed, 64, device="cuda", generator=g).to(torch.float16)
    d["K"] = torch.randn(2, 4, 256 + 128 * seed, 64, device="cuda", generator=g).to(torch.float16)
    d["V"] = torch.randn(2, 4, 256 + 128 * seed, 64, device="cuda", generator=g).to(torch.float16)
    d["moe"] = moe.prepare(num_tokens=40 + seed, hidden_size=256, num_experts=8, intermediate_size=512, topk=2, seed=seed)
    return d


def _mix(ct, d, seed):
    """One pass over the kernels on the current stream; returns the outputs and the variants this thread saw."""
    out, var = {}, {}
    c = torch.empty_like(d["a"]); ct.vec_add_kernel_1d(d["a"], d["b"], c, 1024); out["vadd"] = c; var["vadd"] = ct.last_variant()
    y = torch.empty_like(d["x"]); ct.softmax_tma_kernel(y, d["x"], 1024); out["softmax"] = y; var["softmax"] = ct.last_variant()
    C = torch.empty(512, 512, device="cuda"); ct.matmul_kernel(d["A"], d["B"], C, 64, 64, 64); out["matmul"] = C
    var["matmul"] = ct.last_variant()
    # a different expression per thread: the plans are compiled and looked up under the library's lock
    X = Tiled(d["x"])
    expr = [X * 2.0 + 1.0, T.sin(X) - X, X * X + 0.5, T.exp(X * 0.25)][seed % 4]
    e = torch.empty_like(d["x"]); Tiled(e).assign(expr); out["bcast"] = e; var["bcast"] = ct.last_variant()
    out["sum"] = T.sum(Tiled(d["x"]), dims=1); var["sum"] = ct.last_variant()
    out["fmha"] = fmha.cutile_fmha(d["Q"], d["K"], d["V"], causal=True); var["fmha"] = ct.last_variant()
    m = d["moe"]
    out["moe"] = moe.cutile_moe(m.hidden_states, m.w1, m.w2, m.topk_weights, m.topk_ids, 32, 128, 128)
    var["moe"] = ct.last_variant()
    return out, var


def test_threads_on_their_own_streams_reproduce_the_serial_results(ct):
    data = [_inputs(s) for s in range(NTHREADS)]
    alone = []
    for s in range(NTHREADS):
        out, var = _mix(ct, data[s], s)
        alone.append(({k: v.clone() for k, v in out.items()}, var))
    torch.cuda.synchronize()
    assert alone[0][1]["matmul"].startswith("gemm16_big_128x128x32_ring4_splitk"), alone[0][1]["matmul"]
    assert alone[0][1]["vadd"].startswith("vadd") and alone[0][1]["fmha"].startswith("fmha")
    for s in range(NTHREADS):   # sanity of the serial results themselves, against torch
        assert torch.equal(alone[s][0]["vadd"], data[s]["a"] + data[s]["b"])
        ref = data[s]["B"].float() @ data[s]["A"].float()      # torch holds the transposes: (A * B)' = B' * A'
        assert torch.allclose(alone[s][0]["matmul"], ref, rtol=1e-3, atol=1e-3)

    failures, barrier = [], threading.Barrier(NTHREADS)

    def worker(s):
        try:
            stream = torch.cuda.Stream()
            barrier.wait(timeout=60)
            with torch.cuda.stream(stream):
                for rep in range(REPEATS):
                    out, var = _mix(ct, data[s], s)
                    stream.synchronize()
                    for k, v in out.items():
                        if not torch.equal(v, alone[s][0][k]):
                            bad = int((v != alone[s][0][k]).sum())
                            failures.append(f"thread {s} repeat {rep}: {k} differs from the serial result in {bad} elements")
                    if var != alone[s][1]:
                        failures.append(f"thread {s} repeat {rep}: variants {var} != {alone[s][1]}")
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            failures.append(f"thread {s}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(NTHREADS)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=150)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    torch.cuda.synchronize()
    assert not failures, "\n".join(failures[:10])
