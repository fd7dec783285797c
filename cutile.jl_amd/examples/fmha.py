"""Mirror of examples/fmha.jl:146-293 (cutile_fmha / prepare / run / metric)."""
from __future__ import annotations

import math

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_normal, rand_uniform, time_launches


def cutile_fmha(Q, K, V, *, qk_scale: float | None = None, input_pos: int = 0, tile_m: int = 128,
                tile_n: int = 128, query_group_size: int = 1, causal: bool = False, out=None):
    """fmha.jl:146-168.  Q Julia (D_k, SeqLen_Q, Heads, Batch) = torch (Batch, Heads, SeqLen_Q, D_k);
    allocates and returns Out like the reference (pass ``out`` to reuse a buffer)."""
    Batch, Heads, SeqLen_Q, D_k = Q.shape
    _, KV_Heads, SeqLen_KV, D_v = V.shape
    even_k = (SeqLen_KV % tile_n) == 0
    if qk_scale is None:
        qk_scale = float(np.float32(1.0 / math.sqrt(D_k)))
    Out = torch.empty((Batch, Heads, SeqLen_Q, D_v), dtype=Q.dtype, device=Q.device) if out is None else out
    ct.fmha_kernel(Q, K, V, Out, qk_scale, input_pos, D_k, Heads, tile_m, tile_n, query_group_size,
                   causal, even_k)
    return Out


def prepare(*, benchmark: bool = False, batch: int | None = None, heads: int | None = None,
            seq_q: int | None = None, seq_kv: int | None = None, d_k: int = 64, d_v: int = 64,
            query_group_size: int = 1, causal: bool = True, tile_m: int = 128, tile_n: int = 128,
            T: torch.dtype = torch.float16, seed: int = 5, dist: str = "normal"):
    """fmha.jl:227-255.  ``dist='normal'``: N(0,1) (measured configuration); ``'uniform'``:
    the reference's U(-0.5, 0.5)."""
    batch = (8 if benchmark else 2) if batch is None else batch
    heads = (16 if benchmark else 8) if heads is None else heads
    seq_q = (1024 if benchmark else 128) if seq_q is None else seq_q
    seq_kv = (1024 if benchmark else 128) if seq_kv is None else seq_kv
    kv_heads = heads // query_group_size
    rng = np.random.default_rng(seed)
    gen = (lambda shp: rand_normal(rng, shp, T)) if dist == "normal" else (lambda shp: rand_uniform(rng, shp, T, -0.5, 0.5))
    Q = gen((d_k, seq_q, heads, batch)); K = gen((d_k, seq_kv, kv_heads, batch)); V = gen((d_v, seq_kv, kv_heads, batch))
    return namespace(Q=Q, K=K, V=V, batch=batch, heads=heads, seq_q=seq_q, seq_kv=seq_kv, d_k=d_k, d_v=d_v,
                     query_group_size=query_group_size, causal=causal, tile_m=tile_m, tile_n=tile_n)


def run(data, *, nruns: int = 1, warmup: int = 0):
    """fmha.jl:258-274: the timed region includes allocating Out."""
    d = data
    holder = {}

    def call():
        holder["out"] = cutile_fmha(d.Q, d.K, d.V, tile_m=d.tile_m, tile_n=d.tile_n,
                                    query_group_size=d.query_group_size, causal=d.causal)

    times = time_launches(call, nruns, warmup)
    return namespace(out=holder["out"], times=times)



def ref_fmha(Q, K, V, *, qk_scale: float | None = None, causal: bool = False) -> torch.Tensor:
    """fmha.jl:175-220 on the host in fp32.  Torch shapes (reversed Julia): Q (B, H, M, D), K / V (B, KVH, N, D);
    returns (B, H, M, D_v).  Masked scores are -inf; a row maximum of -inf is replaced by 0."""
    Qf, Kf, Vf = Q.cpu().float(), K.cpu().float(), V.cpu().float()
    B, H, M, D = Qf.shape
    KH, N = Kf.shape[1], Kf.shape[2]
    if qk_scale is None:
        qk_scale = float(np.float32(1.0 / np.sqrt(D)))
    group = H // KH
    out = torch.empty((B, H, M, Vf.shape[3]), dtype=torch.float32)
    mask = torch.triu(torch.ones(M, N, dtype=torch.bool), diagonal=1) if causal else None
    for h in range(H):
        kh = h // group
        scores = torch.matmul(Qf[:, h], Kf[:, kh].transpose(1, 2)) * qk_scale        # (B, M, N)
        if causal:
            scores = scores.masked_fill(mask, float("-inf"))
        smax = scores.amax(dim=2, keepdim=True)
        smax = torch.where(torch.isinf(smax), torch.zeros_like(smax), smax)
        e = torch.exp(scores - smax)
        out[:, h] = torch.matmul(e / e.sum(dim=2, keepdim=True), Vf[:, kh])
    return out


def verify(data, result) -> None:
    """fmha.jl:277-282: ``isapprox(Float32.(out), ref_fmha(...); rtol = 1e-2, atol = 1e-3)``."""
    expected = ref_fmha(data.Q, data.K, data.V, causal=data.causal)
    actual = result.out.cpu().float()
    assert isapprox(actual, expected, rtol=1e-2, atol=1e-3), f"FMHA incorrect! max diff: {float((actual - expected).abs().max())}"


def metric(data):
    """fmha.jl:285-293: the dense count 4*B*H*M*N*D (also for causal runs)."""
    return 4 * data.batch * data.heads * data.seq_q * data.seq_kv * data.d_k, "TFLOPS"


def causal_flops(data):
    """Multiply-adds actually required under the causal mask (Sq == Skv): 4*B*H*D*S*(S+1)/2."""
    S = data.seq_q
    return 4 * data.batch * data.heads * data.d_k * S * (S + 1) // 2


def smoke(orc):
    d = prepare(batch=1, heads=2, seq_q=192, seq_kv=192)
    r = run(d)
    ref = orc.ref_fmha(orc.to_julia(d.Q), orc.to_julia(d.K), orc.to_julia(d.V), causal=True)
    got = orc.to_julia(r.out).astype(np.float32)
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max(), np.abs(got - ref).max()


def test_fmha(batch: int, heads: int, seq_q: int, seq_kv: int, d_k: int, d_v: int, *, causal: bool = False,
              tile_m: int = 128, tile_n: int = 128, query_group_size: int = 1, T: torch.dtype = torch.float16,
              name: str | None = None) -> None:
    """fmha.jl:300-311."""
    name = name or f"fmha B={batch} H={heads} M={seq_q} N={seq_kv} D={d_k} causal={causal} {str(T).replace('torch.', '')}"
    print(f"--- {name} ---")
    data = prepare(batch=batch, heads=heads, seq_q=seq_q, seq_kv=seq_kv, d_k=d_k, d_v=d_v,
                   query_group_size=query_group_size, causal=causal, tile_m=tile_m, tile_n=tile_n, T=T)
    result = run(data)
    verify(data, result)
    print("  passed")


def main() -> None:
    """fmha.jl:314-325."""
    print("--- FMHA Examples ---\n")
    test_fmha(2, 8, 128, 128, 64, 64, causal=False)
    test_fmha(2, 8, 128, 128, 64, 64, causal=True)
    test_fmha(4, 16, 256, 256, 64, 64, causal=True)
    print("\n--- All FMHA examples completed ---")
