"""Mirror of examples/moe.jl:186-383 (invoke_* helpers, cutile_moe, prepare / run / metric)."""
from __future__ import annotations

import numpy as np
import torch

import cutile_jl_amd as ct
from ._harness import isapprox, namespace, rand_normal, time_launches


def invoke_fused_moe_kernel(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids, *, mul_routed_weight,
                            num_token_replicas, tile_m, tile_n, tile_k, b_scale=None, fuse_silu=False):
    """moe.jl:186-199.  ``topk_weights`` Julia (num_tokens, topk) = torch (topk, num_tokens); the reference
    flattens it slot-fastest (moe.jl:193).  ``C`` Julia (dim, topk, num_tokens) is flattened to
    (dim, total_tokens) (moe.jl:196)."""
    C_flat = C.reshape(C.shape[0] * C.shape[1], C.shape[2]) if C.dim() == 3 else C
    launch = ct.fused_moe_silu_kernel if fuse_silu else ct.fused_moe_kernel
    # (the library takes the (num_tokens, topk) matrix as it is and looks (token, slot) up in the kernel, which
    # saves the permuting copy of moe.jl:193 in front of either GEMM; a flattened vector is accepted as well)
    launch(A, B, C_flat, topk_weights, sorted_token_ids, sorted_expert_ids, num_token_replicas,
           mul_routed_weight, tile_m, tile_n, tile_k, b_scale=b_scale)


def invoke_silu_and_mul_kernel(AB, C):
    """moe.jl:202-215: AB Julia (2*inter, total) = torch (total, 2*inter); halves along dim 1."""
    inter = C.shape[1]
    A_half = AB[:, :inter]
    B_half = AB[:, inter:2 * inter]
    tile_n = 1 << (inter - 1).bit_length()
    ct.silu_and_mul_kernel(A_half, B_half, C, tile_n)


def quantize_activations(x):
    """Per-tensor E4M3FN form of an activation matrix, entirely on the device: codes = round-to-nearest-even of
    x / scale with scale = max |x| / 448 (1 for an all-zero tensor); returns (codes, scale as a 1-element fp32
    tensor).  Two launches of the library (``mi_quantize_e4m3fn``)."""
    return ct.quantize_e4m3fn(x)


def cutile_moe(hidden_states, w1, w2, topk_weights, topk_ids, tile_m, tile_n, tile_k, *, w1_scale=None,
               w2_scale=None, aligned=None, device_align=True, fuse_silu=True, fuse_sum=None, fp8_activations=False):
    """moe.jl:218-257.  Torch shapes (reversed Julia): hidden_states (tokens, hidden); w1
    (E, 2*inter, hidden); w2 (E, hidden, inter); topk_weights / topk_ids (topk, tokens), ids
    1-based int64.  ``aligned`` may carry a precomputed (sorted_token_ids, sorted_expert_ids)
    pair on the device to skip the token sort; ``device_align`` (default) sorts on the GPU
    (fixed-capacity outputs, nothing leaves the device), ``device_align=False`` is the reference's
    orchestration with the host round trip of moe.jl:232-233.  ``fuse_silu`` (default) runs the gate / up
    GEMM with SiLU * up as its epilogue: cache1 and the silu_and_mul launch disappear;
    ``fuse_silu=False`` launches the kernels one by one as moe.jl:234-251 does.  ``fuse_sum`` (default: whenever
    it applies -- one or two slots per token, device-side sort, an even hidden size of whole 16-byte rows) lets the
    down projection add every replica's row into the output itself, which the sort launch has zeroed: cache3 and
    the top-k sum launch disappear.  All combinations give bit-identical results.

    ``fp8_activations`` (with E4M3FN weights and their scales; an extension like the fp8 weights themselves): both
    grouped GEMMs multiply fp8 by fp8 on the matrix cores, the operand pairing that ext/DLFP8TypesExt.jl:15-19 gives
    ``mma``.  The activations of either GEMM are quantised per tensor on the device (``quantize_activations``) and
    their scale is folded into the weights' per-channel scales by the same launches; needs blocks of 128 slots, the fused SiLU epilogue and
    hidden / intermediate sizes that are multiples of 16 from 512 up."""
    num_tokens, hidden_size = hidden_states.shape
    num_experts, _, intermediate_size = w2.shape
    topk = topk_ids.shape[0]
    total_tokens = num_tokens * topk
    T, dev = hidden_states.dtype, hidden_states.device
    if fp8_activations:
        if w1_scale is None or w2_scale is None or not fuse_silu:
            raise ValueError("fp8 activations need e4m3 weights with their scales and the fused SiLU epilogue")
        hidden_states, _, w1_scale = ct.quantize_e4m3fn(hidden_states, fold=w1_scale)
    can_fuse_sum = (topk <= 2 and aligned is None and device_align and hidden_size % 8 == 0 and topk_weights.dtype == T)
    if fuse_sum is None:
        fuse_sum = can_fuse_sum
    elif fuse_sum and not can_fuse_sum:
        raise ValueError("fuse_sum needs top-k <= 2, the device-side sort and a hidden size that is a multiple of 8")
    # The three caches of moe.jl:228-230, carved out of one allocation.  The reference zero-fills them; here they
    # are left as allocated: every column of every cache belongs to one (token, slot) replica, the GEMMs write the
    # columns of all replicas (only padding slots write nothing, and nothing reads those), so no fill is ever
    # read.  The one exception is a replica whose expert id lies outside 1..num_experts (the reference raises on
    # those, moe_align_tile_size indexes by them, moe.jl:150-160; the device-side sort drops them): nothing writes
    # its column of cache3, which the top-k sum reads.  cache3 is therefore zeroed -- by the sort launch itself where
    # the sort runs on the GPU, by a fill otherwise -- so that such a replica contributes 0 on every path.
    n1 = 0 if fuse_silu else total_tokens * intermediate_size * 2
    n2, n3 = total_tokens * intermediate_size, 0 if fuse_sum else total_tokens * hidden_size
    caches = torch.empty(n1 + n2 + n3, dtype=T, device=dev)
    cache1 = None if fuse_silu else caches[:n1].view(num_tokens, topk, intermediate_size * 2)
    cache2 = caches[n1:n1 + n2].view(total_tokens, intermediate_size)
    cache3 = None if fuse_sum else caches[n1 + n2:].view(num_tokens, topk, hidden_size)
    out = torch.empty((num_tokens, hidden_size), dtype=T, device=dev)
    if fuse_sum:
        sorted_token_ids, sorted_expert_ids = ct.moe_align_tile_size_device(topk_ids, tile_m, num_experts, clear=out)
    elif aligned is None and device_align:
        clear = cache3 if (cache3.numel() * cache3.element_size()) % 16 == 0 and cache3.data_ptr() % 16 == 0 else None
        if clear is None:
            cache3.zero_()
        sorted_token_ids, sorted_expert_ids = ct.moe_align_tile_size_device(topk_ids, tile_m, num_experts, clear=clear)
    elif aligned is None:
        cache3.zero_()
        tok, exp = ct.moe_align_tile_size(topk_ids.cpu(), tile_m, num_experts)
        sorted_token_ids, sorted_expert_ids = tok.to(dev), exp.to(dev)
    else:
        cache3.zero_()
        sorted_token_ids, sorted_expert_ids = aligned
    if fuse_silu:
        invoke_fused_moe_kernel(hidden_states, w1, cache2, topk_weights, sorted_token_ids, sorted_expert_ids,
                                mul_routed_weight=False, num_token_replicas=topk, tile_m=tile_m, tile_n=tile_n,
                                tile_k=tile_k, b_scale=w1_scale, fuse_silu=True)
    else:
        invoke_fused_moe_kernel(hidden_states, w1, cache1, topk_weights, sorted_token_ids, sorted_expert_ids,
                                mul_routed_weight=False, num_token_replicas=topk, tile_m=tile_m, tile_n=tile_n,
                                tile_k=tile_k, b_scale=w1_scale)
        cache1_flat = cache1.reshape(total_tokens, intermediate_size * 2)
        invoke_silu_and_mul_kernel(cache1_flat, cache2)
    if fp8_activations:
        cache2, _, w2_scale = ct.quantize_e4m3fn(cache2, fold=w2_scale)
    if fuse_sum:
        ct.fused_moe_accumulate_kernel(cache2, w2, out, topk_weights, sorted_token_ids, sorted_expert_ids, tile_m, tile_n,
                                       tile_k, b_scale=w2_scale)
        return out
    invoke_fused_moe_kernel(cache2, w2, cache3, topk_weights, sorted_token_ids, sorted_expert_ids,
                            mul_routed_weight=True, num_token_replicas=1, tile_m=tile_m, tile_n=tile_n,
                            tile_k=tile_k, b_scale=w2_scale)
    ct.moe_sum_topk(cache3, out)  # sum(cache3; dims=2), moe.jl:256
    return out


def prepare(*, benchmark: bool = False, num_tokens: int | None = None, hidden_size: int | None = None,
            num_experts: int | None = None, intermediate_size: int | None = None, topk: int = 8,
            T: torch.dtype = torch.float16, seed: int = 6, router: str = "randperm", weight_std: float = 0.02):
    """moe.jl:311-344.  ``router='randperm'``: the reference's unique random experts with softmax
    of U(0,1) weights; ``'top2_logits'``: the measured configuration (logits ~ N(0,1), top-k,
    softmax over the selected logits).  Activations ~ N(0,1), weights ~ N(0, weight_std)."""
    num_tokens = (256 if benchmark else 48) if num_tokens is None else num_tokens
    hidden_size = (1024 if benchmark else 512) if hidden_size is None else hidden_size
    num_experts = (32 if benchmark else 64) if num_experts is None else num_experts
    intermediate_size = (2048 if benchmark else 1024) if intermediate_size is None else intermediate_size
    rng = np.random.default_rng(seed)
    hidden_states = rand_normal(rng, (hidden_size, num_tokens), T)
    w1 = rand_normal(rng, (hidden_size, intermediate_size * 2, num_experts), T, std=weight_std)
    w2 = rand_normal(rng, (intermediate_size, hidden_size, num_experts), T, std=weight_std)
    logits = None
    if router == "top2_logits":
        logits = rng.standard_normal((num_tokens, num_experts)).astype(np.float32)
        order = np.argsort(-logits, axis=1, kind="stable")[:, :topk]
        sel = np.take_along_axis(logits, order, axis=1).astype(np.float64)
        e = np.exp(sel - sel.max(axis=1, keepdims=True))
        weights = (e / e.sum(axis=1, keepdims=True)).astype(np.float32)
        ids = (order + 1).astype(np.int64)
    else:
        ids = np.stack([rng.permutation(num_experts)[:topk] + 1 for _ in range(num_tokens)]).astype(np.int64)
        raw = np.exp(rng.random((num_tokens, topk), dtype=np.float32))
        weights = raw / raw.sum(axis=1, keepdims=True)
    dev = hidden_states.device
    topk_weights = torch.from_numpy(np.ascontiguousarray(weights.T)).to(T).to(dev)  # Julia (tokens, topk)
    topk_ids = torch.from_numpy(np.ascontiguousarray(ids.T)).to(dev)
    logits = None if logits is None else torch.from_numpy(logits).to(dev)   # (tokens, experts), for the device router
    return namespace(hidden_states=hidden_states, w1=w1, w2=w2, topk_weights=topk_weights, topk_ids=topk_ids, logits=logits,
                     num_tokens=num_tokens, hidden_size=hidden_size, num_experts=num_experts,
                     intermediate_size=intermediate_size, topk=topk, tile_m=128, tile_n=128, tile_k=64)


def quantize_weights(data):
    """Input preparation of the e4m3 configuration: per-(output channel, expert) fp32 scale
    = max |w| over K / 448 (1 for an all-zero channel), codes = round-to-nearest-even E4M3FN of
    w / scale.  Torch shapes: w (E, N, K) -> codes (E, N, K) float8_e4m3fn, scale (E, N) float32."""
    def q(w):
        w32 = w.float()
        amax = w32.abs().amax(dim=2)
        scale = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
        return (w32 / scale[:, :, None]).to(torch.float8_e4m3fn), scale.contiguous()
    w1, s1 = q(data.w1)
    w2, s2 = q(data.w2)
    return namespace(w1=w1, w2=w2, w1_scale=s1, w2_scale=s2)


def run(data, *, nruns: int = 1, warmup: int = 0, **kw):
    """moe.jl:347-367: the timed region is the whole cutile_moe call."""
    d = data
    holder = {}

    def call():
        holder["out"] = cutile_moe(d.hidden_states, d.w1, d.w2, d.topk_weights, d.topk_ids, d.tile_m, d.tile_n,
                                   d.tile_k, **kw)

    times = time_launches(call, nruns, warmup)
    return namespace(out=holder["out"], times=times)



def ref_moe(hidden_states, w1, w2, topk_weights, topk_ids) -> torch.Tensor:
    """moe.jl:264-304 on the host in fp32, expert by expert.  Torch shapes (reversed Julia): hidden_states
    (tokens, hidden); w1 (E, 2*inter, hidden); w2 (E, hidden, inter); topk_weights / topk_ids (topk, tokens),
    ids 1-based.  Returns (tokens, hidden)."""
    hs, w1f, w2f = hidden_states.cpu().float(), w1.cpu().float(), w2.cpu().float()
    tw, ti = topk_weights.cpu().float(), topk_ids.cpu()
    inter = w2f.shape[2]
    result = torch.zeros_like(hs)
    for e in range(w1f.shape[0]):
        slot, tok = torch.nonzero(ti == e + 1, as_tuple=True)
        if tok.numel() == 0:
            continue
        x = hs[tok]                                            # (count, hidden)
        gate = x @ w1f[e, :inter].t()                          # (count, inter)
        up = x @ w1f[e, inter:].t()
        act = gate / (1.0 + torch.exp(-gate)) * up
        y = act @ w2f[e].t()                                   # (count, hidden)
        result.index_add_(0, tok, y * tw[slot, tok].unsqueeze(1))
    return result


def verify(data, result) -> None:
    """moe.jl:370-374: ``isapprox(Float32.(out), ref_moe(...); rtol = 1e-2, atol = 1e-2)``."""
    expected = ref_moe(data.hidden_states, data.w1, data.w2, data.topk_weights, data.topk_ids)
    actual = result.out.cpu().float()
    assert isapprox(actual, expected, rtol=1e-2, atol=1e-2), f"MoE incorrect! max diff: {float((actual - expected).abs().max())}"


def metric(data):
    """moe.jl:377-383."""
    return 2 * data.num_tokens * data.topk * data.hidden_size * data.intermediate_size * 3, "TFLOPS"


def smoke(orc):
    d = prepare(num_tokens=24, hidden_size=256, num_experts=8, intermediate_size=256, topk=2, router="top2_logits")
    r = run(d)
    J = orc.to_julia
    ref = orc.ref_moe(J(d.hidden_states), J(d.w1), J(d.w2), J(d.topk_weights), J(d.topk_ids))
    got = J(r.out).astype(np.float32)
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max(), np.abs(got - ref).max()


def test_moe(num_tokens: int, hidden_size: int, num_experts: int, intermediate_size: int, topk: int, *,
             T: torch.dtype = torch.float16, name: str | None = None) -> None:
    """moe.jl:390-399 (the tile constants are those of ``prepare``)."""
    name = name or (f"moe tokens={num_tokens}, hidden={hidden_size}, experts={num_experts}, inter={intermediate_size}, "
                    f"topk={topk}, {str(T).replace('torch.', '')}")
    print(f"--- {name} ---")
    data = prepare(num_tokens=num_tokens, hidden_size=hidden_size, num_experts=num_experts,
                   intermediate_size=intermediate_size, topk=topk, T=T)
    result = run(data)
    verify(data, result)
    print("  passed")


def main() -> None:
    """moe.jl:402-411."""
    print("--- Mixture of Experts Examples ---\n")
    test_moe(48, 512, 64, 1024, 8)
    test_moe(128, 512, 32, 1024, 4)
    test_moe(64, 1024, 64, 2048, 8)
    print("\n--- All MoE examples completed ---")
