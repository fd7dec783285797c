"""CPU oracle for the cuTile.jl example kernels.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the CPU checking code of the reference's examples (their
``verify`` / ``ref_*`` functions and integer host helpers).  Only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import it; the
product (``cutile.jl_amd``) never does.

Arrays are numpy arrays in the JULIA shape (first dimension fastest in the reference); use
:func:`to_julia` / :func:`from_julia` to convert from / to the reversed-shape row-major
torch tensors the product works on.

Every function cites the reference lines it follows.  What pins each function (so that a
plausible mistake fails a test) is listed in ``tests/test_oracle.py``; summary:

=====================  ======================================================================
function               pinned by
=====================  ======================================================================
vadd, transpose        closed form (IEEE add / permutation); brute force
vadd_gather            out-of-bounds known answer of test/device/gather_scatter.jl:75-113; scalar loops
swizzle_2d             bijection onto the tile grid, brute force; C restatement cross-check
matmul, batch_matmul   float64 ``@``; 64x16x64 case of test/device/tile.jl:1036-1066 by loops
layer_norm_*           invariants (zero-mean/unit-var xhat, sum dx = 0, constant row);
                       ``torch.nn.functional.layer_norm`` + autograd on CPU
softmax                columns sum to 1, shift invariance, ``scipy.special.softmax``
ref_fmha               row 1 of causal output == V[:,1]; brute-force loops on tiny shapes;
                       ``torch.nn.functional.scaled_dot_product_attention`` on CPU
moe_align_tile_size    permutation / grouping / padding invariants; brute force; C cross-check
ref_moe                per-token dense loop on tiny shapes
route_top2             hand-computed answers (distinct logits, an exact tie -> lower id, weights 1/2)
fft_3stage, tables     ``numpy.fft.fft`` (independent library); brute-force DFT sum on tiny sizes
tiled_eval/broadcast   known answers of test/host/broadcast.jl (fills, 0-dim, expansion cases);
                       plain numpy expressions written out by hand; torch CPU for bfloat16
tiled_mapreduce        known answers of test/host/mapreduce.jl (count == 4, any / all, max of
                       fill(-5) == -5); numpy reductions; brute-force loops on tiny arrays
jl_promote             Julia's documented promotion facts (Int32+Int64 -> Int64, Int64+Float32 ->
                       Float32, Float16+Float32 -> Float32, Bool yields, true + true == 2)
philox2x32, rng_fill   Random123's published known-answer vectors for philox2x32 (7 and 10 rounds);
                       slot layout by brute-force loops, for rand! and for randn! / randexp! (which word
                       feeds the radius and which the angle, sine / cosine slots, the Float64 counter
                       pairing); the reference's own properties (test/device/random.jl:421-526:
                       uniqueness, disjoint streams, counter carry)
e4m3fn codec           16 round-trip vectors and fma vectors of
                       test/extensions/DLFP8Types.jl:126-141; all 256 codes vs torch.float8_e4m3fn
e5m2 codec             the same 16 round-trip vectors (DLFP8Types.jl:126-134); all 256 codes and
                       RNE encoding vs torch.float8_e5m2
fp8_matmul             the exact mma case of test/extensions/DLFP8Types.jl:143-152 (operands in
                       {0, 0.5, 1}: integer arithmetic by hand); float64 ``@`` on decoded operands
=====================  ======================================================================

The reference's device rounding (fma contraction, exp2 / reciprocal approximations, f16
rounding of P, atomics order) is produced by NVIDIA's closed ``tileiras`` compiler and is
"parity unpinned" at the bit level; the reference itself only checks it to rtol 1e-2
against the same CPU formulas restated here.  The same holds for the transcendental functions of
the Tiled vocabulary and for randn / randexp (device math library against numpy, a few ulp).
"""
from __future__ import annotations

import math

import numpy as np


# ---- layout helpers ----------------------------------------------------------------------

def to_julia(t) -> np.ndarray:
    """torch tensor (reversed-shape, row-major) -> numpy array in the Julia shape."""
    import torch
    if t.dtype == torch.bfloat16:
        return t.detach().cpu().to(torch.float32).numpy().T
    return t.detach().cpu().numpy().T


def from_julia(a: np.ndarray):
    """numpy array in the Julia shape -> contiguous torch tensor of the reversed shape."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a.T))


def cld(a: int, b: int) -> int:
    return -(-a // b)


# ---- vadd / transpose ----------------------------------------------------------------------

def vadd(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """examples/vadd.jl:127-129: ``Array(a) + Array(b)`` in the arrays' own type (IEEE add;
    Julia's Float16 add widens to Float32 and rounds once, as numpy's float16 add does)."""
    return a + b


def vadd_gather(a: np.ndarray, b: np.ndarray, n_c: int) -> np.ndarray:
    """vec_add_kernel_1d_gather (vadd.jl:31-45) with possibly different lengths: an index
    past the end of ``a`` or ``b`` gathers 0 (src/language/operations.jl:996-1009)."""
    out = np.zeros(n_c, dtype=a.dtype)
    na, nb = min(n_c, a.shape[0]), min(n_c, b.shape[0])
    out[:na] += a[:na]
    out[:nb] += b[:nb]
    return out


def transpose(x: np.ndarray) -> np.ndarray:
    """examples/transpose.jl:58-60: ``transpose(Array(x))``."""
    return np.ascontiguousarray(x.T)


# ---- swizzle -------------------------------------------------------------------------------

def swizzle_2d(M, N, tm, tn, GROUP_SIZE_M, bid):
    """examples/matmul.jl:13-24 (dup. examples/moe.jl:20-31): 1-based bid -> 1-based
    (bid_m, bid_n), grouped ordering."""
    num_bid_m = cld(M, tm)
    num_bid_n = cld(N, tn)
    num_bid_in_group = GROUP_SIZE_M * num_bid_n
    bid0 = bid - 1
    group_id = bid0 // num_bid_in_group
    first_bid_m = group_id * GROUP_SIZE_M
    group_size_m = min(num_bid_m - first_bid_m, GROUP_SIZE_M)
    bid_m = first_bid_m + bid0 % group_size_m + 1
    bid_n = (bid0 % num_bid_in_group) // group_size_m + 1
    return bid_m, bid_n


# ---- matmul --------------------------------------------------------------------------------

def matmul(A: np.ndarray, B: np.ndarray, dtype=np.float64) -> np.ndarray:
    """examples/matmul.jl:98-101: ``Array(A) * Array(B)``; evaluated in ``dtype``
    (float64 = the fp32-reference the tolerances are stated against)."""
    return A.astype(dtype) @ B.astype(dtype)


def batch_matmul(A: np.ndarray, B: np.ndarray, dtype=np.float64) -> np.ndarray:
    """examples/batchmatmul.jl:97-106: per batch ``A[:,:,b] * B[:,:,b]`` (batch is LAST)."""
    M, K, nb = A.shape
    N = B.shape[1]
    out = np.empty((M, N, nb), dtype=dtype, order="F")
    for b in range(nb):
        out[:, :, b] = A[:, :, b].astype(dtype) @ B[:, :, b].astype(dtype)
    return out


# ---- layernorm -----------------------------------------------------------------------------

def layer_norm_fwd(X, W, B, eps, dtype=np.float64):
    """examples/layernorm.jl:284-302.  X is (N, M): reduce along dim 1 (axis 0).  Returns
    (Y, mean (M,), rstd (M,))."""
    X = X.astype(dtype); W = W.astype(dtype); B = B.astype(dtype)
    N = X.shape[0]
    mean = X.sum(axis=0, keepdims=True) / N
    var = ((X - mean) ** 2).sum(axis=0, keepdims=True) / N
    rstd = 1.0 / np.sqrt(var + dtype(eps))
    xhat = (X - mean) * rstd
    Y = xhat * W[:, None] + B[:, None]
    return Y, mean[0], rstd[0]


def layer_norm_bwd(X, W, DY, eps, dtype=np.float64):
    """examples/layernorm.jl:303-313.  Returns (DX (N,M), DW (N,), DB (N,))."""
    X = X.astype(dtype); W = W.astype(dtype); DY = DY.astype(dtype)
    N = X.shape[0]
    mean = X.sum(axis=0, keepdims=True) / N
    var = ((X - mean) ** 2).sum(axis=0, keepdims=True) / N
    rstd = 1.0 / np.sqrt(var + dtype(eps))
    xhat = (X - mean) * rstd
    wdy = W[:, None] * DY
    c1 = (xhat * wdy).sum(axis=0, keepdims=True) / N
    c2 = wdy.sum(axis=0, keepdims=True) / N
    DX = (wdy - (xhat * c1 + c2)) * rstd
    DW = (DY * xhat).sum(axis=1)
    DB = DY.sum(axis=1)
    return DX, DW, DB


# ---- softmax -------------------------------------------------------------------------------

def softmax(x: np.ndarray, dtype=np.float64, rows: int | None = None) -> np.ndarray:
    """examples/softmax.jl:175-188: per column j, ``exp.(col .- max) ./ sum``.  x is (N, M).
    ``rows`` limits the softmax to the first ``rows`` rows (a TILE_SIZE smaller than N:
    the tile at index 1 covers rows 1..TILE_SIZE only, softmax.jl:29-38)."""
    x = x.astype(dtype)
    if rows is not None:
        x = x[:rows]
    mx = x.max(axis=0, keepdims=True)
    e = np.exp(x - mx)
    return e / e.sum(axis=0, keepdims=True)


# ---- FMHA ----------------------------------------------------------------------------------

def ref_fmha(Q, K, V, qk_scale=None, causal=False, dtype=np.float32):
    """examples/fmha.jl:175-220.  Q (D,M,H,B), K (D,N,KH,B), V (Dv,N,KH,B) -> Out (Dv,M,H,B).
    Causal mask: key j (1-based) > query i is -Inf (no input_pos offset in the reference)."""
    Q = Q.astype(dtype); K = K.astype(dtype); V = V.astype(dtype)
    D, M, H, B = Q.shape
    _, N, KH, _ = K.shape
    Dv = V.shape[0]
    if qk_scale is None:
        qk_scale = dtype(1.0 / math.sqrt(D))
    out = np.zeros((Dv, M, H, B), dtype=dtype, order="F")
    group = H // KH
    for b in range(B):
        for h in range(H):
            kh = h // group  # 0-based form of cld(h, H ÷ KH) for 1-based h
            q = Q[:, :, h, b]; k = K[:, :, kh, b]; v = V[:, :, kh, b]
            scores = (q.T @ k) * dtype(qk_scale)  # (M, N)
            if causal:
                i = np.arange(M)[:, None]; j = np.arange(N)[None, :]
                scores = np.where(j > i, -np.inf, scores)
            smax = scores.max(axis=1, keepdims=True)
            smax = np.where(np.isinf(smax), 0.0, smax)
            e = np.exp(scores - smax)
            attn = e / e.sum(axis=1, keepdims=True)
            out[:, :, h, b] = v @ attn.T
    return out


def fmha_general(Q, K, V, qk_scale=None, causal=False, input_pos=0, dtype=np.float64):
    """The kernel's own masking rule (fmha.jl:45-46,92-103): query row i (0-based) sits at
    position ``input_pos + i`` and sees keys ``j <= input_pos + i``.  Equals ref_fmha when
    input_pos == 0.  Used for the decode-offset cases the reference's ref_fmha cannot
    express; pinned against ref_fmha at input_pos == 0 and by the all-keys-visible limit."""
    Q = Q.astype(dtype); K = K.astype(dtype); V = V.astype(dtype)
    D, M, H, B = Q.shape
    _, N, KH, _ = K.shape
    if qk_scale is None:
        qk_scale = 1.0 / math.sqrt(D)
    out = np.zeros((V.shape[0], M, H, B), dtype=dtype, order="F")
    group = H // KH
    for b in range(B):
        for h in range(H):
            kh = h // group
            s = (Q[:, :, h, b].T @ K[:, :, kh, b]) * qk_scale
            if causal:
                i = np.arange(M)[:, None] + input_pos; j = np.arange(N)[None, :]
                s = np.where(j > i, -np.inf, s)
            mx = s.max(axis=1, keepdims=True)
            mx = np.where(np.isinf(mx), 0.0, mx)
            e = np.exp(s - mx)
            out[:, :, h, b] = V[:, :, kh, b] @ (e / e.sum(axis=1, keepdims=True)).T
    return out


# ---- MoE -----------------------------------------------------------------------------------

def moe_align_tile_size(topk_ids: np.ndarray, tile_m: int, num_experts: int):
    """examples/moe.jl:142-183.  topk_ids (num_tokens, topk) of 1-based expert ids.
    Returns (sorted_token_ids int32 1-based with sentinel total+1, sorted_expert_ids int32)."""
    num_tokens, topk = topk_ids.shape
    total = num_tokens * topk
    flat = topk_ids.reshape(-1)  # row-major of (tokens, topk) == slot fastest (moe.jl:148)
    perm = np.argsort(flat, kind="stable") + 1
    counts = np.bincount(flat - 1, minlength=num_experts)
    blocks = -(-counts // tile_m)
    total_blocks = int(blocks.sum())
    tok = np.full(total_blocks * tile_m, total + 1, dtype=np.int32)
    exp = np.zeros(total_blocks, dtype=np.int32)
    cur_block = 0
    cur_tok = 0
    for e in range(num_experts):
        tc, bc = int(counts[e]), int(blocks[e])
        exp[cur_block:cur_block + bc] = e + 1
        start = cur_block * tile_m
        tok[start:start + tc] = perm[cur_tok:cur_tok + tc]
        cur_tok += tc
        cur_block += bc
    return tok, exp


def silu_and_mul(a: np.ndarray, b: np.ndarray, dtype=np.float64) -> np.ndarray:
    """examples/moe.jl:110-128: ``a / (1 + exp(-a)) * b``."""
    a = a.astype(dtype); b = b.astype(dtype)
    return a / (1.0 + np.exp(-a)) * b


def ref_moe(hidden_states, w1, w2, topk_weights, topk_ids, dtype=np.float32, mid=None):
    """examples/moe.jl:264-304.  hidden_states (hidden, tokens); w1 (hidden, 2*inter, E);
    w2 (inter, hidden, E); topk_weights, topk_ids (tokens, topk), ids 1-based.
    ``mid``: what a build that quantises the activations between the two projections does to
    SiLU(gate) * up (a function of the (inter, tokens-of-one-expert) matrix; the reference has
    no such step and passes None)."""
    hs = hidden_states.astype(dtype); w1 = w1.astype(dtype); w2 = w2.astype(dtype)
    tw = topk_weights.astype(dtype)
    hidden, num_tokens = hs.shape
    inter = w2.shape[0]
    E = w1.shape[2]
    result = np.zeros((hidden, num_tokens), dtype=dtype, order="F")
    for eid in range(1, E + 1):
        tok_idx, slot_idx = np.nonzero(topk_ids == eid)
        if tok_idx.size == 0:
            continue
        tokens = hs[:, tok_idx]
        w1e = w1[:, :, eid - 1]
        gate_out = w1e[:, :inter].T @ tokens
        up_out = w1e[:, inter:].T @ tokens
        silu_out = gate_out / (1.0 + np.exp(-gate_out)) * up_out
        if mid is not None:
            silu_out = mid(silu_out).astype(dtype)
        expert_out = w2[:, :, eid - 1].T @ silu_out
        for i, (t, s) in enumerate(zip(tok_idx, slot_idx)):
            result[:, t] += expert_out[:, i] * tw[t, s]
    return result


def route_top2(logits: np.ndarray, topk: int = 2):
    """Router of the measured MoE configuration: top-k experts of each token's logits
    (ties to the lower expert id), softmax over the selected logits.  logits (tokens, E).
    Returns (topk_weights float32 (tokens, topk), topk_ids int64 1-based (tokens, topk))."""
    order = np.argsort(-logits, axis=1, kind="stable")[:, :topk]
    sel = np.take_along_axis(logits, order, axis=1).astype(np.float64)
    e = np.exp(sel - sel.max(axis=1, keepdims=True))
    return (e / e.sum(axis=1, keepdims=True)).astype(np.float32), (order + 1).astype(np.int64)


# ---- FP8 E4M3FN ----------------------------------------------------------------------------

def e4m3fn_decode(code: np.ndarray) -> np.ndarray:
    """OCP FP8 E4M3FN -> float32: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no Inf;
    S.1111.111 is NaN; exponent 0 is subnormal (2^-6 * m/8); max finite 448.  The type the
    reference maps ``Float8_E4M3FN`` to (ext/DLFP8TypesExt.jl:7-9)."""
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    s = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 0x7
    val = np.where(e == 0, (m / 8.0) * 2.0 ** -6, (1.0 + m / 8.0) * np.exp2((e - 7).astype(np.float64)))
    val = np.where((e == 15) & (m == 7), np.nan, val)
    return (s * val).astype(np.float32)


def e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """float -> E4M3FN code, round to nearest even (the reference's default conversion
    rounding, src/compiler/intrinsics/conversions.jl:197), saturating finite values above
    the largest representable magnitude to NaN as the FN format has no Inf."""
    x = np.asarray(x, dtype=np.float64)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    a = np.abs(x)
    out = np.zeros(x.shape, dtype=np.uint8)
    nan = np.isnan(a)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.clip(e, -6, 8)
    quantum = np.exp2(e - 3)  # spacing of representable values in this binade
    q = np.rint(a / quantum)  # rint = round half to even
    val = q * quantum
    # rounding may carry into the next binade; recompute fields from val
    with np.errstate(divide="ignore", invalid="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    e2 = np.clip(e2, -6, 8)
    is_sub = val < 2.0 ** -6
    mant = np.where(is_sub, np.rint(val / 2.0 ** -9), np.rint(val / np.exp2(e2 - 3)) - 8)
    expf = np.where(is_sub, 0, e2 + 7)
    code = (expf.astype(np.int64) << 3) | mant.astype(np.int64)
    overflow = val > 448.0
    code = np.where(overflow | nan, 0x7F, code)
    out = (code.astype(np.uint8) | sign).astype(np.uint8)
    return out


def e5m2_decode(code: np.ndarray) -> np.ndarray:
    """OCP FP8 E5M2 -> float32: 1 sign, 5 exponent (bias 15), 2 mantissa bits; IEEE-style Inf
    (S.11111.00) and NaN; exponent 0 is subnormal (2^-14 * m/4); max finite 57344.  The type the
    reference maps ``Float8_E5M2`` to (ext/DLFP8TypesExt.jl:11-13)."""
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    s = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 2) & 0x1F
    m = c & 0x3
    val = np.where(e == 0, (m / 4.0) * 2.0 ** -14, (1.0 + m / 4.0) * np.exp2((e - 15).astype(np.float64)))
    val = np.where(e == 31, np.where(m == 0, np.inf, np.nan), val)
    return (s * val).astype(np.float32)


def e5m2_encode(x: np.ndarray) -> np.ndarray:
    """float -> E5M2 code, round to nearest even (src/compiler/intrinsics/conversions.jl:197);
    values that round past the largest finite magnitude become Inf, as in IEEE formats."""
    x = np.asarray(x, dtype=np.float64)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    a = np.abs(x)
    nan = np.isnan(a)
    inf = np.isinf(a)
    fin = np.where(nan | inf, 0.0, a)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(fin > 0, fin, 1.0)))
    e = np.clip(e, -14, 15)
    quantum = np.exp2(e - 2)
    val = np.rint(fin / quantum) * quantum
    with np.errstate(divide="ignore", invalid="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    e2 = np.clip(e2, -14, 16)
    is_sub = val < 2.0 ** -14
    mant = np.where(is_sub, np.rint(val / 2.0 ** -16), np.rint(val / np.exp2(e2 - 2)) - 4)
    expf = np.where(is_sub, 0, e2 + 15)
    code = (expf.astype(np.int64) << 2) | mant.astype(np.int64)
    code = np.where(inf | (val > 57344.0), 0x7C, code)
    code = np.where(nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def fp8_matmul(A_codes: np.ndarray, B_codes: np.ndarray, fmt: str = "e4m3fn", dtype=np.float64) -> np.ndarray:
    """``mma`` of fp8 operands (ext/DLFP8TypesExt.jl:15-19 allows them; the product is defined on
    the decoded values, test/extensions/DLFP8Types.jl:143-152: ``Float32.(a) * Float32.(b)``).
    A_codes (M, K) and B_codes (K, N) uint8, Julia shapes; (M, N) float64 out."""
    dec = e4m3fn_decode if fmt == "e4m3fn" else e5m2_decode
    return dec(A_codes).astype(dtype) @ dec(B_codes).astype(dtype)


def quantize_e4m3fn_per_channel(w: np.ndarray):
    """Weight quantisation of the fp8 MoE configuration: w (K, N, E) -> codes (K, N, E) uint8
    and scale (N, E) float32 with scale = amax over K / 448 (1 where the channel is zero)."""
    amax = np.abs(w.astype(np.float32)).max(axis=0)
    scale = np.where(amax > 0, amax / np.float32(448.0), np.float32(1.0)).astype(np.float32)
    codes = e4m3fn_encode(w.astype(np.float32) / scale[None])
    return codes, scale


# ---- FFT -----------------------------------------------------------------------------------

def dft_matrix(size: int) -> np.ndarray:
    """examples/fft.jl:130-140: W[i, j] = exp(-2 pi i * i*j / size), stored (2, size, size) float32
    (Julia shape), real part first."""
    i, j = np.meshgrid(np.arange(size), np.arange(size), indexing="ij")
    W = np.exp(-2j * np.pi * i * j / size)
    return np.stack([W.real, W.imag]).astype(np.float32)


def make_twiddles(factors):
    """examples/fft.jl:143-180.  Returns (W0, W1, W2, T0, T1) in the Julia shapes
    (2,F0,F0), (2,F1,F1), (2,F2,F2), (2,F1F2,F0), (2,F2,F1), float32."""
    F0, F1, F2 = factors
    N, F1F2 = F0 * F1 * F2, F1 * F2
    j, i = np.meshgrid(np.arange(F1F2), np.arange(F0), indexing="ij")      # T0[:, j, i] = exp(-2 pi i * i*j / N)
    t0 = np.exp(-2j * np.pi * i * j / N)
    k, jj = np.meshgrid(np.arange(F2), np.arange(F1), indexing="ij")       # T1[:, k, j] = exp(-2 pi i * j*k / F1F2)
    t1 = np.exp(-2j * np.pi * jj * k / F1F2)
    T0 = np.stack([t0.real, t0.imag]).astype(np.float32)
    T1 = np.stack([t1.real, t1.imag]).astype(np.float32)
    return dft_matrix(F0), dft_matrix(F1), dft_matrix(F2), T0, T1


def fft_3stage(x: np.ndarray, factors, tables=None, dtype=np.complex128) -> np.ndarray:
    """The data flow of fft_kernel (examples/fft.jl:45-121) on x of Julia shape (N, batch), complex:
    three batched products with the DFT matrices, two element-wise twiddle multiplications and the
    reshapes / permutedims between them, written with Fortran-order reshapes so that every line
    matches the Julia one."""
    F0, F1, F2 = factors
    N, F1F2, F0F2, F0F1 = F0 * F1 * F2, F1 * F2, F0 * F2, F0 * F1
    BS = x.shape[1]
    W0, W1, W2, T0, T1 = tables if tables is not None else make_twiddles(factors)
    c = lambda t: (t[0].astype(np.float64) + 1j * t[1].astype(np.float64)).astype(dtype)
    W0, W1, W2, T0, T1 = c(W0), c(W1), c(W2), c(T0), c(T1)
    R = lambda a, shp: np.reshape(a, shp, order="F")
    X = R(x.astype(dtype), (F1F2, F0, BS))                                   # fft.jl:82-83
    X = np.einsum("rib,ik->rkb", X, W0)                                      # :84-85  X * W0
    X = R(X, (N, BS)) * R(T0, (N,))[:, None]                                 # :88-89
    X = np.transpose(R(X, (F2, F1, F0, BS)), (2, 0, 1, 3))                   # :92-93  permutedims (3,1,2,4)
    X = np.einsum("rib,ik->rkb", R(X, (F0F2, F1, BS)), W1)                   # :97-100
    X = R(X, (F0, F1F2, BS)) * R(T1, (F1F2,))[None, :, None]                 # :103-104
    X = np.transpose(R(X, (F0, F2, F1, BS)), (2, 0, 1, 3))                   # :107-108
    X = np.einsum("rib,ik->rkb", R(X, (F0F1, F2, BS)), W2)                   # :112-115
    X = np.transpose(R(X, (F1, F0, F2, BS)), (1, 0, 2, 3))                   # :118-119 permutedims (2,1,3,4)
    return R(X, (N, BS))


# ---- host-level Tiled broadcast / mapreduce ------------------------------------------------
# Julia element types by name; numpy has no bfloat16, those cases are checked against torch.
_JL_FLOATS = ("Float16", "Float32", "Float64")
_JL_NP = {"Float16": np.float16, "Float32": np.float32, "Float64": np.float64, "Int32": np.int32, "Int64": np.int64,
          "Bool": np.bool_}
_NP_JL = {np.dtype(v): k for k, v in _JL_NP.items()}


def jl_promote(a: str, b: str) -> str:
    """Julia's promote_type on {Bool, Int32, Int64, Float16, Float32, Float64} (Base promotion.jl:
    Bool yields to everything, integers yield to floats, the wider of two of a kind wins)."""
    if a == b:
        return a
    if a == "Bool":
        return b
    if b == "Bool":
        return a
    ai, bi = a.startswith("Int"), b.startswith("Int")
    if ai and bi:
        return "Int64"
    if ai:
        return b
    if bi:
        return a
    return _JL_FLOATS[max(_JL_FLOATS.index(a), _JL_FLOATS.index(b))]


def _jl_scalar_type(x) -> str:
    if isinstance(x, (bool, np.bool_)):
        return "Bool"
    if isinstance(x, np.generic):
        return _NP_JL[np.dtype(type(x))]
    return "Int64" if isinstance(x, int) else "Float64"


_TILED_MATH = {"sqrt": np.sqrt, "cbrt": np.cbrt, "exp": np.exp, "exp2": np.exp2, "expm1": np.expm1, "log": np.log,
               "log2": np.log2, "log10": np.log10, "log1p": np.log1p, "sin": np.sin, "cos": np.cos, "tan": np.tan,
               "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan, "sinh": np.sinh, "cosh": np.cosh,
               "tanh": np.tanh, "exp10": lambda v: np.power(v.dtype.type(10), v), "inv": lambda v: v.dtype.type(1) / v,
               "rsqrt": lambda v: v.dtype.type(1) / np.sqrt(v)}


def _jl_shift(name, a, n):
    """Julia's << / >> / >>> on Int32 / Int64 (Base int.jl): counts of the word size or more shift everything
    out (>> keeps the sign), negative counts shift the other way."""
    bits = a.dtype.itemsize * 8
    u = np.dtype(f"uint{bits}")
    n = np.asarray(n, dtype=np.int64)
    a, n = np.broadcast_arrays(a, n)
    k = np.clip(np.abs(n), 0, bits - 1).astype(u)          # in-range count for numpy
    big = np.abs(n) >= bits
    left = np.where(big, 0, (a.view(u) << k).view(a.dtype))
    right_a = np.where(big, np.where(a < 0, -1, 0), a >> k.astype(a.dtype))
    right_l = np.where(big, 0, (a.view(u) >> k).view(a.dtype))
    right = right_a if name == "shr" else right_l
    fwd = left if name == "shl" else right
    back = (right_a if name == "shl" else left)            # a negative count of << is >>, of >> / >>> is <<
    return np.where(n >= 0, fwd, back).astype(a.dtype)
_TILED_CMP = {"lt": np.less, "le": np.less_equal, "gt": np.greater, "ge": np.greater_equal, "eq": np.equal,
              "ne": np.not_equal}


def _jl_max(a, b):
    """Julia's max: NaN wins, +0.0 beats -0.0 (Base math.jl)."""
    with np.errstate(invalid="ignore"):
        r = np.where(np.isnan(a) | np.isnan(b), a + b, np.maximum(a, b)) if a.dtype.kind == "f" else np.maximum(a, b)
    if a.dtype.kind == "f":
        tie = (a == b) & (a == 0)
        r = np.where(tie, np.where(np.signbit(a), b, a), r)
    return r.astype(a.dtype)


def _jl_min(a, b):
    with np.errstate(invalid="ignore"):
        r = np.where(np.isnan(a) | np.isnan(b), a + b, np.minimum(a, b)) if a.dtype.kind == "f" else np.minimum(a, b)
    if a.dtype.kind == "f":
        tie = (a == b) & (a == 0)
        r = np.where(tie, np.where(np.signbit(a), a, b), r)
    return r.astype(a.dtype)


def tiled_eval(text: str, leaves=(), scalars=()):
    """Value and Julia element type of a broadcast tree in the text form of the Tiled API
    (`name(args...)`, `a<i>`, `s<i>`), evaluated like Base.Broadcast does on the CPU: every node in
    its Julia result type (reference: `_eval_bc`, src/broadcast.jl:101-113; element types
    Base.Broadcast.combine_eltypes as used in src/broadcast.jl:28).  `leaves` are numpy arrays in the
    Julia shape; lower-rank leaves expand along trailing dimensions."""
    pos = 0
    rank = max([np.ndim(a) for a in leaves] + [0])

    def parse():
        nonlocal pos
        j = pos
        while pos < len(text) and (text[pos].isalnum() or text[pos] == "_"):
            pos += 1
        name = text[j:pos]
        if pos < len(text) and text[pos] == "(":
            pos += 1
            args = [parse()]
            while text[pos] == ",":
                pos += 1
                args.append(parse())
            assert text[pos] == ")"
            pos += 1
            return apply(name, args)
        if name[0] == "a":
            a = np.asarray(leaves[int(name[1:])])
            a = a.reshape(a.shape + (1,) * (rank - a.ndim))
            return a, _NP_JL[a.dtype]
        x = scalars[int(name[1:])]
        t = _jl_scalar_type(x)
        return np.asarray(x, dtype=_JL_NP[t]), t

    def conv(v, t):
        return v[0].astype(_JL_NP[t]) if v[1] != t else v[0]

    def apply(name, args):
        T = args[0][1]
        for a in args[1:]:
            T = jl_promote(T, a[1])
        isf = T in _JL_FLOATS
        if name in ("add", "sub"):
            R = "Int64" if T == "Bool" else T
            f = np.add if name == "add" else np.subtract
            return f(conv(args[0], R), conv(args[1], R)).astype(_JL_NP[R]), R
        if name == "mul":
            a, b = conv(args[0], T), conv(args[1], T)
            return (np.logical_and(a, b) if T == "Bool" else (a * b).astype(_JL_NP[T])), T
        if name == "div":
            R = T if isf else "Float64"
            return (conv(args[0], R) / conv(args[1], R)).astype(_JL_NP[R]), R
        if name == "neg":
            R = "Int64" if T == "Bool" else T
            return (-conv(args[0], R)).astype(_JL_NP[R]), R
        if name == "pow":
            # ^(x::T, p::Integer) keeps the type of the base (Base intfuncs.jl power_by_squaring; Bool * Bool is
            # Bool): Int32 ^ Int64 is Int32, Bool ^ Int is Bool, Float32 ^ Int is Float32; otherwise promote
            b, x = args
            R = b[1] if x[1] not in _JL_FLOATS else T
            if R == "Bool":
                return np.where(conv(x, "Int64") != 0, b[0], True), R
            if R in _JL_FLOATS:
                return np.power(conv(b, R), conv(x, R)).astype(_JL_NP[R]), R
            return np.power(conv(b, R), conv(x, "Int64")).astype(_JL_NP[R]), R
        if name in _TILED_MATH or name in ("atan2", "hypot"):
            R = T if isf else "Float64"
            # Julia evaluates Float16 functions in Float32 and rounds once (Base math.jl)
            W = "Float32" if R == "Float16" else R
            if name == "atan2":
                r = np.arctan2(conv(args[0], W), conv(args[1], W))
            elif name == "hypot":
                r = np.hypot(conv(args[0], W), conv(args[1], W))
            else:
                r = _TILED_MATH[name](conv(args[0], W))
            return np.asarray(r).astype(_JL_NP[R]), R
        if name in _TILED_CMP:
            return _TILED_CMP[name](conv(args[0], T), conv(args[1], T)), "Bool"
        if name in ("abs", "abs2", "sign", "floor", "ceil", "round", "trunc", "identity"):
            v = conv(args[0], T)
            if T == "Bool" or name == "identity":
                return v, T
            f = {"abs": np.abs, "abs2": lambda q: q * q, "sign": np.sign, "floor": np.floor, "ceil": np.ceil,
                 "round": np.rint, "trunc": np.trunc}[name]
            return (f(v) if isf or name in ("abs", "abs2", "sign") else v).astype(_JL_NP[T]), T
        if name in ("max", "min"):
            return (_jl_max if name == "max" else _jl_min)(*np.broadcast_arrays(conv(args[0], T), conv(args[1], T))), T
        if name in ("fma", "muladd"):
            a, b, c = (conv(v, T) for v in args)
            if isf and T != "Float64":   # one rounding: exact in float64 for Float32 / Float16 operands, then round
                return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(_JL_NP[T]), T
            return (a * b + c).astype(_JL_NP[T]), T
        if name == "clamp":
            x, lo, hi = (conv(v, T) for v in args)
            return np.where(x > hi, hi, np.where(x < lo, lo, x)).astype(_JL_NP[T]), T
        if name == "copysign":
            R = args[0][1]
            a, b = conv(args[0], R), conv(args[1], R)
            if R in _JL_FLOATS:
                return np.copysign(a, b), R
            return np.where(b < 0, -np.abs(a), np.abs(a)).astype(_JL_NP[R]), R
        if name in ("isnan", "isinf", "isfinite", "signbit", "iszero"):
            v = args[0][0]
            if name == "iszero":
                return v == 0, "Bool"
            if v.dtype.kind != "f":
                return np.broadcast_to({"isnan": False, "isinf": False, "isfinite": True}.get(name, False), v.shape) \
                    if name != "signbit" else (v < 0 if v.dtype.kind == "i" else np.zeros(v.shape, bool)), "Bool"
            return {"isnan": np.isnan, "isinf": np.isinf, "isfinite": np.isfinite, "signbit": np.signbit}[name](v), "Bool"
        if name == "not":
            v = conv(args[0], T)
            return (np.logical_not(v) if T == "Bool" else np.invert(v)), T
        if name in ("and", "or", "xor"):
            assert not isf
            f = {"and": np.bitwise_and, "or": np.bitwise_or, "xor": np.bitwise_xor}[name]
            return f(conv(args[0], T), conv(args[1], T)), T
        if name in ("shl", "shr", "lshr"):
            R = "Int64" if args[0][1] == "Bool" else args[0][1]
            assert R in ("Int32", "Int64") and args[1][1] not in _JL_FLOATS
            return _jl_shift(name, np.ascontiguousarray(conv(args[0], R)), conv(args[1], "Int64")), R
        if name == "mul_hi":
            assert not isf
            a, b = conv(args[0], T), conv(args[1], T)
            if T == "Bool":
                return np.zeros(np.broadcast(a, b).shape, bool), T
            bits = 32 if T == "Int32" else 64
            prod = a.astype(object) * b.astype(object)          # exact Python integers
            return np.asarray(prod >> bits, dtype=object).astype(_JL_NP[T]), T
        if name == "ifelse":
            R = jl_promote(args[1][1], args[2][1])
            return np.where(args[0][0], conv(args[1], R), conv(args[2], R)).astype(_JL_NP[R]), R
        if name in ("div_int", "rem", "mod", "fld", "cld"):
            R = "Int64" if T == "Bool" else T
            a, b = conv(args[0], R), conv(args[1], R)
            if R in _JL_FLOATS:
                # Base div.jl: the float quotients come from the exact remainder, round((x - rem(x, y, r)) / y);
                # mod of an exact multiple has the sign of the divisor (Base float.jl)
                def jmod(x, y):
                    m = np.fmod(x, y)
                    m = np.where(m == 0, np.copysign(m, y), np.where((m > 0) != (y > 0), m + y, m))
                    return m
                with np.errstate(all="ignore"):
                    r = {"div_int": lambda: np.rint((a - np.fmod(a, b)) / b), "rem": lambda: np.fmod(a, b), "mod": lambda: jmod(a, b),
                         "fld": lambda: np.rint((a - jmod(a, b)) / b), "cld": lambda: np.rint((a - jmod(a, -b)) / b)}[name]()
            else:
                q = np.floor_divide(a, b)
                r = {"div_int": lambda: np.trunc(a / b).astype(a.dtype), "rem": lambda: np.fmod(a, b),
                     "mod": lambda: np.mod(a, b), "fld": lambda: q,
                     "cld": lambda: -np.floor_divide(-a, b)}[name]()
            return np.asarray(r).astype(_JL_NP[R]), R
        conv_names = {"f16": "Float16", "f32": "Float32", "f64": "Float64", "i32": "Int32", "i64": "Int64", "bool": "Bool"}
        if name in conv_names:
            R = conv_names[name]
            v = args[0][0]
            if R.startswith("Int") and v.dtype.kind == "f":
                v = np.trunc(v)
            return (v != 0 if R == "Bool" else v.astype(_JL_NP[R])), R
        raise KeyError(name)

    value, jl = parse()
    assert pos == len(text)
    return value, jl


def tiled_broadcast(dest_shape, dest_type: str, text: str, leaves=(), scalars=()):
    """`dest .= tree` for a destination of Julia shape `dest_shape` and element type `dest_type`
    (src/broadcast.jl:75-92): axes must match or be 1 (DimensionMismatch -> ValueError), the value is
    converted to the destination's type."""
    rank = len(dest_shape)
    for a in leaves:
        sh = tuple(np.shape(a)) + (1,) * (rank - np.ndim(a))
        for d, v in enumerate(sh):
            if v != 1 and (d >= rank or v != dest_shape[d]):
                raise ValueError("DimensionMismatch")
    value, _ = tiled_eval(text, leaves, scalars)
    value = np.asarray(value)
    value = value.reshape(value.shape + (1,) * (rank - value.ndim)) if value.ndim <= rank else value.reshape(dest_shape)
    return np.broadcast_to(value, dest_shape).astype(_JL_NP[dest_type])


def tiled_mapreduce(f_text, op: str, A: np.ndarray, dims=None, init=None, scalars=()):
    """`mapreduce(f, op, A; dims, init)` with the reference's result-type and `dims` rules
    (src/mapreduce.jl:131-172): T = typeof(f(x)), ET = promote_op(op, T, T) -- `+` turns Bool into
    Int64, "add_sum" / "mul_prod" (what sum / prod pass) also widen Int32 -- dimensions outside
    1:ndims are ignored, reduced dimensions keep extent 1, `dims=None` (Julia's `:`) returns a
    scalar.  Returns (value, Julia element type)."""
    v, T = tiled_eval(f_text, (A,), scalars) if f_text else (np.asarray(A), _NP_JL[np.asarray(A).dtype])
    v = np.broadcast_to(v, np.shape(A))
    ET = T
    if op in ("+", "add_sum") and T == "Bool":
        ET = "Int64"
    if op in ("add_sum", "mul_prod") and T in ("Int32", "Bool"):
        ET = "Int64"
    v = v.astype(_JL_NP[ET])
    N = v.ndim
    region = tuple(range(1, N + 1)) if dims is None else ((dims,) if isinstance(dims, (int, np.integer)) else tuple(dims))
    axes = tuple(d - 1 for d in range(1, N + 1) if d in region)
    if op in ("max", "min"):
        # numpy's max / min propagate NaN like Julia's; ties between +-0.0 are not distinguished by value
        r = (np.max if op == "max" else np.min)(v, axis=axes, keepdims=True) if axes else v
    else:
        f = {"+": np.add, "add_sum": np.add, "*": np.multiply, "mul_prod": np.multiply, "&": np.bitwise_and,
             "|": np.bitwise_or}[op]
        acc = np.float64 if ET in ("Float16", "Float32") else _JL_NP[ET]
        r = f.reduce(v.astype(acc), axis=axes, keepdims=True).astype(_JL_NP[ET]) if axes else v
    if init is not None:
        i = _JL_NP[ET](init)
        g = {"+": np.add, "add_sum": np.add, "*": np.multiply, "mul_prod": np.multiply, "max": np.maximum,
             "min": np.minimum, "&": np.bitwise_and, "|": np.bitwise_or}[op]
        r = g(i, r).astype(_JL_NP[ET])
    if dims is None:
        return r.reshape(-1)[0], ET
    return r, ET


# ---- Philox2x32-7 host RNG fills ---------------------------------------------------------------
PHILOX_M = 0xD256D193      # src/language/random.jl:93
PHILOX_W = 0x9E3779B9      # src/language/random.jl:94 (Weyl key step)
RAND_FILL_TILE = 512       # src/language/random.jl:701


def philox2x32(c1, c2, key, rounds: int = 7):
    """Philox2x32 with `rounds` rounds on uint32 arrays: per round (hi ^ k ^ c2, lo) of the 64-bit
    product c1 * M, the key bumped by W between rounds (src/language/random.jl:100-122).  This is
    Random123's philox2x32 (D. E. Shaw Research, Random123 1.14, `philox.h`); its published
    known-answer vectors (`tests/kat_vectors`) pin this function in tests/test_oracle.py."""
    c1 = np.asarray(c1, np.uint32).copy()
    c2 = np.asarray(c2, np.uint32).copy()
    k = np.broadcast_to(np.asarray(key, np.uint32), c1.shape).copy()
    for r in range(rounds):
        if r:
            k = (k + np.uint32(PHILOX_W)).astype(np.uint32)
        p = c1.astype(np.uint64) * np.uint64(PHILOX_M)
        hi = (p >> np.uint64(32)).astype(np.uint32)
        lo = (p & np.uint64(0xFFFFFFFF)).astype(np.uint32)
        c1, c2 = hi ^ k ^ c2, lo
    return c1, c2


def _u01_f32(u):
    """(u * 2^-32) + 2^-33 in Float32 (src/language/random.jl:136-142)."""
    return (u.astype(np.float32) * np.float32(2.0 ** -32) + np.float32(2.0 ** -33)).astype(np.float32)


def _u01_f64(u):
    """Mantissa construction in [1, 2) minus 1, low bit forced (src/language/random.jl:169-174)."""
    bits = (u >> np.uint64(12)) | np.uint64(0x3FF0000000000001)
    return bits.view(np.float64) - 1.0


def rng_advance_counter(seed: int, counter: int, n: int):
    """`advance_counter!`: UInt32 counter += n, the carry bumps the seed (src/language/random.jl:694-699)."""
    new = (counter + n) & 0xFFFFFFFF
    if new < counter:
        seed = (seed + 1) & 0xFFFFFFFF
    return seed, new


def rng_fill(kind: str, n: int, seed: int, counter: int, dist: str = "rand"):
    """The `n` values a host fill writes for `cuTile.RNG(seed, counter)`: `rand!` / `randn!` /
    `randexp!` (src/language/random.jl:759-818) launch one block per 512 outputs (:703-740); block b
    (0-based) uses the Philox key (b * W) xor seed (:207-224, default stream) and counters
    counter + i.  How a block's Philox outputs (c1, c2) land in its 512 slots depends on the width:
    32-bit: 256 calls, c1 -> slots 0..255, c2 -> 256..511 (:262-286); 64-bit: 512 calls, c1 | c2 << 32
    (:290-305); 16-bit: 128 calls give 256 words (c1 then c2), low halves -> 0..255, high halves ->
    256..511 (:314-324); 8-bit: 64 calls give 128 words, byte q of word m -> slot 128 q + m
    (:326-338).  Floats: `u01` (:136-174).  randn: Box-Muller on the (c1, c2) pair, r = sqrt(-2 log
    u01(c2)), angle = 2 pi u01(c1) -> (r sin, r cos) in slots i and 256 + i, computed in Float32 for
    the 16-bit floats (:369-398, 420-441); Float64 pairs counters i and 256 + i (:449-480).
    randexp: -log(rand) (:500-501).
    `kind`: u8 i8 u16 i16 u32 i32 u64 i64 f16 bf16 f32 f64; bf16 values are returned as float32."""
    width = {"u8": 1, "i8": 1, "u16": 2, "i16": 2, "f16": 2, "bf16": 2, "u32": 4, "i32": 4, "f32": 4, "u64": 8, "i64": 8,
             "f64": 8}[kind]
    nb = cld(n, RAND_FILL_TILE)
    b = np.arange(nb, dtype=np.uint64)
    key = ((b * np.uint64(PHILOX_W)) & np.uint64(0xFFFFFFFF)).astype(np.uint32) ^ np.uint32(seed & 0xFFFFFFFF)

    def calls(count, offset=0):
        ctr = ((np.uint64(counter) + np.uint64(offset) + np.arange(count, dtype=np.uint64)) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
        c1, c2 = philox2x32(np.broadcast_to(ctr, (nb, count)), np.zeros((nb, count), np.uint32), key[:, None])
        return c1, c2

    if dist == "randn":
        if width == 8:
            a1, a2 = calls(256)
            b1, b2 = calls(256, 256)
            f1 = _u01_f64(a1.astype(np.uint64) | (a2.astype(np.uint64) << np.uint64(32)))
            f2 = _u01_f64(b1.astype(np.uint64) | (b2.astype(np.uint64) << np.uint64(32)))
            r = np.sqrt(-2.0 * np.log(f1))
            ang = 2.0 * np.pi * f2
        else:
            c1, c2 = calls(256)
            f1, f2 = _u01_f32(c1), _u01_f32(c2)
            r = np.sqrt(np.float32(-2) * np.log(f2)).astype(np.float32)
            ang = (np.float32(2 * np.pi) * f1).astype(np.float32)
        out = np.concatenate([r * np.sin(ang), r * np.cos(ang)], axis=1)
        if kind == "f16":
            out = out.astype(np.float16)
        elif kind == "bf16":
            out = bf16_round(out.astype(np.float32))
        return out.reshape(-1)[:n]

    if width == 4:
        c1, c2 = calls(256)
        u = np.concatenate([c1, c2], axis=1)
    elif width == 8:
        c1, c2 = calls(512)
        u = c1.astype(np.uint64) | (c2.astype(np.uint64) << np.uint64(32))
    elif width == 2:
        c1, c2 = calls(128)
        raw = np.concatenate([c1, c2], axis=1)
        u = np.concatenate([(raw & np.uint32(0xFFFF)).astype(np.uint16), (raw >> np.uint32(16)).astype(np.uint16)], axis=1)
    else:
        c1, c2 = calls(64)
        raw = np.concatenate([c1, c2], axis=1)
        u = np.concatenate([((raw >> np.uint32(8 * q)) & np.uint32(0xFF)).astype(np.uint8) for q in range(4)], axis=1)
    u = u.reshape(-1)[:n]
    if kind in ("u8", "u16", "u32", "u64"):
        v = u
    elif kind in ("i8", "i16", "i32", "i64"):
        v = u.view({1: np.int8, 2: np.int16, 4: np.int32, 8: np.int64}[width])
    elif kind == "f32":
        v = _u01_f32(u)
    elif kind == "f64":
        v = _u01_f64(u)
    elif kind == "f16":        # (u >> 6) | 0x3C01 as Float16, minus 1 (src/language/random.jl:148-154)
        v = ((u >> np.uint16(6)) | np.uint16(0x3C01)).view(np.float16) - np.float16(1)
    else:                      # bf16: (u >> 9) | 0x3F81 as BFloat16, minus 1 (:155-161); exact in float32
        bits = ((u >> np.uint16(9)) | np.uint16(0x3F81)).astype(np.uint32) << np.uint32(16)
        v = bits.view(np.float32) - np.float32(1)
    if dist == "randexp":
        if kind == "f64":
            return -np.log(v)
        return (-np.log(v.astype(np.float32))).astype(np.float16 if kind == "f16" else np.float32)
    return v


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest-even BFloat16, returned as float32."""
    u = np.asarray(x, np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


# ---- example verify() criteria -------------------------------------------------------------

def isapprox(x: np.ndarray, y: np.ndarray, rtol: float, atol: float = 0.0) -> bool:
    """Julia's ``isapprox`` for arrays: ``norm(x-y) <= max(atol, rtol*max(norm(x), norm(y)))``
    with the 2-norm (used by every example's verify)."""
    wide = np.complex128 if np.iscomplexobj(x) or np.iscomplexobj(y) else np.float64
    x = np.asarray(x, dtype=wide); y = np.asarray(y, dtype=wide)
    d = np.linalg.norm((x - y).ravel())
    return bool(d <= max(atol, rtol * max(np.linalg.norm(x.ravel()), np.linalg.norm(y.ravel()))))
