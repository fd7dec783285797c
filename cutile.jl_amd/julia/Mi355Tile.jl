# Mi355Tile.jl — Julia binding of libmi355tile.so (the C ABI in include/mi355tile.h).
#
# One Julia function per example kernel of cuTile.jl, with the kernel's own name and argument
# order, so an example's host code changes only at the launch line:
#
#     @cuda backend=cuTile blocks=grid matmul_kernel(A, B, C, ct.Constant(tm), ct.Constant(tn), ct.Constant(tk))
# becomes
#     Mi355Tile.matmul_kernel(A, B, C, tm, tn, tk)
#
# Arrays are anything that answers `pointer`, `size`, `strides` and `eltype` with a DEVICE
# pointer: `AMDGPU.ROCArray`, views of it (`SubArray`/`reshape`), or the `DevicePtrArray`
# below for memory obtained from hipMalloc directly.  The default stream argument is the HIP
# null stream; pass `AMDGPU.stream().stream` (a `hipStream_t`) to enqueue on the task's stream,
# which is what the reference does with the task-local CUDA stream (src/launch.jl:862).
#
# This file has not been executed: the build image has no Julia.  It is the binding a
# maintainer would add; the same entry points are exercised through Python ctypes by the
# test-suite.

module Mi355Tile

const libmi355tile = get(ENV, "MI355TILE_LIB",
                         joinpath(@__DIR__, "..", "libmi355tile.so"))

# ---- mi_tile_array (include/mi355tile.h) -------------------------------------------------

const MI_MAX_RANK = 4

struct MiTileArray
    ptr::Ptr{Cvoid}
    dtype::Int32
    ndim::Int32
    sizes::NTuple{MI_MAX_RANK,Int64}
    strides::NTuple{MI_MAX_RANK,Int64}
end

mi_dtype(::Type{Float32}) = Int32(0)
mi_dtype(::Type{Float64}) = Int32(1)
mi_dtype(::Type{Float16}) = Int32(2)
mi_dtype(::Type{Int32})   = Int32(5)
mi_dtype(::Type{Int64})   = Int32(6)
mi_dtype(::Type{Bool})    = Int32(7)
# BFloat16 (BFloat16s.jl / Core.BFloat16) = 3, Float8_E4M3FN = 4 and Float8_E5M2 = 10 (DLFP8Types.jl): add the
# methods in a package extension, the way ext/DLFP8TypesExt.jl adds the cuTile mapping.  matmul_kernel and
# batch_matmul_kernel take both FP8 types as operands (A and B of the same type, C Float32 / Float16 / BFloat16).
mi_dtype(T::Type) = T === UInt8 ? Int32(4) :   # raw e4m3fn bytes
                    error("Mi355Tile: unsupported element type $T")

"A bare device allocation viewed as an N-d column-major array (no GPU package needed)."
struct DevicePtrArray{T,N}
    ptr::Ptr{T}
    dims::NTuple{N,Int}
end
Base.pointer(a::DevicePtrArray) = a.ptr
Base.size(a::DevicePtrArray) = a.dims
Base.strides(a::DevicePtrArray{T,N}) where {T,N} =
    ntuple(i -> prod(a.dims[1:i-1]; init=1), N)
Base.eltype(::DevicePtrArray{T}) where {T} = T

pad4(t::NTuple{N,<:Integer}, fill) where {N} =
    ntuple(i -> i <= N ? Int64(t[i]) : Int64(fill), MI_MAX_RANK)

"Descriptor of `a` — the same (ptr, sizes, strides-in-elements) triple that the reference's
`TileArray(arr)` builds (src/language/types.jl:314-357)."
function descriptor(a; dtype::Int32=mi_dtype(eltype(a)))
    N = length(size(a))
    N <= MI_MAX_RANK || error("Mi355Tile: rank $N > $MI_MAX_RANK")
    MiTileArray(Ptr{Cvoid}(UInt(pointer(a))), dtype, Int32(N),
                pad4(size(a), 1), pad4(strides(a), 0))
end
descriptor(::Nothing; kwargs...) = nothing

struct MiError <: Exception
    code::Cint
    msg::String
end
Base.showerror(io::IO, e::MiError) = print(io, "mi355tile error ", e.code, ": ", e.msg)

function check(rc::Cint)
    rc == 0 && return nothing
    msg = unsafe_string(ccall((:mi_strerror, libmi355tile), Cstring, (Cint,), rc))
    throw(MiError(rc, msg))
end

ref(d::MiTileArray) = Ref(d)
const NULLDESC = Ptr{MiTileArray}(C_NULL)

version() = ccall((:mi_version, libmi355tile), Cint, ())
last_variant() = unsafe_string(ccall((:mi_last_variant, libmi355tile), Cstring, ()))

# ---- examples/vadd.jl ---------------------------------------------------------------------

function vec_add_kernel_1d(a, b, c, tile::Integer; stream::Ptr{Cvoid}=C_NULL)
    da, db, dc = ref(descriptor(a)), ref(descriptor(b)), ref(descriptor(c))
    GC.@preserve a b c check(ccall((:mi_vec_add_kernel_1d, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Ptr{Cvoid}),
        da, db, dc, tile, stream))
end

function vec_add_kernel_2d(a, b, c, tile_x::Integer, tile_y::Integer; stream::Ptr{Cvoid}=C_NULL)
    da, db, dc = ref(descriptor(a)), ref(descriptor(b)), ref(descriptor(c))
    GC.@preserve a b c check(ccall((:mi_vec_add_kernel_2d, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Ptr{Cvoid}),
        da, db, dc, tile_x, tile_y, stream))
end

function vec_add_kernel_1d_gather(a, b, c, tile::Integer; stream::Ptr{Cvoid}=C_NULL)
    da, db, dc = ref(descriptor(a)), ref(descriptor(b)), ref(descriptor(c))
    GC.@preserve a b c check(ccall((:mi_vec_add_kernel_1d_gather, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Ptr{Cvoid}),
        da, db, dc, tile, stream))
end

# ---- examples/transpose.jl ----------------------------------------------------------------

function transpose_kernel(x, y, tm::Integer, tn::Integer; stream::Ptr{Cvoid}=C_NULL)
    dx, dy = ref(descriptor(x)), ref(descriptor(y))
    GC.@preserve x y check(ccall((:mi_transpose_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Ptr{Cvoid}),
        dx, dy, tm, tn, stream))
end

# ---- examples/matmul.jl, examples/batchmatmul.jl ------------------------------------------

function matmul_kernel(A, B, C, tm::Integer, tn::Integer, tk::Integer; stream::Ptr{Cvoid}=C_NULL)
    dA, dB, dC = ref(descriptor(A)), ref(descriptor(B)), ref(descriptor(C))
    GC.@preserve A B C check(ccall((:mi_matmul_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Ptr{Cvoid}),
        dA, dB, dC, tm, tn, tk, stream))
end

function batch_matmul_kernel(A, B, C, tm::Integer, tn::Integer, tk::Integer; stream::Ptr{Cvoid}=C_NULL)
    dA, dB, dC = ref(descriptor(A)), ref(descriptor(B)), ref(descriptor(C))
    GC.@preserve A B C check(ccall((:mi_batch_matmul_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Ptr{Cvoid}),
        dA, dB, dC, tm, tn, tk, stream))
end

function swizzle_2d(M, N, tm, tn, GROUP_SIZE_M, bid)
    bm, bn = Ref{Int32}(0), Ref{Int32}(0)
    ccall((:mi_swizzle_2d, libmi355tile), Cvoid,
          (Int32, Int32, Int32, Int32, Int32, Int32, Ref{Int32}, Ref{Int32}),
          M, N, tm, tn, GROUP_SIZE_M, bid, bm, bn)
    return bm[], bn[]
end

# ---- examples/layernorm.jl ----------------------------------------------------------------

function layer_norm_fwd(X, W, B, Y, Mean, Rstd, eps::Real, TILE_N::Integer; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (X, W, B, Y, Mean, Rstd))
    GC.@preserve X W B Y Mean Rstd check(ccall((:mi_layer_norm_fwd, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ref{MiTileArray}, Ref{MiTileArray}, Cfloat, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], Float32(eps), TILE_N, stream))
end

# The caller zero-fills DW and DB first, as the reference's run_bwd does (layernorm.jl:245-246).
# `Locks` is accepted and ignored (pass the array or `nothing`).
function layer_norm_bwd_dx_partial_dwdb(DX, DY, DW, DB, X, W, Mean, Rstd, Locks,
                                        GROUP_SIZE_M::Integer, TILE_N::Integer;
                                        stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (DX, DY, DW, DB, X, W, Mean, Rstd))
    dl = Locks === nothing ? nothing : ref(descriptor(Locks))
    GC.@preserve DX DY DW DB X W Mean Rstd Locks check(ccall(
        (:mi_layer_norm_bwd_dx_partial_dwdb, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ptr{MiTileArray}, Cint, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8],
        dl === nothing ? NULLDESC : Base.unsafe_convert(Ptr{MiTileArray}, dl),
        GROUP_SIZE_M, TILE_N, stream))
end

function layer_norm_bwd_dwdb(DW, DB, FINAL_DW, FINAL_DB, TILE_M::Integer, TILE_N::Integer;
                             stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (DW, DB, FINAL_DW, FINAL_DB))
    GC.@preserve DW DB FINAL_DW FINAL_DB check(ccall((:mi_layer_norm_bwd_dwdb, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], TILE_M, TILE_N, stream))
end

# The whole backward (zero fill of the partials, layer_norm_bwd_dx_partial_dwdb, layer_norm_bwd_dwdb:
# layernorm.jl:245-251) in one call that allocates nothing: the partial slots live in a static device
# array of the library (N rounded up to a multiple of 4, times GROUP_SIZE_M, at most 524288 floats).
# For callers that can not allocate; calls that overlap on one GPU share the array and race.
function layer_norm_bwd_static(DX, DY, X, W, Mean, Rstd, FINAL_DW, FINAL_DB, GROUP_SIZE_M::Integer,
                               TILE_M::Integer, TILE_N::Integer; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (DX, DY, X, W, Mean, Rstd, FINAL_DW, FINAL_DB))
    GC.@preserve DX DY X W Mean Rstd FINAL_DW FINAL_DB check(ccall(
        (:mi_layer_norm_bwd_static, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], GROUP_SIZE_M, TILE_M, TILE_N, stream))
end

# ---- examples/softmax.jl ------------------------------------------------------------------

function softmax_tma_kernel(output, input, TILE_SIZE::Integer; blocks::Integer=size(input, 2),
                            stream::Ptr{Cvoid}=C_NULL)
    dout, din = ref(descriptor(output)), ref(descriptor(input))
    GC.@preserve output input check(ccall((:mi_softmax_tma_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Ptr{Cvoid}),
        dout, din, TILE_SIZE, blocks, stream))
end

function softmax_chunked_kernel(output, input, n_elems::Integer, TILE_SIZE::Integer;
                                blocks::Integer=size(input, 2), stream::Ptr{Cvoid}=C_NULL)
    dout, din = ref(descriptor(output)), ref(descriptor(input))
    GC.@preserve output input check(ccall((:mi_softmax_chunked_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Ptr{Cvoid}),
        dout, din, n_elems, TILE_SIZE, blocks, stream))
end

# ---- examples/fmha.jl ---------------------------------------------------------------------

function fmha_kernel(Q, K, V, Out, qk_scale::Real, input_pos::Integer, TILE_D::Integer,
                     H::Integer, TILE_M::Integer, TILE_N::Integer, QUERY_GROUP_SIZE::Integer,
                     CAUSAL::Bool, EVEN_K::Bool; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (Q, K, V, Out))
    GC.@preserve Q K V Out check(ccall((:mi_fmha_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cfloat, Int32,
         Cint, Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], Float32(qk_scale), Int32(input_pos), TILE_D, H, TILE_M, TILE_N,
        QUERY_GROUP_SIZE, CAUSAL, EVEN_K, stream))
end

# ---- examples/moe.jl ----------------------------------------------------------------------

"Host routine; `topk_ids` is the (num_tokens, topk) Int64 matrix of 1-based expert ids
(examples/moe.jl:142-183).  Returns (sorted_token_ids, sorted_expert_ids) as host Int32 vectors."
function moe_align_tile_size(topk_ids::Matrix{Int64}, tile_m::Integer, num_experts::Integer)
    nt, topk = size(topk_ids)
    nblocks = Ref{Int64}(0)
    check(ccall((:mi_moe_align_tile_size, libmi355tile), Cint,
        (Ptr{Int64}, Int64, Int64, Cint, Cint, Ptr{Int32}, Ptr{Int32}, Ref{Int64}),
        topk_ids, nt, topk, tile_m, num_experts, C_NULL, C_NULL, nblocks))
    ids = Vector{Int32}(undef, nblocks[] * tile_m)
    experts = Vector{Int32}(undef, nblocks[])
    check(ccall((:mi_moe_align_tile_size, libmi355tile), Cint,
        (Ptr{Int64}, Int64, Int64, Cint, Cint, Ptr{Int32}, Ptr{Int32}, Ref{Int64}),
        topk_ids, nt, topk, tile_m, num_experts, ids, experts, nblocks))
    return ids, experts
end

"Device counterpart: `topk_ids` (num_tokens, topk) Int64 on the device; fills the fixed-capacity
device vectors `sorted_token_ids` (Int32, `tile_m` per block) and `sorted_expert_ids` (Int32, at least
cld(total + min(total, num_experts)*(tile_m-1), tile_m) blocks).  Unused blocks get expert 0."
function moe_align_tile_size_device(topk_ids, tile_m::Integer, num_experts::Integer,
                                    sorted_token_ids, sorted_expert_ids; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (topk_ids, sorted_token_ids, sorted_expert_ids))
    GC.@preserve topk_ids sorted_token_ids sorted_expert_ids check(ccall(
        (:mi_moe_align_tile_size_device, libmi355tile), Cint,
        (Ref{MiTileArray}, Cint, Cint, Ref{MiTileArray}, Ref{MiTileArray}, Ptr{Cvoid}),
        d[1], tile_m, num_experts, d[2], d[3], stream))
end

"Router on the device: fills `topk_ids` (num_tokens, topk) Int64 with the experts of the `topk`
largest `logits[t, :]` (ties to the lower id) and `topk_weights` with the softmax over them."
function moe_route_topk(logits, topk_weights, topk_ids; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (logits, topk_weights, topk_ids))
    GC.@preserve logits topk_weights topk_ids check(ccall(
        (:mi_moe_route_topk, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ptr{Cvoid}),
        d[1], d[2], d[3], stream))
end

# The sort of `moe_align_tile_size_device`, which also fills `clear` (a dense device array of whole 16-byte units) with
# zeros in the same launch: the output that `fused_moe_accumulate_kernel` adds into.
function moe_align_tile_size_device_clear(topk_ids, tile_m::Integer, num_experts::Integer, sorted_token_ids,
                                          sorted_expert_ids, clear; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (topk_ids, sorted_token_ids, sorted_expert_ids, clear))
    GC.@preserve topk_ids sorted_token_ids sorted_expert_ids clear check(ccall(
        (:mi_moe_align_tile_size_device_clear, libmi355tile), Cint,
        (Ref{MiTileArray}, Cint, Cint, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ptr{Cvoid}),
        d[1], tile_m, num_experts, d[2], d[3], d[4], stream))
end

# The down projection and `sum(cache3; dims=2)` (moe.jl:245-256) in one launch: `Out` (N, num_tokens), zeroed
# beforehand, receives every replica's weighted row by packed atomic adds.  `topk_weights` is the (num_tokens, topk)
# matrix, topk = 1 or 2.
function fused_moe_accumulate_kernel(A, B, Out, topk_weights, sorted_token_ids, sorted_expert_ids,
                                     TILE_M::Integer, TILE_N::Integer, TILE_K::Integer;
                                     b_scale=nothing, stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (A, B, Out, topk_weights, sorted_token_ids, sorted_expert_ids))
    ds = b_scale === nothing ? nothing : ref(descriptor(b_scale))
    GC.@preserve A B Out topk_weights sorted_token_ids sorted_expert_ids b_scale check(ccall(
        (:mi_fused_moe_accumulate_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Cint, Cint, Cint, Ptr{MiTileArray}, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], TILE_M, TILE_N, TILE_K,
        ds === nothing ? NULLDESC : Base.unsafe_convert(Ptr{MiTileArray}, ds), stream))
end

# `b_scale` (N, E) Float32 goes with e4m3fn weights only; `nothing` otherwise.  `topk_weights` is either the
# flattened `vec(permutedims(topk_weights))` of moe.jl:193 or the (num_tokens, topk) matrix itself, which saves that copy.
function fused_moe_kernel(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids,
                          num_token_replicas::Integer, mul_routed_weight::Bool,
                          TILE_M::Integer, TILE_N::Integer, TILE_K::Integer;
                          b_scale=nothing, stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids))
    ds = b_scale === nothing ? nothing : ref(descriptor(b_scale))
    GC.@preserve A B C topk_weights sorted_token_ids sorted_expert_ids b_scale check(ccall(
        (:mi_fused_moe_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Cint, Cint,
         Ptr{MiTileArray}, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], num_token_replicas, mul_routed_weight,
        TILE_M, TILE_N, TILE_K,
        ds === nothing ? NULLDESC : Base.unsafe_convert(Ptr{MiTileArray}, ds), stream))
end

# The gate / up GEMM with silu_and_mul_kernel as its epilogue: C is (N/2, total_tokens).
function fused_moe_silu_kernel(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids,
                          num_token_replicas::Integer, mul_routed_weight::Bool,
                          TILE_M::Integer, TILE_N::Integer, TILE_K::Integer;
                          b_scale=nothing, stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids))
    ds = b_scale === nothing ? nothing : ref(descriptor(b_scale))
    GC.@preserve A B C topk_weights sorted_token_ids sorted_expert_ids b_scale check(ccall(
        (:mi_fused_moe_silu_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Cint, Cint,
         Ptr{MiTileArray}, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], num_token_replicas, mul_routed_weight,
        TILE_M, TILE_N, TILE_K,
        ds === nothing ? NULLDESC : Base.unsafe_convert(Ptr{MiTileArray}, ds), stream))
end

function silu_and_mul_kernel(A, B, C, TILE_N::Integer; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (A, B, C))
    GC.@preserve A B C check(ccall((:mi_silu_and_mul_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], TILE_N, stream))
end

"out (H, tokens) = sum over dim 2 of in (H, topk, tokens): the `sum(cache3; dims=2)` of
cutile_moe (examples/moe.jl:256)."
function moe_sum_topk(in, out; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (in, out))
    GC.@preserve in out check(ccall((:mi_moe_sum_topk, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ptr{Cvoid}), d[1], d[2], stream))
end

"Hand the library's shared static arrays (split GEMM / attention partials, sort counts) to capturing streams as well;
the caller keeps replays of such graphs apart from one another and from other launches that use them.  Returns the
previous setting."
scratch_under_capture(allow::Bool) = ccall((:mi_scratch_under_capture, libmi355tile), Cint, (Cint,), allow ? 1 : 0) != 0

"codes (K, columns) E4M3FN and scale[1] = max |x| / 448 of a Float16 / BFloat16 activation matrix x (K, columns):
the fp8 operand `A` of `fused_moe_kernel` when the expert weights are fp8 as well.  `workspace`: 1024 Float32."
function quantize_e4m3fn(x, codes, scale, workspace; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (x, codes, scale, workspace))
    GC.@preserve x codes scale workspace check(ccall((:mi_quantize_e4m3fn, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ptr{Cvoid}), d[1], d[2], d[3], d[4], stream))
end

"The same, and fold_out .= fold_in .* scale[1] (dense Float32 arrays of one shape: the weights' scales that these
activations meet) from the same two launches."
function quantize_e4m3fn_fold(x, codes, scale, workspace, fold_in, fold_out; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (x, codes, scale, workspace, fold_in, fold_out))
    GC.@preserve x codes scale workspace fold_in fold_out check(ccall((:mi_quantize_e4m3fn_fold, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ptr{Cvoid}), d[1], d[2], d[3], d[4], d[5], d[6], stream))
end

# ---- examples/fft.jl ----------------------------------------------------------------------

function fft_kernel(x_packed_in, y_packed_out, W0, W1, W2, T0, T1, N::Integer, F0::Integer, F1::Integer,
                    F2::Integer, BS::Integer, D::Integer; stream::Ptr{Cvoid}=C_NULL)
    d = map(a -> ref(descriptor(a)), (x_packed_in, y_packed_out, W0, W1, W2, T0, T1))
    GC.@preserve x_packed_in y_packed_out W0 W1 W2 T0 T1 check(ccall((:mi_fft_kernel, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray}, Ref{MiTileArray},
         Ref{MiTileArray}, Ref{MiTileArray}, Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Cvoid}),
        d[1], d[2], d[3], d[4], d[5], d[6], d[7], N, F0, F1, F2, BS, D, stream))
end

# ---- host-level Tiled broadcast / mapreduce (src/broadcast.jl, src/mapreduce.jl) ---------

# == struct mi_tile_scalar: dtype, reserved, 8-byte value (Float64 bits or Int64)
struct MiTileScalar
    dtype::Int32
    reserved::Int32
    bits::UInt64
end
MiTileScalar(x::AbstractFloat) = MiTileScalar(mi_dtype(typeof(x)), 0, reinterpret(UInt64, Float64(x)))
MiTileScalar(x::Integer) = MiTileScalar(mi_dtype(typeof(x)), 0, reinterpret(UInt64, Int64(x)))
MiTileScalar(x::Bool) = MiTileScalar(mi_dtype(Bool), 0, UInt64(x))

const MI_OP_ADD, MI_OP_MUL, MI_OP_MAX, MI_OP_MIN, MI_OP_AND, MI_OP_OR = Int32.(0:5)
opcode(::typeof(+)) = MI_OP_ADD
opcode(::typeof(Base.add_sum)) = MI_OP_ADD
opcode(::typeof(*)) = MI_OP_MUL
opcode(::typeof(Base.mul_prod)) = MI_OP_MUL
opcode(::typeof(max)) = MI_OP_MAX
opcode(::typeof(min)) = MI_OP_MIN
opcode(::typeof(&)) = MI_OP_AND
opcode(::typeof(|)) = MI_OP_OR

"`dest .= expr(leaves..., scalars...)`; `expr` is the prefix text form described in mi355tile.h."
function tiled_broadcast(dest, expr::AbstractString, leaves::AbstractVector, scalars::AbstractVector{<:Number};
                         stream::Ptr{Cvoid}=C_NULL)
    descs = [descriptor(a) for a in leaves]
    ptrs = [pointer(descs, i) for i in eachindex(descs)]
    sc = MiTileScalar[MiTileScalar(x) for x in scalars]
    d = ref(descriptor(dest))
    GC.@preserve dest leaves descs ptrs sc check(ccall((:mi_tiled_broadcast, libmi355tile), Cint,
        (Ref{MiTileArray}, Cstring, Ptr{Ptr{MiTileArray}}, Cint, Ptr{MiTileScalar}, Cint, Ptr{Cvoid}),
        d, expr, ptrs, length(ptrs), sc, length(sc), stream))
    return dest
end

"Bytes of device workspace `tiled_mapreduce` needs for these shapes (0 for most)."
function tiled_mapreduce_workspace(dest, src, op::Integer)
    n = Ref{Int64}(0)
    check(ccall((:mi_tiled_mapreduce_workspace, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Cint, Ref{Int64}), ref(descriptor(dest)), ref(descriptor(src)), op, n))
    return n[]
end

"`dest = reduce(op, f.(src))` over the dimensions where `dest` has extent 1; `f_expr === nothing` is identity."
function tiled_mapreduce(dest, src, f_expr::Union{Nothing,AbstractString}, scalars::AbstractVector{<:Number}, op::Integer,
                         workspace=nothing; stream::Ptr{Cvoid}=C_NULL)
    sc = MiTileScalar[MiTileScalar(x) for x in scalars]
    ws = workspace === nothing ? C_NULL : Ptr{Cvoid}(UInt(pointer(workspace)))
    nws = workspace === nothing ? 0 : sizeof(workspace)
    GC.@preserve dest src sc workspace check(ccall((:mi_tiled_mapreduce, libmi355tile), Cint,
        (Ref{MiTileArray}, Ref{MiTileArray}, Cstring, Ptr{MiTileScalar}, Cint, Cint, Ptr{Cvoid}, Int64, Ptr{Cvoid}),
        ref(descriptor(dest)), ref(descriptor(src)), f_expr === nothing ? C_NULL : f_expr, sc, length(sc), op, ws, nws,
        stream))
    return dest
end

# ---- host-level RNG fills (src/language/random.jl:759-818) -------------------------------

mi_dtype(::Type{Int8})  = Int32(8)
mi_dtype(::Type{Int16}) = Int32(9)
mi_dtype(::Type{UInt16}) = Int32(9)
mi_dtype(::Type{UInt32}) = Int32(5)
mi_dtype(::Type{UInt64}) = Int32(6)

"Fill `A` with the Philox2x32-7 stream of `cuTile.RNG(seed, counter)`; dist 0 = rand, 1 = randn, 2 = randexp."
function rng_fill(A, seed::UInt32, counter::UInt32, dist::Integer; stream::Ptr{Cvoid}=C_NULL)
    T = eltype(A)
    d = ref(descriptor(A; dtype = T === UInt8 ? Int32(8) : mi_dtype(T)))
    GC.@preserve A check(ccall((:mi_rng_fill, libmi355tile), Cint,
        (Ref{MiTileArray}, UInt32, UInt32, Cint, Ptr{Cvoid}), d, seed, counter, dist, stream))
    return A
end

end # module
