/*
 * mi355tile.h — C ABI of libmi355tile.so
 *
 * Hand-written HIP kernels for AMD Instinct MI355X (gfx950 / CDNA4) that stand in for
 * the kernels cuTile.jl's examples compile through NVIDIA Tile IR.  There is exactly one
 * entry point per example kernel.  Each takes the example kernel's arguments in the
 * example's own order:
 *
 *   - every `ct.TileArray{T,N}` argument becomes a `const mi_tile_array*`, a plain-data
 *     mirror of the reference's array descriptor (pointer, sizes, strides in ELEMENTS,
 *     first dimension fastest — Julia column-major; reference: src/language/types.jl:283-287,
 *     flattened for launch at src/launch.jl:750-777);
 *   - scalar arguments stay scalars;
 *   - the `ct.Constant(...)` tile-size arguments become plain `int`s;
 *   - a trailing `void* stream` is the hipStream_t to enqueue on (NULL = default stream).
 *     The reference enqueues on the task-local CUDA stream (src/launch.jl:862).
 *
 * The grid is derived inside the library from sizes + tile constants with the formulas
 * the examples use (`cld(M,tm)*cld(N,tn)` …).  Tile constants are semantic parameters
 * (block → data mapping, padding contracts, accumulation grouping); the physical
 * wave / LDS tiling is chosen by the library for CDNA4.
 *
 * Every call is asynchronous, allocates nothing and never throws (the mi_tiled_* entry points
 * compile and load a code object the first time they meet a new expression, see below).  Return value: 0 on
 * success, a negative MI_E_* code for argument errors detected on the host, or a
 * positive hipError_t reported by the launch.  The caller owns all buffers.
 */
#ifndef MI355TILE_H
#define MI355TILE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355TILE_VERSION 100 /* major*10000 + minor*100 + patch */

/* Element types of a mi_tile_array. */
typedef enum mi_dtype {
    MI_F32 = 0,
    MI_F64 = 1,
    MI_F16 = 2,
    MI_BF16 = 3,
    MI_F8E4M3FN = 4, /* OCP FP8 E4M3 "FN": bias 7, no Inf, NaN = S.1111.111, max 448
                        (reference: ext/DLFP8TypesExt.jl:7-9) */
    MI_I32 = 5,
    MI_I64 = 6,
    MI_BOOL = 7,     /* Julia Bool: one byte holding 0 or 1 (Tiled broadcast / mapreduce only) */
    MI_I8 = 8,       /* Int8 / UInt8 and */
    MI_I16 = 9,      /* Int16 / UInt16: RNG fills only (unsigned types share the codes of the signed ones) */
    MI_F8E5M2 = 10   /* OCP FP8 E5M2: bias 15, Inf and NaN as in IEEE (reference: ext/DLFP8TypesExt.jl:11-13);
                        matmul operands only */
} mi_dtype;

/* Error codes (negative).  Positive return values are hipError_t. */
enum {
    MI_OK = 0,
    MI_E_NULL = -1,      /* a required pointer is NULL */
    MI_E_DTYPE = -2,     /* unsupported or mismatching element type */
    MI_E_RANK = -3,      /* wrong number of dimensions */
    MI_E_SHAPE = -4,     /* sizes of the arguments do not agree */
    MI_E_STRIDE = -5,    /* layout not supported (fastest dimension must have stride 1) */
    MI_E_TILE = -6,      /* tile constant not a positive power of two, or unsupported */
    MI_E_GRID = -7,      /* a grid dimension exceeds 2^24-1 (reference: src/launch.jl:743,801-807) */
    MI_E_ALIGN = -8,     /* pointer not aligned to its element size */
    MI_E_ARG = -9,       /* other invalid scalar argument */
    MI_E_UNSUPPORTED = -10,
    MI_E_SCRATCH = -11   /* the problem needs more scratch memory than the library's static buffer holds */
};

#define MI_MAX_RANK 4

/* Mirror of cuTile's TileArray{T,N} (src/language/types.jl:283-287): a device pointer with
 * per-dimension sizes and element strides, dimension 0 here = Julia dimension 1. */
typedef struct mi_tile_array {
    void* ptr;
    int32_t dtype; /* mi_dtype */
    int32_t ndim;
    int64_t sizes[MI_MAX_RANK];
    int64_t strides[MI_MAX_RANK];
} mi_tile_array;

/* ---- library ---------------------------------------------------------------------- */
int mi_version(void);
const char* mi_strerror(int code);
/* Name of the kernel variant chosen by the most recent successful launch on this thread
 * (for profiles and tests; never NULL). */
const char* mi_last_variant(void);
/* Some entry points keep partial results in static device arrays of the library that the streams of a GPU share
 * (the GEMMs split over K, attention split over the keys, the token sort of several workgroups).  Eager launches
 * that use them from different streams are ordered by the library; a launch recorded into a graph can not be (it
 * runs later, as often as the graph is replayed), so by default a capturing stream is not given the arrays and
 * those entry points record their one-piece kernels.  allow != 0 hands the arrays to capturing streams as well: the
 * caller then sees to it that replays of such graphs overlap neither one another nor any other launch of these entry
 * points on the device (the usual serving loop, one graph at a time on one stream, does).  The array in question
 * must have been used by one eager call before (its address is not looked up inside a capture).  Returns the
 * previous setting; process-wide; also set by MI_SCRATCH_UNDER_CAPTURE=1 in the environment.  No counterpart in the
 * reference (its launches own their temporaries). */
int mi_scratch_under_capture(int allow);

/* ---- vadd: examples/vadd.jl ------------------------------------------------------- */
/* vec_add_kernel_1d (vadd.jl:10-17): c = a + b; block `bid` owns elements
 * (bid-1)*tile+1 … bid*tile.  f32 / f64 / f16 / bf16, Int32 / Int64 (wrapping, as Julia's +). */
int mi_vec_add_kernel_1d(const mi_tile_array* a, const mi_tile_array* b, const mi_tile_array* c,
                         int tile, void* stream);
/* vec_add_kernel_2d (vadd.jl:20-28): same on (tile_x, tile_y) tiles of 2-D arrays. */
int mi_vec_add_kernel_2d(const mi_tile_array* a, const mi_tile_array* b, const mi_tile_array* c,
                         int tile_x, int tile_y, void* stream);
/* vec_add_kernel_1d_gather (vadd.jl:31-45): same through per-element indexed gather/scatter;
 * lanes whose index is out of bounds read 0 and their store is dropped
 * (src/language/operations.jl:996-1009,1072-1085). */
int mi_vec_add_kernel_1d_gather(const mi_tile_array* a, const mi_tile_array* b,
                                const mi_tile_array* c, int tile, void* stream);

/* ---- transpose: examples/transpose.jl --------------------------------------------- */
/* transpose_kernel (transpose.jl:11-19): y[j,i] = x[i,j]; x is (m,n), y is (n,m). */
int mi_transpose_kernel(const mi_tile_array* x, const mi_tile_array* y, int tm, int tn,
                        void* stream);

/* ---- matmul: examples/matmul.jl, examples/batchmatmul.jl --------------------------- */
/* matmul_kernel (matmul.jl:28-60): C(M,N) = A(M,K)·B(K,N), fp32 accumulate, 1-D grid of
 * cld(M,tm)*cld(N,tn) blocks ordered by swizzle_2d with GROUP_SIZE_M = 8, ragged edges
 * zero-padded on load and clipped on store.  A,B: f16 / bf16 / f32; C: the input type or
 * f32.  f32 inputs are multiplied in true fp32 (gfx950 has no TF32-class MFMA; the
 * reference rounds f32 operands to TF32 at matmul.jl:49-52).  A,B both MI_F8E4M3FN or both
 * MI_F8E5M2 (the reference's fp8 mma operands, ext/DLFP8TypesExt.jl:15-19; lhs and rhs must share
 * the type, src/compiler/intrinsics/core.jl:589-604): multiplied on the fp8 matrix cores with fp32
 * accumulation, C f32, f16 or bf16. */
int mi_matmul_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                     int tm, int tn, int tk, void* stream);
/* batch_matmul_kernel (batchmatmul.jl:15-56): C(M,N,b) = A(M,K,b)·B(K,N,b), grid
 * (cld(M,tm), cld(N,tn), Batch). */
int mi_batch_matmul_kernel(const mi_tile_array* A, const mi_tile_array* B,
                           const mi_tile_array* C, int tm, int tn, int tk, void* stream);
/* swizzle_2d (matmul.jl:13-24, moe.jl:20-31), host helper: 1-based block id →
 * 1-based (bid_m, bid_n). */
void mi_swizzle_2d(int32_t M, int32_t N, int32_t tm, int32_t tn, int32_t group_size_m,
                   int32_t bid, int32_t* bid_m, int32_t* bid_n);

/* ---- layernorm: examples/layernorm.jl ---------------------------------------------- */
/* layer_norm_fwd (layernorm.jl:27-68).  X,Y (N,M) f32 with N contiguous; W,B (N,);
 * Mean,Rstd (M,).  Two-pass mean / biased variance, rstd = 1/sqrt(var+eps). */
int mi_layer_norm_fwd(const mi_tile_array* X, const mi_tile_array* W, const mi_tile_array* B,
                      const mi_tile_array* Y, const mi_tile_array* Mean,
                      const mi_tile_array* Rstd, float eps, int TILE_N, void* stream);
/* layer_norm_bwd_dx_partial_dwdb (layernorm.jl:118-171).  Writes DX and ADDS partial
 * dW/dB into the GROUP_SIZE_M slots of DW,DB (N, GROUP_SIZE_M), which the caller has
 * zero-filled (layernorm.jl:245-247); row m contributes to slot m mod GROUP_SIZE_M.
 * `Locks` (GROUP_SIZE_M,) i64 is accepted for signature compatibility and not touched:
 * accumulation uses per-workgroup register partials plus device-scope float atomics
 * instead of the reference's CAS spin-lock.  May be NULL. */
int mi_layer_norm_bwd_dx_partial_dwdb(const mi_tile_array* DX, const mi_tile_array* DY,
                                      const mi_tile_array* DW, const mi_tile_array* DB,
                                      const mi_tile_array* X, const mi_tile_array* W,
                                      const mi_tile_array* Mean, const mi_tile_array* Rstd,
                                      const mi_tile_array* Locks, int GROUP_SIZE_M, int TILE_N,
                                      void* stream);
/* layer_norm_bwd_dwdb (layernorm.jl:186-205): FINAL_DW[n] = sum_g DW[n,g], same for DB. */
int mi_layer_norm_bwd_dwdb(const mi_tile_array* DW, const mi_tile_array* DB,
                           const mi_tile_array* FINAL_DW, const mi_tile_array* FINAL_DB,
                           int TILE_M, int TILE_N, void* stream);

/* Whole backward in one call that allocates nothing.  No counterpart in the reference, whose host
 * code allocates the partial buffers itself (layernorm.jl:226-228); for callers that can not
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same result as zero-filling DW / DB (N, GROUP_SIZE_M), mi_layer_norm_bwd_dx_partial_dwdb and
 * mi_layer_norm_bwd_dwdb, with the partial slots held in a file-scope device array of the library
 * (4 MiB per GPU, kept until the process ends; the call's last kernel leaves it zeroed for the
 * next call, so a call is two launches).  Limit: cld(N,4)*4 * GROUP_SIZE_M <= 524288 floats
 * (N = 8192 with 64 slots), MI_E_SCRATCH beyond.  Every call on a GPU uses that GPU's one array:
 * calls that overlap on one GPU (different streams or threads) race.  The array's device address
 * is looked up once per GPU, outside any stream capture: by the first eager call of this or of
 * any other mi_layer_norm_* entry point on that GPU.  A call on a capturing stream before that
 * returns MI_E_UNSUPPORTED (make one eager LayerNorm call first, then capture). */
int mi_layer_norm_bwd_static(const mi_tile_array* DX, const mi_tile_array* DY, const mi_tile_array* X,
                             const mi_tile_array* W, const mi_tile_array* Mean,
                             const mi_tile_array* Rstd, const mi_tile_array* FINAL_DW,
                             const mi_tile_array* FINAL_DB, int GROUP_SIZE_M, int TILE_M, int TILE_N,
                             void* stream);

/* ---- softmax: examples/softmax.jl -------------------------------------------------- */
/* softmax_tma_kernel (softmax.jl:18-42): column softmax of input (N,M), one tile of
 * TILE_SIZE rows per column (rows beyond TILE_SIZE are neither read nor written, as in
 * the reference).  `num_programs` is the reference's launch grid (`blocks=M` at
 * softmax.jl:136); any value >= 1 gives the same result. f32 / f16 / bf16 storage. */
int mi_softmax_tma_kernel(const mi_tile_array* output, const mi_tile_array* input,
                          int TILE_SIZE, int num_programs, void* stream);
/* softmax_chunked_kernel (softmax.jl:48-100): softmax over the rows that the reference's chunk
 * loop visits, 1 .. cld(n_elems, TILE_SIZE)*TILE_SIZE.  Same function of the column as the
 * reference's three chunked passes; columns that fit in registers are read once. */
int mi_softmax_chunked_kernel(const mi_tile_array* output, const mi_tile_array* input,
                              int n_elems, int TILE_SIZE, int num_programs, void* stream);

/* ---- FMHA: examples/fmha.jl --------------------------------------------------------- */
/* fmha_kernel (fmha.jl:20-139).  Q (D,Sq,H,B), K (D,Skv,KVH,B), V (Dv,Skv,KVH,B),
 * Out (Dv,Sq,H,B), f16 or bf16; online softmax in the exp2 domain with fp32 accumulation,
 * P rounded to the storage type before P·V, causal tile skipping, GQA via
 * QUERY_GROUP_SIZE, decode offset input_pos, ragged KV tail when !EVEN_K.
 * Few queries against many keys (decode, chunked prefill: fewer than 1024 workgroups of 128 queries) are split over
 * the keys: the parts go through a 64 MiB static device array of the library and a second kernel adds them.  Launches
 * that use the array from different streams are ordered by an event; a stream under capture runs unsplit.  With
 * grouped heads and at most 64 queries the heads of a group share a query tile, so their keys are read once. */
int mi_fmha_kernel(const mi_tile_array* Q, const mi_tile_array* K, const mi_tile_array* V,
                   const mi_tile_array* Out, float qk_scale, int32_t input_pos, int TILE_D,
                   int H, int TILE_M, int TILE_N, int QUERY_GROUP_SIZE, int CAUSAL, int EVEN_K,
                   void* stream);

/* ---- MoE: examples/moe.jl ------------------------------------------------------------ */
/* moe_align_tile_size (moe.jl:142-183), HOST routine on host memory.  topk_ids is the
 * Julia (num_tokens, topk) Int64 matrix of 1-based expert ids in column-major order.
 * sorted_token_ids_out needs capacity for tile_m * sum_e cld(count_e, tile_m) entries
 * (never more than num_tokens*topk + num_experts*(tile_m-1)); sorted_expert_ids_out one
 * entry per block.  Passing NULL outputs only counts.  Returns 0 or MI_E_*. */
int mi_moe_align_tile_size(const int64_t* topk_ids, int64_t num_tokens, int64_t topk, int tile_m,
                           int num_experts, int32_t* sorted_token_ids_out,
                           int32_t* sorted_expert_ids_out, int64_t* total_blocks_out);
/* Device counterpart of moe_align_tile_size: the same stable counting sort on `stream` (one launch of one
 * workgroup below 8192 replicas; from there on, two launches of up to 64 workgroups whose per-expert counts meet in a static
 * array of the library -- a stream under graph capture is not given that array and sorts with one workgroup),
 * so that cutile_moe needs no host round trip (the reference copies topk_ids to the
 * host, sorts there and copies the result back: moe.jl:232-233).  topk_ids (num_tokens, topk)
 * i64 on the device.  The outputs have fixed capacity, since the block count is only known on
 * the device: sorted_expert_ids needs at least
 * cld(total + min(total, num_experts)*(tile_m-1), tile_m) entries and sorted_token_ids
 * tile_m times as many; unused slots get the sentinel total+1 and unused blocks expert 0, which
 * mi_fused_moe_kernel skips.  Expert ids outside 1..num_experts are dropped (the host routine
 * reports MI_E_ARG for them).  At most 1024 experts and 2^22 replicas. */
int mi_moe_align_tile_size_device(const mi_tile_array* topk_ids, int tile_m, int num_experts,
                                  const mi_tile_array* sorted_token_ids,
                                  const mi_tile_array* sorted_expert_ids, void* stream);
/* The same, and `clear` (a dense device array of whole 16-byte units, any rank and element type) is filled with zeros
 * by the same launch: the output that mi_fused_moe_accumulate_kernel adds into, without a fill launch of its own.
 * No counterpart in the reference (its caches come from CUDA.zeros, moe.jl:228-230). */
int mi_moe_align_tile_size_device_clear(const mi_tile_array* topk_ids, int tile_m, int num_experts,
                                        const mi_tile_array* sorted_token_ids,
                                        const mi_tile_array* sorted_expert_ids, const mi_tile_array* clear,
                                        void* stream);
/* Router on the device: topk_ids[t, :] = the topk = size(topk_ids, 2) experts with the largest
 * logits[t, :] in descending order (ties to the lower expert id, NaN ranks as -Inf), 1-based;
 * topk_weights[t, :] = softmax over those topk logits.  logits (num_tokens, num_experts) f32 / f16 /
 * bf16 with any strides, topk_weights (num_tokens, topk) f32 / f16 / bf16, topk_ids (num_tokens,
 * topk) i64: the inputs cutile_moe takes (moe.jl:218-222).  No counterpart in the reference, whose
 * example draws its routing on the host (moe.jl:323-333); with mi_moe_align_tile_size_device the
 * routed forward pass needs no host step at all.  At most 512 experts, topk <= 64. */
int mi_moe_route_topk(const mi_tile_array* logits, const mi_tile_array* topk_weights,
                      const mi_tile_array* topk_ids, void* stream);
/* fused_moe_kernel (moe.jl:45-105).  A (K,num_tokens), B (K,N,E), C (N,total_tokens),
 * topk_weights (total_tokens,) -- the slot-fastest flattening `vec(permutedims(topk_weights))` of moe.jl:193 -- or
 * the (num_tokens, topk) matrix itself with any strides (the kernel then looks element (token, slot) up directly
 * and the caller saves the permuting copy), sorted_token_ids (M_padded,) i32 1-based with sentinel
 * total_tokens+1, sorted_expert_ids (blocks,) i32 1-based.  A, C, topk_weights f16/bf16.
 * B is f16/bf16, or MI_F8E4M3FN with `b_scale` (N,E) f32 per-output-channel scales
 * (fp8 weights are an extension of this build; b_scale must be NULL otherwise).
 * With fp8 weights A may be MI_F8E4M3FN as well (C and topk_weights stay 16-bit): the products are then formed
 * by the fp8 matrix instruction, fp8 x fp8 with fp32 accumulation -- the operand pairing ext/DLFP8TypesExt.jl:15-19
 * gives `mma` -- and every output channel is multiplied by its b_scale entry (fold an activation scale into it).
 * This form runs on the 128-slot grouped GEMM only: TILE_M a multiple of 128, K a multiple of 16 and at least 512,
 * rows of A and B on 16-byte boundaries; MI_E_UNSUPPORTED otherwise.  The same holds for the two variants below. */
int mi_fused_moe_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                        const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                        const mi_tile_array* sorted_expert_ids, int num_token_replicas,
                        int mul_routed_weight, int TILE_M, int TILE_N, int TILE_K,
                        const mi_tile_array* b_scale, void* stream);
/* The second grouped GEMM of cutile_moe (moe.jl:245-251: mul_routed_weight = true, num_token_replicas = 1) fused
 * with the sum over the top-k slots (moe.jl:256): Out (N, num_tokens), zeroed by the caller, receives every replica's
 * weighted row -- rounded to the activation type first, as cache3 would hold it -- by memory-side packed atomic adds
 * of two adjacent channels (round to nearest even, denormals kept).  topk_weights must be the (num_tokens, topk)
 * matrix with topk = 1 or 2: two terms add up the same in either order, so the result is the one mi_fused_moe_kernel +
 * mi_moe_sum_topk give, bit for bit, and is the same from run to run; MI_E_UNSUPPORTED for more slots.  N even, Out
 * 4-byte aligned with an even column stride (MI_E_ALIGN).  A (K, num_tokens * topk), B, sorted_*, b_scale as for
 * mi_fused_moe_kernel. */
int mi_fused_moe_accumulate_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* Out,
                                   const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                                   const mi_tile_array* sorted_expert_ids, int TILE_M, int TILE_N, int TILE_K,
                                   const mi_tile_array* b_scale, void* stream);
/* The first grouped GEMM of cutile_moe fused with silu_and_mul_kernel (moe.jl:234-251 launch them
 * one after the other through cache1): B holds the gate rows [0, N/2) and the up rows [N/2, N) of
 * every expert, C is (N/2, total_tokens) and receives SiLU(gate) * up.  Both products are rounded
 * to the activation type before the activation, so the result is bit-identical to
 * mi_fused_moe_kernel + mi_silu_and_mul_kernel whenever that GEMM runs the same wide mainloop
 * (it does at the benchmark shape; small problems use a K-split whose fp32 sums are ordered
 * differently); cache1 is never written.  No counterpart in the
 * reference, whose host code launches the two kernels separately; same arguments and checks
 * otherwise. */
int mi_fused_moe_silu_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                             const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                             const mi_tile_array* sorted_expert_ids, int num_token_replicas,
                             int mul_routed_weight, int TILE_M, int TILE_N, int TILE_K,
                             const mi_tile_array* b_scale, void* stream);
/* silu_and_mul_kernel (moe.jl:110-128): C[:,t] = silu(A[:,t]) * B[:,t] in fp32. */
int mi_silu_and_mul_kernel(const mi_tile_array* A, const mi_tile_array* B,
                           const mi_tile_array* C, int TILE_N, void* stream);
/* The top-k combine `sum(cache3; dims=2)` of cutile_moe (moe.jl:256), which the reference
 * hands to CUDA.jl: out (H, tokens) = sum over dim 2 of in (H, topk, tokens), fp32
 * accumulation in slot order. */
int mi_moe_sum_topk(const mi_tile_array* in, const mi_tile_array* out, void* stream);
/* Producer of fp8 activations for the grouped GEMMs above (A of type MI_F8E4M3FN together with fp8 weights: fp8 x fp8
 * on the matrix cores, the operand pairing of ext/DLFP8TypesExt.jl:15-19; the reference leaves making fp8 operands to
 * its caller, so this has no counterpart there).  x (K, columns) f16/bf16 -> codes (K, columns) E4M3FN with one scale
 * for the whole array: scale[0] = max |x| / 448 (1 if x is all zero), codes = round-to-nearest-even of x / scale.
 * `workspace`: at least 1024 floats of the caller's (partial maxima; nothing to clear).  K a multiple of 8, columns on
 * 16-byte (x) and 8-byte (codes) boundaries.  Two launches. */
int mi_quantize_e4m3fn(const mi_tile_array* x, const mi_tile_array* codes, const mi_tile_array* scale,
                       const mi_tile_array* workspace, void* stream);
/* The same, and fold_out = fold_in * scale element by element (dense fp32 arrays of one shape, e.g. the (N, E) scales
 * of the e4m3 weights that these activations meet: the product is what mi_fused_moe_kernel wants as b_scale with fp8
 * activations, and the second launch writes it on the way).  No counterpart in the reference. */
int mi_quantize_e4m3fn_fold(const mi_tile_array* x, const mi_tile_array* codes, const mi_tile_array* scale,
                            const mi_tile_array* workspace, const mi_tile_array* fold_in,
                            const mi_tile_array* fold_out, void* stream);

/* ---- FFT: examples/fft.jl ------------------------------------------------------------- */
/* fft_kernel (fft.jl:22-126): batched complex FFT of N = F0*F1*F2 points as three stages of small
 * DFTs.  x_packed_in, y_packed_out (D, 2N/D, batch) f32: the interleaved (re, im) signals, dense;
 * W0 (2,F0,F0), W1 (2,F1,F1), W2 (2,F2,F2): DFT matrices, T0 (2,F1*F2,F0), T1 (2,F2,F1): twiddles
 * (fft.jl:130-180), all f32 with the (re, im) pair leading.  One workgroup per signal; BS (signals
 * per block of the reference's launch) only has to divide the batch.  N <= 4096; the radix triples
 * compiled in are listed in fft.hip (MI_E_UNSUPPORTED otherwise). */
int mi_fft_kernel(const mi_tile_array* x_packed_in, const mi_tile_array* y_packed_out,
                  const mi_tile_array* W0, const mi_tile_array* W1, const mi_tile_array* W2,
                  const mi_tile_array* T0, const mi_tile_array* T1, int N, int F0, int F1, int F2,
                  int BS, int D, void* stream);

/* ---- Host-level Tiled broadcast and mapreduce ---------------------------------------------------
 * The reference specialises and compiles a kernel per broadcast tree / reduction on first use
 * (src/broadcast.jl:75-129, src/mapreduce.jl:13-129) and caches it (src/launch.jl:663-687).  These
 * entry points do the same through hiprtc: the first call with a new (expression, element types,
 * layout class) generates a fused gfx950 kernel, compiles, loads and caches it (tens of
 * milliseconds, allocates the code object); every later call only launches.  Arrays have 0 to 4
 * dimensions and any element strides; element types f32 f64 f16 bf16 i32 i64 bool.
 *
 * Expressions are text in prefix form:  expr := name(expr{,expr}) | a<i> | s<i>, with a<i> the
 * i-th array leaf and s<i> the i-th scalar; `name` is one of
 *   add sub mul div pow neg abs abs2 sign max min fma muladd clamp copysign floor ceil round trunc
 *   sqrt cbrt inv exp exp2 exp10 expm1 log log2 log10 log1p sin cos tan asin acos atan sinh cosh
 *   tanh atan2 hypot lt le gt ge eq ne isnan isinf isfinite signbit iszero not and or xor ifelse
 *   div_int rem mod fld cld identity f16 bf16 f32 f64 i32 i64 bool rsqrt shl shr lshr mul_hi
 * (Julia's `+` is add, `/` is div, `^` is pow, `÷` is div_int, `Float32(x)` is f32, `<<` `>>` `>>>`
 * are shl shr lshr, ct.rsqrt of src/language/math.jl:16 is rsqrt, ...).  Node
 * types follow Julia's promote_type / float() rules; Float16 and BFloat16 operations are rounded
 * after every step as Julia defines them.  Unknown names return MI_E_UNSUPPORTED. */
typedef struct mi_tile_scalar {
    int32_t dtype;      /* mi_dtype of the Julia number */
    int32_t reserved;
    union {
        double f;       /* value of a float type */
        int64_t i;      /* value of an integer type or Bool */
    } value;
} mi_tile_scalar;

/* dest .= expr(leaves..., scalars...)   (reference: Base.Broadcast.materialize!(::Tiled, bc),
 * src/broadcast.jl:20-24,75-92).  A leaf dimension must equal dest's or be 1 (it then expands);
 * leaves of lower rank expand along the trailing dimensions; MI_E_SHAPE otherwise (the reference
 * throws DimensionMismatch).  The tree's value is converted to dest's element type.  An empty
 * dest launches nothing.  At most 8 leaves, 8 scalars, 128 nodes. */
int mi_tiled_broadcast(const mi_tile_array* dest, const char* expr, const mi_tile_array* const* leaves,
                       int n_leaves, const mi_tile_scalar* scalars, int n_scalars, void* stream);

/* Element type of a tree: Base.Broadcast.combine_eltypes as used by the allocating form
 * (src/broadcast.jl:26-32). */
int mi_tiled_broadcast_eltype(const char* expr, const int32_t* leaf_dtypes, int n_leaves,
                              const int32_t* scalar_dtypes, int n_scalars, int32_t* out_dtype);

/* Reduction operators (src/mapreduce.jl:5-11 lists the reference's). */
enum { MI_OP_ADD = 0, MI_OP_MUL = 1, MI_OP_MAX = 2, MI_OP_MIN = 3, MI_OP_AND = 4, MI_OP_OR = 5 };

/* dest = reduce(op, f.(src)) over the dimensions in which dest has extent 1 and src has not
 * (reference: `_mapreducedim!`, src/mapreduce.jl:66-129, dimension rule of :188-196).  `f_expr`
 * is an expression in a0 (= one element of src) and the scalars, NULL for identity; its value is
 * converted to dest's element type, which is also the accumulator type.  The accumulator starts
 * from op's neutral element (0, 1, typemin, typemax, all-ones, 0); a caller's `init` is applied
 * afterwards as the reference does (src/mapreduce.jl:157-163).  With no reduced dimension this is
 * map.  Reductions with few outputs run in two passes through `workspace` (device memory, 16-byte
 * aligned, at least mi_tiled_mapreduce_workspace() bytes; may be NULL when that is 0); float
 * results are reproducible from run to run.  max / min propagate NaN as Julia does. */
int mi_tiled_mapreduce(const mi_tile_array* dest, const mi_tile_array* src, const char* f_expr,
                       const mi_tile_scalar* scalars, int n_scalars, int op, void* workspace,
                       int64_t workspace_bytes, void* stream);
int mi_tiled_mapreduce_workspace(const mi_tile_array* dest, const mi_tile_array* src, int op, int64_t* bytes);

/* Element type of the result: promote_op(op, T, T) of T = typeof(f(x)) (src/mapreduce.jl:133-137).
 * `widen` != 0 selects Base's add_sum / mul_prod, which widen Int32 and Bool to Int64 (what
 * `sum` / `prod` pass); 0 is plain `+` / `*` as `reduce(+, ...)` passes. */
int mi_tiled_mapreduce_eltype(const char* f_expr, int32_t src_dtype, const int32_t* scalar_dtypes,
                              int n_scalars, int op, int widen, int32_t* out_dtype);

/* ---- Host-level RNG fills -----------------------------------------------------------------------
 * Random.rand!(rng, A) / randn! / randexp! for rng = cuTile.RNG(seed, counter)
 * (reference: src/language/random.jl:759-818 launching the fill kernels of :703-740).  Writes the
 * reference's Philox2x32-7 stream value for value: block b of 512 outputs is keyed with
 * (b * 0x9E3779B9) ^ seed and uses the counters counter + i.  `out` is any dense array, filled in
 * linear order.  dist: 0 = rand (every element type: integers take the raw bits, floats lie in
 * (0, 1]), 1 = randn, 2 = randexp (float types only, MI_E_DTYPE otherwise).  Integer results are
 * bit-exact; randn / randexp go through this library's log / sin / cos. */
int mi_rng_fill(const mi_tile_array* out, uint32_t seed, uint32_t counter, int dist, void* stream);

/* advance_counter! after a fill of n_elements (src/language/random.jl:694-699,776-779): the counter
 * moves by whole blocks of 512 and a wrap increments the seed. */
int mi_rng_advance_counter(uint32_t* seed, uint32_t* counter, int64_t n_elements);

/* Test hooks.  mi_tiled_set_dry_run(1) makes the two entry points stop after compiling (nothing is
 * loaded or launched, no GPU is needed); returns the previous setting.  mi_tiled_compile_count()
 * is the number of kernels compiled so far in this process. */
int mi_tiled_set_dry_run(int on);
int mi_tiled_compile_count(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355TILE_H */
