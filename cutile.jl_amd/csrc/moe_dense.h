// Interface between the MoE entry points (moe.hip) and the grouped GEMM for dense routing (moe_dense.hip).
#pragma once
#include <math.h>

#include "common.h"

namespace mi {
namespace moe {

// One launch of fused_moe_kernel (examples/moe.jl:45-105) as the entry points have validated it.
struct DenseArgs {
    const void* A;                 // activations (K, columns), K contiguous: 16-bit, or E4M3FN bytes when a8
    int64_t lda;
    int num_a_cols;
    const void* B;                 // expert weights (K, N, E), K contiguous: 16-bit, or E4M3FN bytes when w8
    int64_t ldb, sbe;
    unsigned short* C;             // (N, total) / (N/2, total) with the SiLU epilogue / (N, tokens) when accumulating
    int64_t ldc;
    int total_tokens;
    const unsigned short* topk_weights;
    int w_topk;
    int64_t w_s0, w_s1;
    const int* sorted_token_ids;
    int num_slots;
    const int* sorted_expert_ids;
    int num_blocks;                // entries of sorted_expert_ids in use: cld(num_slots, TILE_M)
    const float* b_scale;          // (N, E) fp32 scales of e4m3 weights, or null
    int64_t ld_scale;
    int K, N, num_experts, replicas;
    bool mul_routed_weight;
    int TILE_M;
    int acc_shift;                 // >= 0: accumulate into column (token - 1) >> acc_shift with packed atomic adds
    bool bf16, silu, w8;           // bf16: C (and the routed weights) are bfloat16, else float16
    bool a8;                       // activations are E4M3FN as well: fp8 x fp8 MFMA, every channel times its b_scale entry
};

#ifdef __HIPCC__
// SiLU(x) * y in fp32 as moe.jl:117-124 computes it: the hardware's exponential (2^(-x log2 e), one multiply and one
// transcendental instruction; the reference's kernel is compiled with flush_to_zero and its exp is the device's
// approximate one as well) and the approximate reciprocal.  The barrier keeps the
// fp32 product a value of its own: without it the compiler may fold the final multiply into the
// conversion to f16 (one rounding instead of two) in one kernel and not in another, and the fused
// and the separate path would differ in the last bit now and then.
__device__ __forceinline__ float silu_mul(float x, float y) {
    const float denom = 1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
    float p = x * __builtin_amdgcn_rcpf(denom) * y;
    asm volatile("" : "+v"(p));
    return p;
}

// *p += the two 16-bit floats packed in `pair` (one memory-side atomic; round to nearest even, denormals kept)
__device__ __forceinline__ void atomic_add2(bool bf16, unsigned short* p, unsigned pair) {
    if (bf16) {
        typedef short s2 __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_global_atomic_fadd_v2bf16((s2 __attribute__((address_space(1)))*)p, __builtin_bit_cast(s2, pair));
    } else {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_global_atomic_fadd_v2f16((h2 __attribute__((address_space(1)))*)p, __builtin_bit_cast(h2, pair));
    }
}
#endif

// True if the launch can run on the 128-slot ring kernel (TILE_M a multiple of 128, 16-byte aligned rows, K a multiple
// of 8 and at least 256 -- of 16 and at least 512 for fp8 activations) and routing is dense enough for it to pay.
// 16-bit activations with e4m3 weights are not its case (the streaming kernels widen those); fp8 activations run
// nowhere else.
bool dense_applicable(const DenseArgs& a);
// Launches it and records the variant name.
void dense_launch(const DenseArgs& a, hipStream_t s);

}  // namespace moe
}  // namespace mi
