// Shared pieces of the fused-attention kernels: vector types, per-storage-type MFMA /
// conversion traits, array strides.
#pragma once
#include "common.h"
#include <math.h>

namespace mi {
namespace fmha {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define LDS_PTR(T, p) ((T __attribute__((address_space(3)))*)(p))

struct F16 {
    static __device__ __forceinline__ f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ short cvt(float v) {
        _Float16 h = (_Float16)v;
        return __builtin_bit_cast(short, h);
    }
    static __device__ __forceinline__ float to_f32(short v) { return (float)__builtin_bit_cast(_Float16, v); }
    // cvt(to_f32(q[e]) * s) for the eight elements of q: one mixed-precision fma per element (f16 source, fp32
    // product, rounded once into the low / high half of the result) instead of widen, multiply, narrow
    static __device__ __forceinline__ s16x8 scale8(s16x8 q, float s) {
        typedef unsigned u32x4_ __attribute__((ext_vector_type(4)));
        const u32x4_ in = __builtin_bit_cast(u32x4_, q);
        u32x4_ out;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            unsigned d;
            asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(d) : "v"(in[i]), "v"(s));
            asm("v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(d) : "v"(in[i]), "v"(s));
            out[i] = d;
        }
        return __builtin_bit_cast(s16x8, out);
    }
};
struct BF16 {
    static __device__ __forceinline__ f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ short cvt(float v) {
        unsigned u = __float_as_uint(v);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (short)((u >> 16) | 0x40);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (short)(u >> 16);
    }
    static __device__ __forceinline__ float to_f32(short v) { return __uint_as_float((unsigned)(unsigned short)v << 16); }
    static __device__ __forceinline__ s16x8 scale8(s16x8 q, float s) {
        s16x8 r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = cvt(to_f32(q[e]) * s);
        return r;
    }
};

struct Strides {
    int64_t s1, s2, s3;  // element strides of dims 1..3 (dim 0 is contiguous)
};

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

template <typename E> struct Pack;
template <> struct Pack<F16> {
    static __device__ __forceinline__ unsigned pack(float a, float b) {
        f16x2 v = {(_Float16)a, (_Float16)b};
        return __builtin_bit_cast(unsigned, v);
    }
    // acc + the eight weights of a 16-key chunk (four packed pairs), as rounded: the pairs are added up in f16
    // (three packed adds; the weights are at most 2^8, a sum of four stays far below the f16 range, and its
    // rounding is a quarter of an ulp of the largest weight), the two halves of the result go into the fp32 sum.
    static constexpr bool kChunkSum = true;
    static __device__ __forceinline__ float sum_chunk(const unsigned (&q)[4], float acc) {
        const f16x2 t = (__builtin_bit_cast(f16x2, q[0]) + __builtin_bit_cast(f16x2, q[1])) +
                        (__builtin_bit_cast(f16x2, q[2]) + __builtin_bit_cast(f16x2, q[3]));
        return sum2(__builtin_bit_cast(unsigned, t), 0.f, 0.f, acc);
    }
    // acc + the two weights of the packed pair pk, as rounded.  Two mixed-precision fma (f16 source, fp32
    // sum), not a dot2: the dot2 instructions run on the matrix pipe and wait for the MFMA in flight.
    static __device__ __forceinline__ float sum2(unsigned pk, float, float, float acc) {
        float r;
        asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(pk), "v"(acc));
        asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(r) : "v"(pk));
        return r;
    }
};
template <> struct Pack<BF16> {
    static __device__ __forceinline__ unsigned pack(float a, float b) {
        bf16x2 v = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(unsigned, v);
    }
    // acc + the two weights p0, p1 before rounding (there is no mixed-precision fma for bf16, and widening
    // the rounded pair would take two more instructions; dot2 is avoided for the reason above).
    static constexpr bool kChunkSum = false;
    static __device__ __forceinline__ float sum_chunk(const unsigned (&)[4], float acc) { return acc; }
    static __device__ __forceinline__ float sum2(unsigned, float p0, float p1, float acc) {
        return (acc + p0) + p1;
    }
};

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Software-pipelined kernel for head dimension 64 (fmha_pipe.hip).  `pipe_applicable` says
// whether the problem has the shape that kernel is written for; `pipe_launch` enqueues it.
struct Problem {
    const mi_tile_array *Q, *K, *V, *O;
    int H, group;     // query heads, query heads per KV head
    float scale2;     // qk_scale / ln 2
    int input_pos;
    bool causal, bf16;
};
bool pipe_applicable(const Problem& p);
void pipe_launch(const Problem& p, hipStream_t stream);

}  // namespace fmha
}  // namespace mi
