// Types, element traits and fragment helpers shared by the GEMM kernels.
#pragma once
#include "common.h"

namespace mi {
namespace gemm {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define LDS_PTR(T, p) ((T __attribute__((address_space(3)))*)(p))

// 16-bit element traits: raw storage is `short`; the MFMA picks the interpretation.
struct F16 {
    static __device__ __forceinline__ f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned short from_f32(float v) {
        _Float16 h = (_Float16)v;
        return __builtin_bit_cast(unsigned short, h);
    }
};
struct BF16 {
    static __device__ __forceinline__ f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned short from_f32(float v) {
        unsigned u = __float_as_uint(v);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (unsigned short)(u >> 16);
    }
};

template <typename E, typename OutT> __device__ __forceinline__ OutT cvt_out(float v);
template <> __device__ __forceinline__ float cvt_out<F16, float>(float v) { return v; }
template <> __device__ __forceinline__ float cvt_out<BF16, float>(float v) { return v; }
template <> __device__ __forceinline__ unsigned short cvt_out<F16, unsigned short>(float v) {
    return F16::from_f32(v);
}
template <> __device__ __forceinline__ unsigned short cvt_out<BF16, unsigned short>(float v) {
    return BF16::from_f32(v);
}

// Transposed LDS fragment read.  `base` points at element (row k0, column m0) of an LDS
// tile stored [k][m] with m contiguous and `pitch` elements per row.  The wave gets the
// MFMA column operand for columns m0..m0+31 and the 16 k rows k0..k0+15: lane l holds
// column m0 + l%32 and rows k0 + 8*(l/32) + 0..7.  Two ds_read_b64_tr_b16 per lane: within
// each group of 16 lanes, lane r reads 4 consecutive m of row (r/4) and receives the
// 4 consecutive rows of column (group base + r).
__device__ __forceinline__ s16x8 lds_read_tr_k16(const unsigned short* base, int pitch, int lane) {
    const int g = lane >> 4, r = lane & 15;
    const unsigned short* p = base + (8 * (g >> 1) + (r >> 2)) * pitch + 16 * (g & 1) + 4 * (r & 3);
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 4 * pitch));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}


// Problem description handed from the entry points to the kernel launchers.
struct Problem {
    const void *A, *B;
    void* C;
    int64_t lda, ldb, ldc, sa, sb, sc;
    int M, N, K, batch;
    int in_dtype, out_dtype;
};

// gemm_big.hip: true if the 256x256 direct-to-LDS kernel applies to the problem / launches it.
bool big16_applicable(const Problem& p);
void big16_launch(const Problem& p, hipStream_t s);
// gemm32_big.hip: the same for fp32 operands.
bool big32_applicable(const Problem& p);
void big32_launch(const Problem& p, hipStream_t s);
int64_t big32_cost(const Problem& p);   // its tile choice's estimate, 16 = the 4096^3 product per 4096 of K
// gemm8.hip: fp8 (E4M3FN / E5M2) operands; picks its kernel itself.
void fp8_launch(const Problem& p, hipStream_t s);

}  // namespace gemm
}  // namespace mi
