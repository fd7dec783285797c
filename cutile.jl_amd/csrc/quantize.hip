// Per-tensor E4M3FN quantisation of 16-bit activations, for the fp8 x fp8 form of the MoE's grouped GEMMs (the
// operand pairing ext/DLFP8TypesExt.jl:15-19 gives `mma`; the reference leaves producing fp8 operands to its caller).
//   scale = max |x| / 448 (1 for an all-zero tensor), codes = round-to-nearest-even E4M3FN of x / scale.
// Two launches, no atomics and nothing to clear: the first leaves one partial maximum per workgroup in the caller's
// workspace, the second has every workgroup reduce those (at most 1024 floats) before it converts its share.
#include "common.h"

namespace {

using namespace mi;

typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kQThreads = 256, kQMaxGroups = 1024;

template <bool BF16>
__device__ __forceinline__ float widen(unsigned short h) {
    return BF16 ? __uint_as_float(((unsigned)h) << 16) : (float)__builtin_bit_cast(_Float16, h);
}

// x: rows of `n` elements at stride `ld`; 8 elements per lane and step (whole 16-byte pieces: checked on the host).
template <bool BF16>
__global__ __launch_bounds__(kQThreads) void absmax_kernel(const unsigned short* __restrict__ x, int64_t ld, int64_t n,
                                                           int64_t rows, float* __restrict__ partial) {
    __shared__ float red[kQThreads / 64];
    const int64_t vec_per_row = n / 8, total = vec_per_row * rows;
    float m = 0.f;
    for (int64_t i = (int64_t)blockIdx.x * kQThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kQThreads) {
        const int64_t r = i / vec_per_row, c = i - r * vec_per_row;
        const u16x8 v = *reinterpret_cast<const u16x8*>(x + r * ld + 8 * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(widen<BF16>(v[e])));   // (fmaxf drops a NaN operand: NaNs do not set the scale)
    }
    m = block_reduce<kQThreads / 64>(m, red, MaxOp{}, 0.f);
    if (threadIdx.x == 0) partial[blockIdx.x] = m;
}

template <bool BF16>
__global__ __launch_bounds__(kQThreads) void quantize_kernel(const unsigned short* __restrict__ x, int64_t ld, int64_t n,
                                                             int64_t rows, unsigned char* __restrict__ q, int64_t ldq,
                                                             const float* __restrict__ partial, int groups,
                                                             float* __restrict__ scale_out,
                                                             const float* __restrict__ fold_in, float* __restrict__ fold_out,
                                                             int64_t nfold) {
    __shared__ float red[kQThreads / 64];
    float m = 0.f;
    for (int g = threadIdx.x; g < groups; g += kQThreads) m = fmaxf(m, partial[g]);
    m = block_reduce<kQThreads / 64>(m, red, MaxOp{}, 0.f);
    const float scale = m > 0.f ? m / 448.0f : 1.0f;
    if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = scale;
    // the scale folded into an array of the caller's on the way (the weights' per-channel scales of the GEMM that
    // takes these codes: one multiply there instead of two, and no launch for the product)
    for (int64_t i = (int64_t)blockIdx.x * kQThreads + threadIdx.x; i < nfold; i += (int64_t)gridDim.x * kQThreads)
        fold_out[i] = fold_in[i] * scale;
    const int64_t vec_per_row = n / 8, total = vec_per_row * rows;
    for (int64_t i = (int64_t)blockIdx.x * kQThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kQThreads) {
        const int64_t r = i / vec_per_row, c = i - r * vec_per_row;
        const u16x8 v = *reinterpret_cast<const u16x8*>(x + r * ld + 8 * c);
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = widen<BF16>(v[e]) / scale;   // (a correctly rounded quotient: the kernel is bound by memory)
        // the hardware's OCP-FP8 conversion: round to nearest even, saturating at +-448 (x / scale never exceeds it
        // by more than a rounding)
        unsigned lo = 0, hi = 0;
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
        *reinterpret_cast<u32x2*>(q + r * ldq + 8 * c) = u32x2{lo, hi};
    }
}

}  // namespace

static int dense_f32(const mi_tile_array* a, int64_t* n) {
    MI_CHECK(check_array(a, a->ndim));
    if (a->dtype != MI_F32) return MI_E_DTYPE;
    int64_t run = 1;
    for (int d = 0; d < a->ndim; ++d) {
        if (a->sizes[d] > 1 && a->strides[d] != run) return MI_E_STRIDE;
        run *= a->sizes[d];
    }
    *n = run;
    return MI_OK;
}

static int quantize_impl(const mi_tile_array* x, const mi_tile_array* codes, const mi_tile_array* scale,
                         const mi_tile_array* workspace, const mi_tile_array* fold_in, const mi_tile_array* fold_out,
                         void* stream) {
    MI_CHECK(check_array(x, 2));
    MI_CHECK(check_array(codes, 2));
    MI_CHECK(check_array(scale, 1));
    MI_CHECK(check_array(workspace, 1));
    if ((x->dtype != MI_F16 && x->dtype != MI_BF16) || codes->dtype != MI_F8E4M3FN || scale->dtype != MI_F32 ||
        workspace->dtype != MI_F32)
        return MI_E_DTYPE;
    if (!same_shape(x, codes) || scale->sizes[0] < 1 || workspace->sizes[0] < kQMaxGroups) return MI_E_SHAPE;
    const int64_t n = x->sizes[0], rows = x->sizes[1];
    if ((n > 1 && (x->strides[0] != 1 || codes->strides[0] != 1)) || (workspace->sizes[0] > 1 && workspace->strides[0] != 1))
        return MI_E_STRIDE;
    // whole 16-byte pieces of x, 8-byte pieces of the codes
    if (n % 8 || x->strides[1] % 8 || codes->strides[1] % 8 || !aligned(x->ptr, 16) || !aligned(codes->ptr, 8)) return MI_E_ALIGN;
    int64_t nfold = 0;
    if (fold_in) {
        int64_t nout = 0;
        MI_CHECK(dense_f32(fold_in, &nfold));
        MI_CHECK(dense_f32(fold_out, &nout));
        if (nout != nfold) return MI_E_SHAPE;
    }
    if (n == 0 || rows == 0) return nfold ? MI_E_SHAPE : MI_OK;
    const float* fin = fold_in ? (const float*)fold_in->ptr : nullptr;
    float* fout = fold_out ? (float*)fold_out->ptr : nullptr;
    const int64_t vecs = n / 8 * rows;
    const int groups = (int)(cld(vecs, (int64_t)(4 * kQThreads)) < kQMaxGroups ? cld(vecs, (int64_t)(4 * kQThreads)) : kQMaxGroups);
    hipStream_t s = (hipStream_t)stream;
    if (x->dtype == MI_BF16) {
        hipLaunchKernelGGL(absmax_kernel<true>, dim3(groups), dim3(kQThreads), 0, s, (const unsigned short*)x->ptr, x->strides[1], n, rows,
                           (float*)workspace->ptr);
        hipLaunchKernelGGL(quantize_kernel<true>, dim3(groups), dim3(kQThreads), 0, s, (const unsigned short*)x->ptr, x->strides[1], n, rows,
                           (unsigned char*)codes->ptr, codes->strides[1], (const float*)workspace->ptr, groups, (float*)scale->ptr, fin, fout, nfold);
    } else {
        hipLaunchKernelGGL(absmax_kernel<false>, dim3(groups), dim3(kQThreads), 0, s, (const unsigned short*)x->ptr, x->strides[1], n, rows,
                           (float*)workspace->ptr);
        hipLaunchKernelGGL(quantize_kernel<false>, dim3(groups), dim3(kQThreads), 0, s, (const unsigned short*)x->ptr, x->strides[1], n, rows,
                           (unsigned char*)codes->ptr, codes->strides[1], (const float*)workspace->ptr, groups, (float*)scale->ptr, fin, fout, nfold);
    }
    set_variant("quantize_e4m3fn_per_tensor_2pass");
    return launch_status();
}

extern "C" int mi_quantize_e4m3fn(const mi_tile_array* x, const mi_tile_array* codes, const mi_tile_array* scale,
                                  const mi_tile_array* workspace, void* stream) {
    return quantize_impl(x, codes, scale, workspace, nullptr, nullptr, stream);
}

extern "C" int mi_quantize_e4m3fn_fold(const mi_tile_array* x, const mi_tile_array* codes, const mi_tile_array* scale,
                                       const mi_tile_array* workspace, const mi_tile_array* fold_in,
                                       const mi_tile_array* fold_out, void* stream) {
    if (!fold_in || !fold_out) return MI_E_NULL;
    return quantize_impl(x, codes, scale, workspace, fold_in, fold_out, stream);
}
