// Column softmax: stand-ins for softmax_tma_kernel (examples/softmax.jl:18-42) and
// softmax_chunked_kernel (examples/softmax.jl:48-100) of the reference.
//
// input/output are (N, M) with the softmax dimension N contiguous.  One workgroup owns one
// column at a time.  The single-tile kernel keeps the whole column in registers, so HBM is
// touched exactly once per element each way (algorithmic traffic 2*M*N*sizeof(T)): 16-byte
// loads, wave64 shuffle reductions, one LDS exchange per reduction across the waves of the
// workgroup.  Columns too long for that (more than 16384 elements per 256 lanes' registers) take
// the reference's three passes (max, denominator, normalise), re-reading the column from L2;
// softmax_chunked_kernel uses the register kernel too whenever its column fits.
//
// Numerics follow the reference: fp32 math, max ignores NaN, full-precision exp (not
// exp2), IEEE division, padding rows read as -Inf and are never written.
#include "common.h"
#include <math.h>

namespace {

using namespace mi;

template <typename T> struct Raw;  // 16-byte vectors of the storage type
template <> struct Raw<float> {
    typedef float V __attribute__((ext_vector_type(4)));
    static constexpr int EV = 4;
};
template <> struct Raw<__half> {
    typedef _Float16 V __attribute__((ext_vector_type(8)));
    static constexpr int EV = 8;
};
template <> struct Raw<__hip_bfloat16> {
    typedef unsigned short V __attribute__((ext_vector_type(8)));
    static constexpr int EV = 8;
};

template <typename T> __device__ __forceinline__ float vget(const typename Raw<T>::V& v, int q);
template <> __device__ __forceinline__ float vget<float>(const Raw<float>::V& v, int q) { return v[q]; }
template <> __device__ __forceinline__ float vget<__half>(const Raw<__half>::V& v, int q) {
    return (float)v[q];
}
template <> __device__ __forceinline__ float vget<__hip_bfloat16>(const Raw<__hip_bfloat16>::V& v, int q) {
    return __uint_as_float(((unsigned)v[q]) << 16);
}
template <typename T> __device__ __forceinline__ void vset(typename Raw<T>::V& v, int q, float f);
template <> __device__ __forceinline__ void vset<float>(Raw<float>::V& v, int q, float f) { v[q] = f; }
template <> __device__ __forceinline__ void vset<__half>(Raw<__half>::V& v, int q, float f) {
    v[q] = (_Float16)f;
}
template <> __device__ __forceinline__ void vset<__hip_bfloat16>(Raw<__hip_bfloat16>::V& v, int q, float f) {
    __hip_bfloat16 h = __float2bfloat16(f);
    v[q] = *reinterpret_cast<unsigned short*>(&h);
}

// A 16-byte vector at an address that is aligned for its elements only: global memory takes such accesses, in one
// instruction (a column of 50257 floats starts anywhere).
template <typename V, typename T>
__device__ __forceinline__ V ld_unaligned(const T* p) {
    V v;
    __builtin_memcpy(&v, p, sizeof(V));
    return v;
}
template <typename V, typename T>
__device__ __forceinline__ void st_unaligned(const V& v, T* p) {
    __builtin_memcpy(p, &v, sizeof(V));
}

// ---- single-tile kernel: column cached in registers -----------------------------------
// Capacity BLOCK*VPT*EV elements.  ALIGNED: every column starts on a 16-byte boundary (plain and streaming vector
// accesses); otherwise the vectors inside the column move unaligned and only the one across its end element-wise.
template <typename T, int BLOCK, int VPT, bool ALIGNED, bool STREAM>
__global__ __launch_bounds__(BLOCK) void softmax_regs_kernel(T* __restrict__ out, int64_t ldo,
                                                             const T* __restrict__ in, int64_t ldi,
                                                             int L, int64_t M) {
    constexpr int EV = Raw<T>::EV;
    using V = typename Raw<T>::V;
    constexpr int NW = BLOCK / 64;
    __shared__ float red[NW > 1 ? NW : 1];
    const float NEG_INF = -INFINITY;

    for (int64_t col = blockIdx.x; col < M; col += gridDim.x) {
        const T* ip = in + col * ldi;
        T* op = out + col * ldo;
        float x[VPT][EV];
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int e0 = (threadIdx.x + v * BLOCK) * EV;
            if (e0 + EV <= L) {
                V raw;
                if (ALIGNED) raw = ld_global<STREAM>(reinterpret_cast<const V*>(ip + e0));
                else raw = ld_unaligned<V>(ip + e0);
#pragma unroll
                for (int q = 0; q < EV; ++q) x[v][q] = vget<T>(raw, q);
            } else {
#pragma unroll
                for (int q = 0; q < EV; ++q) x[v][q] = (e0 + q < L) ? to_f32<T>(ip[e0 + q]) : NEG_INF;
            }
        }
        float mx = NEG_INF;
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < EV; ++q) mx = fmaxf(mx, x[v][q]);
        mx = block_reduce<NW>(mx, red, MaxOp{}, NEG_INF);
        float sum = 0.f;
        if constexpr (BLOCK == 1024) {
            // One workgroup holds the CU here, so nothing runs under this loop: 64 library exponentials per lane
            // (about twenty instructions each) were as long as the column's load.  The hardware's 2^x on
            // (x - max) * log2(e), the product formed by one fma: two instructions, and an error of the argument's
            // rounding, |x - max| * 2^-24 relative (3e-6 at 50 below the maximum, where the value is 2e-22).
            const float l2e = 1.4426950408889634f, mxl = mx == NEG_INF ? 0.f : mx * l2e;
#pragma unroll
            for (int v = 0; v < VPT; ++v)
#pragma unroll
                for (int q = 0; q < EV; ++q) {
                    x[v][q] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[v][q], l2e, -mxl));
                    sum += x[v][q];
                }
        } else {
#pragma unroll
            for (int v = 0; v < VPT; ++v)
#pragma unroll
                for (int q = 0; q < EV; ++q) {
                    x[v][q] = expf(x[v][q] - mx);
                    sum += x[v][q];
                }
        }
        sum = block_reduce<NW>(sum, red, SumOp{}, 0.f);
        // one correctly rounded reciprocal per column, then multiplies: within 1.5 ulp of the
        // element-wise quotient, at a tenth of the instructions
        const float rsum = 1.0f / sum;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int e0 = (threadIdx.x + v * BLOCK) * EV;
            if (e0 + EV <= L) {
                V raw;
#pragma unroll
                for (int q = 0; q < EV; ++q) vset<T>(raw, q, x[v][q] * rsum);
                if (ALIGNED) st_global<true>(raw, reinterpret_cast<V*>(op + e0));
                else st_unaligned<V>(raw, op + e0);
            } else {
#pragma unroll
                for (int q = 0; q < EV; ++q)
                    if (e0 + q < L) op[e0 + q] = from_f32<T>(x[v][q] * rsum);
            }
        }
    }
}

// ---- three-pass kernel: any column length ---------------------------------------------
// ALIGNED: every column starts on a 16-byte boundary.  Otherwise a column whose input and output sit at the same
// offset from such a boundary (the usual case: equal leading dimensions) is walked as a scalar head up to the
// boundary, 16-byte vectors, and a scalar tail; columns that do not, element by element.
template <typename T, int BLOCK, bool ALIGNED>
__global__ __launch_bounds__(BLOCK) void softmax_3pass_kernel(T* __restrict__ out, int64_t ldo,
                                                              const T* __restrict__ in, int64_t ldi,
                                                              int64_t L, int64_t M) {
    constexpr int EV = Raw<T>::EV;
    using V = typename Raw<T>::V;
    constexpr int NW = BLOCK / 64;
    __shared__ float red[NW];
    const float NEG_INF = -INFINITY;

    for (int64_t col = blockIdx.x; col < M; col += gridDim.x) {
        const T* ip = in + col * ldi;
        T* op = out + col * ldo;
        int64_t head = 0, nvec = L / EV;
        if (!ALIGNED) {
            const uintptr_t ai = (uintptr_t)ip, ao = (uintptr_t)op;
            if ((ai & 15) == (ao & 15) && ai % sizeof(T) == 0) {
                head = (int64_t)(((16 - (ai & 15)) & 15) / sizeof(T));
                if (head > L) head = L;
                nvec = (L - head) / EV;
            } else {
                head = L;
                nvec = 0;
            }
        }
        const T* ipv = ip + head;
        T* opv = op + head;
        const int64_t nscalar = L - nvec * EV;                       // head and tail elements
        auto at = [&](int64_t e) { return e < head ? e : e + nvec * EV; };   // their positions in the column
        // pass 1: running maximum
        float mx = NEG_INF;
#pragma unroll 4
        for (int64_t v = threadIdx.x; v < nvec; v += BLOCK) {
            V raw = *reinterpret_cast<const V*>(ipv + v * EV);
#pragma unroll
            for (int q = 0; q < EV; ++q) mx = fmaxf(mx, vget<T>(raw, q));
        }
        for (int64_t e = threadIdx.x; e < nscalar; e += BLOCK) mx = fmaxf(mx, to_f32<T>(ip[at(e)]));
        mx = block_reduce<NW>(mx, red, MaxOp{}, NEG_INF);
        // exp(x - max) as the hardware's 2^x of one fma (see the 1024-lane register kernel): a column this long is
        // walked by one workgroup per CU, and the library exponential was most of passes 2 and 3
        const float l2e = 1.4426950408889634f, mxl = mx == NEG_INF ? 0.f : mx * l2e;
        auto ex = [&](float v) { return __builtin_amdgcn_exp2f(__builtin_fmaf(v, l2e, -mxl)); };
        // pass 2: per-lane partial denominators, one reduction at the end
        float den = 0.f;
#pragma unroll 4
        for (int64_t v = threadIdx.x; v < nvec; v += BLOCK) {
            V raw = *reinterpret_cast<const V*>(ipv + v * EV);
#pragma unroll
            for (int q = 0; q < EV; ++q) den += ex(vget<T>(raw, q));
        }
        for (int64_t e = threadIdx.x; e < nscalar; e += BLOCK) den += ex(to_f32<T>(ip[at(e)]));
        den = block_reduce<NW>(den, red, SumOp{}, 0.f);
        const float rden = 1.0f / den;   // (one reciprocal per column, then multiplies, as in the register kernel)
        // pass 3: normalise and store
#pragma unroll 4
        for (int64_t v = threadIdx.x; v < nvec; v += BLOCK) {
            V raw = *reinterpret_cast<const V*>(ipv + v * EV);
            V res;
#pragma unroll
            for (int q = 0; q < EV; ++q) vset<T>(res, q, ex(vget<T>(raw, q)) * rden);
            st_global<true>(res, reinterpret_cast<V*>(opv + v * EV));
        }
        for (int64_t e = threadIdx.x; e < nscalar; e += BLOCK)
            op[at(e)] = from_f32<T>(ex(to_f32<T>(ip[at(e)])) * rden);
    }
}

int check(const mi_tile_array* output, const mi_tile_array* input, int TILE_SIZE, int num_programs) {
    MI_CHECK(check_array(output, 2));
    MI_CHECK(check_array(input, 2));
    if (output->dtype != input->dtype) return MI_E_DTYPE;
    if (input->dtype != MI_F32 && input->dtype != MI_F16 && input->dtype != MI_BF16) return MI_E_DTYPE;
    if (!same_shape(output, input)) return MI_E_SHAPE;
    if (!is_pow2(TILE_SIZE)) return MI_E_TILE;
    if (num_programs < 1 || num_programs > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (input->sizes[0] > 1 && (input->strides[0] != 1 || output->strides[0] != 1)) return MI_E_STRIDE;
    return MI_OK;
}

template <typename T>
bool vec_ok(const mi_tile_array* output, const mi_tile_array* input) {
    constexpr int EV = Raw<T>::EV;
    return aligned(input->ptr, 16) && aligned(output->ptr, 16) &&
           (input->sizes[1] <= 1 || (input->strides[1] % EV == 0 && output->strides[1] % EV == 0));
}

template <typename T, int BLOCK, int VPT>
void launch_regs(const mi_tile_array* output, const mi_tile_array* input, int L, bool al,
                 hipStream_t s) {
    const int64_t M = input->sizes[1];
    // The 1024-lane variants hold a CU's registers with one workgroup (two when a lane keeps 32 elements): a workgroup
    // per CU slot walks the columns, so that the stores of one column, once issued, drain under the loads of the next.
    const int64_t slots = 256 * (VPT * Raw<T>::EV <= 32 ? 2 : 1);
    dim3 grid((unsigned)(BLOCK == 1024 && M > slots ? slots : M)), block(BLOCK);
#define GO(AL, ST)                                                                              \
    hipLaunchKernelGGL((softmax_regs_kernel<T, BLOCK, VPT, AL, ST>), grid, block, 0, s, (T*)output->ptr, \
                       output->strides[1], (const T*)input->ptr, input->strides[1], L, M)
    if (!al) GO(false, false);
    else if (stream_hint(2 * M * (int64_t)L * (int64_t)sizeof(T))) GO(true, true);
    else GO(true, false);
#undef GO
}

template <typename T>
int launch_3pass(const mi_tile_array* output, const mi_tile_array* input, int64_t L, hipStream_t s) {
    const int64_t M = input->sizes[1];
    const bool al = vec_ok<T>(output, input);
    // (few columns: 1024 lanes each, so that a column has sixteen 16-byte loads per lane-slot in flight, not four)
    const bool wide = M < 1024;
    dim3 grid((unsigned)M), block(wide ? 1024 : 256);
#define GO(B, AL)                                                                                          \
    hipLaunchKernelGGL((softmax_3pass_kernel<T, B, AL>), grid, block, 0, s, (T*)output->ptr, output->strides[1], \
                       (const T*)input->ptr, input->strides[1], L, M)
    if (wide && al) GO(1024, true);
    else if (wide) GO(1024, false);
    else if (al) GO(256, true);
    else GO(256, false);
#undef GO
    set_variant(wide ? "softmax_3pass_b1024" : "softmax_3pass_b256");
    return launch_status();
}

// Softmax over the first L64 rows of every column: the register kernel when the column fits
// (one HBM pass), otherwise three passes.
template <typename T>
int launch_len(const mi_tile_array* output, const mi_tile_array* input, int64_t L64, hipStream_t s) {
    constexpr int EV = Raw<T>::EV;
    if (L64 > 65536) return launch_3pass<T>(output, input, L64, s);
    const int L = (int)L64;
    // (a column that is aligned as a whole: its last vector may still cross the end, which the kernel handles)
    const bool al = vec_ok<T>(output, input);
    const int vecs = (int)cld(L, EV);
    if (vecs > 256 * 16) {
        // Up to 65536 elements in the registers of 1024 lanes (64 per lane), one workgroup per CU: one pass over HBM
        // where the three-pass kernel re-reads the column twice (1024 x 50257 fp32: 121 us).
        if (L > 32768) { launch_regs<T, 1024, 64 / EV>(output, input, L, al, s); set_variant("softmax_regs_b1024_e64"); }
        else { launch_regs<T, 1024, 32 / EV>(output, input, L, al, s); set_variant("softmax_regs_b1024_e32"); }
        return launch_status();
    }
    if (vecs <= 64) { launch_regs<T, 64, 1>(output, input, L, al, s); set_variant("softmax_regs_b64_v1"); }
    else if (vecs <= 128) { launch_regs<T, 64, 2>(output, input, L, al, s); set_variant("softmax_regs_b64_v2"); }
    else if (vecs <= 256) { launch_regs<T, 64, 4>(output, input, L, al, s); set_variant("softmax_regs_b64_v4"); }   // one wave per column: no barriers
    else if (vecs <= 512) { launch_regs<T, 256, 2>(output, input, L, al, s); set_variant("softmax_regs_b256_v2"); }
    else if (vecs <= 1024) { launch_regs<T, 256, 4>(output, input, L, al, s); set_variant("softmax_regs_b256_v4"); }
    else if (vecs <= 2048) { launch_regs<T, 256, 8>(output, input, L, al, s); set_variant("softmax_regs_b256_v8"); }
    else { launch_regs<T, 256, 16>(output, input, L, al, s); set_variant("softmax_regs_b256_v16"); }
    return launch_status();
}

}  // namespace

extern "C" int mi_softmax_tma_kernel(const mi_tile_array* output, const mi_tile_array* input,
                                     int TILE_SIZE, int num_programs, void* stream) {
    MI_CHECK(check(output, input, TILE_SIZE, num_programs));
    if (input->sizes[0] == 0 || input->sizes[1] == 0) return MI_OK;
    if (input->sizes[1] > 0x7fffffffLL) return MI_E_GRID;
    hipStream_t s = (hipStream_t)stream;
    const int64_t L = input->sizes[0] < TILE_SIZE ? input->sizes[0] : (int64_t)TILE_SIZE;  // one tile per column
    switch (input->dtype) {
        case MI_F32: return launch_len<float>(output, input, L, s);
        case MI_F16: return launch_len<__half>(output, input, L, s);
        default: return launch_len<__hip_bfloat16>(output, input, L, s);
    }
}

extern "C" int mi_softmax_chunked_kernel(const mi_tile_array* output, const mi_tile_array* input,
                                         int n_elems, int TILE_SIZE, int num_programs, void* stream) {
    MI_CHECK(check(output, input, TILE_SIZE, num_programs));
    if (n_elems < 0) return MI_E_ARG;
    if (input->sizes[0] == 0 || input->sizes[1] == 0) return MI_OK;
    if (input->sizes[1] > 0x7fffffffLL) return MI_E_GRID;
    // The chunk loop visits rows 1 .. cld(n_elems, TILE_SIZE)*TILE_SIZE; rows past the
    // array's end are padding (softmax.jl:58, 65-69).
    int64_t L = cld((int64_t)n_elems, (int64_t)TILE_SIZE) * TILE_SIZE;
    if (L > input->sizes[0]) L = input->sizes[0];
    if (L == 0) return MI_OK;
    hipStream_t s = (hipStream_t)stream;
    switch (input->dtype) {
        // Same function of the column as the reference's three chunked passes; a column that
        // fits in registers is read from HBM once instead.
        case MI_F32: return launch_len<float>(output, input, L, s);
        case MI_F16: return launch_len<__half>(output, input, L, s);
        default: return launch_len<__hip_bfloat16>(output, input, L, s);
    }
}
