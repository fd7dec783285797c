// Batched complex FFT: stand-in for fft_kernel of the reference's examples/fft.jl:22-126, a
// three-stage Cooley-Tukey factorisation N = F0*F1*F2 written there as three small complex
// matrix products with DFT matrices W0, W1, W2 and element-wise twiddles T0, T1.
//
// With the input index n = i2 + F2*i1 + F1*F2*i0 and the output index k = k0 + F0*k1 + F0*F1*k2
// (the reshapes and permutes of fft.jl:45-121 amount to exactly this),
//   Y[k] = sum_i2 W2[i2,k2] T1[i2,k1] sum_i1 W1[i1,k1] T0[i2 + F2*i1, k0] sum_i0 W0[i0,k0] X[n].
// The kernel uses the caller's W and T tables, as the reference does, so any consistent set of
// tables gives the same result as there.
//
// Mapping to CDNA4.  The transform is latency-, not throughput-bound (4096 points x 256 signals
// are 16 MB of traffic and 0.4 GFLOP): one workgroup of 256 lanes per signal, the signal in LDS
// (33 KB with padding), each stage one pass in which a lane gathers the F inputs of a
// sub-transform into registers, multiplies by (its share of the columns of) the DFT matrix,
// whose entries are wave-uniform and arrive through the scalar cache, applies the twiddle and
// scatters back in place; the last stage stores straight to global memory with consecutive
// lanes on consecutive outputs.  1024 lanes per 4096-point signal: four lanes share a
// radix-16 sub-transform.  True fp32 FMAs throughout.
#include "common.h"

namespace {

using namespace mi;

typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kMaxN = 4096;    // points per signal that fit the LDS buffer
__device__ __forceinline__ int pad(int i) { return i + (i >> 8); }  // one element per 256: strides of 256 spread over banks

__device__ __forceinline__ f32x2 cmul(f32x2 a, f32x2 b) {
    return f32x2{a[0] * b[0] - a[1] * b[1], a[0] * b[1] + a[1] * b[0]};
}

constexpr int imin(int a, int b) { return a < b ? a : b; }
// Lanes that share one sub-transform (each computes F/KG of its outputs): as many as the
// workgroup has to spare, but only when whole waves share a k-group, so that the DFT-matrix
// entries a wave needs are wave-uniform and come through the scalar cache.
constexpr int k_groups(int F, int tasks, int threads) {
    return (tasks % 64 == 0 && threads / tasks >= 1) ? imin(F, threads / tasks) : 1;
}

// One stage over the LDS buffer: `tasks` sub-transforms of radix F.  Task t reads its inputs at
// base(t) + stride*i; output k, multiplied by tw(t, k), goes back to the same positions or, in
// the last stage, to global memory through gout(t, k, value).  W is the caller's DFT matrix in
// global memory, out[k] = sum_i in[i] * W[i + F*k] (i fastest).
template <int F, int KG, int THREADS, bool LAST, typename Base, typename Tw, typename Out>
__device__ __forceinline__ void stage(f32x2* buf, const f32x2* __restrict__ W, int tasks, int stride, Base base, Tw tw,
                                      Out gout) {
    constexpr int KPT = F / KG;
    const int items = tasks * KG;
    for (int first = 0; first < items; first += THREADS) {
        const int item = first + (int)threadIdx.x;
        const bool live = item < items;
        const int t = live ? item % tasks : 0;
        const int kg = KG > 1 ? __builtin_amdgcn_readfirstlane(item / tasks) : 0;
        const int b = base(t);
        f32x2 in[F];
#pragma unroll
        for (int i = 0; i < F; ++i) in[i] = buf[pad(b + stride * i)];
        if (KG > 1 && !LAST) __syncthreads();  // every lane of a task has read before any writes in place
        if (live) {
#pragma unroll
            for (int kk = 0; kk < KPT; ++kk) {
                const int k = kg * KPT + kk;
                float re = 0.f, im = 0.f;
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    const f32x2 w = W[i + F * k];
                    re = __builtin_fmaf(in[i][0], w[0], re);
                    re = __builtin_fmaf(-in[i][1], w[1], re);
                    im = __builtin_fmaf(in[i][0], w[1], im);
                    im = __builtin_fmaf(in[i][1], w[0], im);
                }
                const f32x2 o = {re, im};
                if (LAST) gout(t, k, o);
                else buf[pad(b + stride * k)] = cmul(o, tw(t, k));
            }
        }
        if (first + THREADS < items) __syncthreads();
    }
}

template <int F0, int F1, int F2, int THREADS>
__global__ __launch_bounds__(THREADS) void fft_kernel(const f32x2* __restrict__ X, f32x2* __restrict__ Y,
                                                      const f32x2* __restrict__ W0, const f32x2* __restrict__ W1,
                                                      const f32x2* __restrict__ W2, const f32x2* __restrict__ T0,
                                                      const f32x2* __restrict__ T1) {
    constexpr int N = F0 * F1 * F2, F1F2 = F1 * F2;
    __shared__ f32x2 buf[N + (N >> 8) + 1];
    const f32x2* x = X + (size_t)blockIdx.x * N;
    f32x2* y = Y + (size_t)blockIdx.x * N;
    for (int n = threadIdx.x; n < N; n += THREADS) buf[pad(n)] = x[n];
    __syncthreads();
    // stage 0 over i0: task r = i2 + F2*i1, inputs at r + F1F2*i0, twiddle T0[r + F1F2*k0]
    stage<F0, k_groups(F0, F1F2, THREADS), THREADS, false>(
        buf, W0, F1F2, F1F2, [](int r) { return r; }, [&](int r, int k0) { return T0[r + F1F2 * k0]; },
        [](int, int, f32x2) {});
    __syncthreads();
    // stage 1 over i1: task t = i2 + F2*k0, inputs at i2 + F2*i1 + F1F2*k0, twiddle T1[i2 + F2*k1]
    stage<F1, k_groups(F1, F0 * F2, THREADS), THREADS, false>(
        buf, W1, F0 * F2, F2, [](int t) { return (t % F2) + F1F2 * (t / F2); },
        [&](int t, int k1) { return T1[(t % F2) + F2 * k1]; }, [](int, int, f32x2) {});
    __syncthreads();
    // stage 2 over i2: task t = k0 + F0*k1, inputs at i2 + F2*k1 + F1F2*k0, output k0 + F0*k1 + F0F1*k2
    stage<F2, k_groups(F2, F0 * F1, THREADS), THREADS, true>(
        buf, W2, F0 * F1, 1, [](int t) { return F2 * (t / F0) + F1F2 * (t % F0); },
        [](int, int) { return f32x2{1.f, 0.f}; },
        [&](int t, int k2, f32x2 v) { __builtin_nontemporal_store(v, y + t + F0 * F1 * k2); });
}

bool dense3(const mi_tile_array* a) {
    return a->strides[0] == 1 && (a->sizes[1] <= 1 || a->strides[1] == a->sizes[0]) &&
           (a->sizes[2] <= 1 || a->strides[2] == a->sizes[0] * a->sizes[1]);
}

}  // namespace

extern "C" int mi_fft_kernel(const mi_tile_array* x_packed_in, const mi_tile_array* y_packed_out,
                             const mi_tile_array* W0, const mi_tile_array* W1, const mi_tile_array* W2,
                             const mi_tile_array* T0, const mi_tile_array* T1, int N, int F0, int F1, int F2, int BS,
                             int D, void* stream) {
    for (const mi_tile_array* a : {x_packed_in, y_packed_out, W0, W1, W2, T0, T1}) {
        MI_CHECK(check_array(a, 3));
        if (a->dtype != MI_F32) return MI_E_DTYPE;
        if (!dense3(a)) return MI_E_STRIDE;
        if (!aligned(a->ptr, 8)) return MI_E_ALIGN;
    }
    if (F0 < 1 || F1 < 1 || F2 < 1 || BS < 1 || D < 1) return MI_E_ARG;
    if ((int64_t)F0 * F1 * F2 != N || (2 * (int64_t)N) % D != 0) return MI_E_ARG;
    const int64_t batch = x_packed_in->sizes[2];
    if (x_packed_in->sizes[0] != D || x_packed_in->sizes[1] != 2 * (int64_t)N / D || !same_shape(x_packed_in, y_packed_out))
        return MI_E_SHAPE;
    if (batch % BS != 0) return MI_E_SHAPE;
    auto is_table = [](const mi_tile_array* a, int64_t d1, int64_t d2) {
        return a->sizes[0] == 2 && a->sizes[1] == d1 && a->sizes[2] == d2;
    };
    if (!is_table(W0, F0, F0) || !is_table(W1, F1, F1) || !is_table(W2, F2, F2) ||
        !is_table(T0, (int64_t)F1 * F2, F0) || !is_table(T1, F2, F1))
        return MI_E_SHAPE;
    if (batch > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (batch == 0) return MI_OK;
    if (N > kMaxN) return MI_E_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
#define GO(A, B, C)                                                                                              \
    hipLaunchKernelGGL((fft_kernel<A, B, C, (A * B * C >= 2048 ? 1024 : 256)>), dim3((unsigned)batch),            \
                       dim3(A * B * C >= 2048 ? 1024 : 256), 0, s,                                                \
                       (const f32x2*)x_packed_in->ptr, (f32x2*)y_packed_out->ptr, (const f32x2*)W0->ptr,         \
                       (const f32x2*)W1->ptr, (const f32x2*)W2->ptr, (const f32x2*)T0->ptr, (const f32x2*)T1->ptr)
    const int key = (F0 << 16) | (F1 << 8) | F2;
    switch (key) {
        case (16 << 16) | (16 << 8) | 16: GO(16, 16, 16); break;
        case (8 << 16) | (8 << 8) | 8: GO(8, 8, 8); break;
        case (4 << 16) | (4 << 8) | 4: GO(4, 4, 4); break;
        case (2 << 16) | (2 << 8) | 2: GO(2, 2, 2); break;
        case (16 << 16) | (16 << 8) | 8: GO(16, 16, 8); break;
        case (16 << 16) | (8 << 8) | 8: GO(16, 8, 8); break;
        case (8 << 16) | (8 << 8) | 4: GO(8, 8, 4); break;
        case (4 << 16) | (8 << 8) | 2: GO(4, 8, 2); break;
        case (2 << 16) | (4 << 8) | 8: GO(2, 4, 8); break;
        default: return MI_E_UNSUPPORTED;
    }
#undef GO
    set_variant("fft_3stage_lds_1wg_per_signal");
    return launch_status();
}
