// Shared host/device helpers for libmi355tile (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include "../../include/mi355tile.h"

#define MI_MAX_GRID_DIM ((1 << 24) - 1)

namespace mi {

// Host-side record of which kernel variant the last launch on this thread picked.
void set_variant(const char* name);
const char* last_variant_name();   // what the calling thread's last launch set
// True once the caller has promised (mi_scratch_under_capture) that replays of its graphs neither overlap one another
// nor other use of the library's shared static arrays on the device: capturing streams are then given those arrays.
bool scratch_under_capture();

static inline int dtype_size(int dt) {
    switch (dt) {
        case MI_F32: return 4;
        case MI_F64: return 8;
        case MI_F16: return 2;
        case MI_BF16: return 2;
        case MI_F8E4M3FN: return 1;
        case MI_F8E5M2: return 1;
        case MI_I32: return 4;
        case MI_I64: return 8;
        default: return 0;
    }
}

static inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
static inline int64_t cld(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Argument checks shared by every entry point.  Each returns 0 or an MI_E_* code.
static inline int check_array(const mi_tile_array* a, int ndim) {
    if (!a) return MI_E_NULL;
    if (a->ndim != ndim) return MI_E_RANK;
    int es = dtype_size(a->dtype);
    if (es == 0) return MI_E_DTYPE;
    int64_t n = 1;
    for (int i = 0; i < ndim; ++i) {
        if (a->sizes[i] < 0) return MI_E_SHAPE;
        n *= a->sizes[i];
    }
    if (n > 0 && !a->ptr) return MI_E_NULL;
    if (((uintptr_t)a->ptr) % (uintptr_t)es) return MI_E_ALIGN;
    return MI_OK;
}

static inline bool same_shape(const mi_tile_array* a, const mi_tile_array* b) {
    if (a->ndim != b->ndim) return false;
    for (int i = 0; i < a->ndim; ++i)
        if (a->sizes[i] != b->sizes[i]) return false;
    return true;
}

// True when the array is dense column-major (stride[0]==1, stride[i]==prod(sizes[<i])).
static inline bool is_dense(const mi_tile_array* a) {
    int64_t s = 1;
    for (int i = 0; i < a->ndim; ++i) {
        if (a->sizes[i] != 1 && a->strides[i] != s) return false;
        s *= a->sizes[i];
    }
    return true;
}

static inline int64_t numel(const mi_tile_array* a) {
    int64_t n = 1;
    for (int i = 0; i < a->ndim; ++i) n *= a->sizes[i];
    return n;
}

static inline bool aligned(const void* p, size_t a) { return (((uintptr_t)p) % a) == 0; }

static inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? MI_OK : (int)e;
}

#define MI_CHECK(expr)              \
    do {                            \
        int _rc = (expr);           \
        if (_rc != MI_OK) return _rc; \
    } while (0)

}  // namespace mi

#ifdef __HIPCC__
namespace mi {

constexpr int kWave = 64;

// ---- wave64 reductions (six butterfly steps of __shfl_xor) -------------------------------
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
    return v;
}
struct SumOp {
    template <typename T>
    __device__ __forceinline__ T operator()(T a, T b) const { return a + b; }
};
struct MaxOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

// Block-wide all-reduce of one float through LDS. `red` must hold NWAVES floats.
// Contains two barriers; every thread of the block must call it.
template <int NWAVES, typename Op>
__device__ __forceinline__ float block_reduce(float v, float* red, Op op, float ident) {
    v = wave_reduce(v, op);
    if constexpr (NWAVES == 1) return v;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = (lane < NWAVES) ? red[lane] : ident;
#pragma unroll
    for (int off = NWAVES / 2; off >= 1; off >>= 1) r = op(r, __shfl_xor(r, off, 64));
    r = __shfl(r, 0, 64);
    __syncthreads();
    return r;
}

// Storage-type conversion helpers (fp32 compute).
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }
template <> __device__ __forceinline__ float to_f32<__hip_bfloat16>(__hip_bfloat16 v) {
    return __bfloat162float(v);
}
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 from_f32<__hip_bfloat16>(float v) {
    return __float2bfloat16(v);
}

// Streaming (non-temporal) or cached global loads, chosen per launch.  Inputs that fit the 256 MB
// memory-side cache are better read with ordinary loads (they hit when the same buffers come
// round again, and cost nothing extra when they do not); anything larger should not evict it on
// its way through.  Results are written with streaming stores either way: measured on
// 4096x4096 fp32 rows, cached stores were slower whenever the data was not already resident.
template <bool STREAM, typename V>
__device__ __forceinline__ V ld_global(const V* p) {
    return STREAM ? __builtin_nontemporal_load(p) : *p;
}
template <bool STREAM, typename V>
__device__ __forceinline__ void st_global(V v, V* p) {
    if (STREAM) __builtin_nontemporal_store(v, p);
    else *p = v;
}
// Host side of the choice: stream when the bytes one launch touches exceed what the memory-side
// cache can keep next to other tenants.  MI_STREAM_HINT=0 / 1 forces one way (measurements).
inline bool stream_hint(int64_t bytes_touched) {
    static const int forced = [] {
        const char* e = getenv("MI_STREAM_HINT");
        return e ? (e[0] == '0' ? 0 : 1) : -1;
    }();
    if (forced >= 0) return forced != 0;
    return bytes_touched > (224ll << 20);
}

}  // namespace mi
#endif
