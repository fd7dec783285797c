// Vector / matrix addition kernels: stand-ins for vec_add_kernel_1d, vec_add_kernel_2d and
// vec_add_kernel_1d_gather of the reference's examples/vadd.jl:10-45.
//
// The result of c = a + b does not depend on the tile constant (a partial last tile is
// zero-padded on load and clipped on store, src/language/operations.jl:637-646,819-821), so
// the physical mapping is chosen for HBM3E streaming: 16-byte accesses, several independent
// loads in flight per lane before the first use, non-temporal hints because nothing is
// re-read.  Algorithmic traffic: 3 * n * sizeof(T) bytes.
#include "common.h"

namespace {

using namespace mi;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));
typedef unsigned long long u64x2v __attribute__((ext_vector_type(2)));

// One 16-byte vector of T and its element-wise IEEE add.
template <typename T> struct Vec16;
template <> struct Vec16<float> {
    using V = f32x4;
    static constexpr int N = 4;
    static __device__ __forceinline__ V add(V a, V b) { return a + b; }
    static __device__ __forceinline__ float add1(float a, float b) { return a + b; }
};
template <> struct Vec16<double> {
    using V = f64x2;
    static constexpr int N = 2;
    static __device__ __forceinline__ V add(V a, V b) { return a + b; }
    static __device__ __forceinline__ double add1(double a, double b) { return a + b; }
};
template <> struct Vec16<_Float16> {
    using V = f16x8;
    static constexpr int N = 8;
    static __device__ __forceinline__ V add(V a, V b) { return a + b; }
    static __device__ __forceinline__ _Float16 add1(_Float16 a, _Float16 b) { return a + b; }
};
// Integers wrap around, as Julia's + on Int32 / Int64 does: added as unsigned words.
struct i32raw { unsigned v; };
struct i64raw { unsigned long long v; };
template <> struct Vec16<i32raw> {
    using V = u32x4v;
    static constexpr int N = 4;
    static __device__ __forceinline__ V add(V a, V b) { return a + b; }
    static __device__ __forceinline__ i32raw add1(i32raw a, i32raw b) { return i32raw{a.v + b.v}; }
};
template <> struct Vec16<i64raw> {
    using V = u64x2v;
    static constexpr int N = 2;
    static __device__ __forceinline__ V add(V a, V b) { return a + b; }
    static __device__ __forceinline__ i64raw add1(i64raw a, i64raw b) { return i64raw{a.v + b.v}; }
};
// bf16 stored as raw 16-bit words: widen to fp32, add, round to nearest even.
struct bf16raw { unsigned short v; };
__device__ __forceinline__ float bf16_to_f32(unsigned short h) {
    return __uint_as_float(((unsigned)h) << 16);
}
__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
template <> struct Vec16<bf16raw> {
    using V = u16x8;
    static constexpr int N = 8;
    static __device__ __forceinline__ unsigned short add1u(unsigned short a, unsigned short b) {
        return f32_to_bf16_rne(bf16_to_f32(a) + bf16_to_f32(b));
    }
    static __device__ __forceinline__ V add(V a, V b) {
        V r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = add1u(a[i], b[i]);
        return r;
    }
    static __device__ __forceinline__ bf16raw add1(bf16raw a, bf16raw b) {
        return bf16raw{add1u(a.v, b.v)};
    }
};

constexpr int kBlock = 256;

// Streaming kernel: block b owns UNROLL*kBlock consecutive 16-byte vectors.  All UNROLL
// loads of a and of b are issued before the first add so that each lane keeps
// 2*UNROLL*16 bytes in flight.
template <typename T, int UNROLL, bool STREAM>
__global__ __launch_bounds__(kBlock) void vadd_vec_kernel(const T* __restrict__ a,
                                                          const T* __restrict__ b,
                                                          T* __restrict__ c, int64_t nvec) {
    using VT = Vec16<T>;
    using V = typename VT::V;
    const V* av = reinterpret_cast<const V*>(a);
    const V* bv = reinterpret_cast<const V*>(b);
    V* cv = reinterpret_cast<V*>(c);
    const int64_t base = (int64_t)blockIdx.x * (UNROLL * kBlock) + threadIdx.x;
    if (base + (int64_t)(UNROLL - 1) * kBlock < nvec) {
        V x[UNROLL], y[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) x[u] = ld_global<STREAM>(av + base + u * kBlock);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) y[u] = ld_global<STREAM>(bv + base + u * kBlock);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            st_global<true>(VT::add(x[u], y[u]), cv + base + u * kBlock);
    } else {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t i = base + u * kBlock;
            if (i < nvec) cv[i] = VT::add(av[i], bv[i]);
        }
    }
}

// Element-wise kernel with arbitrary element strides: the scalar tail of the streaming
// path, misaligned or strided 1-D arrays, and the gather/scatter variant (each lane forms
// its own 1-based index, reads 0 when it is out of bounds and drops its store).
template <typename T>
__global__ __launch_bounds__(kBlock) void vadd_elem_kernel(const T* __restrict__ a, int64_t sa,
                                                           const T* __restrict__ b, int64_t sb,
                                                           T* __restrict__ c, int64_t sc,
                                                           int64_t first, int64_t n_a, int64_t n_b,
                                                           int64_t n_c) {
    const int64_t i = first + (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_c) return;
    T x = i < n_a ? a[i * sa] : T{};
    T y = i < n_b ? b[i * sb] : T{};
    c[i * sc] = Vec16<T>::add1(x, y);
}

// 2-D strided kernel (dimension 0 contiguous or not); one thread per element, x fastest.
template <typename T>
__global__ __launch_bounds__(kBlock) void vadd_2d_kernel(const T* __restrict__ a, int64_t a0,
                                                         int64_t a1, const T* __restrict__ b,
                                                         int64_t b0, int64_t b1, T* __restrict__ c,
                                                         int64_t c0, int64_t c1, int64_t m,
                                                         int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= m) return;
    // (the second grid dimension holds at most 65535 workgroups: walk dimension 1 with that stride)
    for (int64_t j = blockIdx.y; j < n; j += gridDim.y)
        c[i * c0 + j * c1] = Vec16<T>::add1(a[i * a0 + j * a1], b[i * b0 + j * b1]);
}

// 2-D with dimension 0 contiguous and every column on a 16-byte boundary (a padded leading dimension): a lane owns
// one 16-byte vector of up to four consecutive columns, all loads before the first add.
template <typename T, int UNROLL>
__global__ __launch_bounds__(kBlock) void vadd_2d_vec_kernel(const T* __restrict__ a, int64_t a1, const T* __restrict__ b,
                                                             int64_t b1, T* __restrict__ c, int64_t c1, int64_t mvec,
                                                             int64_t n) {
    using VT = Vec16<T>;
    using V = typename VT::V;
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= mvec) return;
    for (int64_t j0 = (int64_t)blockIdx.y * UNROLL; j0 < n; j0 += (int64_t)gridDim.y * UNROLL) {
        V x[UNROLL], y[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (j0 + u < n) x[u] = ld_global<true>(reinterpret_cast<const V*>(a + (j0 + u) * a1) + i);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (j0 + u < n) y[u] = ld_global<true>(reinterpret_cast<const V*>(b + (j0 + u) * b1) + i);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (j0 + u < n) st_global<true>(VT::add(x[u], y[u]), reinterpret_cast<V*>(c + (j0 + u) * c1) + i);
    }
}

// Dense arrays.  Three arrays that sit at the same offset from a 16-byte boundary (a view such as x[2:end] of each)
// are walked as a scalar head up to the boundary, vectors, and a scalar tail.
template <typename T>
int launch_dense(const void* a0, const void* b0, void* c0, int64_t n, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    constexpr int UNROLL = 4;
    const uintptr_t off = (uintptr_t)a0 & 15;
    const bool same = ((uintptr_t)b0 & 15) == off && ((uintptr_t)c0 & 15) == off && off % sizeof(T) == 0;
    int64_t head = same ? (int64_t)(((16 - off) & 15) / sizeof(T)) : n;
    if (head > n) head = n;
    const T *a = (const T*)a0 + head, *b = (const T*)b0 + head;
    T* c = (T*)c0 + head;
    const int64_t nvec = (n - head) / N;
    if (head > 0) {   // the elements before the boundary (all of them when the arrays do not line up)
        const int64_t blocks = cld(head, (int64_t)kBlock);
        if (blocks > 0x7fffffffLL) return MI_E_GRID;
        hipLaunchKernelGGL((vadd_elem_kernel<T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, (const T*)a0, (int64_t)1,
                           (const T*)b0, (int64_t)1, (T*)c0, (int64_t)1, (int64_t)0, head, head, head);
        set_variant("vadd_elem");
    }
    n -= head;
    if (nvec > 0) {
        const int64_t blocks = cld(nvec, (int64_t)UNROLL * kBlock);
        if (blocks > 0x7fffffffLL) return MI_E_GRID;
        if (stream_hint(3 * n * (int64_t)sizeof(T))) {
            hipLaunchKernelGGL((vadd_vec_kernel<T, UNROLL, true>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                               (const T*)a, (const T*)b, (T*)c, nvec);
            set_variant("vadd_vec16_nt_x4");
        } else {
            hipLaunchKernelGGL((vadd_vec_kernel<T, UNROLL, false>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                               (const T*)a, (const T*)b, (T*)c, nvec);
            set_variant("vadd_vec16_x4");
        }
    }
    const int64_t done = nvec * N;
    if (done < n) {
        const int64_t blocks = cld(n - done, (int64_t)kBlock);
        if (blocks > 0x7fffffffLL) return MI_E_GRID;
        hipLaunchKernelGGL((vadd_elem_kernel<T>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           (const T*)a, (int64_t)1, (const T*)b, (int64_t)1, (T*)c, (int64_t)1,
                           done, n, n, n);
        if (nvec == 0) set_variant("vadd_elem");
    }
    return launch_status();
}

// Gather / scatter with the indices of a tile (vadd.jl:33-45): up to the shortest of the three arrays this is the
// dense sum; past it every lane bounds-checks its index against each array (reads 0, drops its store).
template <typename T>
int launch_gather(const mi_tile_array* a, const mi_tile_array* b, const mi_tile_array* c, hipStream_t s) {
    const int64_t n = c->sizes[0];
    if (n == 0) return MI_OK;
    int64_t common = a->sizes[0] < b->sizes[0] ? a->sizes[0] : b->sizes[0];
    if (n < common) common = n;
    if (!(is_dense(a) && is_dense(b) && is_dense(c))) common = 0;
    if (common > 0) {
        const int rc = launch_dense<T>(a->ptr, b->ptr, c->ptr, common, s);
        if (rc != MI_OK) return rc;
    }
    if (common < n) {
        const int64_t blocks = cld(n - common, (int64_t)kBlock);
        if (blocks > 0x7fffffffLL) return MI_E_GRID;
        hipLaunchKernelGGL((vadd_elem_kernel<T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, (const T*)a->ptr, a->strides[0],
                           (const T*)b->ptr, b->strides[0], (T*)c->ptr, c->strides[0], common, a->sizes[0], b->sizes[0], n);
        if (common == 0) set_variant("vadd_elem");
    }
    return launch_status();
}

template <typename T>
int launch_elem(const mi_tile_array* a, const mi_tile_array* b, const mi_tile_array* c,
                hipStream_t s) {
    const int64_t n = c->sizes[0];
    if (n == 0) return MI_OK;
    const int64_t blocks = cld(n, (int64_t)kBlock);
    if (blocks > 0x7fffffffLL) return MI_E_GRID;
    hipLaunchKernelGGL((vadd_elem_kernel<T>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       (const T*)a->ptr, a->strides[0], (const T*)b->ptr, b->strides[0],
                       (T*)c->ptr, c->strides[0], (int64_t)0, a->sizes[0], b->sizes[0], n);
    set_variant("vadd_elem");
    return launch_status();
}

template <typename T>
int launch_2d(const mi_tile_array* a, const mi_tile_array* b, const mi_tile_array* c,
              hipStream_t s) {
    const int64_t m = c->sizes[0], n = c->sizes[1];
    if (m == 0 || n == 0) return MI_OK;
    constexpr int N = Vec16<T>::N;
    auto cols_vec = [&](const mi_tile_array* x) {
        return (m == 1 || x->strides[0] == 1) && aligned(x->ptr, 16) && (n == 1 || x->strides[1] % N == 0);
    };
    int64_t m_done = 0;
    if (m >= N && cols_vec(a) && cols_vec(b) && cols_vec(c)) {
        const int64_t mvec = m / N, ygroups = cld(n, (int64_t)4);
        hipLaunchKernelGGL((vadd_2d_vec_kernel<T, 4>), dim3((unsigned)cld(mvec, (int64_t)kBlock), (unsigned)(ygroups < 65535 ? ygroups : 65535)),
                           dim3(kBlock), 0, s, (const T*)a->ptr, a->strides[1], (const T*)b->ptr, b->strides[1], (T*)c->ptr,
                           c->strides[1], mvec, n);
        set_variant("vadd_2d_vec16_x4");
        m_done = mvec * N;
        if (m_done == m) return launch_status();
    }
    // every element, or the last m % N rows of every column
    const int64_t mr = m - m_done;
    hipLaunchKernelGGL((vadd_2d_kernel<T>), dim3((unsigned)cld(mr, (int64_t)kBlock), (unsigned)(n < 65535 ? n : 65535)),
                       dim3(kBlock), 0, s, (const T*)a->ptr + m_done * a->strides[0], a->strides[0], a->strides[1],
                       (const T*)b->ptr + m_done * b->strides[0], b->strides[0], b->strides[1],
                       (T*)c->ptr + m_done * c->strides[0], c->strides[0], c->strides[1], mr, n);
    if (m_done == 0) set_variant("vadd_2d_strided");
    return launch_status();
}

#define DISPATCH_DTYPE(dt, CALL)                         \
    switch (dt) {                                        \
        case MI_F32: return CALL(float);                 \
        case MI_F64: return CALL(double);                \
        case MI_F16: return CALL(_Float16);              \
        case MI_BF16: return CALL(bf16raw);              \
        case MI_I32: return CALL(i32raw);                \
        case MI_I64: return CALL(i64raw);                \
        default: return MI_E_DTYPE;                      \
    }

int check3(const mi_tile_array* a, const mi_tile_array* b, const mi_tile_array* c, int ndim) {
    MI_CHECK(check_array(a, ndim));
    MI_CHECK(check_array(b, ndim));
    MI_CHECK(check_array(c, ndim));
    if (a->dtype != b->dtype || a->dtype != c->dtype) return MI_E_DTYPE;
    return MI_OK;
}

}  // namespace

extern "C" int mi_vec_add_kernel_1d(const mi_tile_array* a, const mi_tile_array* b,
                                    const mi_tile_array* c, int tile, void* stream) {
    MI_CHECK(check3(a, b, c, 1));
    if (!is_pow2(tile)) return MI_E_TILE;
    if (!same_shape(a, c) || !same_shape(b, c)) return MI_E_SHAPE;
    const int64_t n = c->sizes[0];
    if (cld(n, (int64_t)tile) > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (n == 0) return MI_OK;
    hipStream_t s = (hipStream_t)stream;
    if (is_dense(a) && is_dense(b) && is_dense(c)) {
#define CALL(T) launch_dense<T>(a->ptr, b->ptr, c->ptr, n, s)
        DISPATCH_DTYPE(c->dtype, CALL)
#undef CALL
    }
#define CALL(T) launch_elem<T>(a, b, c, s)
    DISPATCH_DTYPE(c->dtype, CALL)
#undef CALL
}

extern "C" int mi_vec_add_kernel_1d_gather(const mi_tile_array* a, const mi_tile_array* b,
                                           const mi_tile_array* c, int tile, void* stream) {
    // Sizes may differ here: every lane bounds-checks its index against each array
    // separately, as gather/scatter do.
    MI_CHECK(check3(a, b, c, 1));
    if (!is_pow2(tile)) return MI_E_TILE;
    const int64_t n = c->sizes[0];
    if (cld(n, (int64_t)tile) > MI_MAX_GRID_DIM) return MI_E_GRID;
    hipStream_t s = (hipStream_t)stream;
#define CALL(T) launch_gather<T>(a, b, c, s)
    DISPATCH_DTYPE(c->dtype, CALL)
#undef CALL
}

extern "C" int mi_vec_add_kernel_2d(const mi_tile_array* a, const mi_tile_array* b,
                                    const mi_tile_array* c, int tile_x, int tile_y, void* stream) {
    MI_CHECK(check3(a, b, c, 2));
    if (!is_pow2(tile_x) || !is_pow2(tile_y)) return MI_E_TILE;
    if (!same_shape(a, c) || !same_shape(b, c)) return MI_E_SHAPE;
    const int64_t m = c->sizes[0], n = c->sizes[1];
    if (cld(m, (int64_t)tile_x) > MI_MAX_GRID_DIM || cld(n, (int64_t)tile_y) > MI_MAX_GRID_DIM)
        return MI_E_GRID;
    if (m * n == 0) return MI_OK;
    hipStream_t s = (hipStream_t)stream;
    if (is_dense(a) && is_dense(b) && is_dense(c)) {
#define CALL(T) launch_dense<T>(a->ptr, b->ptr, c->ptr, m * n, s)
        DISPATCH_DTYPE(c->dtype, CALL)
#undef CALL
    }
#define CALL(T) launch_2d<T>(a, b, c, s)
    DISPATCH_DTYPE(c->dtype, CALL)
#undef CALL
}
