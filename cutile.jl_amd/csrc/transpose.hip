// Matrix transpose: stand-in for transpose_kernel of the reference's examples/transpose.jl:11-19,
// y[j,i] = x[i,j] for x (m,n) and y (n,m), both with dimension 0 contiguous.
//
// The result does not depend on the (tm,tn) tile constants, so the physical tile is fixed
// at 64x64 elements per 256-lane workgroup: 16-byte global loads along x's contiguous
// dimension, a padded LDS tile (pitch 65 elements: both the scattered writes and the
// gathered reads hit 64 distinct banks), 16-byte global stores along y's contiguous
// dimension.  Workgroups are numbered so that consecutive ids walk down x's contiguous
// dimension.  Algorithmic traffic: 2 * m * n * sizeof(T) bytes.
#include "common.h"

namespace {

using namespace mi;

constexpr int kTile = 64;
constexpr int kBlock = 256;
constexpr int kPitch = kTile + 1;

template <typename T, int N> struct VecOf {
    typedef T type __attribute__((ext_vector_type(N)));
};

// VEC: true  -> every 16-byte vector is either fully inside or fully outside the matrix
//               and 16-byte aligned (checked on the host);
//      false -> element-wise accesses with per-element bounds checks.
template <typename T, bool VEC>
__global__ __launch_bounds__(kBlock) void transpose_kernel(const T* __restrict__ x, int64_t ldx,
                                                           T* __restrict__ y, int64_t ldy,
                                                           int64_t m, int64_t n) {
    constexpr int V = 16 / sizeof(T);        // elements per 16-byte vector
    constexpr int VR = kTile / V;            // vectors per tile row
    constexpr int RP = kBlock / VR;          // tile rows covered per pass
    constexpr int PASSES = kTile / RP;
    using VT = typename VecOf<T, V>::type;
    __shared__ T lds[kTile * kPitch];

    const int64_t m0 = (int64_t)blockIdx.x * kTile;  // along x dim 0
    const int64_t n0 = (int64_t)blockIdx.y * kTile;  // along x dim 1
    const int vi = threadIdx.x % VR, row = threadIdx.x / VR;

    // Phase 1: x[m0 + V*vi .. +V-1, n0 + r]  ->  lds[i][j] with i along m, j along n.
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int j = row + p * RP;
        const int64_t gi = m0 + vi * V, gj = n0 + j;
        if constexpr (VEC) {
            if (gi < m && gj < n) {
                VT v = __builtin_nontemporal_load(reinterpret_cast<const VT*>(x + gi + gj * ldx));
#pragma unroll
                for (int q = 0; q < V; ++q) lds[(vi * V + q) * kPitch + j] = v[q];
            }
        } else {
#pragma unroll
            for (int q = 0; q < V; ++q)
                if (gi + q < m && gj < n) lds[(vi * V + q) * kPitch + j] = x[gi + q + gj * ldx];
        }
    }
    __syncthreads();
    // Phase 2: y[n0 + V*vi .. +V-1, m0 + r]  <-  lds[r][V*vi .. ].
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int i = row + p * RP;
        const int64_t gj = n0 + vi * V, gi = m0 + i;
        if constexpr (VEC) {
            if (gj < n && gi < m) {
                VT v;
#pragma unroll
                for (int q = 0; q < V; ++q) v[q] = lds[i * kPitch + vi * V + q];
                __builtin_nontemporal_store(v, reinterpret_cast<VT*>(y + gj + gi * ldy));
            }
        } else {
#pragma unroll
            for (int q = 0; q < V; ++q)
                if (gj + q < n && gi < m) y[gj + q + gi * ldy] = lds[i * kPitch + vi * V + q];
        }
    }
}

template <typename T>
int launch(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s) {
    constexpr int V = 16 / sizeof(T);
    const int64_t m = x->sizes[0], n = x->sizes[1];
    const int64_t ldx = x->strides[1], ldy = y->strides[1];
    const int64_t gx = cld(m, (int64_t)kTile), gy = cld(n, (int64_t)kTile);
    if (gy > 65535 || gx > 0x7fffffffLL) return MI_E_GRID;
    const bool vec = (m % V == 0) && (n % V == 0) && (ldx % V == 0) && (ldy % V == 0) &&
                     aligned(x->ptr, 16) && aligned(y->ptr, 16);
    dim3 grid((unsigned)gx, (unsigned)gy), block(kBlock);
    if (vec) {
        hipLaunchKernelGGL((transpose_kernel<T, true>), grid, block, 0, s, (const T*)x->ptr, ldx,
                           (T*)y->ptr, ldy, m, n);
        set_variant("transpose_lds64_vec16");
    } else {
        hipLaunchKernelGGL((transpose_kernel<T, false>), grid, block, 0, s, (const T*)x->ptr, ldx,
                           (T*)y->ptr, ldy, m, n);
        set_variant("transpose_lds64_elem");
    }
    return launch_status();
}

}  // namespace

extern "C" int mi_transpose_kernel(const mi_tile_array* x, const mi_tile_array* y, int tm, int tn,
                                   void* stream) {
    MI_CHECK(check_array(x, 2));
    MI_CHECK(check_array(y, 2));
    if (x->dtype != y->dtype) return MI_E_DTYPE;
    if (!is_pow2(tm) || !is_pow2(tn)) return MI_E_TILE;
    if (x->sizes[0] != y->sizes[1] || x->sizes[1] != y->sizes[0]) return MI_E_SHAPE;
    const int64_t m = x->sizes[0], n = x->sizes[1];
    if (cld(m, (int64_t)tm) > MI_MAX_GRID_DIM || cld(n, (int64_t)tn) > MI_MAX_GRID_DIM)
        return MI_E_GRID;
    if (m == 0 || n == 0) return MI_OK;
    if ((m > 1 && x->strides[0] != 1) || (n > 1 && y->strides[0] != 1)) return MI_E_STRIDE;
    if ((n > 1 && x->strides[1] < m) || (m > 1 && y->strides[1] < n)) return MI_E_STRIDE;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype_size(x->dtype)) {
        case 1: return launch<uint8_t>(x, y, s);
        case 2: return launch<uint16_t>(x, y, s);
        case 4: return launch<uint32_t>(x, y, s);
        case 8: return launch<uint64_t>(x, y, s);
        default: return MI_E_DTYPE;
    }
}
