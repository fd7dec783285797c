// Matrix transpose: stand-in for transpose_kernel of the reference's examples/transpose.jl:11-19,
// y[j,i] = x[i,j] for x (m,n) and y (n,m), both with dimension 0 contiguous.
//
// The result does not depend on the (tm,tn) tile constants, so the physical tiling is the
// library's.  Two kernels:
//   * 1-, 2-, 4- and 8-byte elements with every dimension and stride a multiple of a 16-byte vector
//     (the benchmark case is 4-byte: 128 x 128 tiles of 1024 lanes, 64 x 128 of 256 lanes for
//     small matrices): a V x V block per lane transposed in registers, 16-byte traffic through an
//     XOR-swizzled LDS tile in both directions, workgroup ids walking 8x8 super-tiles
//     (transpose_micro_kernel);
//     sizes that are not multiples of a vector are taken too when the leading dimensions are (edge tiles element-wise);
//   * everything else: 64x64 (large 2- and 4-byte matrices: 128x128) tiles through a padded LDS tile (pitch + 1
//     element: both the scattered writes and the gathered reads hit distinct banks), 16-byte global accesses
//     where alignment allows, element-wise with bounds checks otherwise (transpose_kernel).
// Algorithmic traffic: 2 * m * n * sizeof(T) bytes.
#include "common.h"
#include <stdlib.h>

namespace {

using namespace mi;


template <typename T, int N> struct VecOf {
    typedef T type __attribute__((ext_vector_type(N)));
};

// VEC: true  -> every 16-byte vector is either fully inside or fully outside the matrix
//               and 16-byte aligned (checked on the host);
//      false -> element-wise accesses with per-element bounds checks.
template <typename T, bool VEC, int kTile = 64, int kBlock = 256>
__global__ __launch_bounds__(kBlock) void transpose_kernel(const T* __restrict__ x, int64_t ldx,
                                                           T* __restrict__ y, int64_t ldy,
                                                           int64_t m, int64_t n) {
    constexpr int V = 16 / sizeof(T);        // elements per 16-byte vector
    constexpr int VR = kTile / V;            // vectors per tile row
    constexpr int RP = kBlock / VR;          // tile rows covered per pass
    constexpr int PASSES = kTile / RP;
    using VT = typename VecOf<T, V>::type;
    constexpr int kPitch = kTile + 1;
    __shared__ T lds[kTile * kPitch];

    const int64_t m0 = (int64_t)blockIdx.x * kTile;  // along x dim 0
    const int vi = threadIdx.x % VR, row = threadIdx.x / VR;
    // (the second grid dimension holds at most 65535 workgroups: walk the tile rows along dim 1 with that stride)
    for (int64_t n0 = (int64_t)blockIdx.y * kTile; n0 < n; n0 += (int64_t)gridDim.y * kTile) {
    // Phase 1: x[m0 + V*vi .. +V-1, n0 + r]  ->  lds[i][j] with i along m, j along n.
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int j = row + p * RP;
        const int64_t gi = m0 + vi * V, gj = n0 + j;
        if constexpr (VEC) {
            if (gi < m && gj < n) {
                VT v = ld_global<true>(reinterpret_cast<const VT*>(x + gi + gj * ldx));
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
                st_global<true>(v, reinterpret_cast<VT*>(y + gj + gi * ldy));
            }
        } else {
#pragma unroll
            for (int q = 0; q < V; ++q)
                if (gj + q < n && gi < m) y[gj + q + gi * ldy] = lds[i * kPitch + vi * V + q];
        }
    }
    __syncthreads();   // the tile is free for the next trip
    }
}

// ---- every dimension a multiple of a 16-byte vector: V x V register micro-transpose -----------
// V = 16 / sizeof(T) elements fill a 16-byte vector (2, 4, 8 or 16).  A lane loads a V(m) x V(n) block
// as V vectors along m, transposes it in registers, and passes V vectors along n through an LDS
// tile L[m][n] whose 16-byte slots are XOR-swizzled with (m / V) so that both the writes (lanes
// differ in m) and the reads (lanes differ in n) of a quarter-wave cover all 64 banks.  All LDS
// traffic is 128-bit.
// ORDER selects how workgroup ids walk the tile grid (the workgroups that run at the same
// time decide how large the contiguous spans are that DRAM sees on each side).
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// NT lanes per workgroup.  For 4-byte elements two shapes are used: 128 x 128 tiles with 1024 lanes
// (one 4x4 block per lane) for large matrices -- runs of 512 bytes on both sides, which is what the
// memory system needs to move a strided run at the rate of a linear copy, and two workgroups fill a
// CU -- and 64 x 128 tiles with 256 lanes (five workgroups per CU) when there are too few tiles for
// that.  The 2- and 8-byte shapes are chosen the same way (launch_micro).
// RAGGED: m or n is not a multiple of V (the leading dimensions still are, so every vector inside the matrix is
// aligned: a view of a padded parent).  Tiles on the edge then load and store the vectors that cross it element by
// element; interior tiles are unaffected.
template <typename T, int TM, int TN, bool STREAM = true, int NT = 256, bool RAGGED = false>
__global__ __launch_bounds__(NT) void transpose_micro_kernel(const T* __restrict__ x, int64_t ldx,
                                                              T* __restrict__ y, int64_t ldy, int64_t m,
                                                              int64_t n, int tiles_m, int tiles_n, int order) {
    constexpr int V = 16 / sizeof(T);
    using VT = typename VecOf<T, V>::type;
    __shared__ __attribute__((aligned(16))) T lds[TM * TN];
    constexpr int MB = TM * TN / (V * V * NT);   // V x V micro-blocks per lane
    constexpr int SLOTS = TN / V;                // 16-byte slots per LDS row
    static_assert(MB >= 1 && MB * V * V * NT == TM * TN, "the lanes must tile the block evenly");
    static_assert(SLOTS >= 16 && (SLOTS & (SLOTS - 1)) == 0, "a quarter-wave must find 16 distinct slots");
    int bm, bn;
    {
        const int id = blockIdx.x;
        if (order == 0) { bm = id % tiles_m; bn = id / tiles_m; }
        else if (order == 1) { bn = id % tiles_n; bm = id / tiles_n; }
        else {  // 8 x 8 super-tiles, m fastest inside
            const int sm = (tiles_m + 7) / 8;
            const int st = id / 64, in = id % 64;
            bm = (st % sm) * 8 + (in % 8);
            bn = (st / sm) * 8 + (in / 8);
            if (bm >= tiles_m || bn >= tiles_n) return;
        }
    }
    const int64_t m0 = (int64_t)bm * TM, n0 = (int64_t)bn * TN;
    // A tile that lies wholly inside the matrix is moved without predicates: a predicated load has
    // to be waited for before the other side of its branch may write the same registers, which
    // would leave a lane with one load in flight instead of V.
    const bool interior = m0 + TM <= m && n0 + TN <= n;
#pragma unroll
    for (int k = 0; k < MB; ++k) {
        const int b = threadIdx.x + NT * k;
        const int iv = b % (TM / V), jv = b / (TM / V);
        const int64_t gm = m0 + V * iv, gn = n0 + V * jv;
        VT r[V] = {};
        if (interior) {
#pragma unroll
            for (int c = 0; c < V; ++c) r[c] = ld_global<STREAM>(reinterpret_cast<const VT*>(x + gm + (gn + c) * ldx));
        } else if (gm < m) {
#pragma unroll
            for (int c = 0; c < V; ++c)
                if (gn + c < n) {
                    if (!RAGGED || gm + V <= m) {
                        r[c] = ld_global<STREAM>(reinterpret_cast<const VT*>(x + gm + (gn + c) * ldx));
                    } else {
#pragma unroll
                        for (int q = 0; q < V; ++q)
                            if (gm + q < m) r[c][q] = x[gm + q + (gn + c) * ldx];
                    }
                }
        }
#pragma unroll
        for (int q = 0; q < V; ++q) {
            VT t;                                            // x[m+q, n..n+V-1]
#pragma unroll
            for (int c = 0; c < V; ++c) t[c] = r[c][q];
            const int row = V * iv + q;
            *reinterpret_cast<VT*>(&lds[row * TN + V * (jv ^ (iv & (SLOTS - 1)))]) = t;
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < V * MB; ++k) {
        const int b = threadIdx.x + NT * k;
        const int jv = b % SLOTS, row = b / SLOTS;
        const int64_t gn = n0 + V * jv, gm = m0 + row;
        if (interior || (gn < n && gm < m)) {
            VT t = *reinterpret_cast<const VT*>(&lds[row * TN + V * (jv ^ ((row / V) & (SLOTS - 1)))]);
            if (!RAGGED || interior || gn + V <= n) {
                st_global<true>(t, reinterpret_cast<VT*>(y + gn + gm * ldy));
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (gn + e < n) y[gn + e + gm * ldy] = t[e];
            }
        }
    }
}

template <typename T, int TM, int TN, int NT>
int launch_micro_as(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, const char* name_stream,
                    const char* name_cached, bool ragged);

int launch4(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, bool ragged) {
    const int64_t m = x->sizes[0], n = x->sizes[1];
    if (ragged)
        return cld(m, (int64_t)128) * cld(n, (int64_t)128) >= 1024
                   ? launch_micro_as<unsigned, 128, 128, 1024>(x, y, s, "transpose4_128x128_t1024_regmicro_ragged", "", true)
                   : launch_micro_as<unsigned, 64, 128, 256>(x, y, s, "transpose4_64x128_regmicro_ragged", "", true);
    // measured best on MI355X for 8192^2 fp32: 128 x 128 tiles of 1024 lanes, 8x8 super-tiles (90 us; 64 x 128
    // tiles of 256 lanes 104 us); the big shape needs enough tiles to keep two workgroups on every CU
    int tile = cld(m, (int64_t)128) * cld(n, (int64_t)128) >= 1024 ? 9 : 2, order = 2;
    if (const char* e = getenv("MI_TRANSPOSE_TILE")) tile = atoi(e);    // tuning overrides
    if (const char* e = getenv("MI_TRANSPOSE_ORDER")) order = atoi(e);
    int TM = 64, TN = 128;
    if (tile == 128) { TM = 128; TN = 128; }
    else if (tile == 2) { TM = 64; TN = 128; }
    else if (tile == 3) { TM = 128; TN = 64; }
    else if (tile == 4) { TM = 32; TN = 256; }
    else if (tile == 5) { TM = 64; TN = 256; }
    else if (tile == 6) { TM = 32; TN = 128; }
    else if (tile == 64) { TM = 64; TN = 64; }
    else if (tile == 9) { TM = 128; TN = 128; }   // with 1024 lanes
    const int64_t tm_ = cld(m, (int64_t)TM), tn_ = cld(n, (int64_t)TN);
    int64_t blocks = tm_ * tn_;
    if (order == 2) blocks = ((tm_ + 7) / 8) * ((tn_ + 7) / 8) * 64;
    if (blocks > 0x7fffffffLL || tm_ > 0x3fffffff || tn_ > 0x3fffffff) return MI_E_GRID;
#define T4(A, B)                                                                                          \
    hipLaunchKernelGGL((transpose_micro_kernel<unsigned, A, B>), dim3((unsigned)blocks), dim3(256), 0, s,                \
                       (const unsigned*)x->ptr, x->strides[1], (unsigned*)y->ptr, y->strides[1], m, n,    \
                       (int)tm_, (int)tn_, order)
    if (tile == 9) {
        const bool st = stream_hint(2 * m * n * (int64_t)sizeof(unsigned));
        if (st) hipLaunchKernelGGL((transpose_micro_kernel<unsigned, 128, 128, true, 1024>), dim3((unsigned)blocks), dim3(1024), 0, s,
                                   (const unsigned*)x->ptr, x->strides[1], (unsigned*)y->ptr, y->strides[1], m, n, (int)tm_, (int)tn_, order);
        else hipLaunchKernelGGL((transpose_micro_kernel<unsigned, 128, 128, false, 1024>), dim3((unsigned)blocks), dim3(1024), 0, s,
                                (const unsigned*)x->ptr, x->strides[1], (unsigned*)y->ptr, y->strides[1], m, n, (int)tm_, (int)tn_, order);
        set_variant(st ? "transpose4_128x128_t1024_regmicro" : "transpose4_128x128_t1024_regmicro_cached");
    } else if (TM == 64 && TN == 64) { T4(64, 64); set_variant("transpose4_64x64_regmicro"); }
    else if (TM == 128 && TN == 128) { T4(128, 128); set_variant("transpose4_128x128_regmicro"); }
    else if (TM == 32 && TN == 256) { T4(32, 256); set_variant("transpose4_32x256_regmicro"); }
    else if (TM == 64 && TN == 256) { T4(64, 256); set_variant("transpose4_64x256_regmicro"); }
    else if (TM == 32 && TN == 128) { T4(32, 128); set_variant("transpose4_32x128_regmicro"); }
    else if (TM == 64 && !stream_hint(2 * m * n * (int64_t)sizeof(unsigned))) {
        hipLaunchKernelGGL((transpose_micro_kernel<unsigned, 64, 128, false>), dim3((unsigned)blocks), dim3(256), 0, s,
                           (const unsigned*)x->ptr, x->strides[1], (unsigned*)y->ptr, y->strides[1], m, n,
                           (int)tm_, (int)tn_, order);
        set_variant("transpose4_64x128_regmicro_cached");
    } else if (TM == 64) { T4(64, 128); set_variant("transpose4_64x128_regmicro"); }
    else { T4(128, 64); set_variant("transpose4_128x64_regmicro"); }
#undef T4
    return launch_status();
}

// 2- and 8-byte elements through the same kernel.  `tile` picks the shape (MI_TRANSPOSE_TILE
// overrides it for tuning): the large shapes keep runs of at least 512 bytes on both sides.
template <typename T, int TM, int TN, int NT>
int launch_micro_as(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, const char* name_stream,
                    const char* name_cached, bool ragged) {
    const int64_t m = x->sizes[0], n = x->sizes[1];
    const int64_t tm_ = cld(m, (int64_t)TM), tn_ = cld(n, (int64_t)TN);
    const int64_t blocks = ((tm_ + 7) / 8) * ((tn_ + 7) / 8) * 64;
    if (blocks > 0x7fffffffLL || tm_ > 0x3fffffff || tn_ > 0x3fffffff) return MI_E_GRID;
    const bool st = stream_hint(2 * m * n * (int64_t)sizeof(T));
    if (ragged) {
        hipLaunchKernelGGL((transpose_micro_kernel<T, TM, TN, true, NT, true>), dim3((unsigned)blocks), dim3(NT), 0, s,
                           (const T*)x->ptr, x->strides[1], (T*)y->ptr, y->strides[1], m, n, (int)tm_, (int)tn_, 2);
        set_variant(name_stream);
        return launch_status();
    }
    if (st) hipLaunchKernelGGL((transpose_micro_kernel<T, TM, TN, true, NT>), dim3((unsigned)blocks), dim3(NT), 0, s,
                               (const T*)x->ptr, x->strides[1], (T*)y->ptr, y->strides[1], m, n, (int)tm_, (int)tn_, 2);
    else hipLaunchKernelGGL((transpose_micro_kernel<T, TM, TN, false, NT>), dim3((unsigned)blocks), dim3(NT), 0, s,
                            (const T*)x->ptr, x->strides[1], (T*)y->ptr, y->strides[1], m, n, (int)tm_, (int)tn_, 2);
    set_variant(st ? name_stream : name_cached);
    return launch_status();
}

// measured on MI355X, 8192^2: 8-byte 205 us with 128 x 64 tiles of 1024 lanes (64 x 64 of 256 lanes 221 us; the
// padded-tile kernel 305 us); 2-byte 51 us with 256 x 256 tiles of 1024 lanes (128 x 128 of 256 lanes 56 us; the
// padded-tile kernel 67 us).  At 4096^2 the smaller tiles win, there are too few of the large ones to fill the chip.
int launch8(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, bool ragged) {
    const int64_t m = x->sizes[0], n = x->sizes[1];
    const int64_t t64 = cld(m, (int64_t)64) * cld(n, (int64_t)64);
    if (ragged)
        return t64 >= 1024 ? launch_micro_as<uint64_t, 64, 64, 1024>(x, y, s, "transpose8_64x64_t1024_regmicro_ragged", "", true)
                           : launch_micro_as<uint64_t, 64, 64, 256>(x, y, s, "transpose8_64x64_regmicro_ragged", "", true);
    int tile = t64 >= 8192 ? 3 : t64 >= 1024 ? 2 : 0;
    if (const char* e = getenv("MI_TRANSPOSE_TILE")) tile = atoi(e);
    switch (tile) {
        case 1: return launch_micro_as<uint64_t, 64, 128, 1024>(x, y, s, "transpose8_64x128_t1024_regmicro", "transpose8_64x128_t1024_regmicro_cached", false);
        case 2: return launch_micro_as<uint64_t, 64, 64, 1024>(x, y, s, "transpose8_64x64_t1024_regmicro", "transpose8_64x64_t1024_regmicro_cached", false);
        case 3: return launch_micro_as<uint64_t, 128, 64, 1024>(x, y, s, "transpose8_128x64_t1024_regmicro", "transpose8_128x64_t1024_regmicro_cached", false);
        case 4: return launch_micro_as<uint64_t, 32, 128, 256>(x, y, s, "transpose8_32x128_regmicro", "transpose8_32x128_regmicro_cached", false);
        default: return launch_micro_as<uint64_t, 64, 64, 256>(x, y, s, "transpose8_64x64_regmicro", "transpose8_64x64_regmicro_cached", false);
    }
}

int launch2(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, bool ragged) {
    const int64_t m = x->sizes[0], n = x->sizes[1];
    const int64_t t128 = cld(m, (int64_t)128) * cld(n, (int64_t)128);
    if (ragged)
        return t128 >= 1024 ? launch_micro_as<uint16_t, 128, 256, 512>(x, y, s, "transpose2_128x256_t512_regmicro_ragged", "", true)
                            : launch_micro_as<uint16_t, 128, 128, 256>(x, y, s, "transpose2_128x128_regmicro_ragged", "", true);
    int tile = t128 >= 4096 ? 3 : t128 >= 1024 ? 2 : 0;
    if (const char* e = getenv("MI_TRANSPOSE_TILE")) tile = atoi(e);
    switch (tile) {
        case 1: return launch_micro_as<uint16_t, 256, 128, 512>(x, y, s, "transpose2_256x128_t512_regmicro", "transpose2_256x128_t512_regmicro_cached", false);
        case 2: return launch_micro_as<uint16_t, 128, 256, 512>(x, y, s, "transpose2_128x256_t512_regmicro", "transpose2_128x256_t512_regmicro_cached", false);
        case 3: return launch_micro_as<uint16_t, 256, 256, 1024>(x, y, s, "transpose2_256x256_t1024_regmicro", "transpose2_256x256_t1024_regmicro_cached", false);
        case 4: return launch_micro_as<uint16_t, 256, 128, 256>(x, y, s, "transpose2_256x128_regmicro", "transpose2_256x128_regmicro_cached", false);
        default: return launch_micro_as<uint16_t, 128, 128, 256>(x, y, s, "transpose2_128x128_regmicro", "transpose2_128x128_regmicro_cached", false);
    }
}

// 1-byte, measured: 16384^2 103 us with 256 x 512 tiles of 512 lanes (256 x 256 of 256 lanes 118 us); 8192^2 22 us
// with 256 x 256 (24 us with 256 x 512; the padded-tile kernel 46 us)
int launch1(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, bool ragged) {
    const int64_t m = x->sizes[0], n = x->sizes[1];
    if (ragged) return launch_micro_as<uint8_t, 256, 256, 256>(x, y, s, "transpose1_256x256_regmicro_ragged", "", true);
    int tile = cld(m, (int64_t)256) * cld(n, (int64_t)256) >= 4096 ? 2 : 0;
    if (const char* e = getenv("MI_TRANSPOSE_TILE")) tile = atoi(e);
    switch (tile) {
        case 1: return launch_micro_as<uint8_t, 512, 256, 512>(x, y, s, "transpose1_512x256_t512_regmicro", "transpose1_512x256_t512_regmicro_cached", false);
        case 2: return launch_micro_as<uint8_t, 256, 512, 512>(x, y, s, "transpose1_256x512_t512_regmicro", "transpose1_256x512_t512_regmicro_cached", false);
        default: return launch_micro_as<uint8_t, 256, 256, 256>(x, y, s, "transpose1_256x256_regmicro", "transpose1_256x256_regmicro_cached", false);
    }
}

template <typename T, int TILE, int BLOCK>
int launch_tile(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s) {
    constexpr int V = 16 / sizeof(T);
    const int64_t m = x->sizes[0], n = x->sizes[1];
    const int64_t ldx = x->strides[1], ldy = y->strides[1];
    const int64_t gx = cld(m, (int64_t)TILE), gy = cld(n, (int64_t)TILE);
    if (gx > 0x7fffffffLL) return MI_E_GRID;
    const bool vec = (m % V == 0) && (n % V == 0) && (ldx % V == 0) && (ldy % V == 0) &&
                     aligned(x->ptr, 16) && aligned(y->ptr, 16);
    dim3 grid((unsigned)gx, (unsigned)(gy < 65535 ? gy : 65535)), block(BLOCK);
    if (vec) {
        hipLaunchKernelGGL((transpose_kernel<T, true, TILE, BLOCK>), grid, block, 0, s, (const T*)x->ptr, ldx,
                           (T*)y->ptr, ldy, m, n);
        set_variant(TILE == 64 ? "transpose_lds64_vec16" : "transpose_lds128_vec16");
    } else {
        hipLaunchKernelGGL((transpose_kernel<T, false, TILE, BLOCK>), grid, block, 0, s, (const T*)x->ptr, ldx,
                           (T*)y->ptr, ldy, m, n);
        set_variant(TILE == 64 ? "transpose_lds64_elem" : "transpose_lds128_elem");
    }
    return launch_status();
}

// Sizes or strides that rule out the register micro-transpose.  Large matrices of 2- and 4-byte elements take
// 128 x 128 tiles of 1024 lanes (runs of 256 / 512 bytes instead of 128 / 256).
template <typename T>
int launch(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s) {
    int big = sizeof(T) <= 4 && sizeof(T) >= 2 && cld(x->sizes[0], (int64_t)128) * cld(x->sizes[1], (int64_t)128) >= 512;
    if (const char* e = getenv("MI_TRANSPOSE_FALLBACK_TILE")) big = atoi(e) == 128 && sizeof(T) <= 4;
    if constexpr (sizeof(T) <= 4) {
        if (big) return launch_tile<T, 128, 1024>(x, y, s);
    }
    return launch_tile<T, 64, 256>(x, y, s);
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
    // the register micro-transpose moves whole 16-byte vectors of v elements on both sides
    // 0: not possible; 1: whole vectors everywhere; 2: aligned columns, but m or n is not a multiple of v (edge tiles
    // move the vectors that cross the edge element by element)
    auto micro = [&](int v) {
        if (!((n == 1 || x->strides[1] % v == 0) && (m == 1 || y->strides[1] % v == 0) && aligned(x->ptr, 16) && aligned(y->ptr, 16)))
            return 0;
        return m % v == 0 && n % v == 0 ? 1 : 2;
    };
    switch (dtype_size(x->dtype)) {
        case 1: return micro(16) ? launch1(x, y, s, micro(16) == 2) : launch<uint8_t>(x, y, s);
        case 2: return micro(8) ? launch2(x, y, s, micro(8) == 2) : launch<uint16_t>(x, y, s);
        case 4: return micro(4) ? launch4(x, y, s, micro(4) == 2) : launch<uint32_t>(x, y, s);
        case 8: return micro(2) ? launch8(x, y, s, micro(2) == 2) : launch<uint64_t>(x, y, s);
        default: return MI_E_DTYPE;
    }
}
