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
//   * everything else (columns that start off 16-byte boundaries): 64 x 64 tiles through a padded LDS tile, one element
//     per lane and access with the lanes of a wave consecutive in memory on both sides, workgroup ids banded by XCD
//     (transpose_elem_kernel).
// Algorithmic traffic: 2 * m * n * sizeof(T) bytes.
#include "common.h"
#include <stdlib.h>

namespace {

using namespace mi;


template <typename T, int N> struct VecOf {
    typedef T type __attribute__((ext_vector_type(N)));
};

// ---- columns that start anywhere: one element per lane and access ------------------------------
// No 16-byte vector is aligned in every column, so a lane moves single elements, and what keeps the memory system
// busy is the shape of a wave's access: 64 lanes on 64 consecutive elements of a column, on the load side (lanes
// along m) and on the store side (lanes along n) alike, with all of a lane's loads issued before the first of them is
// used.  (The padded-tile kernel above gives a lane V consecutive elements, as its vector form wants them: element
// by element a wave's access then covers V times the span at 1/V of the density, and the 8191 x 8193 fp32 case ran at
// 3.0 TB/s.)  The tile sits in LDS with rows of TN + 1 elements: the scattered writes of phase 1 (stride TN + 1
// elements between lanes) and the linear reads of phase 2 both spread over the banks.
// A column of a tile starts and ends inside 128-byte lines that the neighbouring tiles along the column share, on the
// load side (neighbours along m) and on the store side (neighbours along n) alike.  Workgroup ids go round the eight
// XCDs, each with an L2 of its own: id % 8 therefore selects a band of tile rows along m, and the ids of one XCD walk
// their band m-fastest, so that the workgroups resident on an XCD at one time cover a compact patch of tiles and both
// kinds of neighbours meet in the same L2 (a shared line is fetched once and written back whole).
template <typename T, int TM, int TN, int NT>
__global__ __launch_bounds__(NT) void transpose_elem_kernel(const T* __restrict__ x, int64_t ldx, T* __restrict__ y,
                                                            int64_t ldy, int64_t m, int64_t n, int tiles_m, int band) {
    constexpr int kPitch = TN + 1;
    __shared__ T lds[TM * kPitch];
    constexpr int LM = TM < NT ? TM : NT, CJ = NT / LM, P1 = TN / CJ;   // phase 1: LM lanes along m, CJ columns per pass
    constexpr int LN = TN < NT ? TN : NT, CI = NT / LN, P2 = TM / CI;   // phase 2: LN lanes along n, CI rows per pass
    static_assert(LM * CJ == NT && CJ * P1 == TN && LN * CI == NT && CI * P2 == TM && LM == TM && LN == TN, "the lanes tile the block");
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int bm = xcd * band + seq % band;
    if (bm >= tiles_m || seq % band >= band) return;   // (the last band may be short; the whole workgroup leaves)
    const int64_t m0 = (int64_t)bm * TM, n0 = (int64_t)(seq / band) * TN;
    const int i1 = threadIdx.x % LM, j1 = threadIdx.x / LM;
    const int j2 = threadIdx.x % LN, i2 = threadIdx.x / LN;
    T v[P1];
    const bool in_m = m0 + i1 < m;
#pragma unroll
    for (int p = 0; p < P1; ++p) {
        const int64_t gj = n0 + j1 + p * CJ;
        v[p] = in_m && gj < n ? x[m0 + i1 + gj * ldx] : T(0);
    }
#pragma unroll
    for (int p = 0; p < P1; ++p) lds[i1 * kPitch + j1 + p * CJ] = v[p];
    __syncthreads();
    const bool in_n = n0 + j2 < n;
#pragma unroll
    for (int p = 0; p < P2; ++p) {
        const int64_t gi = m0 + i2 + p * CI;
        if (in_n && gi < m) y[n0 + j2 + gi * ldy] = lds[(i2 + p * CI) * kPitch + j2];
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

template <typename T, int TM, int TN, int NT>
int launch_elem(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s, const char* name) {
    const int64_t m = x->sizes[0], n = x->sizes[1];
    const int64_t tiles_m = cld(m, (int64_t)TM), tiles_n = cld(n, (int64_t)TN);
    const int64_t band = cld(tiles_m, (int64_t)8);   // tile rows per XCD
    if (tiles_m > 0x7fffffffLL || 8 * band * tiles_n > 0x7fffffffLL) return MI_E_GRID;
    hipLaunchKernelGGL((transpose_elem_kernel<T, TM, TN, NT>), dim3((unsigned)(8 * band * tiles_n)), dim3(NT), 0, s,
                       (const T*)x->ptr, x->strides[1], (T*)y->ptr, y->strides[1], m, n, (int)tiles_m, (int)band);
    set_variant(name);
    return launch_status();
}

// Sizes or strides that rule out the register micro-transpose.
template <typename T>
int launch(const mi_tile_array* x, const mi_tile_array* y, hipStream_t s) {
    int shape = 0;
    if (const char* e = getenv("MI_TRANSPOSE_ELEM_TILE")) shape = atoi(e);
    if (shape == 3) return launch_elem<T, 128, 128, 1024>(x, y, s, "transpose_elem_128x128_t1024");
    return launch_elem<T, 64, 64, 256>(x, y, s, "transpose_elem_64x64_t256");
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
