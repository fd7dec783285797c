// Host-level RNG fills: stand-ins for rand_fill_kernel / randn_fill_kernel / randexp_fill_kernel of the
// reference (src/language/random.jl:703-740) as launched by Random.rand! / randn! / randexp! on a
// cuTile.RNG (src/language/random.jl:759-818).
//
// The stream is the reference's, value for value: one logical block per 512 outputs, block b keyed
// with (b * W) ^ seed, Philox2x32-7 on the counters counter + i, and the reference's placement of a
// block's (c1, c2) outputs in its 512 slots, which depends on the element width:
//   4 bytes: 256 calls, c1 -> slot i, c2 -> slot 256 + i                        (random.jl:262-286)
//   8 bytes: 512 calls, c1 | c2 << 32 -> slot i                                 (random.jl:290-305)
//   2 bytes: 128 calls -> 256 words (c1s then c2s); low half of word m -> slot m,
//            high half -> slot 256 + m                                          (random.jl:314-324)
//   1 byte:   64 calls -> 128 words; byte q of word m -> slot 128 q + m          (random.jl:326-338)
// Integers take the bits, floats go through u01 (random.jl:136-174).  randn is Box-Muller on the
// (c1, c2) pair in Float32 (Float64: the pair of 64-bit words from counters i and 256 + i)
// (random.jl:369-480); randexp is -log(rand) (random.jl:500-501).
//
// Mapping to the chip: a lane runs four Philox calls with consecutive counters, so every store is
// 16 bytes (4-byte types) down to 4 bytes (1-byte types) of consecutive slots; the 64-bit product
// c1 * M is one v_mad_u64_u32.  The Float32 log, square root, sine and cosine are the hardware's
// (as the reference's are, random.jl:358-359): the angle 2 pi u is a fraction of a revolution,
// which is the unit the sine and cosine instructions take, so no range reduction is needed, and
// a standard normal differs from the exactly rounded formula by at most 2e-6 in absolute terms.
// Uniform, normal and exponential fills of 4-byte types then all run at the HBM write rate;
// Float64 normals use the library's log / sincos and are bound by them.
#include "common.h"

namespace {

using namespace mi;

constexpr unsigned kPhiloxM = 0xD256D193u;   // random.jl:93
constexpr unsigned kPhiloxW = 0x9E3779B9u;   // random.jl:94
constexpr int kFillTile = 512;               // RAND_FILL_TILE, random.jl:701

enum Dist { kRand = 0, kRandn = 1, kRandexp = 2 };

__device__ __forceinline__ void philox7(unsigned& c1, unsigned& c2, unsigned k) {
#pragma unroll
    for (int r = 0; r < 7; ++r) {
        if (r) k += kPhiloxW;
        const unsigned long long p = (unsigned long long)c1 * kPhiloxM;
        c1 = (unsigned)(p >> 32) ^ k ^ c2;
        c2 = (unsigned)p;
    }
}

__device__ __forceinline__ float u01_f32(unsigned u) { return __uint2float_rn(u) * 0x1p-32f + 0x1p-33f; }
__device__ __forceinline__ double u01_f64(unsigned long long u) {
    return __longlong_as_double((long long)((u >> 12) | 0x3FF0000000000001ull)) - 1.0;
}
__device__ __forceinline__ unsigned short u01_f16_bits(unsigned short u) {
    const _Float16 v = __builtin_bit_cast(_Float16, (unsigned short)((u >> 6) | 0x3C01u)) - (_Float16)1.0f;
    return __builtin_bit_cast(unsigned short, v);
}
__device__ __forceinline__ unsigned short u01_bf16_bits(unsigned short u) {
    const float v = __uint_as_float((unsigned)((u >> 9) | 0x3F81u) << 16) - 1.0f;   // exact: at most 8 significant bits
    return (unsigned short)(__float_as_uint(v) >> 16);
}
__device__ __forceinline__ unsigned short f32_to_bf16_bits(float x) {
    unsigned u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ unsigned short f32_to_f16_bits(float x) { return __builtin_bit_cast(unsigned short, (_Float16)x); }

// Four consecutive slots starting at `pos` (a multiple of 4): one vector store when they all exist.
template <typename T, bool VEC>
__device__ __forceinline__ void store4(T* out, long long pos, long long n, const T (&v)[4]) {
    if (VEC && pos + 4 <= n) {
        typedef T V4 __attribute__((ext_vector_type(4)));
        V4 w = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(w, reinterpret_cast<V4*>(out + pos));
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) if (pos + e < n) out[pos + e] = v[e];
    }
}

enum Kind { K_INT, K_F32, K_F16, K_BF16, K_F64 };

// WIDTH: bytes per element.  T: unsigned storage type of that width.
template <int WIDTH, typename T, int KIND, int DIST, bool VEC>
__global__ __launch_bounds__(256) void rng_fill_kernel(T* __restrict__ out, long long n, unsigned seed, unsigned counter) {
    // Philox calls per logical block of 512 outputs
    constexpr int CPB = (DIST == kRandn) ? 256 : (WIDTH == 4 ? 256 : WIDTH == 8 ? 512 : WIDTH == 2 ? 128 : 64);
    const long long call0 = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;      // first of this lane's four calls
    const long long b = call0 / CPB;
    const int j = (int)(call0 - b * CPB);
    const long long base = b * kFillTile;
    if (base >= n) return;
    const unsigned key = ((unsigned)b * kPhiloxW) ^ seed;
    unsigned c1[4], c2[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        c1[e] = counter + (unsigned)(j + e);
        c2[e] = 0;
        philox7(c1[e], c2[e], key);
    }
    if constexpr (DIST == kRandn) {
        if constexpr (KIND == K_F64) {
            unsigned d1[4], d2[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                d1[e] = counter + (unsigned)(256 + j + e);
                d2[e] = 0;
                philox7(d1[e], d2[e], key);
            }
            unsigned long long s[4], c[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const double f1 = u01_f64((unsigned long long)c1[e] | ((unsigned long long)c2[e] << 32));
                const double f2 = u01_f64((unsigned long long)d1[e] | ((unsigned long long)d2[e] << 32));
                const double r = sqrt(-2.0 * log(f1)), ang = 6.283185307179586 * f2;
                double sn, cs;
                sincos(ang, &sn, &cs);
                s[e] = (unsigned long long)__double_as_longlong(r * sn);
                c[e] = (unsigned long long)__double_as_longlong(r * cs);
            }
            store4<T, VEC>(out, base + j, n, reinterpret_cast<const T(&)[4]>(s));
            store4<T, VEC>(out, base + 256 + j, n, reinterpret_cast<const T(&)[4]>(c));
        } else {
            T s[4], c[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float f1 = u01_f32(c1[e]), f2 = u01_f32(c2[e]);
                // The hardware's sine and cosine take their argument in revolutions: f1 in (0, 1] is the
                // angle 2 pi f1 of the reference (src/language/random.jl:368-370), with no range reduction.
                const float r = __builtin_amdgcn_sqrtf(-2.0f * __logf(f2));
                const float sn = __builtin_amdgcn_sinf(f1), cs = __builtin_amdgcn_cosf(f1);
                const float n1 = r * sn, n2 = r * cs;
                if constexpr (KIND == K_F32) { s[e] = (T)__float_as_uint(n1); c[e] = (T)__float_as_uint(n2); }
                else if constexpr (KIND == K_F16) { s[e] = (T)f32_to_f16_bits(n1); c[e] = (T)f32_to_f16_bits(n2); }
                else { s[e] = (T)f32_to_bf16_bits(n1); c[e] = (T)f32_to_bf16_bits(n2); }
            }
            store4<T, VEC>(out, base + j, n, s);
            store4<T, VEC>(out, base + 256 + j, n, c);
        }
        return;
    }
    // uniform draw in the element type (then -log for randexp)
    auto fin32 = [](unsigned u) -> unsigned {
        if constexpr (KIND == K_F32) {
            float v = u01_f32(u);
            if constexpr (DIST == kRandexp) v = -__logf(v);
            return __float_as_uint(v);
        } else return u;
    };
    auto fin16 = [](unsigned short u) -> unsigned short {
        if constexpr (KIND == K_F16) {
            unsigned short b = u01_f16_bits(u);
            if constexpr (DIST == kRandexp) b = f32_to_f16_bits(-__logf((float)__builtin_bit_cast(_Float16, b)));
            return b;
        } else if constexpr (KIND == K_BF16) {
            unsigned short b = u01_bf16_bits(u);
            if constexpr (DIST == kRandexp) b = f32_to_bf16_bits(-__logf(__uint_as_float((unsigned)b << 16)));
            return b;
        } else return u;
    };
    if constexpr (WIDTH == 4) {
        T a[4], c[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) { a[e] = (T)fin32(c1[e]); c[e] = (T)fin32(c2[e]); }
        store4<T, VEC>(out, base + j, n, a);
        store4<T, VEC>(out, base + 256 + j, n, c);
    } else if constexpr (WIDTH == 8) {
        T a[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            unsigned long long u = (unsigned long long)c1[e] | ((unsigned long long)c2[e] << 32);
            if constexpr (KIND == K_F64) {
                double v = u01_f64(u);
                if constexpr (DIST == kRandexp) v = -log(v);
                u = (unsigned long long)__double_as_longlong(v);
            }
            a[e] = (T)u;
        }
        store4<T, VEC>(out, base + j, n, a);
    } else if constexpr (WIDTH == 2) {
        T lo1[4], hi1[4], lo2[4], hi2[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo1[e] = (T)fin16((unsigned short)c1[e]); hi1[e] = (T)fin16((unsigned short)(c1[e] >> 16));
            lo2[e] = (T)fin16((unsigned short)c2[e]); hi2[e] = (T)fin16((unsigned short)(c2[e] >> 16));
        }
        store4<T, VEC>(out, base + j, n, lo1);
        store4<T, VEC>(out, base + 128 + j, n, lo2);
        store4<T, VEC>(out, base + 256 + j, n, hi1);
        store4<T, VEC>(out, base + 384 + j, n, hi2);
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            T a[4], c[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) { a[e] = (T)(c1[e] >> (8 * q)); c[e] = (T)(c2[e] >> (8 * q)); }
            store4<T, VEC>(out, base + 128 * q + j, n, a);
            store4<T, VEC>(out, base + 128 * q + 64 + j, n, c);
        }
    }
}

template <int WIDTH, typename T, int KIND, int DIST>
int launch_kind(const mi_tile_array* out, long long n, unsigned seed, unsigned counter, hipStream_t s) {
    constexpr int CPB = (DIST == kRandn) ? 256 : (WIDTH == 4 ? 256 : WIDTH == 8 ? 512 : WIDTH == 2 ? 128 : 64);
    const long long blocks512 = cld(n, (int64_t)kFillTile);
    const long long lanes = blocks512 * (CPB / 4);
    const long long grid = cld(lanes, (int64_t)256);
    if (grid > 0x7fffffffLL) return MI_E_GRID;
    const bool vec = aligned(out->ptr, 4 * WIDTH);
    if (vec) hipLaunchKernelGGL((rng_fill_kernel<WIDTH, T, KIND, DIST, true>), dim3((unsigned)grid), dim3(256), 0, s, (T*)out->ptr, n, seed, counter);
    else hipLaunchKernelGGL((rng_fill_kernel<WIDTH, T, KIND, DIST, false>), dim3((unsigned)grid), dim3(256), 0, s, (T*)out->ptr, n, seed, counter);
    return launch_status();
}

template <int DIST>
int launch_dist(const mi_tile_array* out, long long n, unsigned seed, unsigned counter, hipStream_t s) {
    switch (out->dtype) {
        case MI_F32: return launch_kind<4, unsigned, K_F32, DIST>(out, n, seed, counter, s);
        case MI_F64: return launch_kind<8, unsigned long long, K_F64, DIST>(out, n, seed, counter, s);
        case MI_F16: return launch_kind<2, unsigned short, K_F16, DIST>(out, n, seed, counter, s);
        case MI_BF16: return launch_kind<2, unsigned short, K_BF16, DIST>(out, n, seed, counter, s);
        default: break;
    }
    if constexpr (DIST == kRand) {
        switch (out->dtype) {
            case MI_I32: return launch_kind<4, unsigned, K_INT, kRand>(out, n, seed, counter, s);
            case MI_I64: return launch_kind<8, unsigned long long, K_INT, kRand>(out, n, seed, counter, s);
            case MI_I16: return launch_kind<2, unsigned short, K_INT, kRand>(out, n, seed, counter, s);
            case MI_I8: return launch_kind<1, unsigned char, K_INT, kRand>(out, n, seed, counter, s);
            default: break;
        }
    }
    return MI_E_DTYPE;
}

}  // namespace

extern "C" {

int mi_rng_fill(const mi_tile_array* out, uint32_t seed, uint32_t counter, int dist, void* stream) {
    if (!out) return MI_E_NULL;
    if (out->ndim < 0 || out->ndim > 4) return MI_E_RANK;
    if (dist < kRand || dist > kRandexp) return MI_E_ARG;
    int es = 0;
    switch (out->dtype) {
        case MI_I8: es = 1; break;
        case MI_I16: case MI_F16: case MI_BF16: es = 2; break;
        case MI_I32: case MI_F32: es = 4; break;
        case MI_I64: case MI_F64: es = 8; break;
        default: return MI_E_DTYPE;
    }
    int64_t n = 1;
    for (int d = 0; d < out->ndim; ++d) {
        if (out->sizes[d] < 0) return MI_E_SHAPE;
        n *= out->sizes[d];
    }
    if (n == 0) return MI_OK;
    if (!out->ptr) return MI_E_NULL;
    if (!is_dense(out)) return MI_E_STRIDE;
    if (((uintptr_t)out->ptr) % (uintptr_t)es) return MI_E_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    set_variant(dist == kRand ? "rng_fill_philox2x32_7_rand" : dist == kRandn ? "rng_fill_philox2x32_7_randn" : "rng_fill_philox2x32_7_randexp");
    switch (dist) {
        case kRand: return launch_dist<kRand>(out, n, seed, counter, s);
        case kRandn: return launch_dist<kRandn>(out, n, seed, counter, s);
        default: return launch_dist<kRandexp>(out, n, seed, counter, s);
    }
}

int mi_rng_advance_counter(uint32_t* seed, uint32_t* counter, int64_t n_elements) {
    if (!seed || !counter) return MI_E_NULL;
    if (n_elements < 0) return MI_E_ARG;
    // the fill consumes whole blocks of 512 counters (random.jl:776-779); the carry re-keys (random.jl:694-699)
    const uint32_t step = (uint32_t)(mi::cld(n_elements, (int64_t)kFillTile) * kFillTile);
    const uint32_t next = *counter + step;
    if (next < *counter) *seed += 1;
    *counter = next;
    return MI_OK;
}

}  // extern "C"
