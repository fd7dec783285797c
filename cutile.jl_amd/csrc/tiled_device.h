// Device-side text shared by every kernel the Tiled broadcast / mapreduce entry points build at
// run time (hiprtc).  Host-only header: the text is a string constant.
//
// Element types are named by the values of mi_dtype.  A value of type T lives in registers as its
// carrier (float for Float16 / BFloat16 / Float32, double, int, long long, bool); rnd<T> re-rounds a
// float carrier to T after every operation, which is how Julia defines Float16 / BFloat16 arithmetic.
// max / min follow Julia (NaN wins, -0.0 < +0.0); integer division by zero yields 0 instead of
// throwing; a float -> integer conversion truncates instead of throwing InexactError.
#pragma once

namespace mi {
namespace tiled {

static const char* const kDevicePreamble = R"SRC(
constexpr int DT_F32 = 0, DT_F64 = 1, DT_F16 = 2, DT_BF16 = 3, DT_I32 = 5, DT_I64 = 6, DT_BOOL = 7;
typedef unsigned int u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
struct bf16_t { unsigned short b; };

template <int DT> struct Car { typedef float type; };
template <> struct Car<DT_F64> { typedef double type; };
template <> struct Car<DT_I32> { typedef int type; };
template <> struct Car<DT_I64> { typedef long long type; };
template <> struct Car<DT_BOOL> { typedef bool type; };
template <int DT> using car = typename Car<DT>::type;
template <int DT> constexpr bool is_flt = DT == DT_F32 || DT == DT_F64 || DT == DT_F16 || DT == DT_BF16;
template <int DT> constexpr bool is_int = DT == DT_I32 || DT == DT_I64;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float((u32)v.b << 16); }
__device__ __forceinline__ bf16_t f32_to_bf16(float x) {
    u32 u = __float_as_uint(x);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.b = (unsigned short)((u >> 16) | 0x40u); return r; }
    u += 0x7fffu + ((u >> 16) & 1u);
    r.b = (unsigned short)(u >> 16);
    return r;
}
template <int DT> __device__ __forceinline__ car<DT> rnd(car<DT> x) {
    if constexpr (DT == DT_F16) return (float)(_Float16)x;
    else if constexpr (DT == DT_BF16) return bf16_to_f32(f32_to_bf16(x));
    else return x;
}
template <int DT, typename S> __device__ __forceinline__ car<DT> cvt(S x) {
    if constexpr (DT == DT_BOOL) return x != (S)0;
    else return rnd<DT>((car<DT>)x);
}
template <int DT, typename S> __device__ __forceinline__ car<DT> f_convert(S x) { return cvt<DT>(x); }

// ---- storage <-> carrier ----
__device__ __forceinline__ float to_car(float v) { return v; }
__device__ __forceinline__ double to_car(double v) { return v; }
__device__ __forceinline__ float to_car(_Float16 v) { return (float)v; }
__device__ __forceinline__ float to_car(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ int to_car(int v) { return v; }
__device__ __forceinline__ long long to_car(long long v) { return v; }
__device__ __forceinline__ bool to_car(unsigned char v) { return v != 0; }
template <typename ST, typename C> __device__ __forceinline__ ST to_sto(C v);
template <> __device__ __forceinline__ float to_sto<float, float>(float v) { return v; }
template <> __device__ __forceinline__ double to_sto<double, double>(double v) { return v; }
template <> __device__ __forceinline__ _Float16 to_sto<_Float16, float>(float v) { return (_Float16)v; }
template <> __device__ __forceinline__ bf16_t to_sto<bf16_t, float>(float v) { return f32_to_bf16(v); }
template <> __device__ __forceinline__ int to_sto<int, int>(int v) { return v; }
template <> __device__ __forceinline__ long long to_sto<long long, long long>(long long v) { return v; }
template <> __device__ __forceinline__ unsigned char to_sto<unsigned char, bool>(bool v) { return v ? 1 : 0; }

// ---- global memory: V consecutive elements, as the widest vectors their bytes allow ----
template <bool NT, typename T> __device__ __forceinline__ T ldg(const T* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p); else return *p;
}
template <bool NT, typename T> __device__ __forceinline__ void stg(T* p, T v) {
    if constexpr (NT) __builtin_nontemporal_store(v, p); else *p = v;
}
template <int BYTES, bool NT> __device__ __forceinline__ void copy_in(void* dst, const void* src) {
    if constexpr (BYTES >= 16) {
#pragma unroll
        for (int i = 0; i < BYTES / 16; ++i) { u32x4 t = ldg<NT>((const u32x4*)src + i); __builtin_memcpy((char*)dst + 16 * i, &t, 16); }
    } else if constexpr (BYTES == 8) { u32x2 t = ldg<NT>((const u32x2*)src); __builtin_memcpy(dst, &t, 8); }
    else if constexpr (BYTES == 4) { u32 t = ldg<NT>((const u32*)src); __builtin_memcpy(dst, &t, 4); }
    else if constexpr (BYTES == 2) { unsigned short t = ldg<NT>((const unsigned short*)src); __builtin_memcpy(dst, &t, 2); }
    else { *(unsigned char*)dst = ldg<NT>((const unsigned char*)src); }
}
template <int BYTES, bool NT> __device__ __forceinline__ void copy_out(void* dst, const void* src) {
    if constexpr (BYTES >= 16) {
#pragma unroll
        for (int i = 0; i < BYTES / 16; ++i) { u32x4 t; __builtin_memcpy(&t, (const char*)src + 16 * i, 16); stg<NT>((u32x4*)dst + i, t); }
    } else if constexpr (BYTES == 8) { u32x2 t; __builtin_memcpy(&t, src, 8); stg<NT>((u32x2*)dst, t); }
    else if constexpr (BYTES == 4) { u32 t; __builtin_memcpy(&t, src, 4); stg<NT>((u32*)dst, t); }
    else if constexpr (BYTES == 2) { unsigned short t; __builtin_memcpy(&t, src, 2); stg<NT>((unsigned short*)dst, t); }
    else { stg<NT>((unsigned char*)dst, *(const unsigned char*)src); }
}
// Loads elements [0, V) of a run that has `left` elements before the array ends (stride st).
// VEC: the run starts on a vector boundary and st == 1, so a full run moves as one vector.
template <typename ST, int V, bool VEC, bool NT>
__device__ __forceinline__ void load_run(const ST* p, long long left, long long st, ST (&r)[V]) {
    if constexpr (VEC) {
        if (left >= V) { copy_in<V * (int)sizeof(ST), NT>(r, p); return; }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) if (e < left) r[e] = p[e * st];
}
template <typename ST, int V, bool VEC, bool NT>
__device__ __forceinline__ void store_run(ST* p, long long left, long long st, const ST (&r)[V]) {
    if constexpr (VEC) {
        if (left >= V) { copy_out<V * (int)sizeof(ST), NT>(p, r); return; }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) if (e < left) p[e * st] = r[e];
}

// ---- functions of the expression language (template argument: the type the operation works in) ----
template <int DT> __device__ __forceinline__ car<DT> f_identity(car<DT> a) { return a; }
template <int DT> __device__ __forceinline__ car<DT> f_add(car<DT> a, car<DT> b) { return rnd<DT>(a + b); }
template <int DT> __device__ __forceinline__ car<DT> f_sub(car<DT> a, car<DT> b) { return rnd<DT>(a - b); }
template <int DT> __device__ __forceinline__ car<DT> f_mul(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_BOOL) return a && b; else return rnd<DT>(a * b);
}
template <int DT> __device__ __forceinline__ car<DT> f_div(car<DT> a, car<DT> b) { return rnd<DT>(a / b); }
template <int DT> __device__ __forceinline__ car<DT> f_neg(car<DT> a) { return -a; }
template <int DT> __device__ __forceinline__ car<DT> f_abs(car<DT> a) {
    if constexpr (DT == DT_BOOL) return a;
    else if constexpr (DT == DT_F64) return __builtin_fabs(a);
    else if constexpr (is_flt<DT>) return __builtin_fabsf(a);
    else return a < 0 ? -a : a;
}
template <int DT> __device__ __forceinline__ car<DT> f_abs2(car<DT> a) {
    if constexpr (DT == DT_BOOL) return a; else return rnd<DT>(a * a);
}
template <int DT> __device__ __forceinline__ car<DT> f_sign(car<DT> a) {
    if constexpr (DT == DT_BOOL) return a;
    else return a > 0 ? (car<DT>)1 : a < 0 ? (car<DT>)-1 : a;
}
template <int DT> __device__ __forceinline__ bool sgn(car<DT> a) {
    if constexpr (DT == DT_F64) return __builtin_signbit(a);
    else if constexpr (is_flt<DT>) return __builtin_signbitf(a);
    else if constexpr (DT == DT_BOOL) return false;
    else return a < 0;
}
template <int DT> __device__ __forceinline__ car<DT> f_max(car<DT> a, car<DT> b) {
    if constexpr (is_flt<DT>) return __builtin_elementwise_maximum(a, b);   // IEEE 754-2019 maximum: v_maximum3_f32
    else return a > b ? a : b;
}
template <int DT> __device__ __forceinline__ car<DT> f_min(car<DT> a, car<DT> b) {
    if constexpr (is_flt<DT>) return __builtin_elementwise_minimum(a, b);
    else return a < b ? a : b;
}
template <int DT> __device__ __forceinline__ car<DT> f_fma(car<DT> a, car<DT> b, car<DT> c) {
    if constexpr (DT == DT_F64) return __builtin_fma(a, b, c);
    else if constexpr (is_flt<DT>) return rnd<DT>(__builtin_fmaf(a, b, c));
    else if constexpr (DT == DT_BOOL) return (a && b) || c;
    else return a * b + c;
}
template <int DT> __device__ __forceinline__ car<DT> f_clamp(car<DT> x, car<DT> lo, car<DT> hi) { return x > hi ? hi : x < lo ? lo : x; }
template <int DT> __device__ __forceinline__ car<DT> f_copysign(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_F64) return __builtin_copysign(a, b);
    else if constexpr (is_flt<DT>) return __builtin_copysignf(a, b);
    else if constexpr (DT == DT_BOOL) return a;
    else { const car<DT> m = a < 0 ? -a : a; return b < 0 ? -m : m; }
}
#define MI_ROUNDING(NAME, FF, FD)                                                   \
    template <int DT> __device__ __forceinline__ car<DT> NAME(car<DT> a) {          \
        if constexpr (DT == DT_F64) return FD(a);                                   \
        else if constexpr (is_flt<DT>) return FF(a);                                \
        else return a;                                                              \
    }
MI_ROUNDING(f_floor, floorf, floor)
MI_ROUNDING(f_ceil, ceilf, ceil)
MI_ROUNDING(f_round, rintf, rint)
MI_ROUNDING(f_trunc, truncf, trunc)
#define MI_MATH1(NAME, FF, FD)                                                      \
    template <int DT> __device__ __forceinline__ car<DT> NAME(car<DT> a) {          \
        if constexpr (DT == DT_F64) return FD(a); else return rnd<DT>(FF(a));       \
    }
#define MI_MATH2(NAME, FF, FD)                                                      \
    template <int DT> __device__ __forceinline__ car<DT> NAME(car<DT> a, car<DT> b) { \
        if constexpr (DT == DT_F64) return FD(a, b); else return rnd<DT>(FF(a, b)); \
    }
MI_MATH1(f_sqrt, sqrtf, sqrt)
MI_MATH1(f_cbrt, cbrtf, cbrt)
MI_MATH1(f_exp, expf, exp)
MI_MATH1(f_exp2, exp2f, exp2)
MI_MATH1(f_exp10, exp10f, exp10)
MI_MATH1(f_expm1, expm1f, expm1)
MI_MATH1(f_log, logf, log)
MI_MATH1(f_log2, log2f, log2)
MI_MATH1(f_log10, log10f, log10)
MI_MATH1(f_log1p, log1pf, log1p)
MI_MATH1(f_sin, sinf, sin)
MI_MATH1(f_cos, cosf, cos)
MI_MATH1(f_tan, tanf, tan)
MI_MATH1(f_asin, asinf, asin)
MI_MATH1(f_acos, acosf, acos)
MI_MATH1(f_atan, atanf, atan)
MI_MATH1(f_sinh, sinhf, sinh)
MI_MATH1(f_cosh, coshf, cosh)
MI_MATH1(f_tanh, tanhf, tanh)
MI_MATH2(f_atan2, atan2f, atan2)
MI_MATH2(f_hypot, hypotf, hypot)
template <int DT> __device__ __forceinline__ car<DT> f_inv(car<DT> a) { return rnd<DT>((car<DT>)1 / a); }
template <int DT, typename X> __device__ __forceinline__ car<DT> f_pow(car<DT> a, X x) {
    if constexpr (DT == DT_BOOL) return x ? a : true;
    else if constexpr (DT == DT_F64) return pow(a, (double)x);
    else if constexpr (is_flt<DT>) return rnd<DT>(powf(a, (float)x));
    else {   // integers: power by squaring; negative exponents only make sense for +-1
        long long n = (long long)x;
        if (n < 0) return a == 1 ? (car<DT>)1 : a == -1 ? (car<DT>)((n & 1) ? -1 : 1) : (car<DT>)0;
        car<DT> r = 1, b = a;
        while (n) { if (n & 1) r *= b; b *= b; n >>= 1; }
        return r;
    }
}
template <int DT> __device__ __forceinline__ bool f_lt(car<DT> a, car<DT> b) { return a < b; }
template <int DT> __device__ __forceinline__ bool f_le(car<DT> a, car<DT> b) { return a <= b; }
template <int DT> __device__ __forceinline__ bool f_gt(car<DT> a, car<DT> b) { return a > b; }
template <int DT> __device__ __forceinline__ bool f_ge(car<DT> a, car<DT> b) { return a >= b; }
template <int DT> __device__ __forceinline__ bool f_eq(car<DT> a, car<DT> b) { return a == b; }
template <int DT> __device__ __forceinline__ bool f_ne(car<DT> a, car<DT> b) { return a != b; }
template <int DT> __device__ __forceinline__ bool f_isnan(car<DT> a) { if constexpr (is_flt<DT>) return a != a; else return false; }
template <int DT> __device__ __forceinline__ bool f_isinf(car<DT> a) {
    if constexpr (is_flt<DT>) return f_abs<DT>(a) == (car<DT>)__builtin_huge_valf(); else return false;
}
template <int DT> __device__ __forceinline__ bool f_isfinite(car<DT> a) {
    if constexpr (is_flt<DT>) return f_abs<DT>(a) < (car<DT>)__builtin_huge_valf(); else return true;
}
template <int DT> __device__ __forceinline__ bool f_signbit(car<DT> a) { return sgn<DT>(a); }
template <int DT> __device__ __forceinline__ bool f_iszero(car<DT> a) { return a == (car<DT>)0; }
template <int DT> __device__ __forceinline__ car<DT> f_not(car<DT> a) { if constexpr (DT == DT_BOOL) return !a; else return ~a; }
template <int DT> __device__ __forceinline__ car<DT> f_and(car<DT> a, car<DT> b) { return (car<DT>)(a & b); }
template <int DT> __device__ __forceinline__ car<DT> f_or(car<DT> a, car<DT> b) { return (car<DT>)(a | b); }
template <int DT> __device__ __forceinline__ car<DT> f_xor(car<DT> a, car<DT> b) { return (car<DT>)(a ^ b); }
template <int DT> __device__ __forceinline__ car<DT> f_ifelse(bool c, car<DT> a, car<DT> b) { return c ? a : b; }
// Julia's div (toward zero), rem (sign of the dividend), mod (sign of the divisor), fld, cld.  For floats
// Julia derives the quotients from the exact remainder, round((x - rem(x, y, r)) / y) (Base div.jl), which
// differs from rounding x / y where the division itself rounds across an integer (1.0 / 0.1 is 10.0, but
// div(1.0, 0.1) and fld(1.0, 0.1) are 9.0); mod of an exact multiple takes the sign of the divisor.
template <int DT> __device__ __forceinline__ car<DT> f_rem(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_F64) return fmod(a, b);
    else if constexpr (is_flt<DT>) return rnd<DT>(fmodf(a, b));
    else return (b == 0 || b == -1) ? (car<DT>)0 : a % b;
}
template <int DT> __device__ __forceinline__ car<DT> f_mod(car<DT> a, car<DT> b) {
    car<DT> r = f_rem<DT>(a, b);
    if constexpr (is_flt<DT> || DT == DT_F64) {
        if (r == (car<DT>)0) return (car<DT>)copysign((double)r, (double)b);
    }
    if (r != (car<DT>)0 && ((r < (car<DT>)0) != (b < (car<DT>)0))) r = rnd<DT>(r + b);
    return r;
}
template <int DT> __device__ __forceinline__ car<DT> f_divi(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_F64) return rint((a - fmod(a, b)) / b);
    else if constexpr (is_flt<DT>) return rnd<DT>(rintf((a - f_rem<DT>(a, b)) / b));
    else return b == 0 ? (car<DT>)0 : (b == -1 ? -a : a / b);
}
template <int DT> __device__ __forceinline__ car<DT> f_fld(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_F64) return rint((a - f_mod<DT>(a, b)) / b);
    else if constexpr (is_flt<DT>) return rnd<DT>(rintf((a - f_mod<DT>(a, b)) / b));
    else { const car<DT> q = f_divi<DT>(a, b); return (b != 0 && (a % (b == -1 ? 1 : b)) != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; }
}
template <int DT> __device__ __forceinline__ car<DT> f_cld(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_F64) return rint((a - f_mod<DT>(a, -b)) / b);
    else if constexpr (is_flt<DT>) return rnd<DT>(rintf((a - f_mod<DT>(a, -b)) / b));
    else { const car<DT> q = f_divi<DT>(a, b); return (b != 0 && (a % (b == -1 ? 1 : b)) != 0 && ((a < 0) == (b < 0))) ? q + 1 : q; }
}

template <int DT> __device__ __forceinline__ car<DT> f_rsqrt(car<DT> a) {
    if constexpr (DT == DT_F64) return 1.0 / sqrt(a); else return rnd<DT>(1.0f / sqrtf(a));
}
// Julia's shifts: a count of the word size or more shifts everything out (>> keeps the sign), a
// negative count shifts the other way.
template <int DT> struct UCar { typedef unsigned int type; };
template <> struct UCar<DT_I64> { typedef unsigned long long type; };
template <int DT> __device__ __forceinline__ car<DT> shift_left(car<DT> a, long long n) {
    constexpr int B = 8 * (int)sizeof(car<DT>);
    return n >= B ? (car<DT>)0 : (car<DT>)((typename UCar<DT>::type)a << n);
}
template <int DT, bool ARITH> __device__ __forceinline__ car<DT> shift_right(car<DT> a, long long n) {
    constexpr int B = 8 * (int)sizeof(car<DT>);
    if constexpr (ARITH) return n >= B ? (car<DT>)(a < 0 ? -1 : 0) : (car<DT>)(a >> n);
    else return n >= B ? (car<DT>)0 : (car<DT>)((typename UCar<DT>::type)a >> n);
}
template <int DT> __device__ __forceinline__ car<DT> f_shl(car<DT> a, long long n) {
    return n >= 0 ? shift_left<DT>(a, n) : shift_right<DT, true>(a, n < -64 ? 64 : -n);
}
template <int DT> __device__ __forceinline__ car<DT> f_shr(car<DT> a, long long n) {
    return n >= 0 ? shift_right<DT, true>(a, n) : shift_left<DT>(a, n < -64 ? 64 : -n);
}
template <int DT> __device__ __forceinline__ car<DT> f_lshr(car<DT> a, long long n) {
    return n >= 0 ? shift_right<DT, false>(a, n) : shift_left<DT>(a, n < -64 ? 64 : -n);
}
// High half of the full product (Base.mul_hi).
template <int DT> __device__ __forceinline__ car<DT> f_mul_hi(car<DT> a, car<DT> b) {
    if constexpr (DT == DT_I32) return (int)(((long long)a * (long long)b) >> 32);
    else if constexpr (DT == DT_I64) return (long long)(((__int128)a * (__int128)b) >> 64);
    else return false;
}

// ---- wave64 exchange of any carrier ----
template <typename C> __device__ __forceinline__ C xor_lane(C v, int m) {
    if constexpr (sizeof(C) == 8) {
        u32 w[2]; __builtin_memcpy(w, &v, 8);
        w[0] = (u32)__shfl_xor((int)w[0], m, 64); w[1] = (u32)__shfl_xor((int)w[1], m, 64);
        C r; __builtin_memcpy(&r, w, 8); return r;
    } else if constexpr (sizeof(C) == 4) {
        u32 w; __builtin_memcpy(&w, &v, 4); w = (u32)__shfl_xor((int)w, m, 64);
        C r; __builtin_memcpy(&r, &w, 4); return r;
    } else {
        return (C)(__shfl_xor((int)v, m, 64) != 0);
    }
}
)SRC";

}  // namespace tiled
}  // namespace mi
