// Mixture-of-experts kernels: stand-ins for fused_moe_kernel (examples/moe.jl:45-105),
// silu_and_mul_kernel (moe.jl:110-128) and the top-k combine `sum(cache3; dims=2)`
// (moe.jl:256) of the reference.
//
// fused_moe_kernel is a token-gather grouped GEMM: for the block of TILE_M sorted token
// slots `bid_m` (all routed to expert sorted_expert_ids[bid_m]; padding slots carry the
// sentinel total_tokens+1) and a strip of output channels,
//     C[n, token_id] = sum_k B[k, n, expert] * A[k, cld(token_id, replicas)]  (* routed weight).
// Both operands are K-contiguous in memory, so both MFMA operands are plain 16-byte LDS
// reads.  The MFMA column operand (lane % 32) carries n, which makes every store of C a run
// of 32 consecutive channels; the row operand carries the token slot.  Token tiles of 32
// slots that hold only padding are skipped, so the usual case of ~16 tokens per expert
// costs one 32-row MFMA tile instead of TILE_M/32.  The kernel is bound by streaming the
// expert weights from HBM (each weight is used by only the block's few tokens); weights
// may be f16/bf16 or OCP FP8 E4M3 with one fp32 scale per (n, expert), which are widened to
// f16 on their way into LDS (every e4m3 value is exact in f16) and scaled in the epilogue.
#include "common.h"
#include <math.h>

namespace {

using namespace mi;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct F16 {
    static __device__ __forceinline__ f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned short cvt(float v) {
        _Float16 h = (_Float16)v;
        return __builtin_bit_cast(unsigned short, h);
    }
    static __device__ __forceinline__ float widen(unsigned short h) {
        return (float)__builtin_bit_cast(_Float16, h);
    }
};
struct BF16 {
    static __device__ __forceinline__ f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ unsigned short cvt(float v) {
        unsigned u = __float_as_uint(v);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (unsigned short)(u >> 16);
    }
    static __device__ __forceinline__ float widen(unsigned short h) { return __uint_as_float(((unsigned)h) << 16); }
};

// Two E4M3FN bytes (the low or high half of `w`) -> two f16, exactly.  The byte's 7 magnitude
// bits land in f16's exponent/mantissa fields shifted by 7, which gives value * 2^-8 for
// normals and subnormals alike (bias 7 vs 15); the factor 2^8 is applied by an exact f16
// multiply.  (NaN codes never occur in weights.)
__device__ __forceinline__ unsigned e4m3x2_to_f16x2(unsigned w16) {
    const unsigned x = (w16 & 0xffu) | ((w16 & 0xff00u) << 8);       // bytes at bits 0-7 and 16-23
    const unsigned bits = ((x & 0x007f007fu) << 7) | ((x & 0x00800080u) << 8);
    f16x2 h = __builtin_bit_cast(f16x2, bits);
    h = h * (f16x2){(_Float16)256.0f, (_Float16)256.0f};
    return __builtin_bit_cast(unsigned, h);
}

constexpr int kNT = 128;  // output channels per workgroup (4 waves x 32)
constexpr int kKT = 64;   // K step
constexpr int kMaxMT = 4; // token tiles of 32 per workgroup (TILE_M <= 128)

// E: activation/output element traits; W8: weights are E4M3FN bytes (else same type as A).
template <typename E, bool W8>
__global__ __launch_bounds__(256) void fused_moe_kernel(
    const unsigned short* __restrict__ A, int64_t lda, int num_a_cols, const void* __restrict__ Bv, int64_t ldb,
    int64_t sbe, unsigned short* __restrict__ C, int64_t ldc, int total_tokens,
    const unsigned short* __restrict__ topk_weights, const int* __restrict__ sorted_token_ids, int num_slots,
    const int* __restrict__ sorted_expert_ids, const float* __restrict__ b_scale, int64_t ld_scale, int K, int N,
    int num_experts, int replicas, bool mul_routed_weight, int TILE_M, int n_blocks, bool vecA, bool vecB) {
    __shared__ __attribute__((aligned(16))) unsigned short Bs[kNT * kKT];          // [n][k], 16-byte chunks XOR-swizzled
    __shared__ __attribute__((aligned(16))) unsigned short As[32 * kMaxMT * kKT];  // [slot][k], same swizzle
    __shared__ int s_tok[32 * kMaxMT];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hb = lane >> 5;
    // consecutive workgroups share the token block (and therefore the activations in L2)
    const int bid_m = blockIdx.x / n_blocks, bid_n = blockIdx.x % n_blocks;
    const int n0 = bid_n * kNT;
    const int slot0 = bid_m * TILE_M;
    const int expert = sorted_expert_ids[bid_m] - 1;
    const bool expert_ok = expert >= 0 && expert < num_experts;

    for (int i = tid; i < TILE_M; i += 256) {
        const int s = slot0 + i;
        s_tok[i] = s < num_slots ? sorted_token_ids[s] : 0;  // 1-based; 0 / >total = no token
    }
    __syncthreads();
    // number of 32-slot tiles that contain at least one real token
    int mt_used = 0;
    for (int i = 0; i < TILE_M; ++i) {
        const int t = s_tok[i];
        if (t >= 1 && t <= total_tokens) mt_used = i / 32 + 1;
    }
    if (mt_used == 0 || !expert_ok) return;  // uniform across the workgroup

    const unsigned char* B8 = (const unsigned char*)Bv + (int64_t)expert * sbe;
    const unsigned short* B16 = (const unsigned short*)Bv + (int64_t)expert * sbe;

    f32x16 acc[kMaxMT];
#pragma unroll
    for (int i = 0; i < kMaxMT; ++i) acc[i] = f32x16{0};

    // staging registers: B tile 128 n x 64 k = 1024 chunks of 8 elements -> 4 per thread;
    // A tile up to 128 slots x 64 k -> up to 4 per thread.
    s16x8 breg[4], areg[kMaxMT];
    auto load_tiles = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i, n = id >> 3, c = id & 7;
            const int gn = n0 + n, gk = k0 + 8 * c;
            s16x8 v = {0};
            if (gn < N && gk < K) {
                if (W8) {
                    const unsigned char* p = B8 + gk + (int64_t)gn * ldb;
                    u32x2 raw = {0, 0};
                    if (vecB && gk + 8 <= K) raw = *reinterpret_cast<const u32x2*>(p);
                    else {
                        unsigned long long acc8 = 0;
                        for (int e = 0; e < 8; ++e)
                            if (gk + e < K) acc8 |= (unsigned long long)p[e] << (8 * e);
                        raw[0] = (unsigned)acc8;
                        raw[1] = (unsigned)(acc8 >> 32);
                    }
                    u32x4 w;
                    w[0] = e4m3x2_to_f16x2(raw[0] & 0xffffu);
                    w[1] = e4m3x2_to_f16x2(raw[0] >> 16);
                    w[2] = e4m3x2_to_f16x2(raw[1] & 0xffffu);
                    w[3] = e4m3x2_to_f16x2(raw[1] >> 16);
                    v = __builtin_bit_cast(s16x8, w);
                } else {
                    const unsigned short* p = B16 + gk + (int64_t)gn * ldb;
                    if (vecB && gk + 8 <= K) v = *reinterpret_cast<const s16x8*>(p);
                    else
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[e] = (gk + e < K) ? (short)p[e] : (short)0;
                }
            }
            breg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < kMaxMT; ++i) {
            s16x8 v = {0};
            if (i < mt_used) {
                const int id = tid + 256 * i, slot = id >> 3, c = id & 7;
                const int tok = slot < TILE_M ? s_tok[slot] : 0;
                const int gk = k0 + 8 * c;
                if (tok >= 1 && tok <= total_tokens && gk < K) {
                    const int col = (tok + replicas - 1) / replicas - 1;  // cld(token_id, replicas), 0-based
                    if (col < num_a_cols) {
                        const unsigned short* p = A + gk + (int64_t)col * lda;
                        if (vecA && gk + 8 <= K) v = *reinterpret_cast<const s16x8*>(p);
                        else
#pragma unroll
                            for (int e = 0; e < 8; ++e) v[e] = (gk + e < K) ? (short)p[e] : (short)0;
                    }
                }
            }
            areg[i] = v;
        }
    };
    load_tiles(0);

    for (int k0 = 0; k0 < K; k0 += kKT) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i, n = id >> 3, c = id & 7;
            *reinterpret_cast<s16x8*>(&Bs[n * kKT + 8 * (c ^ (n & 7))]) = breg[i];
        }
#pragma unroll
        for (int i = 0; i < kMaxMT; ++i)
            if (i < mt_used) {
                const int id = tid + 256 * i, slot = id >> 3, c = id & 7;
                *reinterpret_cast<s16x8*>(&As[slot * kKT + 8 * (c ^ (slot & 7))]) = areg[i];
            }
        __syncthreads();
        if (k0 + kKT < K) load_tiles(k0 + kKT);
#pragma unroll
        for (int ks = 0; ks < kKT / 16; ++ks) {
            const int c = 2 * ks + hb;
            const int n = wave * 32 + (lane & 31);
            s16x8 bf = *reinterpret_cast<const s16x8*>(&Bs[n * kKT + 8 * (c ^ (n & 7))]);
#pragma unroll
            for (int mt = 0; mt < kMaxMT; ++mt)
                if (mt < mt_used) {
                    const int slot = 32 * mt + (lane & 31);
                    s16x8 af = *reinterpret_cast<const s16x8*>(&As[slot * kKT + 8 * (c ^ (slot & 7))]);
                    acc[mt] = E::mfma32(af, bf, acc[mt]);
                }
        }
    }

    // epilogue: rows = token slots 8*(r/4) + 4*hb + r%4, column = channel n0 + wave*32 + lane%32
    const int gn = n0 + wave * 32 + (lane & 31);
    if (gn >= N) return;
    float ch_scale = 1.f;
    if (W8) ch_scale = b_scale[gn + (int64_t)expert * ld_scale];
#pragma unroll
    for (int mt = 0; mt < kMaxMT; ++mt)
        if (mt < mt_used) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int slot = 32 * mt + 8 * (r >> 2) + 4 * hb + (r & 3);
                if (slot >= TILE_M) continue;
                const int tok = s_tok[slot];
                if (tok < 1 || tok > total_tokens) continue;
                float v = acc[mt][r];
                if (W8) v *= ch_scale;
                if (mul_routed_weight) v *= E::widen(topk_weights[tok - 1]);
                C[gn + (int64_t)(tok - 1) * ldc] = E::cvt(v);
            }
        }
}

// ---- SiLU(a) * b -------------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const unsigned short* __restrict__ A, int64_t lda,
                                                           const unsigned short* __restrict__ B, int64_t ldb,
                                                           unsigned short* __restrict__ C, int64_t ldc, int rows,
                                                           bool vec) {
    const int64_t col = blockIdx.y;
    const unsigned short* a = A + col * lda;
    const unsigned short* b = B + col * ldb;
    unsigned short* c = C + col * ldc;
    const int i0 = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (i0 >= rows) return;
    auto f = [](float x, float y) {
        const float denom = 1.0f + expf(-x);
        return x * __builtin_amdgcn_rcpf(denom) * y;  // approximate reciprocal, moe.jl:117-124
    };
    if (vec && i0 + 8 <= rows) {
        s16x8 va = *reinterpret_cast<const s16x8*>(a + i0), vb = *reinterpret_cast<const s16x8*>(b + i0), vc;
#pragma unroll
        for (int e = 0; e < 8; ++e)
            vc[e] = (short)E::cvt(f(E::widen((unsigned short)va[e]), E::widen((unsigned short)vb[e])));
        *reinterpret_cast<s16x8*>(c + i0) = vc;
    } else {
        for (int e = 0; e < 8 && i0 + e < rows; ++e) c[i0 + e] = E::cvt(f(E::widen(a[i0 + e]), E::widen(b[i0 + e])));
    }
}

// ---- sum over the top-k slots ---------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void moe_sum_topk_kernel(const unsigned short* __restrict__ in, int64_t s1,
                                                           int64_t s2, unsigned short* __restrict__ out,
                                                           int64_t ldo, int H, int topk) {
    const int64_t tok = blockIdx.y;
    const int h = blockIdx.x * 256 + threadIdx.x;
    if (h >= H) return;
    const unsigned short* p = in + h + tok * s2;
    float acc = 0.f;
    for (int k = 0; k < topk; ++k) acc += E::widen(p[k * s1]);
    out[h + tok * ldo] = E::cvt(acc);
}

bool is16(int dt) { return dt == MI_F16 || dt == MI_BF16; }

}  // namespace

extern "C" int mi_fused_moe_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                                   const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                                   const mi_tile_array* sorted_expert_ids, int num_token_replicas,
                                   int mul_routed_weight, int TILE_M, int TILE_N, int TILE_K,
                                   const mi_tile_array* b_scale, void* stream) {
    MI_CHECK(check_array(A, 2));
    MI_CHECK(check_array(B, 3));
    MI_CHECK(check_array(C, 2));
    MI_CHECK(check_array(topk_weights, 1));
    MI_CHECK(check_array(sorted_token_ids, 1));
    MI_CHECK(check_array(sorted_expert_ids, 1));
    if (!is16(A->dtype) || C->dtype != A->dtype || topk_weights->dtype != A->dtype) return MI_E_DTYPE;
    const bool w8 = B->dtype == MI_F8E4M3FN;
    if (!w8 && B->dtype != A->dtype) return MI_E_DTYPE;
    if (w8 != (b_scale != nullptr)) return MI_E_ARG;
    if (sorted_token_ids->dtype != MI_I32 || sorted_expert_ids->dtype != MI_I32) return MI_E_DTYPE;
    if (!is_pow2(TILE_M) || !is_pow2(TILE_N) || !is_pow2(TILE_K)) return MI_E_TILE;
    if (TILE_M > 32 * kMaxMT) return MI_E_UNSUPPORTED;
    if (num_token_replicas < 1) return MI_E_ARG;
    const int64_t K = B->sizes[0], N = B->sizes[1], E = B->sizes[2];
    if (A->sizes[0] != K || C->sizes[0] != N) return MI_E_SHAPE;
    const int64_t slots = sorted_token_ids->sizes[0], total = C->sizes[1];
    const int64_t m_blocks = cld(slots, (int64_t)TILE_M);
    if (sorted_expert_ids->sizes[0] < m_blocks) return MI_E_SHAPE;
    if (mul_routed_weight && topk_weights->sizes[0] < total) return MI_E_SHAPE;
    if (w8) {
        MI_CHECK(check_array(b_scale, 2));
        if (b_scale->dtype != MI_F32) return MI_E_DTYPE;
        if (b_scale->sizes[0] != N || b_scale->sizes[1] != E) return MI_E_SHAPE;
        if (N > 1 && b_scale->strides[0] != 1) return MI_E_STRIDE;
    }
    if ((K > 1 && (A->strides[0] != 1 || B->strides[0] != 1)) || (N > 1 && C->strides[0] != 1)) return MI_E_STRIDE;
    if (slots > 1 && sorted_token_ids->strides[0] != 1) return MI_E_STRIDE;
    if (m_blocks > 1 && sorted_expert_ids->strides[0] != 1) return MI_E_STRIDE;
    if (total > 1 && topk_weights->strides[0] != 1) return MI_E_STRIDE;
    if (K > 0x7fffffff || N > 0x7fffffff || total > 0x7ffffffe || slots > 0x7fffffff) return MI_E_SHAPE;
    if (m_blocks * cld(N, (int64_t)TILE_N) > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (m_blocks == 0 || N == 0) return MI_OK;
    const int n_blocks = (int)cld(N, (int64_t)kNT);
    if (m_blocks * n_blocks > 0x7fffffffLL) return MI_E_GRID;
    const bool vecA = aligned(A->ptr, 16) && A->strides[1] % 8 == 0;
    const int bdiv = w8 ? 8 : 8;
    const bool vecB = aligned(B->ptr, w8 ? 8 : 16) && B->strides[1] % bdiv == 0 && B->strides[2] % bdiv == 0;
    dim3 grid((unsigned)(m_blocks * n_blocks));
    hipStream_t s = (hipStream_t)stream;
#define LAUNCH(ET, W8)                                                                                              \
    hipLaunchKernelGGL((fused_moe_kernel<ET, W8>), grid, dim3(256), 0, s, (const unsigned short*)A->ptr,           \
                       A->strides[1], (int)A->sizes[1], (const void*)B->ptr, B->strides[1], B->strides[2],          \
                       (unsigned short*)C->ptr, C->strides[1], (int)total, (const unsigned short*)topk_weights->ptr, \
                       (const int*)sorted_token_ids->ptr, (int)slots, (const int*)sorted_expert_ids->ptr,           \
                       w8 ? (const float*)b_scale->ptr : nullptr, w8 ? b_scale->strides[1] : 0, (int)K, (int)N,     \
                       (int)E, num_token_replicas, mul_routed_weight != 0, TILE_M, n_blocks, vecA, vecB)
    if (A->dtype == MI_F16) {
        if (w8) LAUNCH(F16, true);
        else LAUNCH(F16, false);
    } else {
        if (w8) LAUNCH(BF16, true);
        else LAUNCH(BF16, false);
    }
#undef LAUNCH
    set_variant(w8 ? "fused_moe_n128_k64_w8a16" : "fused_moe_n128_k64");
    return launch_status();
}

extern "C" int mi_silu_and_mul_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                                      int TILE_N, void* stream) {
    MI_CHECK(check_array(A, 2));
    MI_CHECK(check_array(B, 2));
    MI_CHECK(check_array(C, 2));
    if (!is16(A->dtype) || B->dtype != A->dtype || C->dtype != A->dtype) return MI_E_DTYPE;
    if (!is_pow2(TILE_N)) return MI_E_TILE;
    if (!same_shape(A, B) || A->sizes[1] != C->sizes[1]) return MI_E_SHAPE;
    // one tile of TILE_N rows per column (moe.jl:112-113,126): rows past TILE_N are untouched
    int64_t rows = C->sizes[0] < A->sizes[0] ? C->sizes[0] : A->sizes[0];
    if (rows > TILE_N) rows = TILE_N;
    const int64_t cols = C->sizes[1];
    if (cols > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (rows == 0 || cols == 0) return MI_OK;
    if (rows > 1 && (A->strides[0] != 1 || B->strides[0] != 1 || C->strides[0] != 1)) return MI_E_STRIDE;
    if (cols > 65535) return MI_E_UNSUPPORTED;
    const bool vec = aligned(A->ptr, 16) && aligned(B->ptr, 16) && aligned(C->ptr, 16) && A->strides[1] % 8 == 0 &&
                     B->strides[1] % 8 == 0 && C->strides[1] % 8 == 0;
    dim3 grid((unsigned)cld(rows, (int64_t)2048), (unsigned)cols);
    hipStream_t s = (hipStream_t)stream;
    if (A->dtype == MI_F16)
        hipLaunchKernelGGL((silu_and_mul_kernel<F16>), grid, dim3(256), 0, s, (const unsigned short*)A->ptr,
                           A->strides[1], (const unsigned short*)B->ptr, B->strides[1], (unsigned short*)C->ptr,
                           C->strides[1], (int)rows, vec);
    else
        hipLaunchKernelGGL((silu_and_mul_kernel<BF16>), grid, dim3(256), 0, s, (const unsigned short*)A->ptr,
                           A->strides[1], (const unsigned short*)B->ptr, B->strides[1], (unsigned short*)C->ptr,
                           C->strides[1], (int)rows, vec);
    set_variant("silu_and_mul_vec8");
    return launch_status();
}

extern "C" int mi_moe_sum_topk(const mi_tile_array* in, const mi_tile_array* out, void* stream) {
    MI_CHECK(check_array(in, 3));
    MI_CHECK(check_array(out, 2));
    if (!is16(in->dtype) || out->dtype != in->dtype) return MI_E_DTYPE;
    const int64_t H = in->sizes[0], topk = in->sizes[1], T = in->sizes[2];
    if (out->sizes[0] != H || out->sizes[1] != T) return MI_E_SHAPE;
    if (H > 1 && (in->strides[0] != 1 || out->strides[0] != 1)) return MI_E_STRIDE;
    if (H == 0 || T == 0) return MI_OK;
    if (T > 65535 || H > 0x7fffffff || topk > 0x7fffffff) return MI_E_UNSUPPORTED;
    dim3 grid((unsigned)cld(H, (int64_t)256), (unsigned)T);
    hipStream_t s = (hipStream_t)stream;
    if (in->dtype == MI_F16)
        hipLaunchKernelGGL((moe_sum_topk_kernel<F16>), grid, dim3(256), 0, s, (const unsigned short*)in->ptr,
                           in->strides[1], in->strides[2], (unsigned short*)out->ptr, out->strides[1], (int)H,
                           (int)topk);
    else
        hipLaunchKernelGGL((moe_sum_topk_kernel<BF16>), grid, dim3(256), 0, s, (const unsigned short*)in->ptr,
                           in->strides[1], in->strides[2], (unsigned short*)out->ptr, out->strides[1], (int)H,
                           (int)topk);
    set_variant("moe_sum_topk");
    return launch_status();
}
