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
#include "moe_dense.h"
#include "shared_scratch.h"
#include <math.h>
#include <type_traits>

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
    // *p += the two values packed in `pair` (one memory-side atomic; round to nearest even, denormals kept)
    static __device__ __forceinline__ void atomic_add2(unsigned short* p, unsigned pair) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_global_atomic_fadd_v2f16((h2 __attribute__((address_space(1)))*)p, __builtin_bit_cast(h2, pair));
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
    static __device__ __forceinline__ void atomic_add2(unsigned short* p, unsigned pair) {
        typedef short s2 __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_global_atomic_fadd_v2bf16((s2 __attribute__((address_space(1)))*)p, __builtin_bit_cast(s2, pair));
    }
};

// Four E4M3FN bytes -> four values of the activation type.  gfx950's FP8 is the OCP E4M3FN
// format; its conversion instruction with scale 1 is exact for f16 (every e4m3 value,
// subnormals included, is an f16 value).  For bf16 activations the f16 pair is widened and
// truncated, also exactly (e4m3 has 3 mantissa bits).
template <typename E> struct Fp8;
template <> struct Fp8<F16> {
    static __device__ __forceinline__ void cvt4(unsigned w, unsigned& lo, unsigned& hi) {
        lo = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
        hi = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
    }
};
template <> struct Fp8<BF16> {
    static __device__ __forceinline__ unsigned f16x2_to_bf16x2(f16x2 h) {
        const unsigned a = __float_as_uint((float)h[0]) >> 16, b = __float_as_uint((float)h[1]) & 0xffff0000u;
        return a | b;
    }
    static __device__ __forceinline__ void cvt4(unsigned w, unsigned& lo, unsigned& hi) {
        lo = f16x2_to_bf16x2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
        hi = f16x2_to_bf16x2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
    }
};

using mi::moe::silu_mul;   // SiLU(x) * y as moe.jl:117-124 computes it, shared with the dense-routing kernel

constexpr int kTT = 32;   // token slots per workgroup (one MFMA row tile)

// Workgroup barrier that waits for the wave's LDS accesses only (lgkmcnt(0); vmcnt and expcnt at their
// maxima).  __syncthreads() also waits for every global load in flight, which would turn the weight
// tiles requested one and two steps ahead into synchronous loads.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// E: activation/output element traits; W8: weights are E4M3FN bytes (else same type as A).
// NTW: waves side by side along n (workgroup strip = 32*NTW channels); the other 4/NTW waves
// split each K step between them and their accumulators are added through LDS at the end.
// kKT: K step.  Two shapes are used: (NTW=4, kKT=128) when N is large enough to give every CU
// several strips, and (NTW=1, kKT=256) for small N, where 32-channel strips with a 4-way
// in-workgroup K split keep ~4x more workgroups (and bytes) in flight.
// Workgroup = (one tile of up to 32 consecutive sorted slots, one strip of 32*NTW channels).
// With ~16 tokens per expert most 32-slot tiles of a TILE_M block hold only padding; their
// workgroups leave at once, so the expert's weight strip is streamed by exactly as many
// workgroups as it has (started) 32-token tiles.  Small register footprint -> many
// workgroups per CU, each with the next weight tile already in flight.
// SILU (wide shape only): the workgroup's 128 weight rows are 64 gate channels [n0, n0 + 64) and
// the 64 up channels N/2 + [n0, n0 + 64) of the gate / up projection; the epilogue rounds both
// products to the activation type exactly as the separate kernels would, applies SiLU(gate) * up
// (moe.jl:110-128) and writes N/2 channels, so the intermediate never goes to memory.
// TS: 32-slot tiles of one expert block that a workgroup multiplies with the same weight tile
// (wide shapes only).  With more than 32 tokens per expert TS = 2 streams an expert's weights once
// per 64 tokens instead of once per 32, at the price of one workgroup per CU less.
// FAST: the workgroup's tiles lie wholly inside the arrays and everything is 16-byte aligned (checked on
// the host for the whole launch): loads without predicates.  A compile-time property, because with both
// load paths in one loop body the compiler has to wait for every outstanding load at their join, which
// empties the look-ahead.
template <typename E, bool W8, int NTW, int kKT, bool SILU = false, int TS = 1, bool FAST = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(TS == 1 ? 4 : 3))) void fused_moe_kernel(
    const unsigned short* __restrict__ A, int64_t lda, int num_a_cols, const void* __restrict__ Bv, int64_t ldb,
    int64_t sbe, unsigned short* __restrict__ C, int64_t ldc, int total_tokens,
    const unsigned short* __restrict__ topk_weights, const int* __restrict__ sorted_token_ids, int num_slots,
    const int* __restrict__ sorted_expert_ids, const float* __restrict__ b_scale, int64_t ld_scale, int K, int N,
    int num_experts, int replicas, bool mul_routed_weight, int TILE_M, int tile_slots, int n_blocks, bool vecA,
    bool vecB, int w_topk, int64_t w_s0, int64_t w_s1, int acc_shift) {
    constexpr int kNT = 32 * NTW, KW = 4 / NTW;
    // B tile [n][k], 16-byte chunks XOR-swizzled.  E4M3 weights stay raw bytes here (half the LDS
    // traffic and footprint) and are widened after the fragment read; see b_offset8 below.
    constexpr int kBsBytes = (W8 ? 1 : 2) * kNT * kKT, kRedBytes = KW > 1 ? 4 * 64 * 16 * 4 : 0;
    __shared__ __attribute__((aligned(16))) unsigned char Bs_raw[kBsBytes > kRedBytes ? kBsBytes : kRedBytes];
    unsigned short* Bs = reinterpret_cast<unsigned short*>(Bs_raw);
    constexpr int kTTS = kTT * TS;   // token slots per workgroup
    __shared__ __attribute__((aligned(16))) unsigned short As[kTTS * kKT];  // [slot][k], same swizzle

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hb = lane >> 5;
    const int wn = wave % NTW, wk = wave / NTW;  // position along n / along the K split
    // Consecutive workgroups share the token tile (and therefore the activations in L2).  The tiles
    // are walked sub-tile-major: first the leading 32 slots of every TILE_M block, which always hold
    // a token, then the second 32 slots of every block, and so on.  With ~16 tokens per expert all
    // the workgroups that have work are thus dispatched first and stream from the start; in slot
    // order three quarters of every dispatch round would be padding tiles that leave at once, and
    // the weight streams would take several rounds to build up.
    const int t_lin = blockIdx.x / n_blocks, bid_n = blockIdx.x % n_blocks;
    const int gpb = TILE_M / tile_slots / TS, m_blocks = (gridDim.x / n_blocks) / gpb;   // groups of TS tiles per block
    // (Dense routing, TS > 1: an expert with more than 32 * TS tokens has a second group with work, which streams
    // the same weights again.  In slot order the groups of a block are n_blocks workgroups apart -- the same XCD,
    // the same dispatch round -- so the second reader finds part of the lines in that XCD's L2.  Handing every XCD a
    // contiguous range of (group, strip) pairs instead, so that the strips of a group share their activation tile
    // in one L2 as well, cut the fabric traffic of the down projection by a fifth and made it a fifth slower.)
    const int grp = TS > 1 ? t_lin : (t_lin % m_blocks) * gpb + t_lin / m_blocks;
    static_assert(!SILU || NTW == 4, "the fused SiLU epilogue pairs waves 0,1 (gate) with waves 2,3 (up)");
    const int half_n = N / 2;
    const int n0 = bid_n * (SILU ? kNT / 2 : kNT);
    // global weight row of tile row n
    auto row_of = [&](int n) { return SILU ? (n < 64 ? n0 + n : half_n + n0 + n - 64) : n0 + n; };
    auto row_ok = [&](int n) { return SILU ? (n0 + (n & 63) < half_n) : (n0 + n < N); };
    const int slot0 = grp * tile_slots * TS;        // tile_slots = min(TILE_M, 32) divides TILE_M (32 when TS > 1)
    const int expert = sorted_expert_ids[slot0 / TILE_M] - 1;

    // A tile's 32 token ids live in registers, slot i in lanes i and i + 32 of every wave (LDS is
    // exactly the two operand tiles, which is what lets a fourth workgroup fit on a CU).
    int my_tok[TS];
    unsigned live = 0;   // tiles of the workgroup that hold a token; the same in every wave
#pragma unroll
    for (int ts = 0; ts < TS; ++ts) {
        const int i = lane & 31, sl = slot0 + kTT * ts + i;
        int t = (i < tile_slots && sl < num_slots) ? sorted_token_ids[sl] : 0;  // 1-based; 0 / >total = no token
        if (t < 1 || t > total_tokens) t = 0;
        my_tok[ts] = t;
        if (__ballot(t != 0) != 0ull) live |= 1u << ts;
    }
    auto tok_of = [&](int ts, int slot) { return __shfl(my_tok[ts], slot, 64); };
    if (!live || expert < 0 || expert >= num_experts) return;
    // The routed weight of the lane's slot is requested now and handed round by shuffles in the epilogue: loaded
    // there (sixteen dependent gathers per lane) it added a memory round trip to the end of every workgroup.
    unsigned short my_w[TS];
#pragma unroll
    for (int ts = 0; ts < TS; ++ts) {
        // weight of replica t0 = token * w_topk + slot: element (token, slot) of the (num_tokens, topk) matrix
        // (the flattened, slot-fastest vector of moe.jl:193 is the case w_topk = 1)
        const int t0 = my_tok[ts] - 1, tk = t0 / w_topk;
        my_w[ts] = (mul_routed_weight && my_tok[ts]) ? topk_weights[tk * w_s0 + (t0 - tk * w_topk) * w_s1] : (unsigned short)0;
    }
    auto weight_of = [&](int ts, int slot) { return E::widen((unsigned short)__shfl((int)my_w[ts], slot, 64)); };

    const unsigned char* B8 = (const unsigned char*)Bv + (int64_t)expert * sbe;
    const unsigned short* B16 = (const unsigned short*)Bv + (int64_t)expert * sbe;

    f32x16 acc[TS];
#pragma unroll
    for (int ts = 0; ts < TS; ++ts) acc[ts] = f32x16{0};
    // staging registers for the next B tile (128 n x kKT k) and A tile (32 slots x kKT k)
    constexpr int CPR = kKT / 8;            // 16-byte chunks per LDS tile row
    constexpr int EPB = W8 ? 16 : 8;        // weight elements per 16-byte global chunk
    constexpr int CPRB = kKT / EPB;         // 16-byte global chunks per weight row
    constexpr int NB = kNT * CPRB / 256;    // weight chunks per thread
    constexpr int NA = kTTS * CPR / 256;    // A chunks per thread
    // One staging set: the tile of the next step is requested right after this step's tile has gone to LDS
    // and is waited for at the next step's LDS write.  Keeping two weight tiles per workgroup in flight was
    // measured and is markedly slower (52 us against 29 us for the down projection; 46 against 27 us for
    // the e4m3 gate / up projection): four workgroups per CU already have 64 to 128 KB per CU in flight, and
    // twice that is the whole L2 of an XCD in outstanding lines.
    constexpr int DEPTH = 1;
    u32x4 breg0[NB];
    s16x8 areg0[NA];
    int a_col[NA];
    // Workgroups whose whole tile is inside the arrays (the usual case) load without predicates: a
    // predicated load is waited for before the other side of its branch may write the same
    // registers, which would leave a lane with one load in flight at a time.  Slots without a token
    // read column 0 there; their accumulator rows are never stored.
    constexpr bool fast = FAST;
    auto load_b = [&](int k0, u32x4* breg) {
        if constexpr (fast) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int id = tid + 256 * i, n = id / CPRB, c = id % CPRB;
                const int64_t off = k0 + EPB * c + (int64_t)row_of(n) * ldb;
                // (dense routing: a second group of the block may be streaming the same strip on this XCD right
                // now, so the lines are left to the L2; otherwise every weight is read once and passes it by)
                if constexpr (TS > 1)
                    breg[i] = W8 ? *reinterpret_cast<const u32x4*>(B8 + off) : *reinterpret_cast<const u32x4*>(B16 + off);
                else
                    breg[i] = W8 ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B8 + off))
                                 : __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B16 + off));
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int id = tid + 256 * i, n = id / CPRB, c = id % CPRB;
            const int gn = row_of(n), gk = k0 + EPB * c;
            u32x4 v = {0, 0, 0, 0};
            if (row_ok(n) && gk < K) {
                if (W8) {
                    const unsigned char* p = B8 + gk + (int64_t)gn * ldb;
                    if (vecB && gk + 16 <= K) v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
                    else
                        for (int e = 0; e < 16; ++e)
                            if (gk + e < K) v[e >> 2] |= (unsigned)p[e] << (8 * (e & 3));
                } else {
                    const unsigned short* p = B16 + gk + (int64_t)gn * ldb;
                    if (vecB && gk + 8 <= K) v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
                    else
                        for (int e = 0; e < 8; ++e)
                            if (gk + e < K) v[e >> 1] |= (unsigned)p[e] << (16 * (e & 1));
                }
            }
            breg[i] = v;
        }
    };
    auto load_a = [&](int k0, s16x8* areg) {
        if constexpr (fast) {
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                const int gk = k0 + 8 * ((tid + 256 * i) % CPR);
                areg[i] = *reinterpret_cast<const s16x8*>(A + gk + (int64_t)(a_col[i] < 0 ? 0 : a_col[i]) * lda);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            s16x8 v = {0};
            const int gk = k0 + 8 * ((tid + 256 * i) % CPR);
            if (a_col[i] >= 0 && gk < K) {
                const unsigned short* p = A + gk + (int64_t)a_col[i] * lda;
                if (vecA && gk + 8 <= K) v = *reinterpret_cast<const s16x8*>(p);
                else
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = (gk + e < K) ? (short)p[e] : (short)0;
            }
            areg[i] = v;
        }
    };
    // Raw-byte tile of the e4m3 path: row n = kKT bytes in 16-byte chunks.  Chunk c sits at
    // c ^ sw(n) and its two 8-byte halves are swapped for rows with bit 4 set, which makes the
    // 8-byte fragment reads of 32 lanes (rows n .. n+31, one half) cover all 64 banks exactly once.
    auto b_sw = [](int n) { return kKT == 128 ? ((n >> 1) & 7) : (n & 15); };

    // One K step: staged tiles -> LDS, refill the weight staging set with the tile DEPTH steps ahead and the
    // activation set with the next tile, MFMAs.
    // The K tiles are walked from a start that differs from workgroup to workgroup (and wraps): workgroups
    // that run at the same time would otherwise all read the same few hundred bytes of every weight row
    // at the same moment, i.e. the same slice of every 4 KB of address space.
    const int nsteps = (K + kKT - 1) / kKT;
    // (the narrow shape only: 27.9 against 29.5 us there, 49 against 45 us on the wide shape)
    const unsigned rot_seed = (unsigned)(3 * expert + grp);
    const int rot = NTW != 1 ? 0 : (nsteps & (nsteps - 1)) == 0 ? (int)(rot_seed & (unsigned)(nsteps - 1)) : (int)(rot_seed % (unsigned)nsteps);   // (not a function of the strip: the fused-SiLU and the plain kernel then add in the same order)
    auto k_of = [&](int it) {
        int st = it + rot;
        if (st >= nsteps) st -= nsteps;
        return st * kKT;
    };
    // LB / LA: this step requests a weight tile / an activation tile.  Compile-time, and the loops below are
    // peeled accordingly: after a load that is issued under a run-time condition the compiler has to assume
    // the older loads are the youngest ones in flight and waits for everything.
    auto step = [&](int it, u32x4* breg, auto lb, auto la) {
        constexpr bool LB = decltype(lb)::value, LA = decltype(la)::value;
        s16x8* areg = areg0;
        lds_barrier();   // the previous step's fragment reads are done
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int id = tid + 256 * i, n = id / CPRB, c = id % CPRB;
            if (W8) {
                const u32x4 v = breg[i];
                const u32x4 sw = ((n >> 4) & 1) ? u32x4{v[2], v[3], v[0], v[1]} : v;
                *reinterpret_cast<u32x4*>(&Bs_raw[n * kKT + 16 * (c ^ b_sw(n))]) = sw;
            } else {
                *reinterpret_cast<u32x4*>(&Bs[n * kKT + 8 * (c ^ (n & 15))]) = breg[i];
            }
        }
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const int id = tid + 256 * i, sl = id / CPR, c = id % CPR;
            *reinterpret_cast<s16x8*>(&As[sl * kKT + 8 * (c ^ (sl & 15))]) = areg[i];
        }
        lds_barrier();
        // (activations first: loads return in order, and the next step needs its activations together with a
        // weight tile requested a step earlier -- were the activations the youngest request, waiting for
        // them would also wait for the weight tile of the step after)
        if constexpr (LA) load_a(k_of(it + 1), areg);
        if constexpr (LB) load_b(k_of(it + DEPTH), breg);
#pragma unroll
        for (int kq = 0; kq < kKT / 16 / KW; ++kq) {
            const int ks = wk * (kKT / 16 / KW) + kq;
            const int c = 2 * ks + hb;
            const int n = wn * 32 + (lane & 31);
            const int slot = lane & 31;
            s16x8 bf;
            if (W8) {   // k elements 16 ks + 8 hb .. +7 are half hb of chunk ks
                const u32x2 raw = *reinterpret_cast<const u32x2*>(&Bs_raw[n * kKT + 16 * (ks ^ b_sw(n)) + 8 * (hb ^ ((n >> 4) & 1))]);
                unsigned w0, w1, w2, w3;
                Fp8<E>::cvt4(raw[0], w0, w1);
                Fp8<E>::cvt4(raw[1], w2, w3);
                bf = __builtin_bit_cast(s16x8, u32x4{w0, w1, w2, w3});
            } else {
                bf = *reinterpret_cast<const s16x8*>(&Bs[n * kKT + 8 * (c ^ (n & 15))]);
            }
#pragma unroll
            for (int ts = 0; ts < TS; ++ts) {
                if (TS > 1 && !((live >> ts) & 1u)) continue;
                s16x8 af = *reinterpret_cast<const s16x8*>(&As[(kTT * ts + slot) * kKT + 8 * (c ^ (slot & 15))]);
                acc[ts] = E::mfma32(af, bf, acc[ts]);
            }
        }
    };
    // The first weight tile only needs the expert and the strip: request it before the columns of the activation
    // tile are worked out from the token ids.
    load_b(k_of(0), breg0);
    const bool rep_pow2 = (replicas & (replicas - 1)) == 0;
    const int rep_shift = __builtin_ctz((unsigned)replicas);
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        a_col[i] = -1;
        const int sl = (tid + 256 * i) / CPR;
        // (a chunk index covers 256 / CPR consecutive slots, which divides a tile: the tile is known at compile time)
        static_assert(kTT % (256 / CPR) == 0, "a chunk index must not straddle two slot tiles");
        int tok = tok_of((256 * i / CPR) / kTT, sl & 31);
        if (tok) {
            // cld(token_id, replicas), 0-based (a shift for the usual power of two)
            const int col = rep_pow2 ? ((tok + replicas - 1) >> rep_shift) - 1 : (tok + replicas - 1) / replicas - 1;
            if (col < num_a_cols) a_col[i] = col;
        }
    }
    load_a(k_of(0), areg0);
    using Y = std::true_type;
    using No = std::false_type;
    {
        int it = 0;
        for (; it + 1 < nsteps; ++it) step(it, breg0, Y{}, Y{});
        step(it, breg0, No{}, No{});
    }
    if (KW > 1) {  // add the K-split partial accumulators: wave (wn, wk) -> wave (wn, 0), one slot tile at a time
        float* red = reinterpret_cast<float*>(Bs_raw);  // 4 waves x 64 lanes x 16 floats = 16 KB <= sizeof(Bs_raw)
#pragma unroll
        for (int ts = 0; ts < TS; ++ts) {
            if (!((live >> ts) & 1u)) continue;   // same decision in every wave
            __syncthreads();                      // the operand tiles (or the previous exchange) are no longer read
            if (wk > 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) red[(wave * 16 + r) * 64 + lane] = acc[ts][r];
            }
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int q = 1; q < KW; ++q)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[ts][r] += red[((wn + NTW * q) * 16 + r) * 64 + lane];
            }
        }
        if (wk > 0) return;
    }

    // epilogue: rows = token slots 8*(r/4) + 4*hb + r%4, column = channel n0 + wn*32 + lane%32
#pragma unroll
    for (int ts = 0; ts < TS; ++ts) {
        if (!((live >> ts) & 1u)) continue;   // same decision in every wave
        int toks[16];   // gathered with every lane of the wave active
        float wts[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            toks[r] = tok_of(ts, 8 * (r >> 2) + 4 * hb + (r & 3));
            wts[r] = mul_routed_weight ? weight_of(ts, 8 * (r >> 2) + 4 * hb + (r & 3)) : 1.f;
        }
        if constexpr (SILU) {
            const int nt = wn * 32 + (lane & 31);               // tile row of this lane's channel
            const bool ok = row_ok(nt);
            float ch_scale = 1.f;
            if (W8 && ok) ch_scale = b_scale[row_of(nt) + (int64_t)expert * ld_scale];
            // both halves rounded to the activation type, as the unfused GEMM stores them
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = acc[ts][r];
                if (W8) v *= ch_scale;
                if (mul_routed_weight && toks[r]) v *= wts[r];
                acc[ts][r] = E::widen(E::cvt(v));
            }
            __syncthreads();   // every wave is done with the operand tiles (and with the previous tile's exchange)
            float* up = reinterpret_cast<float*>(Bs_raw);        // 2 waves x 16 x 64 floats = 8 KB
            if (wn >= 2) {
#pragma unroll
                for (int r = 0; r < 16; ++r) up[((wn - 2) * 16 + r) * 64 + lane] = acc[ts][r];
            }
            __syncthreads();
            if (wn < 2 && ok) {
                const int gc = n0 + nt;                          // output channel, < N / 2
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int tok = toks[r];
                    if (!tok) continue;
                    const float g = acc[ts][r], u = up[(wn * 16 + r) * 64 + lane];
                    C[gc + (int64_t)(tok - 1) * ldc] = E::cvt(silu_mul(g, u));
                }
            }
        } else if (acc_shift >= 0) {
            // Accumulating form: C is (N, num_tokens) and column (token_id - 1) >> acc_shift receives the replica's
            // value as rounded to the storage type, by a packed atomic add of two adjacent channels: lanes 2i and
            // 2i + 1 exchange their values, the even lane sends the even rows and the odd lane the odd ones.
            const int gn = n0 + wn * 32 + (lane & 31);
            float ch_scale = 1.f;
            if (W8 && gn < N) ch_scale = b_scale[gn + (int64_t)expert * ld_scale];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int tok = toks[r];
                float v = acc[ts][r];
                if (W8) v *= ch_scale;
                if (mul_routed_weight) v *= wts[r];
                const unsigned own = (tok && gn < N) ? (unsigned)E::cvt(v) : 0u;
                const unsigned nbr = (unsigned)__shfl_xor((int)own, 1, 64);
                if ((((unsigned)r ^ (unsigned)lane) & 1u) == 0u && tok && gn < N) {
                    const unsigned pair = (lane & 1) ? (nbr | (own << 16)) : (own | (nbr << 16));
                    E::atomic_add2(C + (gn & ~1) + (int64_t)((tok - 1) >> acc_shift) * ldc, pair);
                }
            }
        } else {
            const int gn = n0 + wn * 32 + (lane & 31);
            if (gn < N) {
                float ch_scale = 1.f;
                if (W8) ch_scale = b_scale[gn + (int64_t)expert * ld_scale];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int tok = toks[r];
                    if (!tok) continue;
                    float v = acc[ts][r];
                    if (W8) v *= ch_scale;
                    if (mul_routed_weight) v *= wts[r];
                    C[gn + (int64_t)(tok - 1) * ldc] = E::cvt(v);
                }
            }
        }
    }
}

// ---- SiLU(a) * b -------------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const unsigned short* __restrict__ A, int64_t lda,
                                                           const unsigned short* __restrict__ B, int64_t ldb,
                                                           unsigned short* __restrict__ C, int64_t ldc, int rows,
                                                           int64_t cols, bool vec) {
    const int i0 = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (i0 >= rows) return;
    auto f = [](float x, float y) { return silu_mul(x, y); };
    // (the second grid dimension holds at most 65535 workgroups: walk the columns with that stride)
    for (int64_t col = blockIdx.y; col < cols; col += gridDim.y) {
    const unsigned short* a = A + col * lda;
    const unsigned short* b = B + col * ldb;
    unsigned short* c = C + col * ldc;
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
}

// ---- sum over the top-k slots ---------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void moe_sum_topk_kernel(const unsigned short* __restrict__ in, int64_t s1,
                                                           int64_t s2, unsigned short* __restrict__ out,
                                                           int64_t ldo, int H, int topk, int64_t T) {
    const int h = blockIdx.x * 256 + threadIdx.x;
    if (h >= H) return;
    for (int64_t tok = blockIdx.y; tok < T; tok += gridDim.y) {
        const unsigned short* p = in + h + tok * s2;
        float acc = 0.f;
        for (int k = 0; k < topk; ++k) acc += E::widen(p[k * s1]);
        out[h + tok * ldo] = E::cvt(acc);
    }
}

// The same with eight channels per lane (16-byte loads and stores) and every slot's load issued before the first
// add; a lane walks (token, channel group) pairs, so a launch has a few hundred workgroups however the two extents
// are split.  The slots are added in ascending order in fp32, as above: same bits.
template <typename E, int TOPK>
__global__ __launch_bounds__(256) void moe_sum_topk_vec_kernel(const unsigned short* __restrict__ in, int64_t s1,
                                                               int64_t s2, unsigned short* __restrict__ out,
                                                               int64_t ldo, int hvec, int topk, int64_t items) {
    typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
    for (int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x; it < items; it += (int64_t)gridDim.x * 256) {
        const int64_t tok = it / hvec;
        const int h = (int)(it - tok * hvec) * 8;
        const unsigned short* p = in + h + tok * s2;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (TOPK > 0) {
            u16x8 v[TOPK > 0 ? TOPK : 1];
#pragma unroll
            for (int k = 0; k < TOPK; ++k) v[k] = *reinterpret_cast<const u16x8*>(p + k * s1);
#pragma unroll
            for (int k = 0; k < TOPK; ++k)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] += E::widen(v[k][e]);
        } else {
            for (int k = 0; k < topk; ++k) {
                const u16x8 v = *reinterpret_cast<const u16x8*>(p + k * s1);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] += E::widen(v[e]);
            }
        }
        u16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = E::cvt(acc[e]);
        *reinterpret_cast<u16x8*>(out + h + tok * ldo) = o;
    }
}

bool is16(int dt) { return dt == MI_F16 || dt == MI_BF16; }

}  // namespace

static int fused_moe_impl(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                          const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                          const mi_tile_array* sorted_expert_ids, int num_token_replicas, int mul_routed_weight,
                          int TILE_M, int TILE_N, int TILE_K, const mi_tile_array* b_scale, bool silu, void* stream,
                          bool accumulate = false) {
    MI_CHECK(check_array(A, 2));
    MI_CHECK(check_array(B, 3));
    MI_CHECK(check_array(C, 2));
    if (!topk_weights) return MI_E_NULL;
    if (topk_weights->ndim != 1 && topk_weights->ndim != 2) return MI_E_RANK;
    MI_CHECK(check_array(topk_weights, topk_weights->ndim));
    MI_CHECK(check_array(sorted_token_ids, 1));
    MI_CHECK(check_array(sorted_expert_ids, 1));
    // activations: 16-bit, or E4M3FN together with E4M3FN weights (fp8 x fp8 on the matrix cores, the operand pairing
    // of ext/DLFP8TypesExt.jl:15-19); C and the routed weights are 16-bit either way
    const bool a8 = A->dtype == MI_F8E4M3FN;
    if (!is16(C->dtype) || topk_weights->dtype != C->dtype) return MI_E_DTYPE;
    if (!a8 && A->dtype != C->dtype) return MI_E_DTYPE;
    const bool w8 = B->dtype == MI_F8E4M3FN;
    if (!w8 && (a8 || B->dtype != A->dtype)) return MI_E_DTYPE;
    if (w8 != (b_scale != nullptr)) return MI_E_ARG;
    if (sorted_token_ids->dtype != MI_I32 || sorted_expert_ids->dtype != MI_I32) return MI_E_DTYPE;
    if (!is_pow2(TILE_M) || !is_pow2(TILE_N) || !is_pow2(TILE_K)) return MI_E_TILE;
    if (num_token_replicas < 1) return MI_E_ARG;
    const int64_t K = B->sizes[0], N = B->sizes[1], E = B->sizes[2];
    if (silu && (N % 2)) return MI_E_SHAPE;
    if (A->sizes[0] != K || C->sizes[0] != (silu ? N / 2 : N)) return MI_E_SHAPE;
    // accumulating form: C is (N, num_tokens), and the replicas of a token are added into its column
    int acc_shift = -1;
    if (accumulate) {
        if (topk_weights->ndim != 2 || !mul_routed_weight || silu) return MI_E_ARG;
        const int64_t topk = topk_weights->sizes[1];
        if (topk != 1 && topk != 2) return MI_E_UNSUPPORTED;   // (two terms add up the same in either order; more would not)
        if (C->sizes[1] != topk_weights->sizes[0]) return MI_E_SHAPE;
        if (N % 2 || C->strides[1] % 2 || !aligned(C->ptr, 4)) return MI_E_ALIGN;
        acc_shift = (int)topk - 1;
    }
    const int64_t slots = sorted_token_ids->sizes[0], total = accumulate ? C->sizes[1] * topk_weights->sizes[1] : C->sizes[1];
    const int64_t m_blocks = cld(slots, (int64_t)TILE_M);
    if (sorted_expert_ids->sizes[0] < m_blocks) return MI_E_SHAPE;
    // routed weights: the flattened vector of moe.jl:193, or the (num_tokens, topk) matrix itself with any strides
    const bool w2d = topk_weights->ndim == 2;
    const int64_t w_topk = w2d && topk_weights->sizes[1] > 0 ? topk_weights->sizes[1] : 1;
    if (mul_routed_weight && (w2d ? topk_weights->sizes[0] * topk_weights->sizes[1] != total : topk_weights->sizes[0] < total)) return MI_E_SHAPE;
    if (w_topk > 0x7fffffff) return MI_E_SHAPE;
    if (w8) {
        MI_CHECK(check_array(b_scale, 2));
        if (b_scale->dtype != MI_F32) return MI_E_DTYPE;
        if (b_scale->sizes[0] != N || b_scale->sizes[1] != E) return MI_E_SHAPE;
        if (N > 1 && b_scale->strides[0] != 1) return MI_E_STRIDE;
    }
    if ((K > 1 && (A->strides[0] != 1 || B->strides[0] != 1)) || (N > 1 && C->strides[0] != 1)) return MI_E_STRIDE;
    if (slots > 1 && sorted_token_ids->strides[0] != 1) return MI_E_STRIDE;
    if (m_blocks > 1 && sorted_expert_ids->strides[0] != 1) return MI_E_STRIDE;
    if (!w2d && total > 1 && topk_weights->strides[0] != 1) return MI_E_STRIDE;
    if (K > 0x7fffffff || N > 0x7fffffff || total > 0x7ffffffe || slots > 0x7fffffff) return MI_E_SHAPE;
    if (m_blocks * cld(N, (int64_t)TILE_N) > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (m_blocks == 0 || N == 0) return MI_OK;
    hipStream_t s = (hipStream_t)stream;
    {   // dense routing: the grouped GEMM on 128 x 128 tiles fed by a ring of LDS stages (moe_dense.hip), same bits
        mi::moe::DenseArgs d;
        d.A = A->ptr; d.lda = A->strides[1]; d.num_a_cols = (int)A->sizes[1];
        d.B = B->ptr; d.ldb = B->strides[1]; d.sbe = B->strides[2];
        d.C = (unsigned short*)C->ptr; d.ldc = C->strides[1]; d.total_tokens = (int)total;
        d.topk_weights = (const unsigned short*)topk_weights->ptr; d.w_topk = (int)w_topk;
        d.w_s0 = w2d ? topk_weights->strides[0] : (int64_t)1; d.w_s1 = w2d ? topk_weights->strides[1] : (int64_t)0;
        d.sorted_token_ids = (const int*)sorted_token_ids->ptr; d.num_slots = (int)slots;
        d.sorted_expert_ids = (const int*)sorted_expert_ids->ptr; d.num_blocks = (int)m_blocks;
        d.b_scale = w8 ? (const float*)b_scale->ptr : nullptr; d.ld_scale = w8 ? b_scale->strides[1] : 0;
        d.K = (int)K; d.N = (int)N; d.num_experts = (int)E; d.replicas = num_token_replicas;
        d.mul_routed_weight = mul_routed_weight != 0; d.TILE_M = TILE_M; d.acc_shift = acc_shift;
        d.bf16 = C->dtype == MI_BF16; d.silu = silu; d.w8 = w8; d.a8 = a8;
        if (mi::moe::dense_applicable(d)) {
            mi::moe::dense_launch(d, s);
            return launch_status();
        }
        // fp8 activations have no other kernel: blocks of 128 slots (or multiples), K a multiple of 16 from 512 up,
        // rows on 16-byte boundaries
        if (a8) return MI_E_UNSUPPORTED;
    }
    const int tile_slots = TILE_M < kTT ? TILE_M : kTT;
    const int64_t tiles = m_blocks * (TILE_M / tile_slots);
    // Wide strips (128 channels) when they already give the chip >= ~3 workgroups per CU,
    // counting one started 32-slot tile per TILE_M block; otherwise 32-channel strips with an
    // in-workgroup K split.
    // Dense routing (more than 32 tokens per expert on average): two slot tiles per workgroup, and
    // wide strips throughout -- every block then has two or more tiles with tokens, which gives the
    // wide shape its workgroups, and a weight strip is streamed once per 64 tokens.
    const bool dense = tile_slots == kTT && (TILE_M / kTT) % 2 == 0 && total >= (int64_t)kTT * E;
    const bool narrow = !silu && !dense && m_blocks * cld(N, (int64_t)128) < 768 && K >= 512;
    const int n_blocks = silu ? (int)cld(N / 2, (int64_t)64) : (int)cld(N, (int64_t)(narrow ? 32 : 128));
    // (Two tiles per workgroup cover 64 tokens; with that many per expert on average every second expert has a
    // third tile, whose workgroup streams the expert's weights once more.  A variant that takes the whole 128-slot
    // block per workgroup reads every weight once and is no faster -- 69 against 66 us for the gate / up projection
    // at 256 tokens, top-8 of 32 experts: at two workgroups per CU, which is what its registers and LDS allow, too
    // few weight tiles are in flight.  32-channel strips for the dense down projection are slower as well: 63 us
    // with one tile per workgroup and 49 us with two, against 43 us for the wide shape.)
    const int ts = dense ? 2 : 1;
    if (tiles * n_blocks > 0x7fffffffLL) return MI_E_GRID;
    const bool vecA = aligned(A->ptr, 16) && A->strides[1] % 8 == 0;
    const bool vecB = aligned(B->ptr, 16) && B->strides[1] % (w8 ? 16 : 8) == 0 && B->strides[2] % (w8 ? 16 : 8) == 0;
    dim3 grid((unsigned)(tiles / ts * n_blocks));
    // every tile of the launch inside the arrays and 16-byte aligned: the kernels without load predicates
    // (a K step of 512 for the e4m3 down projection, whose steps move half the weight bytes: 29.8 us against 20.4)
    const int kt = narrow ? 256 : 128;
    const bool fast = vecA && vecB && K % kt == 0 && (silu ? (N / 2) % 64 == 0 : N % (narrow ? 32 : 128) == 0);
#define LAUNCH(ET, W8, NTW, KT, SILU, TS)                                                                           \
    do {                                                                                                            \
        if (fast) LAUNCH1(ET, W8, NTW, KT, SILU, TS, true);                                                         \
        else LAUNCH1(ET, W8, NTW, KT, SILU, TS, false);                                                             \
    } while (0)
#define LAUNCH1(ET, W8, NTW, KT, ...)                                                                               \
    hipLaunchKernelGGL((fused_moe_kernel<ET, W8, NTW, KT, ##__VA_ARGS__>), grid, dim3(256), 0, s, (const unsigned short*)A->ptr, \
                       A->strides[1], (int)A->sizes[1], (const void*)B->ptr, B->strides[1], B->strides[2],          \
                       (unsigned short*)C->ptr, C->strides[1], (int)total, (const unsigned short*)topk_weights->ptr, \
                       (const int*)sorted_token_ids->ptr, (int)slots, (const int*)sorted_expert_ids->ptr,           \
                       w8 ? (const float*)b_scale->ptr : nullptr, w8 ? b_scale->strides[1] : 0, (int)K, (int)N,     \
                       (int)E, num_token_replicas, mul_routed_weight != 0, TILE_M, tile_slots, n_blocks, vecA, vecB,     \
                       (int)w_topk, w2d ? topk_weights->strides[0] : (int64_t)1, w2d ? topk_weights->strides[1] : (int64_t)0, acc_shift)
#define LAUNCH_SHAPE(ET, W8)                                  \
    do {                                                      \
        if (silu && ts == 2) LAUNCH(ET, W8, 4, 128, true, 2); \
        else if (silu) LAUNCH(ET, W8, 4, 128, true, 1);       \
        else if (narrow) LAUNCH(ET, W8, 1, 256, false, 1);    \
        else if (ts == 2) LAUNCH(ET, W8, 4, 128, false, 2);   \
        else LAUNCH(ET, W8, 4, 128, false, 1);                \
    } while (0)
    if (A->dtype == MI_F16) {
        if (w8) LAUNCH_SHAPE(F16, true);
        else LAUNCH_SHAPE(F16, false);
    } else {
        if (w8) LAUNCH_SHAPE(BF16, true);
        else LAUNCH_SHAPE(BF16, false);
    }
#undef LAUNCH_SHAPE
#undef LAUNCH
#undef LAUNCH1
    if (silu && ts == 2) set_variant(w8 ? "fused_moe_silu_t64_n64x2_k128_w8a16" : "fused_moe_silu_t64_n64x2_k128");
    else if (silu) set_variant(w8 ? "fused_moe_silu_t32_n64x2_k128_w8a16" : "fused_moe_silu_t32_n64x2_k128");
    else if (narrow) set_variant(w8 ? "fused_moe_t32_n32_k256_ksplit4_w8a16" : "fused_moe_t32_n32_k256_ksplit4");
    else if (ts == 2) set_variant(w8 ? "fused_moe_t64_n128_k128_w8a16" : "fused_moe_t64_n128_k128");
    else set_variant(w8 ? "fused_moe_t32_n128_k128_w8a16" : "fused_moe_t32_n128_k128");
    return launch_status();
}

extern "C" int mi_fused_moe_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                                   const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                                   const mi_tile_array* sorted_expert_ids, int num_token_replicas,
                                   int mul_routed_weight, int TILE_M, int TILE_N, int TILE_K,
                                   const mi_tile_array* b_scale, void* stream) {
    return fused_moe_impl(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids, num_token_replicas, mul_routed_weight,
                          TILE_M, TILE_N, TILE_K, b_scale, false, stream);
}

extern "C" int mi_fused_moe_silu_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                                        const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                                        const mi_tile_array* sorted_expert_ids, int num_token_replicas,
                                        int mul_routed_weight, int TILE_M, int TILE_N, int TILE_K,
                                        const mi_tile_array* b_scale, void* stream) {
    return fused_moe_impl(A, B, C, topk_weights, sorted_token_ids, sorted_expert_ids, num_token_replicas, mul_routed_weight,
                          TILE_M, TILE_N, TILE_K, b_scale, true, stream);
}

extern "C" int mi_fused_moe_accumulate_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* Out,
                                              const mi_tile_array* topk_weights, const mi_tile_array* sorted_token_ids,
                                              const mi_tile_array* sorted_expert_ids, int TILE_M, int TILE_N, int TILE_K,
                                              const mi_tile_array* b_scale, void* stream) {
    return fused_moe_impl(A, B, Out, topk_weights, sorted_token_ids, sorted_expert_ids, 1, 1, TILE_M, TILE_N, TILE_K, b_scale,
                          false, stream, true);
}

// ---- on-device moe_align_tile_size ------------------------------------------------------------
// Counting sort by expert of the replica ids (slot-fastest flattening of topk_ids, examples/moe.jl:148-150), stable:
// the ids of one expert ascend exactly as the sortperm of moe.jl:150 orders them.
//
// A workgroup of sixteen waves sorts a contiguous segment of the replicas, every wave a contiguous part of it:
//   pass 1: the wave counts its replicas per expert (LDS atomics on its own row of a table);
//   scan:   thread e turns expert e's sixteen counts into the first slot of every wave's share of the expert;
//   pass 2: the wave walks its part again, 64 replicas at a time: a replica's slot is the wave's cursor for its expert
//           plus the number of earlier lanes with the same expert (ballots alone, one per bit of the expert id), and
//           the first lane of every expert advances the cursor.
// The passes have no workgroup barrier inside (a wave touches only its own row of the table).
//
// One workgroup is one compute unit, and the sort is bound by that unit's instruction issue (10 us at 8192
// replicas, 40 us at 32768).  Larger batches therefore take two launches of up to 64 workgroups: the first counts
// every workgroup's segment per expert, and the workgroup that arrives last (a ticket, no waiting) scans the counts
// into the first slot of every (workgroup, expert) pair, labels the blocks and fills the sentinels' share; the
// second launch is the one-workgroup kernel per segment with those first slots in place of its own scan.
// The counts travel through a static array of the library (a captured stream is not given it and sorts with one
// workgroup).  The outputs have fixed capacity: unused slots hold the sentinel total+1, unused blocks expert 0,
// which the GEMM kernel skips.
constexpr int kAlignMaxExperts = 1024;
constexpr int kAlignThreads = 1024, kAlignWaves = kAlignThreads / 64;
constexpr int kAlignBatch = 8;            // chunks of 64 replicas whose ids a lane requests together: one memory round trip per batch
constexpr int kAlignMaxWgs = 64;
constexpr int kAlignPairs = 16384;        // (workgroup, expert) pairs of the two-launch sort
constexpr int kAlignOneWgReplicas = 8191; // up to here one launch of one workgroup is the faster sort (8192: 10 us either way, and the
                                          // workgroups that clear an array on the way have the two launches to hide in)
// counts [kAlignPairs] | first slot inside the expert [kAlignPairs] | first slot of the expert [kAlignMaxExperts] | ticket
constexpr int kAlignScratchInts = 2 * kAlignPairs + kAlignMaxExperts + 64;
static __device__ __align__(256) int moe_align_scratch[kAlignScratchInts];
static SharedScratch g_align_scratch[16];

struct AlignArgs {
    const long long* topk_ids;
    int64_t ld_slot;
    int num_tokens, topk;
    float inv_topk;
    int tile_m, num_experts;
    int* sorted_token_ids;
    int cap_slots;
    int* sorted_expert_ids;
    int cap_blocks;
    u32x4* clear;
    int64_t clear_n16;
    int sort_wgs;        // workgroups that sort; the ones behind them zero `clear`
    int wg_chunks;       // chunks of 64 replicas in a workgroup's segment: a multiple of kAlignWaves
};

// Expert (0-based) of replica r, -1 for a replica at or past `limit` or an id outside 1..num_experts (such a replica takes
// no slot).  r < 2^22: the float quotient is off by one at most.
__device__ __forceinline__ int align_expert_of(const AlignArgs& a, int r, int limit) {
    if (r >= limit) return -1;
    int tok = (int)((float)r * a.inv_topk), slot = r - tok * a.topk;
    if (slot < 0) { --tok; slot += a.topk; }
    if (slot >= a.topk) { ++tok; slot -= a.topk; }
    const long long v = a.topk_ids[tok + (int64_t)slot * a.ld_slot];
    return (v >= 1 && v <= a.num_experts) ? (int)v - 1 : -1;
}

// Exclusive scan over the experts of their block counts (thread e holds expert e's): shuffles inside a wave, the waves'
// totals through LDS.  Every thread of the workgroup calls it.
__device__ __forceinline__ int align_scan_blocks(int nb, int* wave_total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = nb;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int first = incl - nb;
#pragma unroll
    for (int w = 0; w < kAlignWaves; ++w) first += w < wave ? wave_total[w] : 0;
    return first;
}

__device__ __forceinline__ void align_clear(const AlignArgs& a) {
    const int64_t wgs = gridDim.x - a.sort_wgs;
    for (int64_t i = (int64_t)(blockIdx.x - a.sort_wgs) * kAlignThreads + threadIdx.x; i < a.clear_n16; i += wgs * kAlignThreads)
        a.clear[i] = u32x4{0, 0, 0, 0};
}

// MULTI: the second launch of the two-launch sort (`start`, `rel`: what the first launch left in the static array).
template <bool MULTI>
__global__ __launch_bounds__(kAlignThreads) void moe_align_kernel(const AlignArgs a, const int* __restrict__ start,
                                                                  const int* __restrict__ rel) {
    __shared__ int tbl[kAlignWaves][kAlignMaxExperts];   // per (wave, expert): count, then next free slot
    __shared__ int s_blocks, wave_total[kAlignWaves];
    // Workgroups past the sorting ones only zero their share of the array the caller wants cleared on the way (e.g.
    // the output that the accumulating down projection adds into).
    if ((int)blockIdx.x >= a.sort_wgs) {
        align_clear(a);
        return;
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, total = a.num_tokens * a.topk;
    const int cpw = a.wg_chunks / kAlignWaves;
    const int seg0 = ((int)blockIdx.x * a.wg_chunks + wave * cpw) * 64, seg1 = seg0 + cpw * 64 < total ? seg0 + cpw * 64 : total;
    // The ids of the wave's first kAlignBatch chunks stay in registers between the passes (a workgroup's segment of up
    // to 8192 replicas is read once), and are requested before the table is cleared.
    int ecache[kAlignBatch];
#pragma unroll
    for (int i = 0; i < kAlignBatch; ++i) ecache[i] = align_expert_of(a, seg0 + 64 * i + lane, seg1);
    for (int e = tid; e < a.num_experts; e += kAlignThreads) {
#pragma unroll
        for (int w = 0; w < kAlignWaves; ++w) tbl[w][e] = 0;
    }
    if (!MULTI)
        for (int i = tid; i < a.cap_slots; i += kAlignThreads) a.sorted_token_ids[i] = total + 1;
    __syncthreads();
    // ---- pass 1
#pragma unroll
    for (int i = 0; i < kAlignBatch; ++i)
        if (ecache[i] >= 0) atomicAdd(&tbl[wave][ecache[i]], 1);
    for (int r0 = seg0 + 64 * kAlignBatch; r0 < seg1; r0 += 64 * kAlignBatch) {
        int eb[kAlignBatch];
#pragma unroll
        for (int i = 0; i < kAlignBatch; ++i) eb[i] = align_expert_of(a, r0 + 64 * i + lane, seg1);
#pragma unroll
        for (int i = 0; i < kAlignBatch; ++i)
            if (eb[i] >= 0) atomicAdd(&tbl[wave][eb[i]], 1);
    }
    __syncthreads();
    // ---- the first slot of every wave's share of every expert (thread e owns expert e)
    if (MULTI) {
        if (tid < a.num_experts) {
            int slot = start[tid] + rel[(int)blockIdx.x * a.num_experts + tid];
#pragma unroll
            for (int w = 0; w < kAlignWaves; ++w) {
                const int c = tbl[w][tid];
                tbl[w][tid] = slot;
                slot += c;
            }
        }
    } else {
        int cnt = 0;
        if (tid < a.num_experts) {
#pragma unroll
            for (int w = 0; w < kAlignWaves; ++w) cnt += tbl[w][tid];
        }
        const int nb = (cnt + a.tile_m - 1) / a.tile_m;
        const int first = align_scan_blocks(nb, wave_total);
        if (tid < a.num_experts) {
            int slot = first * a.tile_m;
#pragma unroll
            for (int w = 0; w < kAlignWaves; ++w) {
                const int c = tbl[w][tid];
                tbl[w][tid] = slot;
                slot += c;
            }
            for (int b = first; b < first + nb && b < a.cap_blocks; ++b) a.sorted_expert_ids[b] = tid + 1;
        }
        if (tid == kAlignThreads - 1) s_blocks = first + nb < a.cap_blocks ? first + nb : a.cap_blocks;
    }
    __syncthreads();
    if (!MULTI)
        for (int b = s_blocks + tid; b < a.cap_blocks; b += kAlignThreads) a.sorted_expert_ids[b] = 0;

    // ---- pass 2
    const unsigned long long lt = lane ? (~0ull >> (64 - lane)) : 0ull;
    const int id_bits = 32 - __builtin_clz((unsigned)(a.num_experts > 1 ? a.num_experts - 1 : 1));
    volatile int* cur = tbl[wave];   // (this wave's row only; its LDS accesses execute in order)
    for (int b0 = seg0; b0 < seg1; b0 += 64 * kAlignBatch) {
        int eb[kAlignBatch];
#pragma unroll
        for (int i = 0; i < kAlignBatch; ++i) eb[i] = b0 == seg0 ? ecache[i] : align_expert_of(a, b0 + 64 * i + lane, seg1);
#pragma unroll
        for (int i = 0; i < kAlignBatch; ++i) {
            const int r0 = b0 + 64 * i;
            if (r0 >= seg1) break;   // (the same decision in every lane)
            const int r = r0 + lane, e = eb[i];
            // the lanes of this chunk that hold the same expert: one ballot per bit of the expert id
            unsigned long long m = __ballot(e >= 0);
            for (int b = 0; b < id_bits; ++b) {
                const unsigned long long bal = __ballot((e >> b) & 1);
                m &= ((e >> b) & 1) ? bal : ~bal;
            }
            const int rank = __popcll(m & lt);
            int base = 0;
            if (e >= 0) base = cur[e];
            // every lane has read its cursor before the first lane of each expert moves it on
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_wave_barrier();
            if (e >= 0) {
                if (rank == 0) cur[e] = base + __popcll(m);
                const int pos = base + rank;
                if (pos < a.cap_slots) a.sorted_token_ids[pos] = r + 1;
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// First launch of the two-launch sort: per-expert counts of every workgroup's segment; the last workgroup to arrive
// turns them into first slots (scratch: counts | rel | start | ticket, see kAlignScratchInts).
__global__ __launch_bounds__(kAlignThreads) void moe_align_count_kernel(const AlignArgs a, int* __restrict__ scratch) {
    __shared__ int hist[kAlignMaxExperts];
    __shared__ int pairs[kAlignPairs];
    __shared__ int s_ticket, s_blocks, wave_total[kAlignWaves];
    if ((int)blockIdx.x >= a.sort_wgs) {
        align_clear(a);
        return;
    }
    const int tid = threadIdx.x, total = a.num_tokens * a.topk, E = a.num_experts, G = a.sort_wgs;
    int* counts = scratch;
    int* rel = scratch + kAlignPairs;
    int* start = scratch + 2 * kAlignPairs;
    int* ticket = scratch + 2 * kAlignPairs + kAlignMaxExperts;
    const int seg0 = (int)blockIdx.x * a.wg_chunks * 64, seg1 = seg0 + a.wg_chunks * 64 < total ? seg0 + a.wg_chunks * 64 : total;
    for (int e = tid; e < E; e += kAlignThreads) hist[e] = 0;
    __syncthreads();
    for (int r0 = seg0; r0 < seg1; r0 += kAlignThreads * 4) {
        int eb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) eb[i] = align_expert_of(a, r0 + kAlignThreads * i + tid, seg1);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (eb[i] >= 0) atomicAdd(&hist[eb[i]], 1);
    }
    // this workgroup's share of the sentinels (the second launch writes the ids over them)
    for (int i = (int)blockIdx.x * kAlignThreads + tid; i < a.cap_slots; i += G * kAlignThreads) a.sorted_token_ids[i] = total + 1;
    __syncthreads();
    // Counts go out with device-scope stores and come in with device-scope loads: they pass by the L2 of the writer's
    // and the reader's XCD, and no cache is written back or invalidated as a fence would have it.
    if (tid < E) __hip_atomic_store(&counts[(int)blockIdx.x * E + tid], hist[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0): the stores have reached memory
    __syncthreads();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != G - 1) return;
    if (tid == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next sort
    for (int i = tid; i < G * E; i += kAlignThreads) pairs[i] = __hip_atomic_load(&counts[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    int cnt = 0;
    if (tid < E) {
        for (int g = 0; g < G; ++g) {
            const int c = pairs[g * E + tid];
            pairs[g * E + tid] = cnt;
            cnt += c;
        }
    }
    const int nb = (cnt + a.tile_m - 1) / a.tile_m;
    const int first = align_scan_blocks(nb, wave_total);
    if (tid < E) {
        start[tid] = first * a.tile_m;
        for (int b = first; b < first + nb && b < a.cap_blocks; ++b) a.sorted_expert_ids[b] = tid + 1;
    }
    if (tid == kAlignThreads - 1) s_blocks = first + nb < a.cap_blocks ? first + nb : a.cap_blocks;
    __syncthreads();
    for (int i = tid; i < G * E; i += kAlignThreads) rel[i] = pairs[i];
    for (int b = s_blocks + tid; b < a.cap_blocks; b += kAlignThreads) a.sorted_expert_ids[b] = 0;
}

static int moe_align_device_impl(const mi_tile_array* topk_ids, int tile_m, int num_experts, const mi_tile_array* sorted_token_ids,
                                 const mi_tile_array* sorted_expert_ids, const mi_tile_array* clear, void* stream) {
    MI_CHECK(check_array(topk_ids, 2));
    MI_CHECK(check_array(sorted_token_ids, 1));
    MI_CHECK(check_array(sorted_expert_ids, 1));
    if (topk_ids->dtype != MI_I64 || sorted_token_ids->dtype != MI_I32 || sorted_expert_ids->dtype != MI_I32)
        return MI_E_DTYPE;
    if (!is_pow2(tile_m)) return MI_E_TILE;
    if (num_experts < 1) return MI_E_ARG;
    if (num_experts > kAlignMaxExperts) return MI_E_UNSUPPORTED;
    const int64_t num_tokens = topk_ids->sizes[0], topk = topk_ids->sizes[1], total = num_tokens * topk;
    if (total > (1 << 22)) return MI_E_UNSUPPORTED;  // one workgroup sorts; larger batches use the host routine
    if (num_tokens > 1 && topk_ids->strides[0] != 1) return MI_E_STRIDE;
    const int64_t cap_blocks = sorted_expert_ids->sizes[0], cap_slots = sorted_token_ids->sizes[0];
    // worst case: every expert's last block is one replica short of empty
    const int64_t used = total < num_experts ? total : (int64_t)num_experts;
    const int64_t need_blocks = cld(total + used * (tile_m - 1), (int64_t)tile_m);
    if (cap_blocks < need_blocks || cap_slots < cap_blocks * tile_m) return MI_E_SHAPE;
    if ((cap_slots > 1 && sorted_token_ids->strides[0] != 1) || (cap_blocks > 1 && sorted_expert_ids->strides[0] != 1))
        return MI_E_STRIDE;
    if (cap_slots > 0x7fffffff) return MI_E_SHAPE;
    int64_t clear_n16 = 0;
    if (clear) {   // a dense array of whole 16-byte units
        MI_CHECK(check_array(clear, clear->ndim));
        int64_t n = 1, run = 1;
        for (int d = 0; d < clear->ndim; ++d) {
            if (clear->sizes[d] > 1 && clear->strides[d] != run) return MI_E_STRIDE;
            run *= clear->sizes[d];
            n *= clear->sizes[d];
        }
        const int64_t bytes = n * dtype_size(clear->dtype);
        if (bytes % 16 || !aligned(clear->ptr, 16)) return MI_E_ALIGN;
        clear_n16 = bytes / 16;
    }
    if (cap_blocks == 0 && clear_n16 == 0) return MI_OK;
    const int64_t clear_wgs = clear_n16 ? (cld(clear_n16, (int64_t)(4 * kAlignThreads)) < 256 ? cld(clear_n16, (int64_t)(4 * kAlignThreads)) : 256) : 0;
    AlignArgs a;
    a.topk_ids = (const long long*)topk_ids->ptr;
    a.ld_slot = topk > 1 ? topk_ids->strides[1] : 0;
    a.num_tokens = (int)num_tokens;
    a.topk = (int)topk;
    a.inv_topk = topk > 0 ? 1.0f / (float)topk : 0.f;
    a.tile_m = tile_m;
    a.num_experts = num_experts;
    a.sorted_token_ids = (int*)sorted_token_ids->ptr;
    a.cap_slots = (int)cap_slots;
    a.sorted_expert_ids = (int*)sorted_expert_ids->ptr;
    a.cap_blocks = (int)cap_blocks;
    a.clear = clear ? (u32x4*)clear->ptr : nullptr;
    a.clear_n16 = clear_n16;
    const int64_t chunks = cld(total, (int64_t)64);
    // Two launches of several workgroups: every workgroup at least 1024 replicas, (workgroup, expert) pairs within the
    // static array.
    int64_t wgs = kAlignPairs / num_experts < kAlignMaxWgs ? kAlignPairs / num_experts : kAlignMaxWgs;
    if (wgs > cld(total, (int64_t)kAlignThreads)) wgs = cld(total, (int64_t)kAlignThreads);
    if (total > kAlignOneWgReplicas && wgs >= 2 && cap_blocks > 0) {
        ScratchLease lease;
        if (int* scratch = (int*)lease.acquire(g_align_scratch, HIP_SYMBOL(moe_align_scratch), (hipStream_t)stream)) {
            a.wg_chunks = (int)(cld(cld(chunks, wgs), (int64_t)kAlignWaves) * kAlignWaves);
            a.sort_wgs = (int)cld(chunks, (int64_t)a.wg_chunks);
            hipLaunchKernelGGL(moe_align_count_kernel, dim3((unsigned)(a.sort_wgs + clear_wgs)), dim3(kAlignThreads), 0, (hipStream_t)stream, a, scratch);
            const int sort_wgs = a.sort_wgs;
            a.clear_n16 = 0;   // (the first launch has cleared)
            hipLaunchKernelGGL(moe_align_kernel<true>, dim3((unsigned)sort_wgs), dim3(kAlignThreads), 0, (hipStream_t)stream, a,
                               scratch + 2 * kAlignPairs, scratch + kAlignPairs);
            set_variant("moe_align_device_count_place");
            return launch_status();
        }
    }
    a.sort_wgs = 1;
    a.wg_chunks = (int)((chunks > 0 ? cld(chunks, (int64_t)kAlignWaves) : 1) * kAlignWaves);
    hipLaunchKernelGGL(moe_align_kernel<false>, dim3((unsigned)(1 + clear_wgs)), dim3(kAlignThreads), 0, (hipStream_t)stream, a,
                       (const int*)nullptr, (const int*)nullptr);
    set_variant("moe_align_device_1wg");
    return launch_status();
}

extern "C" int mi_moe_align_tile_size_device(const mi_tile_array* topk_ids, int tile_m, int num_experts,
                                             const mi_tile_array* sorted_token_ids,
                                             const mi_tile_array* sorted_expert_ids, void* stream) {
    return moe_align_device_impl(topk_ids, tile_m, num_experts, sorted_token_ids, sorted_expert_ids, nullptr, stream);
}

extern "C" int mi_moe_align_tile_size_device_clear(const mi_tile_array* topk_ids, int tile_m, int num_experts,
                                                   const mi_tile_array* sorted_token_ids,
                                                   const mi_tile_array* sorted_expert_ids, const mi_tile_array* clear,
                                                   void* stream) {
    if (!clear) return MI_E_NULL;
    return moe_align_device_impl(topk_ids, tile_m, num_experts, sorted_token_ids, sorted_expert_ids, clear, stream);
}

// ---- on-device router ---------------------------------------------------------------------------
// The routing that examples/moe.jl leaves to its caller (moe.jl:311-344 draws random experts on
// the host): the top-k experts of every token's logits, ties to the lower expert id, and the
// softmax over the k selected logits.  One wave per token; lane l holds experts l, l + 64, ...;
// k rounds of a wave-wide argmax over the experts not yet taken.  NaN logits rank as -Inf.
constexpr int kRoutePerLane = 8;  // up to 512 experts

__device__ __forceinline__ float route_load(const void* p, int dtype, int64_t i) {
    if (dtype == MI_F32) return ((const float*)p)[i];
    if (dtype == MI_F16) return F16::widen(((const unsigned short*)p)[i]);
    return BF16::widen(((const unsigned short*)p)[i]);
}

__global__ __launch_bounds__(256) void moe_route_kernel(const void* __restrict__ logits, int ldt, int64_t ls_tok,
                                                        int64_t ls_exp, int num_tokens, int E, int k,
                                                        void* __restrict__ weights, int wdt, int64_t ws_slot,
                                                        long long* __restrict__ ids, int64_t is_slot) {
    const int lane = threadIdx.x & 63, token = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (token >= num_tokens) return;  // whole waves leave
    float v[kRoutePerLane];
    unsigned taken = 0;
#pragma unroll
    for (int j = 0; j < kRoutePerLane; ++j) {
        const int e = lane + 64 * j;
        v[j] = -INFINITY;
        if (e < E) {
            const float x = route_load(logits, ldt, token * ls_tok + e * ls_exp);
            if (x == x) v[j] = x;
        } else {
            taken |= 1u << j;
        }
    }
    float mine = -INFINITY, top = -INFINITY;
    int mine_id = 0;
    for (int s = 0; s < k; ++s) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < kRoutePerLane; ++j) {
            const int e = lane + 64 * j;
            if (!((taken >> j) & 1u) && (v[j] > bv || (v[j] == bv && e < bi))) {
                bv = v[j];
                bi = e;
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ov > bv || (ov == bv && oi < bi)) {
                bv = ov;
                bi = oi;
            }
        }
        if ((bi & 63) == lane) taken |= 1u << (bi >> 6);  // k <= E: some expert is always left
        if (lane == s) {
            mine = bv;
            mine_id = bi;
        }
        if (s == 0) top = bv;
    }
    const float ex = lane < k ? expf(mine - top) : 0.f;
    float sum = ex;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane < k) {
        const float w = ex / sum;
        const int64_t wi = token + lane * ws_slot;
        if (wdt == MI_F32) ((float*)weights)[wi] = w;
        else if (wdt == MI_F16) ((unsigned short*)weights)[wi] = F16::cvt(w);
        else ((unsigned short*)weights)[wi] = BF16::cvt(w);
        ids[token + lane * is_slot] = mine_id + 1;
    }
}

extern "C" int mi_moe_route_topk(const mi_tile_array* logits, const mi_tile_array* topk_weights,
                                 const mi_tile_array* topk_ids, void* stream) {
    MI_CHECK(check_array(logits, 2));
    MI_CHECK(check_array(topk_weights, 2));
    MI_CHECK(check_array(topk_ids, 2));
    auto is_float = [](int d) { return d == MI_F32 || d == MI_F16 || d == MI_BF16; };
    if (!is_float(logits->dtype) || !is_float(topk_weights->dtype) || topk_ids->dtype != MI_I64) return MI_E_DTYPE;
    const int64_t num_tokens = logits->sizes[0], E = logits->sizes[1], k = topk_ids->sizes[1];
    if (topk_ids->sizes[0] != num_tokens || topk_weights->sizes[0] != num_tokens || topk_weights->sizes[1] != k)
        return MI_E_SHAPE;
    if (k < 1 || k > E) return MI_E_ARG;
    if (E > 64 * kRoutePerLane || k > 64) return MI_E_UNSUPPORTED;
    if (num_tokens > 1 && (topk_weights->strides[0] != 1 || topk_ids->strides[0] != 1)) return MI_E_STRIDE;
    if (num_tokens == 0) return MI_OK;
    if (cld(num_tokens, (int64_t)4) > MI_MAX_GRID_DIM) return MI_E_GRID;
    hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)cld(num_tokens, (int64_t)4)), dim3(256), 0, (hipStream_t)stream,
                       (const void*)logits->ptr, logits->dtype, logits->strides[0], logits->strides[1], (int)num_tokens,
                       (int)E, (int)k, (void*)topk_weights->ptr, topk_weights->dtype, topk_weights->strides[1],
                       (long long*)topk_ids->ptr, topk_ids->strides[1]);
    set_variant("moe_route_topk_wave_per_token");
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
    const bool vec = aligned(A->ptr, 16) && aligned(B->ptr, 16) && aligned(C->ptr, 16) && A->strides[1] % 8 == 0 &&
                     B->strides[1] % 8 == 0 && C->strides[1] % 8 == 0;
    dim3 grid((unsigned)cld(rows, (int64_t)2048), (unsigned)(cols < 65535 ? cols : 65535));
    hipStream_t s = (hipStream_t)stream;
    if (A->dtype == MI_F16)
        hipLaunchKernelGGL((silu_and_mul_kernel<F16>), grid, dim3(256), 0, s, (const unsigned short*)A->ptr,
                           A->strides[1], (const unsigned short*)B->ptr, B->strides[1], (unsigned short*)C->ptr,
                           C->strides[1], (int)rows, cols, vec);
    else
        hipLaunchKernelGGL((silu_and_mul_kernel<BF16>), grid, dim3(256), 0, s, (const unsigned short*)A->ptr,
                           A->strides[1], (const unsigned short*)B->ptr, B->strides[1], (unsigned short*)C->ptr,
                           C->strides[1], (int)rows, cols, vec);
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
    if (H > 0x7fffffff || topk > 0x7fffffff) return MI_E_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if (H % 8 == 0 && aligned(in->ptr, 16) && aligned(out->ptr, 16) && in->strides[1] % 8 == 0 && in->strides[2] % 8 == 0 &&
        out->strides[1] % 8 == 0) {
        const int64_t items = (H / 8) * T;
        const int64_t blocks = cld(items, (int64_t)256);
        dim3 vgrid((unsigned)(blocks < 4096 ? blocks : 4096));
#define SUMV(ET, K)                                                                                                         \
    hipLaunchKernelGGL((moe_sum_topk_vec_kernel<ET, K>), vgrid, dim3(256), 0, s, (const unsigned short*)in->ptr, in->strides[1], \
                       in->strides[2], (unsigned short*)out->ptr, out->strides[1], (int)(H / 8), (int)topk, items)
#define SUMV_K(ET)                       \
    do {                                 \
        if (topk == 2) SUMV(ET, 2);      \
        else if (topk == 4) SUMV(ET, 4); \
        else if (topk == 8) SUMV(ET, 8); \
        else SUMV(ET, 0);                \
    } while (0)
        if (in->dtype == MI_F16) SUMV_K(F16);
        else SUMV_K(BF16);
#undef SUMV_K
#undef SUMV
        set_variant("moe_sum_topk_vec8");
        return launch_status();
    }
    dim3 grid((unsigned)cld(H, (int64_t)256), (unsigned)(T < 65535 ? T : 65535));
    if (in->dtype == MI_F16)
        hipLaunchKernelGGL((moe_sum_topk_kernel<F16>), grid, dim3(256), 0, s, (const unsigned short*)in->ptr,
                           in->strides[1], in->strides[2], (unsigned short*)out->ptr, out->strides[1], (int)H,
                           (int)topk, T);
    else
        hipLaunchKernelGGL((moe_sum_topk_kernel<BF16>), grid, dim3(256), 0, s, (const unsigned short*)in->ptr,
                           in->strides[1], in->strides[2], (unsigned short*)out->ptr, out->strides[1], (int)H,
                           (int)topk, T);
    set_variant("moe_sum_topk");
    return launch_status();
}
