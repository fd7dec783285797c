// FP8 GEMM for MI355X: C(M,N) = A(M,K) * B(K,N), column-major, A and B both OCP E4M3FN or both E5M2
// (one byte per element), fp32 accumulation on the fp8 matrix cores, C stored as f32, f16 or bf16.
// The reference lets Float8_E4M3FN / Float8_E5M2 tiles be `mma` operands with an f16 or f32
// accumulator (ext/DLFP8TypesExt.jl:15-19; lhs and rhs must share the type,
// src/compiler/intrinsics/core.jl:589-604); matmul_kernel (examples/matmul.jl:28-60) always
// accumulates in fp32 and converts on the store.
//
// Two kernels:
//   gemm8_big      256(m) x 256(n) workgroup tile, 4 waves of 128x128 = 4x4 tiles of
//                  v_mfma_f32_32x32x64_f8f6f4 (K = 64 per instruction, the 5 PFLOP/s rate), K walked in
//                  steps of 64 bytes through a ring of four 32 KB LDS stages filled by direct
//                  global->LDS transfers: the data movement of the 16-bit kernel (gemm_big.hip) at one
//                  byte per element, so a stage carries twice the K.  K >= 512; rows of any alignment, and
//                  sizes that are not multiples of 16 as in gemm_big.hip (register-fed last K step).
//   gemm8_generic  64x64 tile, register staged, v_mfma_f32_32x32x16_fp8_fp8: any shape / stride.
//
// Operand order inside a K step.  A dot product does not depend on the order of its terms, so the
// kernels only make sure that byte q of the A operand and byte q of the B operand of a lane carry the
// same k; which k the hardware associates with a byte position never enters.
//
// LDS layouts of gemm8_big (per stage):
//   B tile [256 n][64 k]: row = 64 bytes = four 16-byte chunks, chunk c of row n at position
//     c ^ ((n >> 2) & 3); lane (n, half h) reads chunks 2h and 2h+1 with two ds_read_b128.
//   A tile [64 k][256 m]: row = 256 bytes = sixteen chunks, chunk c of row k at position
//     c ^ (2 * (k & 7)).  Fragments come from ds_read_b64_tr_b8: the 16 lanes of a group read an 8 (k) x
//     16 (m) block of bytes (lane r: row r/2, half r%2 of the 16-byte chunk) and lane r receives
//     column r, 8 consecutive k; four such reads give a lane its 32 k of the step.  With the
//     swizzle the 8 rows x 2 chunks that the two groups of a half-wave touch are 16 different
//     16-byte positions: all 64 banks once.
#include "gemm_direct.h"

namespace {

using namespace mi;
using namespace mi::gemm;

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef unsigned char u8;

// FMT: 0 = E4M3FN, 1 = E5M2 (the encodings of the instruction's cbsz / blgp fields).
template <int FMT>
__device__ __forceinline__ f32x16 mfma_k64(i32x8 rows, i32x8 cols, f32x16 c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rows, cols, c, FMT, FMT, 0, 0, 0, 0);
}
template <int FMT>
__device__ __forceinline__ f32x16 mfma_k16(long rows, long cols, f32x16 c) {
    if constexpr (FMT == 0) return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(rows, cols, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(rows, cols, c, 0, 0, 0);
}

template <int OD> struct Out;
template <> struct Out<MI_F32> {
    using T = float;
    static __device__ __forceinline__ T cvt(float v) { return v; }
};
template <> struct Out<MI_F16> {
    using T = unsigned short;
    static __device__ __forceinline__ T cvt(float v) { return F16::from_f32(v); }
};
template <> struct Out<MI_BF16> {
    using T = unsigned short;
    static __device__ __forceinline__ T cvt(float v) { return BF16::from_f32(v); }
};

// ---- generic kernel ---------------------------------------------------------------------------
// Workgroup tile 64(m) x 64(n), K step 64, 4 waves as 2x2 of 32x32.  A is written to LDS transposed,
// byte by byte ([m][k]), so both fragments are plain 8-byte reads.
constexpr int GT8 = 64, GK8 = 64, G8_PITCH = GK8 + 16;

template <int FMT, int OD>
__global__ __launch_bounds__(256) void gemm8_generic(const u8* __restrict__ A, int64_t lda, int64_t sa,
                                                     const u8* __restrict__ B, int64_t ldb, int64_t sb,
                                                     typename Out<OD>::T* __restrict__ C, int64_t ldc, int64_t sc,
                                                     int M, int N, int K, int tiles_m, int tiles_mn, bool vecA,
                                                     bool vecB) {
    __shared__ __attribute__((aligned(16))) u8 At[GT8 * G8_PITCH];  // [m][k]
    __shared__ __attribute__((aligned(16))) u8 Bs[GT8 * G8_PITCH];  // [n][k]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bz = blockIdx.x / tiles_mn, L = blockIdx.x - bz * tiles_mn;
    const int bm = L % tiles_m, bn = L / tiles_m;
    const int64_t m0 = (int64_t)bm * GT8, n0 = (int64_t)bn * GT8;
    A += (int64_t)bz * sa;
    B += (int64_t)bz * sb;
    C += (int64_t)bz * sc;
    const int wm = (wave & 1) * 32, wn = (wave >> 1) * 32;
    const int ak = tid >> 2, am = (tid & 3) * 16;   // A tile: row k, 16 consecutive m
    const int bnn = tid >> 2, bk = (tid & 3) * 16;  // B tile: column n, 16 consecutive k
    f32x16 acc = {0};

    for (int k0 = 0; k0 < K; k0 += GK8) {
        union { u32x4 v; u8 b[16]; } va, vb;
        va.v = u32x4{0, 0, 0, 0};
        vb.v = u32x4{0, 0, 0, 0};
        {
            const int64_t gm = m0 + am;
            const int gk = k0 + ak;
            if (gk < K) {
                const u8* p = A + gm + (int64_t)gk * lda;
                if (vecA && gm + 16 <= M) va.v = *reinterpret_cast<const u32x4*>(p);
                else
#pragma unroll
                    for (int q = 0; q < 16; ++q) va.b[q] = (gm + q < M) ? p[q] : (u8)0;
            }
            const int64_t gn = n0 + bnn;
            const int gk2 = k0 + bk;
            if (gn < N) {
                const u8* p = B + gk2 + gn * ldb;
                if (vecB && gk2 + 16 <= K) vb.v = *reinterpret_cast<const u32x4*>(p);
                else
#pragma unroll
                    for (int q = 0; q < 16; ++q) vb.b[q] = (gk2 + q < K) ? p[q] : (u8)0;
            }
        }
        __syncthreads();  // the previous iteration's fragment reads are done
#pragma unroll
        for (int q = 0; q < 16; ++q) At[(am + q) * G8_PITCH + ak] = va.b[q];
        *reinterpret_cast<u32x4*>(&Bs[bnn * G8_PITCH + bk]) = vb.v;
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < GK8 / 16; ++ks) {
            const long fn = *reinterpret_cast<const long*>(&Bs[(wn + (lane & 31)) * G8_PITCH + ks * 16 + 8 * (lane >> 5)]);
            const long fm = *reinterpret_cast<const long*>(&At[(wm + (lane & 31)) * G8_PITCH + ks * 16 + 8 * (lane >> 5)]);
            acc = mfma_k16<FMT>(fn, fm, acc);
        }
    }
    const int64_t gm = m0 + wm + (lane & 31);
    if (gm < M) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t gn = n0 + wn + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (gn < N) C[gm + gn * ldc] = Out<OD>::cvt(acc[r]);
        }
    }
}

// ---- direct-to-LDS kernel ---------------------------------------------------------------------
constexpr int BK8 = 64;                 // k per step (= bytes per B row of a stage)
constexpr int BT8 = 256;                // tile edge
constexpr int STAGE8 = BT8 * BK8;       // bytes per operand and stage (16 KB)

__device__ __attribute__((aligned(16))) const unsigned zeros16b[4] = {0u, 0u, 0u, 0u};

struct Lane8 {
    int kA, kB;          // first k, within a stage, of the lane's chunk in A transfer 0 (transfer j: + 16 j) / in a B transfer
    unsigned goffA;      // byte offset of the lane's chunk within a wave-wide 1 KB transfer of A (4 rows of k)
    int64_t goffB[4];    // the same for the wave's four B transfers (16 rows of n each)
    unsigned fb[2];      // LDS byte offset of the two chunks of the B fragment (+ 32*j*BK8 for n tile j)
    unsigned fa[4];      // LDS byte offset of the first transpose read of the A fragment, m tile i (+ 8*t*BT8 for read t)
};

struct Frag8 {
    i32x8 a[4], b[4];
};

template <bool TAIL = false>
__device__ __forceinline__ void issue_B8(const char* Bg, u8* Bs, int wave, const Lane8& ln, int k_left = 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const char* g = Bg + ln.goffB[j];
        if (TAIL && ln.kB >= k_left) g = (const char*)zeros16b;
        gload_lds16(g, Bs + (wave + 4 * j) * 1024);
    }
}
template <bool TAIL = false>
__device__ __forceinline__ void issue_A8(const char* Ag, int64_t lda, u8* As, int wave, const Lane8& ln, int k_left = 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const char* g = Ag + (int64_t)(16 * j) * lda + ln.goffA;
        if (TAIL && ln.kA + 16 * j >= k_left) g = (const char*)zeros16b;
        gload_lds16(g, As + (wave + 4 * j) * 1024);
    }
}

__device__ __forceinline__ void load_b_frags(const u8* Bs, const Lane8& ln, Frag8& f) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const i32x4 lo = *reinterpret_cast<const i32x4*>(Bs + ln.fb[0] + 32 * j * BK8);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(Bs + ln.fb[1] + 32 * j * BK8);
        f.b[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}
template <int I0>
__device__ __forceinline__ void load_a_frags(const u8* As, const Lane8& ln, Frag8& f) {
#pragma unroll
    for (int i = I0; i < I0 + 2; ++i) {
        const u8* p = As + ln.fa[i];
        const i32x2 t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(i32x2, p));
        const i32x2 t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(i32x2, p + 8 * BT8));
        const i32x2 t2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(i32x2, p + 16 * BT8));
        const i32x2 t3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(i32x2, p + 24 * BT8));
        f.a[i] = i32x8{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
    }
}

template <int FMT, int I0>
__device__ __forceinline__ void mma8(const i32x8 (&a)[4], const i32x8 (&b)[4], f32x16 (&acc)[4][4]) {
#pragma unroll
    for (int i = I0; i < I0 + 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma_k64<FMT>(b[j], a[i], acc[i][j]);
}

// Spread NRD LDS reads and NDMA transfers over the 8 MFMAs of a half step.
template <int NRD, int NDMA>
__device__ __forceinline__ void interleave8() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        if (NRD >= 8) __builtin_amdgcn_sched_group_barrier(SG_DSRD, NRD / 8, 0);
        if (NDMA && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
}

// One K step of 64 on stage (AsX, BsX); the next step's data is in (AsY, BsY).
//   first half : MFMAs of m tiles 0, 1 | read the A fragments of m tiles 2, 3 | issue the A transfers of step s+3
//   barrier      (every wave has read everything it needs from BsX)
//   second half: MFMAs of m tiles 2, 3 | read the next stage's B fragments and A fragments 0, 1 | issue the B transfers of step s+4 into BsX
// f holds the A fragments; the B fragments alternate between bcur and bnext.
template <int FMT, bool DMA_A, bool DMA_B, int VMCNT, bool LAST, bool TAIL>
__device__ __forceinline__ void k_step8(const u8* AsX, u8* BsX, const u8* AsY, const u8* BsY, u8* AsA, const char* Ag_next3,
                                        const char* Bg_next4, int64_t lda, int wave, const Lane8& ln, Frag8& f,
                                        Frag8& fnext, f32x16 (&acc)[4][4], int k_left3) {
    if (DMA_A) issue_A8<TAIL>(Ag_next3, lda, AsA, wave, ln, k_left3);
    load_a_frags<2>(AsX, ln, f);
    mma8<FMT, 0>(f.a, f.b, acc);
    interleave8<8, DMA_A ? 4 : 0>();
    if (!LAST) stage_barrier<VMCNT>();
    if (DMA_B) issue_B8<TAIL>(Bg_next4, BsX, wave, ln, k_left3 - BK8);
    if (!LAST) {
        load_b_frags(BsY, ln, fnext);
        load_a_frags<0>(AsY, ln, fnext);
    }
    mma8<FMT, 2>(f.a, f.b, acc);
    interleave8<LAST ? 0 : 16, DMA_B ? 4 : 0>();
}

template <int FMT, int OD>
__global__ __launch_bounds__(256) void gemm8_big(const u8* __restrict__ A, int64_t lda, int64_t sa,
                                                 const u8* __restrict__ B, int64_t ldb, int64_t sb,
                                                 typename Out<OD>::T* __restrict__ C, int64_t ldc, int64_t sc, int M,
                                                 int N, int K, int tiles_m, int tiles_n, int batch, int kpeel) {
    // K: the extent the transfers walk (a multiple of 16); kpeel: values of k behind it for the register-fed step
    using OutT = typename Out<OD>::T;
    __shared__ __attribute__((aligned(1024))) u8 As0[STAGE8], As1[STAGE8], As2[STAGE8], As3[STAGE8];
    __shared__ __attribute__((aligned(1024))) u8 Bs0[STAGE8], Bs1[STAGE8], Bs2[STAGE8], Bs3[STAGE8];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups whose ids are congruent mod 8 share an XCD and its L2: each XCD gets a contiguous run of
    // (batch-major) tiles, walked in groups of four m tiles.
    const int total = tiles_m * tiles_n, total_all = total * batch;
    int L = blockIdx.x;
    if (total_all % 8 == 0) L = (L & 7) * (total_all >> 3) + (L >> 3);
    const int bz = L / total;
    L -= bz * total;
    constexpr int GM = 4;
    const int per_group = GM * tiles_n;
    const int first_m = (L / per_group) * GM;
    const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int bm = first_m + (L % per_group) % gsz, bn = (L % per_group) / gsz;
    const int wm = (wave & 1) * 128, wn = (wave >> 1) * 128;

    Lane8 ln;
    {
        const int g = lane >> 4, r = lane & 15, h = lane >> 5;
        // B transfer: 16 rows of n x 64 bytes; lane -> row lane/4, LDS position lane%4.  Rows past N
        // re-read row N-1 (their products land in accumulators that are never stored).
        const int first = bn * BT8 + 16 * wave;
        const int cb = (lane & 3) ^ ((lane >> 4) & 3);     // chunk that belongs at the lane's LDS position
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int row = 64 * j + (lane >> 2);
            if (first + row > N - 1) row = N - 1 - first;
            ln.goffB[j] = (int64_t)row * ldb + 16 * cb;
        }
        ln.kB = 16 * cb;
        // A transfer: 4 rows of k x 256 bytes; lane -> row lane/16, LDS position lane%16.  Chunks of 16 m
        // that start past the edge re-read the last chunk that starts inside.
        const int ka = 4 * wave + (lane >> 4);
        ln.kA = ka;
        int ca = (lane & 15) ^ (2 * (ka & 7));
        if (bm * BT8 + 16 * ca >= M) ca = (M - 1 - bm * BT8) / 16;
        ln.goffA = (unsigned)((int64_t)(lane >> 4) * lda + 16 * ca);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int n = wn + (lane & 31);
            ln.fb[t] = n * BK8 + 16 * ((2 * h + t) ^ ((n >> 2) & 3));
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = 32 * (g >> 1) + (r >> 1);                 // first of the lane's four read rows (+ 8 t)
            const int m = wm + 32 * i + 16 * (g & 1) + 8 * (r & 1);
            ln.fa[i] = k * BT8 + 16 * ((m >> 4) ^ (2 * (k & 7))) + (m & 15);
        }
    }
    // wave-uniform byte pointers to this wave's first rows of the k = 0 stage
    const char* Ab = (const char*)(A + (int64_t)bz * sa + (int64_t)bm * BT8) + (int64_t)(4 * wave) * lda;
    const char* Bb = (const char*)(B + (int64_t)bz * sb + (int64_t)bn * BT8 * ldb) + (int64_t)(16 * wave) * ldb;
    C += (int64_t)bz * sc;
    const int64_t a_step = (int64_t)BK8 * lda;  // next K step of A: 64 rows down
    const int64_t b_step = BK8;                 // next K step of B: 64 bytes along the row

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x16{0};

    const int KT = 4 * ((K + 4 * BK8 - 1) / (4 * BK8));  // steps, in whole groups of four; >= 8 (K >= 512 is checked on the host)
    Frag8 f0, f1;
    issue_B8(Bb, Bs0, wave, ln);
    issue_A8(Ab, lda, As0, wave, ln);
    issue_B8(Bb + b_step, Bs1, wave, ln);
    issue_A8(Ab + a_step, lda, As1, wave, ln);
    issue_B8(Bb + 2 * b_step, Bs2, wave, ln);
    issue_A8(Ab + 2 * a_step, lda, As2, wave, ln);
    issue_B8(Bb + 3 * b_step, Bs3, wave, ln);
    constexpr int PER_STAGE = 8;   // transfers per wave and stage
    stage_barrier<2 * PER_STAGE + 4>();
    load_b_frags(Bs0, ln, f0);
    load_a_frags<0>(As0, ln, f0);

#define KSTEP(X, Y, AA, FC, FN, DA, DB, VM, LAST, TAIL, s)                                                           \
    k_step8<FMT, DA, DB, (VM) * PER_STAGE, LAST, TAIL>(As##X, Bs##X, As##Y, Bs##Y, As##AA, Ab + (int64_t)((s) + 3) * a_step, \
                                                       Bb + (int64_t)((s) + 4) * b_step, lda, wave, ln, FC, FN, acc,   \
                                                       K - ((s) + 3) * BK8)
    int s = 0;
    for (; s + 12 <= KT; s += 4) {
        KSTEP(0, 1, 3, f0, f1, true, true, 2, false, false, s);
        KSTEP(1, 2, 0, f1, f0, true, true, 2, false, false, s + 1);
        KSTEP(2, 3, 1, f0, f1, true, true, 2, false, false, s + 2);
        KSTEP(3, 0, 2, f1, f0, true, true, 2, false, false, s + 3);
    }
    // the group that requests the last four stages (the only ones that can reach past K)
    KSTEP(0, 1, 3, f0, f1, true, true, 2, false, true, s);
    KSTEP(1, 2, 0, f1, f0, true, true, 2, false, true, s + 1);
    KSTEP(2, 3, 1, f0, f1, true, true, 2, false, true, s + 2);
    KSTEP(3, 0, 2, f1, f0, true, true, 2, false, true, s + 3);
    s += 4;
    // last four steps: only the A half of the final stage is still to be requested
    KSTEP(0, 1, 3, f0, f1, true, false, 2, false, true, s);
    KSTEP(1, 2, 0, f1, f0, false, false, 1, false, false, s + 1);
    KSTEP(2, 3, 1, f0, f1, false, false, 0, false, false, s + 2);
    KSTEP(3, 0, 2, f1, f0, false, false, 0, true, false, s + 3);
#undef KSTEP

    if (kpeel > 0) {   // (same for the whole grid)
        // k = K .. K + kpeel - 1 as the first values of one 64-wide MFMA step: the lower half-wave holds k 0..31 of its
        // row of B / column of A (here: up to 16 values, then zeros), the upper half-wave zeros.
        const u8* Ap = A + (int64_t)bz * sa + (int64_t)K * lda;
        const u8* Bp = B + (int64_t)bz * sb + K;
        const bool lower = lane < 32;
        auto gather = [&](const u8* p, int64_t step, bool live) {
            i32x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const unsigned byte = live && q < kpeel ? p[q * step] : 0u;
                v[q >> 2] |= (int)(byte << (8 * (q & 3)));
            }
            return v;
        };
        i32x8 pa[4], pb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = (int64_t)bn * BT8 + wn + 32 * j + (lane & 31);
            pb[j] = gather(Bp + (n < N ? n : 0) * ldb, 1, lower && n < N);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t m = (int64_t)bm * BT8 + wm + 32 * i + (lane & 31);
            pa[i] = gather(Ap + (m < M ? m : 0), lda, lower && m < M);
        }
        mma8<FMT, 0>(pa, pb, acc);
        mma8<FMT, 2>(pa, pb, acc);
    }

    // Epilogue: a half-wave holds 32 consecutive m of one column of C.
    const unsigned lane_off = (unsigned)((lane & 31) + (int64_t)(4 * (lane >> 5)) * ldc);
    OutT* Cw = C + (int64_t)bm * BT8 + wm + ((int64_t)bn * BT8 + wn) * ldc;
    if ((bm + 1) * BT8 <= M && (bn + 1) * BT8 <= N) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    OutT* cu = Cw + 32 * i + (int64_t)(32 * j + 8 * (r >> 2) + (r & 3)) * ldc;
                    __builtin_nontemporal_store(Out<OD>::cvt(acc[i][j][r]), cu + lane_off);
                }
    } else {
        int m_left = M - (bm * BT8 + wm + (lane & 31)), n_left = N - (bn * BT8 + wn + 4 * (lane >> 5));
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    asm volatile("" : "+v"(m_left), "+v"(n_left));   // keeps each test next to its store
                    const int dn = 32 * j + 8 * (r >> 2) + (r & 3);
                    if (32 * i < m_left && dn < n_left) {
                        float v = acc[i][j][r];
                        asm volatile("" : "+v"(v));
                        __builtin_nontemporal_store(Out<OD>::cvt(v), Cw + 32 * i + (int64_t)dn * ldc + lane_off);
                    }
                }
    }
}

template <int FMT, int OD>
void launch_big(const Problem& p, hipStream_t s) {
    const int tiles_m = (p.M + BT8 - 1) / BT8, tiles_n = (p.N + BT8 - 1) / BT8;
    // The extent of K that the transfers walk: whole chunks of 16, and not the last row of A when a chunk of A can
    // straddle the end of a row (M not a multiple of 16: the chunk then reads on into the next row, which must exist).
    const int kd = p.M % 16 ? (p.K - 1) / 16 * 16 : p.K / 16 * 16;
    hipLaunchKernelGGL((gemm8_big<FMT, OD>), dim3((unsigned)(tiles_m * tiles_n * p.batch)), dim3(256), 0, s,
                       (const u8*)p.A, p.lda, p.sa, (const u8*)p.B, p.ldb, p.sb, (typename Out<OD>::T*)p.C, p.ldc,
                       p.sc, p.M, p.N, kd, tiles_m, tiles_n, p.batch, p.K - kd);
}

template <int FMT, int OD>
void launch_generic(const Problem& p, hipStream_t s) {
    const int tiles_m = (p.M + GT8 - 1) / GT8, tiles_n = (p.N + GT8 - 1) / GT8;
    const bool vecA = aligned(p.A, 16) && p.lda % 16 == 0 && p.sa % 16 == 0;
    const bool vecB = aligned(p.B, 16) && p.ldb % 16 == 0 && p.sb % 16 == 0;
    hipLaunchKernelGGL((gemm8_generic<FMT, OD>), dim3((unsigned)(tiles_m * tiles_n * p.batch)), dim3(256), 0, s,
                       (const u8*)p.A, p.lda, p.sa, (const u8*)p.B, p.ldb, p.sb, (typename Out<OD>::T*)p.C, p.ldc,
                       p.sc, p.M, p.N, p.K, tiles_m, tiles_m * tiles_n, vecA, vecB);
}

template <int FMT>
void dispatch(const Problem& p, hipStream_t s, bool big) {
#define GO(OD) (big ? launch_big<FMT, OD>(p, s) : launch_generic<FMT, OD>(p, s))
    if (p.out_dtype == MI_F32) GO(MI_F32);
    else if (p.out_dtype == MI_F16) GO(MI_F16);
    else GO(MI_BF16);
#undef GO
}

bool big8_applicable(const Problem& p) {
    // Any alignment of the rows, any M, N and K from 512 on (sizes that are not multiples of 16: the K tail, and with a
    // ragged M the last rows of A, are one register-fed MFMA step); enough tiles of 256 x 256 to give every XCD work.
    return p.M >= 16 && p.N >= 1 && p.K >= 512 + 16 * (p.M % 16 != 0 || p.K % 16 != 0) &&
           p.lda >= p.M && p.ldb >= p.K && p.ldc >= p.M && p.sa >= 0 && p.sb >= 0 && p.sc >= 0 &&
           p.ldc < (1 << 26) && p.lda < (1 << 27) && p.ldb < (1 << 27) && tiles_of(p, BT8, BT8) >= 8 &&
           tiles_of(p, BT8, BT8) < (1 << 30);
}

}  // namespace

namespace mi {
namespace gemm {

void fp8_launch(const Problem& p, hipStream_t s) {
    static const int force = [] { const char* e = getenv("MI_GEMM_KERNEL"); return e ? atoi(e) : 0; }();   // 1: generic
    const bool big = big8_applicable(p) && force != 1;
    if (p.in_dtype == MI_F8E4M3FN) dispatch<0>(p, s, big);
    else dispatch<1>(p, s, big);
    set_variant(big ? "gemm8_big_256x256x64_ring4" : "gemm8_generic_64x64x64");
}

}  // namespace gemm
}  // namespace mi
