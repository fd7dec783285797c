// Large-tile f16/bf16 GEMM for MI355X: C(M,N) = A(M,K) * B(K,N), column-major, fp32 accumulate.
//
// Workgroup tile 256(m) x 256(n); 4 waves as 2x2, each 128x128 = 4x4 MFMA 32x32x16 tiles
// (256 accumulator registers per lane, one wave per SIMD).  K is walked in steps of 32
// through a ring of four LDS stages (4 x 32 KB) filled by direct global->LDS transfers
// (global_load_lds, 16 bytes per lane, no staging registers).  The transfers for step s+3 /
// s+4 are issued while step s is multiplied, a few at a time between the MFMAs, so the L2 /
// fabric see a steady stream and every transfer has two to three steps (> 1 us) to land.
// One workgroup barrier per step; the barrier waits only for the oldest stage in flight
// (s_waitcnt vmcnt(16)), never for the stream to drain.
//
// LDS layouts (per stage):
//   B tile [256 n][32 k]: row = 64 bytes = four 16-byte chunks; chunk c of row n sits at
//     position c ^ ((n >> 2) & 3), so the 16 rows a quarter-wave reads with ds_read_b128 cover
//     all 64 banks.
//   A tile [32 k][256 m]: row = 512 bytes; chunk c of row k sits at position c ^ (4*(k & 3)),
//     so the 4 rows x 32 bytes each 16-lane group of a transpose read (ds_read_b64_tr_b16)
//     touches, and the two groups of a half-wave, land on 8 distinct 32-byte bank groups.
//   Both swizzles are applied on the global side: the lane whose LDS slot is `pos` fetches
//   the chunk that belongs there.
//
// The MFMA row operand carries n (B fragments, plain 16-byte reads), the column operand
// (lane % 32) carries m (A fragments through the transpose read); a half-wave therefore
// holds 32 consecutive m of one column of C and every store is a full 128-byte line.
//
// Workgroups are numbered so that the tiles resident on one XCD (ids congruent mod 8) form a
// 4 x 8 block of tiles and share A row panels / B column panels in that XCD's L2.
//
// Requires K >= 256.  Tiles that reach past M or N re-read the last valid rows / chunks on the way in and clip
// their stores.  K is walked in whole groups of four steps (128); in the last group the 16-byte chunks at
// k >= K are fetched from a 16-byte block of zeros instead (both operands, so padding never meets a non-finite value).
// Rows need no alignment: the transfers take any element-aligned address (a dense matrix with an odd leading
// dimension: 0.94-1.12 PFLOP/s at 4096^3 against 1.15 with aligned rows).  Sizes that are not multiples of 8:
//   * K: the transfers cover the whole chunks of 8, k < Kd; the remaining 1 to 8 values of k are one more MFMA step
//     whose fragments come straight from global memory into registers, element by element with zeros past the edges;
//   * M: the chunk of A that straddles the end of a row reads on into the next row (its surplus only reaches rows of
//     C that are never stored); so that no such read passes the end of the array, the last row of A is always
//     left to the register-fed step (Kd <= K - 1 then).
#include "gemm_direct.h"
#include "shared_scratch.h"

namespace {

using namespace mi;
using namespace mi::gemm;

// The tile is (64*I) m x (64*J) n, a wave's part (32*I) x (32*J): I = J = 4 is the 256x256 tile described
// above; 256x128 (I = 4, J = 2: half the B stage, half the accumulators) and 128x128 (I = J = 2: 64 KB of
// LDS, two workgroups per CU) serve problems that would otherwise give too few workgroups to the chip.
// An A stage of 32 k x (64*I) m moves as 4*I transfers of 1 KB, each 8/I rows of k; a row is 8*I chunks.
constexpr int BK = 32;

// Source of every chunk that lies past K.
__device__ __attribute__((aligned(16))) const unsigned zeros16[4] = {0u, 0u, 0u, 0u};

struct Lane {
    int kA, kB;             // first k, within a stage, of the lane's chunk in A transfer 0 (transfer j: + 32/I*j) / in a B transfer
    unsigned goffA;         // byte offset of this lane's 16-byte chunk within a wave-wide 1 KB transfer of A
    int64_t goffB[4];       // the same for the wave's four B transfers (rows past the matrix edge re-read the last row)
    unsigned fb[2];         // LDS element offset of the B fragment, k16 sub-step 0/1 (+ 32*j*BK for n tile j)
    unsigned fa[4];         // LDS element offset of the A fragment, m tile i (+ 16*ks*64*I for sub-step ks)
};

struct Frag {
    s16x8 a[4], b[4];   // (b[j] for j < J)
};

// B stage: 64*J rows x 64 B = 4*J transfers of 1 KB (16 rows each); wave w takes transfers w, w+4, ...
// TAIL: k_left = K - (first k of the stage); chunks at or past it come from the zero block.
template <int J, bool TAIL = false>
__device__ __forceinline__ void issue_B(const char* Bg, int64_t ldb2, unsigned short* Bs, int wave, const Lane& ln,
                                        int k_left = 0) {
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const char* g = Bg + ln.goffB[j];
        if (TAIL && ln.kB >= k_left) g = (const char*)zeros16;
        gload_lds16(g, Bs + (wave + 4 * j) * 512);
    }
}
// A stage: 32 rows x 128*I B = 4*I transfers of 1 KB (8/I rows each); wave w takes transfers w, w+4, ...
template <int I, bool TAIL = false>
__device__ __forceinline__ void issue_A(const char* Ag, int64_t lda2, unsigned short* As, int wave, const Lane& ln,
                                        int k_left = 0) {
#pragma unroll
    for (int j = 0; j < I; ++j) {
        const char* g = Ag + (int64_t)(32 / I * j) * lda2 + ln.goffA;
        if (TAIL && ln.kA + 32 / I * j >= k_left) g = (const char*)zeros16;
        gload_lds16(g, As + (wave + 4 * j) * 512);
    }
}

template <int I, int J>
__device__ __forceinline__ void load_frags(const unsigned short* As, const unsigned short* Bs, const Lane& ln, int ks,
                                           Frag& f) {
    constexpr int BTM = 64 * I;
#pragma unroll
    for (int j = 0; j < J; ++j) f.b[j] = *reinterpret_cast<const s16x8*>(Bs + ln.fb[ks] + 32 * j * BK);
#pragma unroll
    for (int i = 0; i < I; ++i) {
        const unsigned short* p = As + ln.fa[i] + 16 * ks * BTM;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 4 * BTM));
        f.a[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

template <typename E, int I, int J>
__device__ __forceinline__ void mma16(const Frag& f, f32x16 (&acc)[I][J]) {
#pragma unroll
    for (int i = 0; i < I; ++i)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[i][j] = E::mfma32(f.b[j], f.a[i], acc[i][j]);
}

// Spread the 2*I + J LDS reads and (if NDMA) the I (A) or J (B) global->LDS transfers of a half step
// over its I*J MFMAs.
template <int I, int J, int NDMA, bool FRAGS>
__device__ __forceinline__ void interleave16() {
    if constexpr (I == 2) {   // 4 MFMAs, 6 reads, 2 transfers
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
            if (FRAGS) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
            if (FRAGS && i < 2) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
            if (NDMA && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
        }
    } else if constexpr (J == 4) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
            if (FRAGS && i < 12) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
            if (NDMA && (i & 3) == 1) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
            if (FRAGS) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
            if (FRAGS && i < 2) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
            if (NDMA == 4 && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
            if (NDMA == 2 && (i & 3) == 1) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}

// One K step of 32 on stage (AsX, BsX); the next step's data is in (AsY, BsY).
//   first half : MFMAs of sub-step 0 | read sub-step 1 fragments | issue A transfers (into stage AsA)
//   barrier
//   second half: MFMAs of sub-step 1 | read next stage's sub-step 0 fragments | issue B transfers (into BsX)
// TAIL: the stages requested here may reach past K; k_left3 = K - (first k of step s+3).
template <typename E, int I, int J, bool DMA_A, bool DMA_B, int VMCNT, bool LAST, bool TAIL>
__device__ __forceinline__ void k_step(const unsigned short* AsX, unsigned short* BsX, const unsigned short* AsY,
                                       const unsigned short* BsY, unsigned short* AsA, const char* Ag_next3,
                                       const char* Bg_next4, int64_t lda2, int64_t ldb2, int wave, const Lane& ln,
                                       Frag& f0, Frag& f1, f32x16 (&acc)[I][J], int k_left3) {
    if (DMA_A) issue_A<I, TAIL>(Ag_next3, lda2, AsA, wave, ln, k_left3);
    load_frags<I, J>(AsX, BsX, ln, 1, f1);
    mma16<E, I, J>(f0, acc);
    interleave16<I, J, DMA_A ? I : 0, true>();
    if (!LAST) stage_barrier<VMCNT>();
    if (DMA_B) issue_B<J, TAIL>(Bg_next4, ldb2, BsX, wave, ln, k_left3 - BK);
    if (!LAST) load_frags<I, J>(AsY, BsY, ln, 0, f0);
    mma16<E, I, J>(f1, acc);
    interleave16<I, J, DMA_B ? J : 0, !LAST>();
}

template <typename E, typename OutT, int I, int J>
__global__ __launch_bounds__(256) void gemm16_big(const unsigned short* __restrict__ A, int64_t lda, int64_t sa,
                                                  const unsigned short* __restrict__ B, int64_t ldb, int64_t sb,
                                                  OutT* __restrict__ C, int64_t ldc, int64_t sc, int M, int N, int K,
                                                  int tiles_m, int tiles_n, int batch, int ksplit, int kchunk, int kpeel) {
    // K: the extent the transfers walk (a multiple of 8); kpeel: values of k behind it for the register-fed step
    constexpr int BTM = 64 * I, STAGE_A = BTM * BK, BTN = 64 * J, STAGE_B = BTN * BK;
    __shared__ __attribute__((aligned(1024))) unsigned short As0[STAGE_A], As1[STAGE_A], As2[STAGE_A], As3[STAGE_A];
    __shared__ __attribute__((aligned(1024))) unsigned short Bs0[STAGE_B], Bs1[STAGE_B], Bs2[STAGE_B], Bs3[STAGE_B];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // One-dimensional grid over (tile, batch).  Workgroups whose ids are congruent mod 8 share an XCD and
    // its L2: give each XCD a contiguous run of (batch-major) tiles, so that it works on neighbouring
    // tiles of as few batch entries as possible.
    // With a split over K (ksplit > 1) consecutive workgroups are the ksplit parts of one tile; part ks walks
    // k = ks * kchunk ... and writes its sums to slice (batch entry * ksplit + ks) of C, which is then the
    // caller's partial-sum buffer.
    const int total = tiles_m * tiles_n, total_all = total * batch;
    int L = blockIdx.x, ks_part = 0;
    if (ksplit > 1) {
        ks_part = L % ksplit;
        L /= ksplit;
        K = K - ks_part * kchunk < kchunk ? K - ks_part * kchunk : kchunk;
    }
    if (total_all % 8 == 0) L = (L & 7) * (total_all >> 3) + (L >> 3);
    const int bz = L / total;
    L -= bz * total;
    constexpr int GM = 4;
    const int per_group = GM * tiles_n;
    const int first_m = (L / per_group) * GM;
    const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int bm = first_m + (L % per_group) % gsz, bn = (L % per_group) / gsz;
    const int wm = (wave & 1) * (32 * I), wn = (wave >> 1) * (32 * J);

    Lane ln;
    {
        const int hb = lane >> 5, g = lane >> 4, r = lane & 15;
        // B transfer: lane -> row lane/4 of its 16-row block, LDS position lane%4; rows n = 16*blk + lane/4.
        // In a tile that reaches past N the rows beyond the edge re-read row N-1 (their products land in
        // accumulators that are never stored), so every transfer stays inside the matrix.
        {
            const int first = bn * BTN + 16 * wave;              // first row of the wave's transfer 0
#pragma unroll
            for (int j = 0; j < J; ++j) {
                int row = 64 * j + (lane >> 2);                  // relative to `first`
                if (first + row > N - 1) row = N - 1 - first;    // (may be negative: still inside the tile's rows)
                ln.goffB[j] = ((int64_t)row * ldb + 8 * ((lane & 3) ^ ((lane >> 4) & 3))) * 2;
            }
        }
        // A transfer: lane -> row lane/(8*I) of its block of 8/I rows, LDS position lane%(8*I); rows
        // k = 8/I*blk + lane/(8*I).  Chunks of 8 m that start past the edge re-read the last chunk that starts inside.
        const int ka = 8 / I * wave + lane / (8 * I);
        ln.kA = ka;
        ln.kB = 8 * ((lane & 3) ^ ((lane >> 4) & 3));
        int ca = (lane % (8 * I)) ^ (4 * (ka & 3));
        if (bm * BTM + 8 * ca >= M) ca = (M - 1 - bm * BTM) / 8;
        ln.goffA = (unsigned)(((int64_t)(lane / (8 * I)) * lda + 8 * ca) * 2);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int n = wn + (lane & 31);
            ln.fb[ks] = n * BK + 8 * ((2 * ks + hb) ^ ((n >> 2) & 3));
        }
#pragma unroll
        for (int i = 0; i < I; ++i) {
            const int k = 8 * (g >> 1) + (r >> 2);
            const int m = wm + 32 * i + 16 * (g & 1) + 4 * (r & 3);
            ln.fa[i] = k * BTM + 8 * ((m >> 3) ^ (4 * (r >> 2))) + (m & 7);
        }
    }
    const int64_t lda2 = lda * 2, ldb2 = ldb * 2;
    // wave-uniform byte pointers to this wave's first rows of the k = 0 stage
    const int64_t k_first = (int64_t)ks_part * kchunk;
    const char* Ab = (const char*)(A + (int64_t)bz * sa + (int64_t)bm * BTM) + ((int64_t)(8 / I * wave) + k_first) * lda2;
    const char* Bb = (const char*)(B + (int64_t)bz * sb + (int64_t)bn * BTN * ldb + k_first) + (int64_t)(16 * wave) * ldb2;
    C += ((int64_t)bz * ksplit + ks_part) * sc;
    const int64_t a_step = (int64_t)BK * lda2;  // next K step of A: 32 rows down
    const int64_t b_step = (int64_t)BK * 2;     // next K step of B: 32 elements along the row

    f32x16 acc[I][J];
#pragma unroll
    for (int i = 0; i < I; ++i)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[i][j] = f32x16{0};

    const int KT = 4 * ((K + 4 * BK - 1) / (4 * BK));  // steps, in whole groups of four; >= 8 (K >= 256 is checked on the host)
    Frag f0, f1;
    // prologue: stages 0..2 and the B half of stage 3 (I + J transfers per wave and stage); wait for stage 0
    issue_B<J>(Bb, ldb2, Bs0, wave, ln);
    issue_A<I>(Ab, lda2, As0, wave, ln);
    issue_B<J>(Bb + b_step, ldb2, Bs1, wave, ln);
    issue_A<I>(Ab + a_step, lda2, As1, wave, ln);
    issue_B<J>(Bb + 2 * b_step, ldb2, Bs2, wave, ln);
    issue_A<I>(Ab + 2 * a_step, lda2, As2, wave, ln);
    issue_B<J>(Bb + 3 * b_step, ldb2, Bs3, wave, ln);
    constexpr int PER_STAGE = I + J;   // transfers per wave and stage: the waits below leave 2, 1 or 0 stages in flight
    stage_barrier<2 * PER_STAGE + J>();
    load_frags<I, J>(As0, Bs0, ln, 0, f0);

#define KSTEP(X, Y, AA, DA, DB, VM, LAST, TAIL, s)                                                                \
    k_step<E, I, J, DA, DB, (VM) * PER_STAGE, LAST, TAIL>(As##X, Bs##X, As##Y, Bs##Y, As##AA, Ab + (int64_t)((s) + 3) * a_step,      \
                                      Bb + (int64_t)((s) + 4) * b_step, lda2, ldb2, wave, ln, f0, f1, acc,       \
                                      K - ((s) + 3) * BK)
    int s = 0;
    for (; s + 12 <= KT; s += 4) {
        KSTEP(0, 1, 3, true, true, 2, false, false, s);
        KSTEP(1, 2, 0, true, true, 2, false, false, s + 1);
        KSTEP(2, 3, 1, true, true, 2, false, false, s + 2);
        KSTEP(3, 0, 2, true, true, 2, false, false, s + 3);
    }
    // the group that requests the last four stages (the only ones that can reach past K)
    KSTEP(0, 1, 3, true, true, 2, false, true, s);
    KSTEP(1, 2, 0, true, true, 2, false, true, s + 1);
    KSTEP(2, 3, 1, true, true, 2, false, true, s + 2);
    KSTEP(3, 0, 2, true, true, 2, false, true, s + 3);
    s += 4;
    // last four steps: only the A half of the final stage is still to be requested
    KSTEP(0, 1, 3, true, false, 2, false, true, s);
    KSTEP(1, 2, 0, false, false, 1, false, false, s + 1);
    KSTEP(2, 3, 1, false, false, 0, false, false, s + 2);
    KSTEP(3, 0, 2, false, false, 0, true, false, s + 3);
#undef KSTEP

    if (kpeel > 0) {   // (same for the whole grid)
        // k = K .. K + kpeel - 1 as the first values of one 16-wide MFMA step: the lower half-wave holds k 0..7 of its
        // row of B / column of A, the upper half-wave zeros.
        const unsigned short* Ap = A + (int64_t)bz * sa + (int64_t)K * lda;
        const unsigned short* Bp = B + (int64_t)bz * sb + K;
        Frag fp;
        const bool lower = lane < 32;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int64_t n = (int64_t)bn * BTN + wn + 32 * j + (lane & 31);
#pragma unroll
            for (int q = 0; q < 8; ++q) fp.b[j][q] = lower && q < kpeel && n < N ? (short)Bp[n * ldb + q] : (short)0;
        }
#pragma unroll
        for (int i = 0; i < I; ++i) {
            const int64_t m = (int64_t)bm * BTM + wm + 32 * i + (lane & 31);
#pragma unroll
            for (int q = 0; q < 8; ++q) fp.a[i][q] = lower && q < kpeel && m < M ? (short)Ap[m + (int64_t)q * lda] : (short)0;
        }
        mma16<E, I, J>(fp, acc);
    }

    // Epilogue.  The lane's own offset (m within the wave tile, plus its 4*hb rows of n) is a
    // 32-bit element offset; the part of n that is uniform across the wave goes into the base.
    const unsigned lane_off = (unsigned)((lane & 31) + (int64_t)(4 * (lane >> 5)) * ldc);
    OutT* Cw = C + (int64_t)bm * BTM + wm + ((int64_t)bn * BTN + wn) * ldc;
    if ((bm + 1) * BTM <= M && (bn + 1) * BTN <= N) {   // interior tile (same for the whole workgroup)
#pragma unroll
        for (int i = 0; i < I; ++i)
#pragma unroll
            for (int j = 0; j < J; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    OutT* cu = Cw + 32 * i + (int64_t)(32 * j + 8 * (r >> 2) + (r & 3)) * ldc;
                    __builtin_nontemporal_store(cvt_out<E, OutT>(acc[i][j][r]), cu + lane_off);
                }
    } else {                                          // edge tile: clip to the matrix
        int m_left = M - (bm * BTM + wm + (lane & 31)), n_left = N - (bn * BTN + wn + 4 * (lane >> 5));
#pragma unroll
        for (int i = 0; i < I; ++i)
#pragma unroll
            for (int j = 0; j < J; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    // the empty statement keeps each test next to its store (256 hoisted lane masks would
                    // not fit the scalar registers)
                    asm volatile("" : "+v"(m_left), "+v"(n_left));
                    const int dn = 32 * j + 8 * (r >> 2) + (r & 3);
                    if (32 * i < m_left && dn < n_left) {
                        float v = acc[i][j][r];
                        asm volatile("" : "+v"(v));   // convert after the test, not 256 values ahead of it
                        __builtin_nontemporal_store(cvt_out<E, OutT>(v), Cw + 32 * i + (int64_t)dn * ldc + lane_off);
                    }
                }
    }
}

// The extent of K that the transfers walk: whole chunks of 8, and not the last row of A when a chunk of A can straddle
// the end of a row (M not a multiple of 8).
int dma_extent(const Problem& p) { return p.M % 8 ? (p.K - 1) / 8 * 8 : p.K / 8 * 8; }

template <typename E, typename OutT, int I, int J>
void launch(const Problem& p, hipStream_t s) {
    const int tiles_m = (p.M + 64 * I - 1) / (64 * I), tiles_n = (p.N + 64 * J - 1) / (64 * J);
    hipLaunchKernelGGL((gemm16_big<E, OutT, I, J>), dim3((unsigned)(tiles_m * tiles_n * p.batch)), dim3(256), 0,
                       s, (const unsigned short*)p.A, p.lda, p.sa, (const unsigned short*)p.B, p.ldb, p.sb,
                       (OutT*)p.C, p.ldc, p.sc, p.M, p.N, dma_extent(p), tiles_m, tiles_n, p.batch, 1, 0, p.K - dma_extent(p));
}

// ---- split over K for problems with few tiles and a long K ---------------------------------------------------
// A 512 x 512 x 4096 product is 16 tiles of 128 x 128: sixteen workgroups walk 128 K steps each while 240 CUs
// idle.  Split into ksplit parts along K, ksplit times as many workgroups walk a part each and write fp32 partial
// sums; a second kernel adds the parts in fixed order (results do not depend on timing) and converts.  The entry
// point has no workspace argument (it mirrors the reference's kernel signature), so the partial sums live in a
// static device array of the library, 16 MiB per GPU.  Launches that use it are ordered by an event when they
// come from different streams; a stream that is being captured into a graph does not use it.
constexpr int64_t kSplitFloats = 4 * 1024 * 1024;
static __device__ __align__(256) float splitk_scratch[kSplitFloats];

template <typename OutT>
__global__ __launch_bounds__(256) void splitk_reduce(const float* __restrict__ part, int ksplit, OutT* __restrict__ C,
                                                     int64_t ldc, int64_t sc, int M, int N, int batch, bool bf16) {
    // one lane: 4 consecutive m of one column (M is a multiple of 8)
    const int64_t quads = (int64_t)(M / 4) * N * batch;
    const int64_t MN = (int64_t)M * N;
    for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += (int64_t)gridDim.x * 256) {
        const int m4 = (int)(q % (M / 4)), n = (int)((q / (M / 4)) % N), bz = (int)(q / ((int64_t)(M / 4) * N));
        const float* src = part + (int64_t)bz * ksplit * MN + (int64_t)n * M + 4 * m4;
        // parts added in index order (the result does not depend on timing); four loads in flight at a time
        f32x4 acc = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src));
        int ks = 1;
        for (; ks + 4 <= ksplit; ks += 4) {
            f32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + (ks + u) * MN));
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += v[u];
        }
        for (; ks < ksplit; ++ks) acc += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + ks * MN));
        OutT* dst = C + (int64_t)bz * sc + (int64_t)n * ldc + 4 * m4;
        if constexpr (sizeof(OutT) == 4) {
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = acc[e];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = bf16 ? BF16::from_f32(acc[e]) : F16::from_f32(acc[e]);
        }
    }
}

SharedScratch g_split[16];

// Parts and part length for the problem, or 0 if a split does not apply.
int pick_split(const Problem& p, int* kchunk) {
    static const int force = [] { const char* e = getenv("MI_GEMM_SPLITK"); return e ? atoi(e) : -1; }();   // 0 = never, n = n parts
    if (force == 0 || p.M % 8 || p.K % 8) return 0;   // (the parts and the kernel that adds them move whole vectors)
    const int64_t tiles = tiles_of(p, 128, 128);
    // (up to half a tile per CU: 2048 x 768 x 8192, 96 tiles, 59 -> 41 us with two parts; 1152 x 1024 x 16384 107 -> 55 us
    // with three; beyond 128 tiles the estimate below never favours a split)
    if (tiles > 128 || p.K < 1024) return 0;
    // Estimated times in us: one launch walks K / 32 steps of 0.18 us; the split pays a second launch, the partial
    // sums written and read again (at about 3 bytes per ns), and walks a part's steps only.
    const double t_plain = 3.0 + 0.18 * (p.K / 32.0);
    const double mn_bytes = 4.0 * p.M * p.N * p.batch;
    int best = 0;
    double t_best = 0.85 * t_plain;   // (a split has to be clearly better)
    for (int parts = force > 1 ? force : 2; parts <= (force > 1 ? force : 16); ++parts) {
        if (parts * tiles > 512) break;
        const int chunk = ((p.K + parts - 1) / parts + 127) / 128 * 128;        // whole groups of four K steps
        const int n = (p.K + chunk - 1) / chunk;
        if (n < 2 || chunk < 256 || p.K - (n - 1) * chunk < 256 || (int64_t)n * p.M * p.N * p.batch > kSplitFloats) continue;
        const double t = 7.0 + 0.18 * (chunk / 32.0) + (n + 1) * mn_bytes / 3.0e6 + (n * tiles > 256 ? 0.18 * (chunk / 32.0) : 0.0);
        if (t < t_best || (force > 1 && !best)) {
            t_best = t;
            best = n;
            *kchunk = chunk;
        }
    }
    return best;
}

template <typename E>
bool launch_split(const Problem& p, hipStream_t s, int parts, int kchunk) {
    ScratchLease lease;   // ends behind the reduce launch
    float* scratch = (float*)lease.acquire(g_split, HIP_SYMBOL(splitk_scratch), s);
    if (!scratch) return false;
    const int tiles_m = (p.M + 127) / 128, tiles_n = (p.N + 127) / 128;
    const int64_t MN = (int64_t)p.M * p.N;
    hipLaunchKernelGGL((gemm16_big<E, float, 2, 2>), dim3((unsigned)(tiles_m * tiles_n * p.batch * parts)), dim3(256), 0, s,
                       (const unsigned short*)p.A, p.lda, p.sa, (const unsigned short*)p.B, p.ldb, p.sb, scratch,
                       (int64_t)p.M, MN, p.M, p.N, p.K, tiles_m, tiles_n, p.batch, parts, kchunk, 0);
    const int64_t quads = MN / 4 * p.batch;
    const unsigned blocks = (unsigned)((quads + 255) / 256 < 2048 ? (quads + 255) / 256 : 2048);
    if (p.out_dtype == MI_F32)
        hipLaunchKernelGGL((splitk_reduce<float>), dim3(blocks), dim3(256), 0, s, scratch, parts, (float*)p.C, p.ldc,
                           p.sc, p.M, p.N, p.batch, false);
    else
        hipLaunchKernelGGL((splitk_reduce<unsigned short>), dim3(blocks), dim3(256), 0, s, scratch, parts,
                           (unsigned short*)p.C, p.ldc, p.sc, p.M, p.N, p.batch, p.out_dtype == MI_BF16);
    return true;
}

}  // namespace

namespace mi {
namespace gemm {

bool big16_applicable(const Problem& p) {
    if (p.in_dtype != MI_F16 && p.in_dtype != MI_BF16) return false;
    const int64_t tiles = tiles_of(p, 128, 128);   // (from 16 tiles of 128x128 on, this kernel is no slower than 64x64 tiles)
    int split = 0, kchunk = 0;
    return p.M >= 8 && p.N >= 1 && p.K >= 256 + 8 * (p.K % 8 != 0 || p.M % 8 != 0) && p.ldc < (1 << 26) &&
           // (the kernel's 32-bit lane offsets assume rows that follow each other upwards in memory)
           p.lda >= p.M && p.ldb >= p.K && p.ldc >= p.M && p.sa >= 0 && p.sb >= 0 && p.sc >= 0 &&
           p.lda < (1 << 26) && p.ldb < (1 << 26) && tiles < (1 << 30) &&
           // (fewer than 16 tiles only when the split over K multiplies the workgroups)
           (tiles >= 16 || (split = pick_split(p, &kchunk), (int64_t)split * tiles >= 16));
}

void big16_launch(const Problem& p, hipStream_t s) {
    const bool f32out = p.out_dtype == MI_F32;
    const int t = pick_direct_tile(p);
    int kchunk = 0;
    const int parts = t == 22 ? pick_split(p, &kchunk) : 0;
    if (parts > 1 && (p.in_dtype == MI_F16 ? launch_split<F16>(p, s, parts, kchunk) : launch_split<BF16>(p, s, parts, kchunk))) {
        static const char* names[17] = {"", "", "gemm16_big_128x128x32_ring4_splitk2", "gemm16_big_128x128x32_ring4_splitk3",
            "gemm16_big_128x128x32_ring4_splitk4", "gemm16_big_128x128x32_ring4_splitk5", "gemm16_big_128x128x32_ring4_splitk6",
            "gemm16_big_128x128x32_ring4_splitk7", "gemm16_big_128x128x32_ring4_splitk8", "gemm16_big_128x128x32_ring4_splitk9",
            "gemm16_big_128x128x32_ring4_splitk10", "gemm16_big_128x128x32_ring4_splitk11", "gemm16_big_128x128x32_ring4_splitk12",
            "gemm16_big_128x128x32_ring4_splitk13", "gemm16_big_128x128x32_ring4_splitk14", "gemm16_big_128x128x32_ring4_splitk15",
            "gemm16_big_128x128x32_ring4_splitk16"};
        set_variant(names[parts]);
        return;
    }
#define BIG(E, O) (t == 22 ? launch<E, O, 2, 2>(p, s) : t == 42 ? launch<E, O, 4, 2>(p, s) : launch<E, O, 4, 4>(p, s))
    if (p.in_dtype == MI_F16) {
        if (f32out) BIG(F16, float);
        else BIG(F16, unsigned short);
    } else {
        if (f32out) BIG(BF16, float);
        else BIG(BF16, unsigned short);
    }
#undef BIG
    set_variant(t == 22 ? "gemm16_big_128x128x32_ring4" : t == 42 ? "gemm16_big_256x128x32_ring4" : "gemm16_big_256x256x32_ring4");
}

}  // namespace gemm
}  // namespace mi
