// Large-tile fp32 GEMM for MI355X: C(M,N) = A(M,K) * B(K,N), column-major, v_mfma_f32_32x32x2_f32
// (true fp32 products and sums; gfx950 has no TF32-class MFMA, the reference rounds fp32 operands to
// TF32, matmul.jl:49-52).
//
// The fp32 sibling of the 16-bit direct-to-LDS kernel, byte for byte the same data movement: a
// workgroup tile of (64*I) m x (64*J) n on 4 waves as 2x2, K walked in steps of 16 floats through a
// ring of four LDS stages filled by global_load_lds (16 bytes per lane, no staging registers), the
// transfers for step s+3 / s+4 issued between the MFMAs of step s, one barrier per step that waits
// only for the oldest stage in flight.  I = J = 4 is a 256x256 tile (256 accumulator registers, one
// wave per SIMD); 256x128, 128x128 and 64x64 (I = J = 1, 32 KB of LDS) serve problems with few tiles:
// the fp32 MFMA is slow enough (64 cycles for 32x32x2) that a small problem is bound by the MFMA work
// of its busiest CU, so the tile that spreads the work over most CUs wins.
//
// LDS layouts (per stage):
//   B tile [64*J n][16 k]: row = 64 bytes = four 16-byte chunks; chunk c of row n sits at position
//     c ^ ((n >> 2) & 3), so the 16 rows a quarter-wave reads with ds_read_b128 cover all 64 banks.
//   A tile [16 k][64*I m]: row = 256*I bytes; chunk c of row k sits at position c ^ (8 * ((k >> 2) & 1)),
//     so the two rows (k and k + 4) the halves of a wave read with ds_read_b32 fall on different banks.
//   Both swizzles are applied on the global side.
//
// Operands of the MFMA (k = 2 per instruction, lane half h = lane / 32 carries one k each): within a
// group of 8 k, half h takes k = 8u + 4h + q for the q-th of four MFMAs.  B: one 16-byte read gives
// a lane its four q for one n; A: four 4-byte reads per m tile.  Any pairing of k with (q, h) gives
// the same sums as long as A and B agree.
//
// Requires K >= 128.  Tiles that reach past M or N re-read the last valid rows / chunks on the way in and clip
// their stores; in the last group of four steps the chunks at k >= K come from a 16-byte block of zeros (both
// operands).  Rows of any (4-byte) alignment; M and K that are not multiples of 4 as in gemm_big.hip: the K tail --
// and, with a ragged M, the last row of A -- is one register-fed group of MFMAs behind the ring.
#include "gemm_direct.h"

namespace {

using namespace mi;
using namespace mi::gemm;

constexpr int BK = 16;

// Source of every chunk that lies past K.
__device__ __attribute__((aligned(16))) const unsigned zeros16[4] = {0u, 0u, 0u, 0u};

struct Lane {
    int kA, kB;             // first k, within a stage, of the lane's chunk in A transfer 0 (transfer j: + 16/I*j) / in a B transfer
    unsigned goffA[4];      // byte offset of this lane's 16-byte chunk within the wave's A transfer j
    int64_t goffB[4];       // the same for the wave's B transfers (rows past the matrix edge re-read the last row)
    unsigned fb[2];         // LDS float offset of the B fragment, group of 8 k u = 0/1 (+ 32*j*BK for n tile j)
    unsigned fa[4];         // LDS float offset of the A fragment, m tile i (+ (8*u + q)*64*I for group u, MFMA q)
};

struct Frag {
    f32x4 b[4];             // b[j][q]
    float a[4][4];          // a[i][q]
};

// B stage: 64*J rows x 64 B = 4*J transfers of 1 KB (16 rows each); wave w takes transfers w, w+4, ...
// TAIL: k_left = K - (first k of the stage); chunks at or past it come from the zero block.
template <int J, bool TAIL = false>
__device__ __forceinline__ void issue_B(const char* Bg, float* Bs, int wave, const Lane& ln, int k_left = 0) {
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const char* g = Bg + ln.goffB[j];
        if (TAIL && ln.kB >= k_left) g = (const char*)zeros16;
        gload_lds16(g, Bs + (wave + 4 * j) * 256);
    }
}
// A stage: 16 rows x 256*I B = 4*I transfers of 1 KB (4/I rows each); wave w takes transfers w, w+4, ...
template <int I, bool TAIL = false>
__device__ __forceinline__ void issue_A(const char* Ag, int64_t lda4, float* As, int wave, const Lane& ln,
                                        int k_left = 0) {
#pragma unroll
    for (int j = 0; j < I; ++j) {
        const char* g = Ag + (int64_t)(16 / I * j) * lda4 + ln.goffA[j];
        if (TAIL && ln.kA + 16 / I * j >= k_left) g = (const char*)zeros16;
        gload_lds16(g, As + (wave + 4 * j) * 256);
    }
}

template <int I, int J>
__device__ __forceinline__ void load_frags(const float* As, const float* Bs, const Lane& ln, int u, Frag& f) {
    constexpr int BTM = 64 * I;
#pragma unroll
    for (int j = 0; j < J; ++j) f.b[j] = *reinterpret_cast<const f32x4*>(Bs + ln.fb[u] + 32 * j * BK);
#pragma unroll
    for (int i = 0; i < I; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) f.a[i][q] = As[ln.fa[i] + (8 * u + q) * BTM];
}

template <int I, int J>
__device__ __forceinline__ void mma(const Frag& f, f32x16 (&acc)[I][J]) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < I; ++i)
#pragma unroll
            for (int j = 0; j < J; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.b[j][q], f.a[i][q], acc[i][j], 0, 0, 0);
}

// Spread the J + 4*I LDS reads and the NDMA global->LDS transfers of a half step over its 4*I*J MFMAs.
template <int I, int J, int NDMA, bool FRAGS>
__device__ __forceinline__ void interleave() {
    constexpr int NM = 4 * I * J, ND = J + 4 * I;
    static_assert(ND <= 2 * NM, "at most two reads per MFMA slot");
#pragma unroll
    for (int i = 0; i < NM; ++i) {
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        if (FRAGS && i < ND) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
        if (FRAGS && i + NM < ND) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
        if (NDMA && NM >= 8 && i % (NM / 4) == 1 && i / (NM / 4) < NDMA) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
        if (NDMA && NM < 8 && i < NDMA) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
}

// One K step of 16 on stage (AsX, BsX); the next step's data is in (AsY, BsY).
//   first half : MFMAs of k group 0 | read group 1 fragments | issue A transfers (into stage AsA)
//   barrier
//   second half: MFMAs of k group 1 | read next stage's group 0 fragments | issue B transfers (into BsX)
// TAIL: the stages requested here may reach past K; k_left3 = K - (first k of step s+3).
template <int I, int J, bool DMA_A, bool DMA_B, int VMCNT, bool LAST, bool TAIL>
__device__ __forceinline__ void k_step(const float* AsX, float* BsX, const float* AsY, const float* BsY, float* AsA,
                                       const char* Ag_next3, const char* Bg_next4, int64_t lda4, int wave,
                                       const Lane& ln, Frag& f0, Frag& f1, f32x16 (&acc)[I][J], int k_left3) {
    if (DMA_A) issue_A<I, TAIL>(Ag_next3, lda4, AsA, wave, ln, k_left3);
    load_frags<I, J>(AsX, BsX, ln, 1, f1);
    mma<I, J>(f0, acc);
    interleave<I, J, DMA_A ? I : 0, true>();
    if (!LAST) stage_barrier<VMCNT>();
    if (DMA_B) issue_B<J, TAIL>(Bg_next4, BsX, wave, ln, k_left3 - BK);
    if (!LAST) load_frags<I, J>(AsY, BsY, ln, 0, f0);
    mma<I, J>(f1, acc);
    interleave<I, J, DMA_B ? J : 0, !LAST>();
}

template <int I, int J>
__global__ __launch_bounds__(256) void gemm32_big(const float* __restrict__ A, int64_t lda, int64_t sa,
                                                  const float* __restrict__ B, int64_t ldb, int64_t sb,
                                                  float* __restrict__ C, int64_t ldc, int64_t sc, int M, int N, int K,
                                                  int tiles_m, int tiles_n, int batch, int kpeel) {
    // K: the extent the transfers walk (a multiple of 4); kpeel: values of k behind it for the register-fed MFMAs
    constexpr int BTM = 64 * I, STAGE_A = BTM * BK, BTN = 64 * J, STAGE_B = BTN * BK;
    __shared__ __attribute__((aligned(1024))) float As0[STAGE_A], As1[STAGE_A], As2[STAGE_A], As3[STAGE_A];
    __shared__ __attribute__((aligned(1024))) float Bs0[STAGE_B], Bs1[STAGE_B], Bs2[STAGE_B], Bs3[STAGE_B];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // One-dimensional grid over (tile, batch).  Workgroups whose ids are congruent mod 8 share an XCD and
    // its L2: give each XCD a contiguous run of (batch-major) tiles, so that it works on neighbouring
    // tiles of as few batch entries as possible (8 entries on 8 XCDs: one each).
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
    const int wm = (wave & 1) * (32 * I), wn = (wave >> 1) * (32 * J);

    Lane ln;
    {
        const int h = lane >> 5;
        // B transfer: lane -> row lane/4 of its 16-row block, LDS position lane%4; rows n = 16*blk + lane/4.
        // In a tile that reaches past N the rows beyond the edge re-read row N-1 (their products land in
        // accumulators that are never stored), so every transfer stays inside the matrix.
        ln.kB = 4 * ((lane & 3) ^ ((lane >> 4) & 3));
        {
            const int first = bn * BTN + 16 * wave;              // first row of the wave's transfer 0
#pragma unroll
            for (int j = 0; j < J; ++j) {
                int row = 64 * j + (lane >> 2);                  // relative to `first`
                if (first + row > N - 1) row = N - 1 - first;    // (may be negative: still inside the tile's rows)
                ln.goffB[j] = ((int64_t)row * ldb + ln.kB) * 4;
            }
        }
        // A transfer: lane -> row lane/(16*I) of its block of 4/I rows, LDS position lane%(16*I); rows
        // k = 4/I*blk + lane/(16*I).  Chunks of 4 m that start past the edge re-read the last chunk that starts inside.
        const int r_in = lane / (16 * I);
        ln.kA = 4 / I * wave + r_in;
#pragma unroll
        for (int j = 0; j < I; ++j) {
            const int k = 4 / I * (wave + 4 * j) + r_in;
            int ca = (lane % (16 * I)) ^ (8 * ((k >> 2) & 1));
            if (bm * BTM + 4 * ca >= M) ca = (M - 1 - bm * BTM) / 4;
            ln.goffA[j] = (unsigned)(((int64_t)r_in * lda + 4 * ca) * 4);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int n = wn + (lane & 31);
            ln.fb[u] = n * BK + 4 * ((2 * u + h) ^ ((n >> 2) & 3));
        }
#pragma unroll
        for (int i = 0; i < I; ++i) {
            const int m = wm + 32 * i + (lane & 31);
            ln.fa[i] = 4 * h * BTM + 4 * ((m >> 2) ^ (8 * h)) + (m & 3);
        }
    }
    const int64_t lda4 = lda * 4;
    // wave-uniform byte pointers to this wave's first rows of the k = 0 stage
    const char* Ab = (const char*)(A + (int64_t)bz * sa + (int64_t)bm * BTM) + (int64_t)(4 / I * wave) * lda4;
    const char* Bb = (const char*)(B + (int64_t)bz * sb + ((int64_t)bn * BTN + 16 * wave) * ldb);
    C += (int64_t)bz * sc;
    const int64_t a_step = (int64_t)BK * lda4;  // next K step of A: 16 rows down
    const int64_t b_step = (int64_t)BK * 4;     // next K step of B: 16 floats along the row

    f32x16 acc[I][J];
#pragma unroll
    for (int i = 0; i < I; ++i)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[i][j] = f32x16{0};

    const int KT = 4 * ((K + 4 * BK - 1) / (4 * BK));  // steps, in whole groups of four; >= 8 (K >= 128 is checked on the host)
    Frag f0, f1;
    // prologue: stages 0..2 and the B half of stage 3 (I + J transfers per wave and stage); wait for stage 0
    issue_B<J>(Bb, Bs0, wave, ln);
    issue_A<I>(Ab, lda4, As0, wave, ln);
    issue_B<J>(Bb + b_step, Bs1, wave, ln);
    issue_A<I>(Ab + a_step, lda4, As1, wave, ln);
    issue_B<J>(Bb + 2 * b_step, Bs2, wave, ln);
    issue_A<I>(Ab + 2 * a_step, lda4, As2, wave, ln);
    issue_B<J>(Bb + 3 * b_step, Bs3, wave, ln);
    constexpr int PER_STAGE = I + J;   // transfers per wave and stage: the waits below leave 2, 1 or 0 stages in flight
    stage_barrier<2 * PER_STAGE + J>();
    load_frags<I, J>(As0, Bs0, ln, 0, f0);

#define KSTEP(X, Y, AA, DA, DB, VM, LAST, TAIL, s)                                                                \
    k_step<I, J, DA, DB, (VM) * PER_STAGE, LAST, TAIL>(As##X, Bs##X, As##Y, Bs##Y, As##AA,                       \
                                                       Ab + (int64_t)((s) + 3) * a_step,                         \
                                                       Bb + (int64_t)((s) + 4) * b_step, lda4, wave, ln, f0, f1, \
                                                       acc, K - ((s) + 3) * BK)
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
        // k = K .. K + kpeel - 1 as the q-th k of the lower half-wave in four MFMAs; the upper half-wave holds zeros
        const float* Ap = A + (int64_t)bz * sa + (int64_t)K * lda;
        const float* Bp = B + (int64_t)bz * sb + K;
        Frag fp;
        const bool lower = lane < 32;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int64_t n = (int64_t)bn * BTN + wn + 32 * j + (lane & 31);
#pragma unroll
            for (int q = 0; q < 4; ++q) fp.b[j][q] = lower && q < kpeel && n < N ? Bp[n * ldb + q] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < I; ++i) {
            const int64_t m = (int64_t)bm * BTM + wm + 32 * i + (lane & 31);
#pragma unroll
            for (int q = 0; q < 4; ++q) fp.a[i][q] = lower && q < kpeel && m < M ? Ap[m + (int64_t)q * lda] : 0.f;
        }
        mma<I, J>(fp, acc);
    }

    // Epilogue.  The lane's own offset (m within the wave tile, plus its 4*h rows of n) is a 32-bit
    // element offset; the part of n that is uniform across the wave goes into the base.
    const unsigned lane_off = (unsigned)((lane & 31) + (int64_t)(4 * (lane >> 5)) * ldc);
    float* Cw = C + (int64_t)bm * BTM + wm + ((int64_t)bn * BTN + wn) * ldc;
    if ((bm + 1) * BTM <= M && (bn + 1) * BTN <= N) {   // interior tile (same for the whole workgroup)
#pragma unroll
        for (int i = 0; i < I; ++i)
#pragma unroll
            for (int j = 0; j < J; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float* cu = Cw + 32 * i + (int64_t)(32 * j + 8 * (r >> 2) + (r & 3)) * ldc;
                    __builtin_nontemporal_store(acc[i][j][r], cu + lane_off);
                }
    } else {                                            // edge tile: clip to the matrix
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
                    if (32 * i < m_left && dn < n_left)
                        __builtin_nontemporal_store(acc[i][j][r], Cw + 32 * i + (int64_t)dn * ldc + lane_off);
                }
    }
}

template <int I, int J>
void launch(const Problem& p, hipStream_t s) {
    const int tiles_m = (p.M + 64 * I - 1) / (64 * I), tiles_n = (p.N + 64 * J - 1) / (64 * J);
    // The extent of K that the transfers walk: whole chunks of 4, and not the last row of A when a chunk of A can
    // straddle the end of a row (M not a multiple of 4: the chunk then reads on into the next row, which must exist).
    const int kd = p.M % 4 ? (p.K - 1) / 4 * 4 : p.K / 4 * 4;
    hipLaunchKernelGGL((gemm32_big<I, J>), dim3((unsigned)(tiles_m * tiles_n * p.batch)), dim3(256), 0, s,
                       (const float*)p.A, p.lda, p.sa, (const float*)p.B, p.ldb, p.sb, (float*)p.C, p.ldc, p.sc, p.M,
                       p.N, kd, tiles_m, tiles_n, p.batch, p.K - kd);
}

}  // namespace

namespace mi {
namespace gemm {

bool big32_applicable(const Problem& p) {
    if (p.in_dtype != MI_F32 || p.out_dtype != MI_F32) return false;
    return p.M >= 4 && p.N >= 1 && p.K >= 128 + 4 * (p.M % 4 != 0 || p.K % 4 != 0) && p.ldc < (1 << 26) &&
           // (the kernel's 32-bit lane offsets assume rows that follow each other upwards in memory)
           p.lda >= p.M && p.ldb >= p.K && p.ldc >= p.M && p.sa >= 0 && p.sb >= 0 && p.sc >= 0 &&
           p.lda < (1 << 26) && p.ldb < (1 << 26) && tiles_of(p, 64, 64) >= 16 &&
           tiles_of(p, 64, 64) < (1 << 30);
}

// Tile size for fp32.  The kernel is bound by MFMA time, so a candidate costs (rounds of 256 workgroups)
// x (MFMAs per wave and step, I*J); co-resident workgroups of the small tiles simply add up.  The
// smallest tile moves four times the bytes per flop of 128x128 through L2, so it is only taken when it
// at least halves that cost (1024^3: 64 tiles of 128x128 take 63 us).  Ties go to the larger tile.
int pick_tile32(const Problem& p, int64_t* cost = nullptr) {
    static const int force = [] { const char* e = getenv("MI_GEMM_BIG_TILE"); return e ? atoi(e) : 0; }();   // 44, 42, 22 or 11
    auto rounds = [&](int btm, int btn) { return (tiles_of(p, btm, btn) + 255) / 256; };
    const int64_t c44 = rounds(256, 256) * 16, c42 = rounds(256, 128) * 8, c22 = rounds(128, 128) * 4, c11 = rounds(64, 64);
    const int64_t best = c44 <= c42 && c44 <= c22 ? c44 : c42 <= c22 ? c42 : c22;
    if (cost) *cost = 2 * c11 <= best ? 2 * c11 : best;
    if (force == 44 || force == 42 || force == 22 || force == 11) return force;
    if (2 * c11 <= best) return 11;
    return best == c44 ? 44 : best == c42 ? 42 : 22;
}

// The tile choice's estimate: 16 per round of 256 x 256 tiles (the 4096^3 product).
int64_t big32_cost(const Problem& p) {
    int64_t c = 0;
    (void)pick_tile32(p, &c);
    return c;
}

void big32_launch(const Problem& p, hipStream_t s) {
    const int t = pick_tile32(p);
    if (t == 11) launch<1, 1>(p, s);
    else if (t == 22) launch<2, 2>(p, s);
    else if (t == 42) launch<4, 2>(p, s);
    else launch<4, 4>(p, s);
    set_variant(t == 11   ? "gemm32_big_64x64x16_ring4"
                : t == 22 ? "gemm32_big_128x128x16_ring4"
                : t == 42 ? "gemm32_big_256x128x16_ring4"
                          : "gemm32_big_256x256x16_ring4");
}

}  // namespace gemm
}  // namespace mi
