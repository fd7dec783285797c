// Token-gather grouped GEMM of the MoE for dense routing (fused_moe_kernel, examples/moe.jl:45-105, at the
// reference example's own routing -- top-8 of 32 experts, moe.jl:311-344 -- and at prefill sizes): with tens to
// hundreds of tokens per expert the product is no longer a weight stream with a few MFMAs attached (moe.hip) but a
// GEMM per expert, and takes the big GEMM's structure (gemm_big.hip):
//
//   workgroup tile = 128 sorted slots of one expert x 64 * J weight rows (channels); 4 waves as 2 (slots) x 2
//   (channels), each 64 slots x 32 * J channels = 2 x J MFMA 32x32x16 tiles; K walked in steps of 32 through a ring of
//   LDS stages filled by direct global->LDS transfers with no staging registers (J = 2: four stages of 16 KB, J = 4:
//   three of 24 KB; two workgroups per CU either way); the token rows of a stage are gathered (every lane of a
//   transfer carries the address of its own token's row), the weight rows carry the expert's offset; the transfers of
//   later steps are issued between the MFMAs of a step; one barrier per step that waits for the oldest stage in
//   flight only.
//
// Both operands are K-contiguous, so both LDS tiles are [row][32 k] with the 16-byte chunks of a row XOR-swizzled
// by (row >> 2) & 3, and both fragments are plain 16-byte reads.  What bounds the K walk is the LDS pipe (128 bytes
// per clock and CU for fragment reads and transfer writes together): with J = 2 a step of two workgroups needs 768
// of its cycles against 512 of the matrix pipe, with J = 4 1152 against 1024.  k is walked in ascending order with
// the k <-> lane map of the streaming kernel (moe.hip), whichever operand the lanes of the result carry, so every
// output element is accumulated in the same order as there and the two kernels give the same bits.
//
// 32-slot tiles that hold only padding are never multiplied: a wave whose slots are all padding only takes part in
// the transfers and barriers.  Workgroups are persistent (two per CU) and walk the tiles of their XCD's range with a
// stride; what a tile needs to know (expert, token ids) is requested a tile ahead, and a tile's stores and the next
// tile's ring fill are issued back to back.  Within a run of blocks of one expert the tiles are numbered strip-major,
// so the workgroups of an XCD work on a few weight strips of all of the expert's blocks at a time: a strip is
// fetched into that L2 once, and the blocks' token rows stay there while the strips pass.
//
// Epilogues: plain (optionally times the routed weight) and SiLU(gate) * up (the tile's weight rows are gate channels
// and the up channels that go with them, arranged so that a lane holds both halves of an output element) have the
// slot in the lane: a lane holds runs of four channels of its token's row, two lane-half swaps make them runs of
// eight, and the stores are 16 bytes per lane.  The accumulating form (packed atomic adds into the token's output
// column, one or two slots per token) has the channel in the lane, so that an atomic instruction covers whole
// 128-byte lines.
#include <type_traits>

#include "gemm_direct.h"
#include "moe_dense.h"

namespace {

using namespace mi;
using namespace mi::gemm;
using mi::moe::DenseArgs;

constexpr int BK = 32;
constexpr int kRows = 128;            // slots, and weight rows, per workgroup tile
constexpr int kStage = kRows * BK;    // elements of one operand stage (8 KB)
constexpr int MODE_PLAIN = 0, MODE_SILU = 1, MODE_ACC = 2;

// Source of every chunk that lies past K.
__device__ __attribute__((aligned(16))) const unsigned zeros16d[4] = {0u, 0u, 0u, 0u};

__device__ __forceinline__ float widen16(bool bf16, unsigned short h) {
    return bf16 ? __uint_as_float(((unsigned)h) << 16) : (float)__builtin_bit_cast(_Float16, h);
}

// J: MFMA column tiles (32 channels each) per wave.  J = 2: tile of 128 weight rows, ring of four stages of 16 KB;
// J = 4: 256 weight rows, ring of three stages of 24 KB.  Either way two workgroups fit a CU.
template <int J>
struct DLane {
    const char* gT[2];   // global address, at k = 0, of the lane's 16-byte chunk in the wave's two token transfers
    const char* gW[J];   // the same in its J weight transfers
    int kC;              // first k, within a stage, of that chunk
    unsigned fT[2], fW[2];   // LDS element offset of the token / weight fragment of sub-step 0 / 1 (+ 32 * BK per 32-row tile)
};

template <int J>
struct DFrag {
    s16x8 t[2], w[J];
};

// An operand stage of 64 * N rows x 64 B is 4 * N transfers of 1 KB (16 rows each); wave w takes transfers w, w + 4, ...
// TAIL: k_left = K - (first k of the stage); chunks at or past it come from the zero block.
template <bool TAIL, int N>
__device__ __forceinline__ void issueN(const char* const (&g)[N], int64_t koff, unsigned short* S, int wave, int kC,
                                       int k_left) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const char* p = g[j] + koff;
        if (TAIL && kC >= k_left) p = (const char*)zeros16d;
        gload_lds16(p, S + (wave + 4 * j) * 512);
    }
}

template <int LIVE, int J>
__device__ __forceinline__ void load_frags(const unsigned short* Ts, const unsigned short* Ws, const DLane<J>& ln, int ks,
                                           DFrag<J>& f) {
    if (LIVE == 0) return;
#pragma unroll
    for (int j = 0; j < J; ++j) f.w[j] = *reinterpret_cast<const s16x8*>(Ws + ln.fW[ks] + 32 * j * BK);
#pragma unroll
    for (int i = 0; i < LIVE; ++i) f.t[i] = *reinterpret_cast<const s16x8*>(Ts + ln.fT[ks] + 32 * i * BK);
}

// SLOT_LANE: the MFMA column operand (lane % 32 of the result) carries the slot and the rows the channel: a lane
// then holds four consecutive channels of one token's row in four consecutive registers.  Otherwise the lane carries
// the channel and the rows the slots.  The products and the order in which an element's k are added are the same.
template <typename E, int LIVE, bool SLOT_LANE, int J>
__device__ __forceinline__ void mma(const DFrag<J>& f, f32x16 (&acc)[2][J]) {
#pragma unroll
    for (int i = 0; i < LIVE; ++i)
#pragma unroll
        for (int j = 0; j < J; ++j)
            acc[i][j] = SLOT_LANE ? E::mfma32(f.w[j], f.t[i], acc[i][j]) : E::mfma32(f.t[i], f.w[j], acc[i][j]);
}

// Spread the fragment reads (2 + J) and the transfers (NDMA) of a half step over its 2 * J MFMAs.
template <int LIVE, int J, int NDMA, bool FRAGS>
__device__ __forceinline__ void interleave() {
    if constexpr (LIVE == 2) {
#pragma unroll
        for (int i = 0; i < 2 * J; ++i) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
            if (FRAGS && i < 2 + J) __builtin_amdgcn_sched_group_barrier(SG_DSRD, 1, 0);
            if (NDMA && (i * NDMA) / (2 * J) != ((i + 1) * NDMA) / (2 * J)) __builtin_amdgcn_sched_group_barrier(SG_VMEM, 1, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}

// One K step of 32 on stage X; the next step's data is in stage Y.
//   first half : MFMAs of sub-step 0 | read sub-step 1 fragments | token transfers of a later step (into stage TsA)
//   barrier
//   second half: MFMAs of sub-step 1 | read the next stage's sub-step 0 fragments | weight transfers of a later step (into WsX)
// The ring of four stages (J = 2) requests tokens three steps ahead and weights four; the ring of three (J = 4) two
// and three.  koffT / koffW: byte offsets along a row of the stages requested; k_leftT / k_leftW: K less their first k.
template <typename E, int LIVE, bool SLOT_LANE, int J, bool DMA_T, bool DMA_W, int VMCNT, bool LAST, bool TAIL>
__device__ __forceinline__ void k_step(const unsigned short* TsX, unsigned short* WsX, const unsigned short* TsY,
                                       const unsigned short* WsY, unsigned short* TsA, int64_t koffT, int64_t koffW,
                                       int wave, const DLane<J>& ln, DFrag<J>& f0, DFrag<J>& f1, f32x16 (&acc)[2][J],
                                       int k_leftT, int k_leftW) {
    if (DMA_T) issueN<TAIL, 2>(ln.gT, koffT, TsA, wave, ln.kC, k_leftT);
    load_frags<LIVE, J>(TsX, WsX, ln, 1, f1);
    mma<E, LIVE, SLOT_LANE, J>(f0, acc);
    interleave<LIVE, J, DMA_T ? 2 : 0, true>();
    if (!LAST) stage_barrier<VMCNT>();
    if (DMA_W) issueN<TAIL, J>(ln.gW, koffW, WsX, wave, ln.kC, k_leftW);
    if (!LAST) load_frags<LIVE, J>(TsY, WsY, ln, 0, f0);
    mma<E, LIVE, SLOT_LANE, J>(f1, acc);
    interleave<LIVE, J, DMA_W ? J : 0, !LAST>();
}

// ---- 16-bit operands, 64 k per stage -----------------------------------------------------------------------------
// The same walk with stages of 64 k: a stage row is a whole 128-byte line, so every line of the operands is requested
// once, by one transfer (with rows of 64 bytes a line is requested twice, a step apart, and the second request finds
// the first still on its way).  A transfer is 8 rows x 128 B; chunk c of row r sits at position c ^ ((r >> 1) & 7): the
// 16 rows of a quarter-wave's fragment read alternate between the two halves of the banks and the eight rows of a
// half take eight different positions.  Per stage a wave issues four token transfers and 2 * J weight transfers; a K
// step is four MFMA sub-steps around one barrier.  Twice the LDS per stage: a ring of four (J = 2, 128 KB) or three
// (J = 4, 144 KB) stages and one workgroup per CU, whose waves have a SIMD's registers to themselves.
constexpr int BKW = 64;
constexpr int kStageTW = kRows * BKW;   // elements of a token stage (16 KB)

template <int J>
struct WLane {
    const char* gT[4];       // global address, at k = 0, of the lane's 16-byte chunk in the wave's four token transfers
    const char* gW[2 * J];   // the same in its 2 * J weight transfers
    int kC;                  // first k, within a stage, of that chunk
    unsigned fT[4], fW[4];   // LDS element offset of the token / weight fragment of sub-step 0 .. 3 (+ 32 * BKW per 32-row tile)
};

// The weight transfers of a wide stage, non-temporal where the launch reads every weight line once (one block per
// expert): a line that is requested as a whole, once, need not stay anywhere behind the transfer.  (With the 64-byte rows
// of the narrow stages the second half of a line would be fetched from memory again.)
// (a template parameter, not a run-time flag: a branch around the transfers would end the block of instructions in
// which they are spread between the MFMAs -- measured, 56.5 -> 65.5 us on the gate / up projection)
template <bool TAIL, int N, bool STREAM>
__device__ __forceinline__ void issueWt(const char* const (&g)[N], int64_t koff, unsigned short* S, int wave, int kC,
                                        int k_left) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const char* p = g[j] + koff;
        if (TAIL && kC >= k_left) p = (const char*)zeros16d;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p,
                                         (__attribute__((address_space(3))) void*)(S + (wave + 4 * j) * 512), 16, 0, STREAM ? 2 : 0);
    }
}

template <int LIVE, int J>
__device__ __forceinline__ void load_fragsW(const unsigned short* Ts, const unsigned short* Ws, const WLane<J>& ln, int ss,
                                            DFrag<J>& f) {
    if (LIVE == 0) return;
#pragma unroll
    for (int j = 0; j < J; ++j) f.w[j] = *reinterpret_cast<const s16x8*>(Ws + ln.fW[ss] + 32 * j * BKW);
#pragma unroll
    for (int i = 0; i < LIVE; ++i) f.t[i] = *reinterpret_cast<const s16x8*>(Ts + ln.fT[ss] + 32 * i * BKW);
}

// One K step of 64 on stage X; the next step's data is in stage Y.
//   sub-step 0: MFMAs | read sub-step 1 fragments | token transfers of a later step (into stage TsA)
//   sub-steps 1, 2: MFMAs | read the next sub-step's fragments
//   barrier
//   sub-step 3: MFMAs | read the next stage's sub-step 0 fragments | weight transfers of a later step (into WsX)
template <typename E, int LIVE, bool SLOT_LANE, int J, bool DMA_T, bool DMA_W, int VMCNT, bool LAST, bool TAIL, bool STREAM>
__device__ __forceinline__ void k_stepW(const unsigned short* TsX, unsigned short* WsX, const unsigned short* TsY,
                                        const unsigned short* WsY, unsigned short* TsA, int64_t koffT, int64_t koffW,
                                        int wave, const WLane<J>& ln, DFrag<J>& f0, DFrag<J>& f1, f32x16 (&acc)[2][J],
                                        int k_leftT, int k_leftW) {
    if (DMA_T) issueN<TAIL, 4>(ln.gT, koffT, TsA, wave, ln.kC, k_leftT);
    load_fragsW<LIVE, J>(TsX, WsX, ln, 1, f1);
    mma<E, LIVE, SLOT_LANE, J>(f0, acc);
    interleave<LIVE, J, DMA_T ? 4 : 0, true>();
    load_fragsW<LIVE, J>(TsX, WsX, ln, 2, f0);
    mma<E, LIVE, SLOT_LANE, J>(f1, acc);
    interleave<LIVE, J, 0, true>();
    load_fragsW<LIVE, J>(TsX, WsX, ln, 3, f1);
    mma<E, LIVE, SLOT_LANE, J>(f0, acc);
    interleave<LIVE, J, 0, true>();
    if (!LAST) stage_barrier<VMCNT>();
    if (DMA_W) issueWt<TAIL, 2 * J, STREAM>(ln.gW, koffW, WsX, wave, ln.kC, k_leftW);
    if (!LAST) load_fragsW<LIVE, J>(TsY, WsY, ln, 0, f0);
    mma<E, LIVE, SLOT_LANE, J>(f1, acc);
    interleave<LIVE, J, DMA_W ? 2 * J : 0, !LAST>();
}

// ---- fp8 x fp8 (E4M3FN activations and weights) on v_mfma_f32_32x32x64_f8f6f4 ------------------------------------
// A stage has the same bytes as for 16-bit operands (rows of 64 B, four swizzled 16-byte chunks) and therefore twice
// the k: one stage is one K step of the instruction, whose operand is 32 bytes per lane -- chunks 2 * hb and 2 * hb + 1
// of the lane's row, two 16-byte reads at the offsets the 16-bit kernel reads in its two sub-steps.  Tokens and weights
// use the same byte <-> k map, which is all a dot product asks for.  The LDS bytes per MFMA cycle are those of the
// 16-bit kernel (the instruction takes twice as long and multiplies four times as much), so this is the same loop at
// twice the K per step.
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

template <int J>
struct DFrag8 {
    i32x8 t[2], w[J];
};

template <int LIVE, int J>
__device__ __forceinline__ void load_frags8(const unsigned short* Ts, const unsigned short* Ws, const DLane<J>& ln, DFrag8<J>& f) {
    if (LIVE == 0) return;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const i32x4 lo = *reinterpret_cast<const i32x4*>(Ws + ln.fW[0] + 32 * j * BK);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(Ws + ln.fW[1] + 32 * j * BK);
        f.w[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
#pragma unroll
    for (int i = 0; i < LIVE; ++i) {
        const i32x4 lo = *reinterpret_cast<const i32x4*>(Ts + ln.fT[0] + 32 * i * BK);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(Ts + ln.fT[1] + 32 * i * BK);
        f.t[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

// the MFMAs of slot tile I of a step
template <int LIVE, bool SLOT_LANE, int J, int I>
__device__ __forceinline__ void mma8(const DFrag8<J>& f, f32x16 (&acc)[2][J]) {
    if (I >= LIVE) return;
#pragma unroll
    for (int j = 0; j < J; ++j)
        acc[I][j] = SLOT_LANE ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.w[j], f.t[I], acc[I][j], 0, 0, 0, 0, 0, 0)
                              : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.t[I], f.w[j], acc[I][j], 0, 0, 0, 0, 0, 0);
}

template <int LIVE, int J, int NRD, int NDMA>
__device__ __forceinline__ void interleave8() {
    if constexpr (LIVE == 2) {
#pragma unroll
        for (int i = 0; i < J; ++i) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
            if (NRD) __builtin_amdgcn_sched_group_barrier(SG_DSRD, NRD / J, 0);
            if (NDMA) __builtin_amdgcn_sched_group_barrier(SG_VMEM, NDMA / J > 0 ? NDMA / J : 1, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}

// One K step of 64 on stage X, whose fragments are in `cur`; the next step's data is in stage Y.
//   first half : MFMAs of slot tile 0 | token transfers of step s + 3 (into stage TsA)
//   barrier
//   second half: MFMAs of slot tile 1 | read the next stage's fragments into `nxt` | weight transfers of step s + 4 (into WsX)
template <int LIVE, bool SLOT_LANE, int J, bool DMA_T, bool DMA_W, int VMCNT, bool LAST, bool TAIL>
__device__ __forceinline__ void k_step8(unsigned short* WsX, const unsigned short* TsY, const unsigned short* WsY,
                                        unsigned short* TsA, int64_t koffT, int64_t koffW, int wave, const DLane<J>& ln,
                                        const DFrag8<J>& cur, DFrag8<J>& nxt, f32x16 (&acc)[2][J], int k_leftT, int k_leftW) {
    if (DMA_T) issueN<TAIL, 2>(ln.gT, koffT, TsA, wave, ln.kC, k_leftT);
    mma8<LIVE, SLOT_LANE, J, 0>(cur, acc);
    interleave8<LIVE, J, 0, DMA_T ? 2 : 0>();
    if (!LAST) stage_barrier<VMCNT>();
    if (DMA_W) issueN<TAIL, J>(ln.gW, koffW, WsX, wave, ln.kC, k_leftW);
    if (!LAST) load_frags8<LIVE, J>(TsY, WsY, ln, nxt);
    mma8<LIVE, SLOT_LANE, J, 1>(cur, acc);
    interleave8<LIVE, J, LAST ? 0 : 2 * (2 + J), DMA_W ? J : 0>();
}

struct Stages {
    unsigned short *T0, *T1, *T2, *T3, *W0, *W1, *W2, *W3;
};

constexpr int64_t kStepBytes = BK * 2;   // bytes along a row per K step

// What a tile requests before its first step.  Ring of four: stages 0..2 and the weight half of stage 3; ring of three:
// stages 0, 1 and the weight half of stage 2.
template <int J>
__device__ __forceinline__ void ring_fill(const Stages& st, int wave, const DLane<J>& ln) {
    issueN<false, J>(ln.gW, 0, st.W0, wave, ln.kC, 0);
    issueN<false, 2>(ln.gT, 0, st.T0, wave, ln.kC, 0);
    issueN<false, J>(ln.gW, kStepBytes, st.W1, wave, ln.kC, 0);
    issueN<false, 2>(ln.gT, kStepBytes, st.T1, wave, ln.kC, 0);
    issueN<false, J>(ln.gW, 2 * kStepBytes, st.W2, wave, ln.kC, 0);
    if constexpr (J == 2) {
        issueN<false, 2>(ln.gT, 2 * kStepBytes, st.T2, wave, ln.kC, 0);
        issueN<false, J>(ln.gW, 3 * kStepBytes, st.W3, wave, ln.kC, 0);
    }
}

// The K walk of one tile whose ring has been filled.  Its first wait leaves the youngest transfers of the fill in
// flight (all but stage 0): whatever the wave requested before the ring fill (the previous tile's stores, the next
// tile's token ids) is older and completes first.
template <typename E, int LIVE, bool SLOT_LANE, int J>
__device__ __forceinline__ void main_loop(const Stages& st, int K, int wave, const DLane<J>& ln, f32x16 (&acc)[2][J]) {
    DFrag<J> f0, f1;
    constexpr int PER = 2 + J;   // transfers per wave and stage
    if constexpr (J == 2) {
        const int KT = 4 * ((K + 4 * BK - 1) / (4 * BK));   // steps, in whole groups of four; >= 8 (K >= 256 is checked on the host)
        stage_barrier<2 * PER + J>();
        load_frags<LIVE, J>(st.T0, st.W0, ln, 0, f0);
#define KSTEP(X, Y, AA, DT, DW, VM, LAST, TAIL, s)                                                                          \
    k_step<E, LIVE, SLOT_LANE, J, DT, DW, (VM) * PER, LAST, TAIL>(st.T##X, st.W##X, st.T##Y, st.W##Y, st.T##AA,            \
                                                               (int64_t)((s) + 3) * kStepBytes, (int64_t)((s) + 4) * kStepBytes, \
                                                               wave, ln, f0, f1, acc, K - ((s) + 3) * BK, K - ((s) + 4) * BK)
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
        // last four steps: only the token half of the final stage is still to be requested
        KSTEP(0, 1, 3, true, false, 2, false, true, s);
        KSTEP(1, 2, 0, false, false, 1, false, false, s + 1);
        KSTEP(2, 3, 1, false, false, 0, false, false, s + 2);
        KSTEP(3, 0, 2, false, false, 0, true, false, s + 3);
#undef KSTEP
    } else {
        // Ring of three: step s requests the tokens of step s + 2 (into the stage freed half a step ago) and, behind
        // its barrier, the weights of step s + 3 (into its own stage).  At the barrier of step s the transfers
        // younger than the tokens of step s + 1 are the weights of s + 2 and the tokens of s + 2: J + 2.
        const int KT = 3 * ((K + 3 * BK - 1) / (3 * BK));   // steps, in whole groups of three (up to two of zeros); >= 9
        stage_barrier<PER + J>();
        load_frags<LIVE, J>(st.T0, st.W0, ln, 0, f0);
#define KSTEP(X, Y, AA, DT, DW, VM, LAST, TAIL, s)                                                                          \
    k_step<E, LIVE, SLOT_LANE, J, DT, DW, VM, LAST, TAIL>(st.T##X, st.W##X, st.T##Y, st.W##Y, st.T##AA,                    \
                                                       (int64_t)((s) + 2) * kStepBytes, (int64_t)((s) + 3) * kStepBytes,    \
                                                       wave, ln, f0, f1, acc, K - ((s) + 2) * BK, K - ((s) + 3) * BK)
        int s = 0;
        for (; s + 9 <= KT; s += 3) {
            KSTEP(0, 1, 2, true, true, PER, false, false, s);
            KSTEP(1, 2, 0, true, true, PER, false, false, s + 1);
            KSTEP(2, 0, 1, true, true, PER, false, false, s + 2);
        }
        // the group that requests the last stages (the only ones that can reach past K)
        KSTEP(0, 1, 2, true, true, PER, false, true, s);
        KSTEP(1, 2, 0, true, true, PER, false, true, s + 1);
        KSTEP(2, 0, 1, true, true, PER, false, true, s + 2);
        s += 3;
        // last three steps: only the tokens of the final stage are still to be requested
        KSTEP(0, 1, 2, true, false, PER, false, true, s);
        KSTEP(1, 2, 0, false, false, 0, false, false, s + 1);
        KSTEP(2, 0, 1, false, false, 0, true, false, s + 2);
#undef KSTEP
    }
}

constexpr int64_t kStepBytesW = BKW * 2;   // bytes along a row per K step of 64

template <int J, bool STREAM>
__device__ __forceinline__ void ring_fillW(const Stages& st, int wave, const WLane<J>& ln) {
    issueWt<false, 2 * J, STREAM>(ln.gW, 0, st.W0, wave, ln.kC, 0);
    issueN<false, 4>(ln.gT, 0, st.T0, wave, ln.kC, 0);
    issueWt<false, 2 * J, STREAM>(ln.gW, kStepBytesW, st.W1, wave, ln.kC, 0);
    issueN<false, 4>(ln.gT, kStepBytesW, st.T1, wave, ln.kC, 0);
    issueWt<false, 2 * J, STREAM>(ln.gW, 2 * kStepBytesW, st.W2, wave, ln.kC, 0);
    if constexpr (J == 2) {
        issueN<false, 4>(ln.gT, 2 * kStepBytesW, st.T2, wave, ln.kC, 0);
        issueWt<false, 2 * J, STREAM>(ln.gW, 3 * kStepBytesW, st.W3, wave, ln.kC, 0);
    }
}

// The K walk in steps of 64: the rings, the look-ahead and the waits of main_loop with PER = 4 + 2 * J transfers per wave
// and stage.  K >= 512 is checked on the host (at least two groups of steps, and a ring fill that stays inside K).
template <typename E, int LIVE, bool SLOT_LANE, int J, bool STREAM>
__device__ __forceinline__ void main_loopW(const Stages& st, int K, int wave, const WLane<J>& ln, f32x16 (&acc)[2][J]) {
    DFrag<J> f0, f1;
    constexpr int PER = 4 + 2 * J;
    if constexpr (J == 2) {
        const int KT = 4 * ((K + 4 * BKW - 1) / (4 * BKW));
        stage_barrier<2 * PER + 2 * J>();
        load_fragsW<LIVE, J>(st.T0, st.W0, ln, 0, f0);
#define KSTEP(X, Y, AA, DT, DW, VM, LAST, TAIL, s)                                                                          \
    k_stepW<E, LIVE, SLOT_LANE, J, DT, DW, (VM) * PER, LAST, TAIL, STREAM>(st.T##X, st.W##X, st.T##Y, st.W##Y, st.T##AA,           \
                                                                (int64_t)((s) + 3) * kStepBytesW, (int64_t)((s) + 4) * kStepBytesW, \
                                                                wave, ln, f0, f1, acc, K - ((s) + 3) * BKW, K - ((s) + 4) * BKW)
        int s = 0;
        for (; s + 12 <= KT; s += 4) {
            KSTEP(0, 1, 3, true, true, 2, false, false, s);
            KSTEP(1, 2, 0, true, true, 2, false, false, s + 1);
            KSTEP(2, 3, 1, true, true, 2, false, false, s + 2);
            KSTEP(3, 0, 2, true, true, 2, false, false, s + 3);
        }
        KSTEP(0, 1, 3, true, true, 2, false, true, s);
        KSTEP(1, 2, 0, true, true, 2, false, true, s + 1);
        KSTEP(2, 3, 1, true, true, 2, false, true, s + 2);
        KSTEP(3, 0, 2, true, true, 2, false, true, s + 3);
        s += 4;
        KSTEP(0, 1, 3, true, false, 2, false, true, s);
        KSTEP(1, 2, 0, false, false, 1, false, false, s + 1);
        KSTEP(2, 3, 1, false, false, 0, false, false, s + 2);
        KSTEP(3, 0, 2, false, false, 0, true, false, s + 3);
#undef KSTEP
    } else {
        const int KT = 3 * ((K + 3 * BKW - 1) / (3 * BKW));
        stage_barrier<PER + 2 * J>();
        load_fragsW<LIVE, J>(st.T0, st.W0, ln, 0, f0);
#define KSTEP(X, Y, AA, DT, DW, VM, LAST, TAIL, s)                                                                          \
    k_stepW<E, LIVE, SLOT_LANE, J, DT, DW, VM, LAST, TAIL, STREAM>(st.T##X, st.W##X, st.T##Y, st.W##Y, st.T##AA,                   \
                                                        (int64_t)((s) + 2) * kStepBytesW, (int64_t)((s) + 3) * kStepBytesW, \
                                                        wave, ln, f0, f1, acc, K - ((s) + 2) * BKW, K - ((s) + 3) * BKW)
        int s = 0;
        for (; s + 9 <= KT; s += 3) {
            KSTEP(0, 1, 2, true, true, PER, false, false, s);
            KSTEP(1, 2, 0, true, true, PER, false, false, s + 1);
            KSTEP(2, 0, 1, true, true, PER, false, false, s + 2);
        }
        KSTEP(0, 1, 2, true, true, PER, false, true, s);
        KSTEP(1, 2, 0, true, true, PER, false, true, s + 1);
        KSTEP(2, 0, 1, true, true, PER, false, true, s + 2);
        s += 3;
        KSTEP(0, 1, 2, true, false, PER, false, true, s);
        KSTEP(1, 2, 0, false, false, 0, false, false, s + 1);
        KSTEP(2, 0, 1, false, false, 0, true, false, s + 2);
#undef KSTEP
    }
}

// The K walk with fp8 operands: the ring of four, a stage per K step of 64.
template <int LIVE, bool SLOT_LANE, int J>
__device__ __forceinline__ void main_loop8(const Stages& st, int K, int wave, const DLane<J>& ln, f32x16 (&acc)[2][J]) {
    static_assert(J == 2, "fp8 operands take the ring of four stages");
    constexpr int BK8 = 64, PER = 2 + J;
    const int KT = 4 * ((K + 4 * BK8 - 1) / (4 * BK8));   // steps, in whole groups of four; >= 8 (K >= 512 is checked on the host)
    DFrag8<J> f0, f1;
    stage_barrier<2 * PER + J>();
    load_frags8<LIVE, J>(st.T0, st.W0, ln, f0);
#define KSTEP(X, Y, AA, CUR, NXT, DT, DW, VM, LAST, TAIL, s)                                                             \
    k_step8<LIVE, SLOT_LANE, J, DT, DW, (VM) * PER, LAST, TAIL>(st.W##X, st.T##Y, st.W##Y, st.T##AA,                     \
                                                                (int64_t)((s) + 3) * kStepBytes, (int64_t)((s) + 4) * kStepBytes, \
                                                                wave, ln, CUR, NXT, acc, K - ((s) + 3) * BK8, K - ((s) + 4) * BK8)
    int s = 0;
    for (; s + 12 <= KT; s += 4) {
        KSTEP(0, 1, 3, f0, f1, true, true, 2, false, false, s);
        KSTEP(1, 2, 0, f1, f0, true, true, 2, false, false, s + 1);
        KSTEP(2, 3, 1, f0, f1, true, true, 2, false, false, s + 2);
        KSTEP(3, 0, 2, f1, f0, true, true, 2, false, false, s + 3);
    }
    KSTEP(0, 1, 3, f0, f1, true, true, 2, false, true, s);
    KSTEP(1, 2, 0, f1, f0, true, true, 2, false, true, s + 1);
    KSTEP(2, 3, 1, f0, f1, true, true, 2, false, true, s + 2);
    KSTEP(3, 0, 2, f1, f0, true, true, 2, false, true, s + 3);
    s += 4;
    KSTEP(0, 1, 3, f0, f1, true, false, 2, false, true, s);
    KSTEP(1, 2, 0, f1, f0, false, false, 1, false, false, s + 1);
    KSTEP(2, 3, 1, f0, f1, false, false, 0, false, false, s + 2);
    KSTEP(3, 0, 2, f1, f0, false, false, 0, true, false, s + 3);
#undef KSTEP
}

// Barrier that waits for the wave's LDS accesses only (the transfers, loads and stores in flight stay in flight).
__device__ __forceinline__ void lds_only_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// What a workgroup reads about a tile ahead of time (raw values: looking at them would wait for the loads).
struct Meta {
    int sb, bid_n;          // 128-slot block and channel strip
    int expert_raw;         // sorted_expert_ids entry (1-based, 0 = unused block)
    int t0, t1, tm;         // sorted_token_ids entries of the rows of this lane's two transfers / of slot `tid`
    int tw[4];              // (stages of 64 k) entries of the rows of this lane's four transfers
};

// Stores one 32-slot x 32-channel tile held slot-per-lane (o[r]: channel 8 * (r / 4) + 4 * hb + r % 4 of the lane's
// slot) as 16-byte pieces: four registers are four consecutive channels; the two half-waves of a lane pair (l, l + 32)
// hold the two halves of every group of eight, and two lane-half swaps per pair of groups leave every lane with eight
// consecutive channels of its slot's row.  `row`: the slot's output row at the tile's first channel; n_left: channels
// from there to the end of the row.
template <typename E>
__device__ __forceinline__ void store_tile_slot_lane(const float (&o)[16], unsigned short* row, bool valid, int n_left,
                                                     bool vec_ok, int hb) {
    unsigned P[4][2];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        P[q][0] = (unsigned)E::from_f32(o[4 * q]) | ((unsigned)E::from_f32(o[4 * q + 1]) << 16);
        P[q][1] = (unsigned)E::from_f32(o[4 * q + 2]) | ((unsigned)E::from_f32(o[4 * q + 3]) << 16);
    }
#pragma unroll
    for (int q = 0; q < 4; q += 2) {
        // lower half-wave: own group q, then the partner's half of it; upper: the partner's half of group q + 1, then own
        const auto s0 = __builtin_amdgcn_permlane32_swap(P[q][0], P[q + 1][0], false, false);
        const auto s1 = __builtin_amdgcn_permlane32_swap(P[q][1], P[q + 1][1], false, false);
        const u32x4 v = {s0[0], s1[0], s0[1], s1[1]};
        const int c = 8 * q + 8 * hb;   // first of this lane's eight channels
        if (valid) {
            if (vec_ok && c + 8 <= n_left) {
                // (an ordinary store: what is written here is read again by the next launch -- the down projection
                // or the sum over the slots -- and a streaming store would send it past the L2 it can be found in;
                // measured 1-7 % on both launches, most at 16 384 tokens)
                *reinterpret_cast<u32x4*>(row + c) = v;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (c + e < n_left) row[c + e] = (unsigned short)(v[e >> 1] >> (16 * (e & 1)));
            }
        }
    }
}

// Stores of one tile.
// A8: the products are those of unscaled fp8 codes and every channel is multiplied by its fp32 scale first (scale_of:
// b_scale entry of a weight row of the tile's expert, 1 for rows past N).
template <typename E, int MODE, int J, bool A8>
__device__ __forceinline__ void epilogue(const DenseArgs& a, const f32x16 (&acc)[2][J], int nlive, const int* s_tok,
                                         const float* s_wt, int bid_n, int ws, int wn, int lane, bool vec_ok, int expert) {
    const int hb = lane >> 5;
    auto scale_of = [&](int row) { return (A8 && row < a.N && expert >= 0 && expert < a.num_experts) ? a.b_scale[row + (int64_t)expert * a.ld_scale] : 1.f; };
    // slot-in-lane layouts: register r of a column tile is weight row (tile's first row) + 8 * (r / 4) + 4 * hb + r % 4
    float sc[A8 ? J : 1][A8 ? 16 : 1];
    if constexpr (A8 && MODE != MODE_ACC) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            int row0;
            if (MODE == MODE_SILU) row0 = (j >= J / 2 ? a.N / 2 : 0) + bid_n * (32 * J) + 16 * J * wn + 32 * (j % (J / 2));
            else row0 = bid_n * (64 * J) + 32 * J * wn + 32 * j;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ch = 8 * (r >> 2) + 4 * hb + (r & 3);
                // (a gate row past N / 2 belongs to no output channel: its scale is never used)
                sc[j][r] = scale_of(row0 + ch);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        if (i >= nlive) break;
        // token and routed weight of slot lane % 32 of this 32-slot tile
        const int tokv = s_tok[64 * ws + 32 * i + (lane & 31)];
        const float wtv = s_wt[64 * ws + 32 * i + (lane & 31)];
        if constexpr (MODE == MODE_SILU) {
            // lane = slot; register r of gate tile jj and of up tile J / 2 + jj are the same output channel
#pragma unroll
            for (int jj = 0; jj < J / 2; ++jj) {
                const int ch0 = bid_n * (32 * J) + 16 * J * wn + 32 * jj;   // first output channel of the pair of tiles, < N / 2
                float o[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float g = acc[i][jj][r], u = acc[i][J / 2 + jj][r];
                    if constexpr (A8) {
                        g *= sc[jj][r];
                        u *= sc[J / 2 + jj][r];
                    }
                    if (a.mul_routed_weight) {
                        g *= wtv;
                        u *= wtv;
                    }
                    // both halves rounded to the activation type, as the unfused GEMM stores them
                    g = widen16(a.bf16, E::from_f32(g));
                    u = widen16(a.bf16, E::from_f32(u));
                    o[r] = mi::moe::silu_mul(g, u);
                }
                store_tile_slot_lane<E>(o, a.C + (int64_t)(tokv ? tokv - 1 : 0) * a.ldc + ch0, tokv != 0, a.N / 2 - ch0, vec_ok, hb);
            }
        } else if constexpr (MODE == MODE_PLAIN) {
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const int ch0 = bid_n * (64 * J) + 32 * J * wn + 32 * j;
                float o[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float v = acc[i][j][r];
                    if constexpr (A8) v *= sc[j][r];
                    o[r] = a.mul_routed_weight ? v * wtv : v;
                }
                store_tile_slot_lane<E>(o, a.C + (int64_t)(tokv ? tokv - 1 : 0) * a.ldc + ch0, tokv != 0, a.N - ch0, vec_ok, hb);
            }
        } else {
            // lane = channel; rows of a 32 x 32 tile = slots 8 * (r / 4) + 4 * hb + r % 4.  Two neighbouring MFMA column
            // tiles are 64 consecutive channels: swapping the upper half of the first one's register with the lower half
            // of the second one's gives one register with all 64 channels of row R and one with those of row R + 4.
            // Column (token_id - 1) >> acc_shift receives the replica's value as rounded to the storage type, by a
            // packed atomic add of two adjacent channels: even lanes send row R, odd lanes row R + 4, each row 128
            // consecutive bytes.
#pragma unroll
            for (int jp = 0; jp < J; jp += 2) {
                const int gn = bid_n * (64 * J) + 32 * J * wn + 32 * jp + lane;
                // (before the swap a lane holds channel lane % 32 of both column tiles)
                const int gn0 = bid_n * (64 * J) + 32 * J * wn + 32 * jp + (lane & 31);
                const float s0 = scale_of(gn0), s1 = scale_of(gn0 + 32);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int R = 8 * (r >> 2) + (r & 3);
                    const int tokA = __builtin_amdgcn_readlane(tokv, R), tokB = __builtin_amdgcn_readlane(tokv, R + 4);
                    float v0 = acc[i][jp][r], v1 = acc[i][jp + 1][r];
                    if constexpr (A8) {
                        v0 *= s0;
                        v1 *= s1;
                    }
                    if (a.mul_routed_weight) {
                        const float wA = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wtv), R));
                        const float wB = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wtv), R + 4));
                        const float w = hb ? wB : wA;
                        v0 *= w;
                        v1 *= w;
                    }
                    const auto sw = __builtin_amdgcn_permlane32_swap((unsigned)E::from_f32(v0), (unsigned)E::from_f32(v1), false, false);
                    const unsigned rowA = sw[0], rowB = sw[1];   // this lane's channel of row R / of row R + 4
                    const unsigned nbrA = (unsigned)__shfl_xor((int)rowA, 1, 64), nbrB = (unsigned)__shfl_xor((int)rowB, 1, 64);
                    const int tok = (lane & 1) ? tokB : tokA;
                    const unsigned pair = (lane & 1) ? (nbrB | (rowB << 16)) : (rowA | (nbrA << 16));
                    if (tok && gn < a.N)
                        mi::moe::atomic_add2(a.bf16, a.C + (gn & ~1) + (int64_t)((tok - 1) >> a.acc_shift) * a.ldc, pair);
                }
            }
        }
    }
}

// Persistent workgroups: the launch has at most two per CU, and each walks the tiles of its XCD's range with a
// stride.  A tile's stores, and the next tile's ring fill right behind them, are in flight while nothing else of the
// workgroup is: the next tile's K walk starts as soon as its first stage has landed, and what a tile needs to know
// (expert, token ids) is requested one tile ahead.
// WIDE: stages of 64 k (16-bit operands only): twice the LDS, one workgroup per CU; STREAM: their weight transfers are
// non-temporal.
template <typename E, int MODE, int J, bool A8 = false, bool WIDE = false, bool STREAM = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WIDE ? 1 : 2, WIDE ? 1 : 2))) void moe_dense_kernel(const DenseArgs a, int n_blocks) {
    static_assert(!(WIDE && A8), "fp8 stages are 64 k already");
    static_assert(WIDE || !STREAM, "only whole lines are streamed");
    constexpr int ES = A8 ? 1 : 2;          // bytes per operand element
    constexpr int EPC = 16 / ES;            // elements per 16-byte chunk
    constexpr int kStageT = WIDE ? kStageTW : kStage;               // elements of a token stage
    constexpr int kStageW = 64 * J * (WIDE ? BKW : BK);             // elements of a weight stage: 64 * J rows
    constexpr int kLast = J == 2 ? 1 : 0;  // the ring of three has no fourth stage
    __shared__ __attribute__((aligned(1024))) unsigned short Ts0[kStageT], Ts1[kStageT], Ts2[kStageT], Ts3[kLast ? kStageT : 8];
    __shared__ __attribute__((aligned(1024))) unsigned short Ws0[kStageW], Ws1[kStageW], Ws2[kStageW], Ws3[kLast ? kStageW : 8];
    __shared__ int s_tok[2][kRows];      // 1-based replica id of every slot, 0 = no token (two tiles: current and next)
    __shared__ float s_wt[2][kRows];     // its routed weight (1 where none is applied)
    __shared__ unsigned s_live[2][2];    // per half of the block: bit i = its 32-slot tile i holds a token
    const int tid = threadIdx.x, lane = tid & 63, hb = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ws = wave & 1, wn = wave >> 1;   // the wave's half of the slots / of the channels

    // Blocks in use: up to and including the last block that names an expert (the on-device sort fills a
    // fixed-capacity array and marks the rest with expert 0).
    int used = a.num_blocks;
    if (a.num_blocks <= 4096) {
        used = 0;
        for (int b0 = 0; b0 < a.num_blocks; b0 += 64) {
            const int b = b0 + lane;
            const int e = b < a.num_blocks ? a.sorted_expert_ids[b] : 0;
            const unsigned long long m = __ballot(e >= 1 && e <= a.num_experts);
            if (m) used = b0 + 64 - __builtin_clzll(m);
        }
    }
    // Workgroup ids congruent mod 8 share an XCD; XCD x takes tiles [x * per, (x + 1) * per) of the (block, strip)
    // pairs in use, strips of a block consecutive, and its workgroups walk that range with a stride.
    const int bpb = a.TILE_M / kRows;                       // 128-slot tiles per TILE_M block
    const int tiles_all = used * bpb * n_blocks;
    const int per = (tiles_all + 7) >> 3;
    const int nslot = gridDim.x >> 3;
    const int lo = (blockIdx.x & 7) * per, hi = lo + per < tiles_all ? lo + per : tiles_all;
    int cur = lo + (blockIdx.x >> 3);
    if (cur >= hi) return;

    const int r0 = 16 * wave + (lane >> 2), r1 = 64 + r0;   // rows of this lane's chunks in the wave's two transfers
    const int rw0 = 8 * wave + (lane >> 3);                  // (stages of 64 k) row of its chunk in the first of four transfers, then every 32
    // Tile idx -> (128-slot block, strip).  Blocks of one expert that follow each other form a run (cut at multiples
    // of 64 blocks, so that one look at 64 expert ids finds it); the tiles of a run are numbered strip-major: all
    // blocks of the expert for strip 0, then for strip 1, ...  The workgroups of an XCD work on consecutive tiles,
    // i.e. on a few strips of every block of an expert at a time: a weight strip is fetched into the L2 once for all
    // of the expert's blocks, and the blocks' token rows stay there while the strips pass.
    int win = -1, win_e = 0;   // the window of 64 blocks whose expert ids this lane holds one of
    const int sub_used = used * bpb;
    auto load_meta = [&](int idx) {
        Meta m;
        const int lb = idx / n_blocks, w = lb >> 6, q = lb & 63;
        if (w != win) {   // (the same decision in every lane)
            const int b = (w << 6) + lane;
            win_e = b < sub_used ? a.sorted_expert_ids[b / bpb] : -1;
            win = w;
        }
        const int e_lb = __shfl(win_e, q, 64);
        const unsigned long long same = __ballot(win_e == e_lb);
        const unsigned long long below = ~same & ((1ull << q) - 1ull), above = ~same & ~((2ull << q) - 1ull);
        const int b0 = (w << 6) + (below ? 64 - __builtin_clzll(below) : 0);
        const int b1 = (w << 6) + ((q < 63 && above) ? __builtin_ctzll(above) : 64);
        const int nb = b1 - b0, t = idx - b0 * n_blocks;   // 0 <= t < nb * n_blocks
        m.bid_n = t / nb;
        m.sb = b0 + (t - m.bid_n * nb);
        const int slot0 = m.sb * kRows, last = a.num_slots - 1;
        m.expert_raw = e_lb;
        if constexpr (WIDE) {
#pragma unroll
            for (int j = 0; j < 4; ++j) m.tw[j] = a.sorted_token_ids[slot0 + rw0 + 32 * j < last ? slot0 + rw0 + 32 * j : last];
        } else {
            m.t0 = a.sorted_token_ids[slot0 + r0 < last ? slot0 + r0 : last];
            m.t1 = a.sorted_token_ids[slot0 + r1 < last ? slot0 + r1 : last];
        }
        m.tm = a.sorted_token_ids[slot0 + (tid & 127) < last ? slot0 + (tid & 127) : last];
        return m;
    };
    using LaneT = typename std::conditional<WIDE, WLane<J>, DLane<J>>::type;
    LaneT ln;
    if constexpr (WIDE) {
        // the lane's LDS position in a transfer is lane % 8 of row lane / 8; rows 8 * (wave + 4 * j) + lane / 8 all have
        // (row >> 1) & 7 = (4 * wave + lane / 16) & 7
        const int chunk = (lane & 7) ^ ((4 * wave + (lane >> 4)) & 7);
        ln.kC = EPC * chunk;
#pragma unroll
        for (int ss = 0; ss < 4; ++ss) {
            const int sw = 8 * ((2 * ss + hb) ^ (((lane & 31) >> 1) & 7));   // (tile rows 64 * ws and 32 * J * wn are multiples of 16)
            ln.fT[ss] = (64 * ws + (lane & 31)) * BKW + sw;
            ln.fW[ss] = (32 * J * wn + (lane & 31)) * BKW + sw;
        }
    } else {
        const int chunk = (lane & 3) ^ ((lane >> 4) & 3);   // global chunk that belongs at this lane's LDS position
        ln.kC = EPC * chunk;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int sw = 8 * ((2 * ks + hb) ^ (((lane & 31) >> 2) & 3));
            ln.fT[ks] = (64 * ws + (lane & 31)) * BK + sw;
            ln.fW[ks] = (32 * J * wn + (lane & 31)) * BK + sw;
        }
    }
    // Addresses of a tile's transfers from what was read about it; returns this thread's slot's token (0 = none;
    // every slot of a block without a valid expert counts as empty, and such a tile reads expert 1's rows).
    auto setup = [&](const Meta& m, LaneT& L) {
        const int slot0 = m.sb * kRows;
        int expert = m.expert_raw - 1;
        const bool ok = expert >= 0 && expert < a.num_experts;
        if (!ok) expert = 0;
        auto fix = [&](int raw, int r) { return (ok && slot0 + r < a.num_slots && raw >= 1 && raw <= a.total_tokens) ? raw : 0; };
        const int chunk = L.kC / EPC;
        if constexpr (WIDE) {
            const char* Bx = (const char*)a.B + (int64_t)expert * a.sbe * ES;
            const int half_n = a.N / 2;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int t = fix(m.tw[j], rw0 + 32 * j);
                const int c = t ? (t - 1) / a.replicas : 0;   // slots without a token read column 0
                L.gT[j] = (const char*)a.A + ((int64_t)c * a.lda + EPC * chunk) * ES;
            }
#pragma unroll
            for (int j = 0; j < 2 * J; ++j) {
                // tile row R: wave column R / (32 * J), MFMA tile (R / 32) % J of it, channel R % 32 of that
                const int R = 32 * j + rw0, wcol = R / (32 * J), tj = (R >> 5) % J;
                int row;
                if (MODE == MODE_SILU) {
                    int ch = m.bid_n * (32 * J) + 16 * J * wcol + 32 * (tj % (J / 2)) + (R & 31);
                    if (ch > half_n - 1) ch = half_n - 1;
                    row = tj >= J / 2 ? half_n + ch : ch;
                } else {
                    row = m.bid_n * (64 * J) + R;
                    if (row > a.N - 1) row = a.N - 1;
                }
                L.gW[j] = Bx + ((int64_t)row * a.ldb + EPC * chunk) * ES;
            }
            return fix(m.tm, tid & 127);
        } else {
        const int t0 = fix(m.t0, r0), t1 = fix(m.t1, r1);
        const int c0 = t0 ? (t0 - 1) / a.replicas : 0, c1 = t1 ? (t1 - 1) / a.replicas : 0;   // slots without a token read column 0
        L.gT[0] = (const char*)a.A + ((int64_t)c0 * a.lda + EPC * chunk) * ES;
        L.gT[1] = (const char*)a.A + ((int64_t)c1 * a.lda + EPC * chunk) * ES;
        const char* Bx = (const char*)a.B + (int64_t)expert * a.sbe * ES;
        const int half_n = a.N / 2;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            // tile row R: wave column R / (32 * J), MFMA tile (R / 32) % J of it, channel R % 32 of that
            const int R = 64 * j + r0, wcol = R / (32 * J), tj = (R >> 5) % J;
            int row;
            if (MODE == MODE_SILU) {   // tiles 0 .. J/2 - 1 of a wave are gate channels, the others the up channels that go with them
                int ch = m.bid_n * (32 * J) + 16 * J * wcol + 32 * (tj % (J / 2)) + (R & 31);
                if (ch > half_n - 1) ch = half_n - 1;
                row = tj >= J / 2 ? half_n + ch : ch;
            } else {
                row = m.bid_n * (64 * J) + R;
                if (row > a.N - 1) row = a.N - 1;
            }
            L.gW[j] = Bx + ((int64_t)row * a.ldb + EPC * chunk) * ES;
        }
        return fix(m.tm, tid & 127);
        }
    };
    auto routed_weight = [&](int tm) {
        float w = 1.f;
        if (a.mul_routed_weight && tm) {
            // weight of replica q = token * w_topk + slot: element (token, slot) of the (num_tokens, topk) matrix (the
            // flattened, slot-fastest vector of moe.jl:193 is the case w_topk = 1)
            const int q = tm - 1, tk = q / a.w_topk;
            w = widen16(a.bf16, a.topk_weights[tk * a.w_s0 + (q - tk * a.w_topk) * a.w_s1]);
        }
        return w;
    };
    auto publish = [&](int p, int tm, float w) {   // waves 0 and 1 hold the 128 slots
        if (tid < kRows) {
            s_tok[p][tid] = tm;
            s_wt[p][tid] = w;
        }
        const unsigned long long has = __ballot(tm != 0);
        if (wave < 2 && lane == 0) s_live[p][wave] = ((has & 0xffffffffull) ? 1u : 0u) | ((has >> 32) ? 2u : 0u);
    };
    // (tile 1 of a half without tile 0 does not occur with sorted slots; it is multiplied as two tiles)
    auto live_of = [&](int p) { const unsigned l = s_live[p][ws]; return l == 0 ? 0 : l == 1 ? 1 : 2; };

    // whole 16-byte pieces of C's rows can be stored as such
    const bool vec_ok = ((uintptr_t)a.C % 16) == 0 && a.ldc % 8 == 0;
    const Stages st{Ts0, Ts1, Ts2, Ts3, Ws0, Ws1, Ws2, Ws3};
    Meta mc = load_meta(cur), mn = mc;
    int p = 0;
    {
        const int tm = setup(mc, ln);
        publish(0, tm, routed_weight(tm));
    }
    __syncthreads();
    int nlive = live_of(0);
    int nxt = cur + nslot;
    bool have_next = nxt < hi;
    if (have_next) mn = load_meta(nxt);
    if constexpr (WIDE) ring_fillW<J, STREAM>(st, wave, ln);
    else ring_fill<J>(st, wave, ln);
    for (;;) {
        f32x16 acc[2][J];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < J; ++j) acc[i][j] = f32x16{0};
        constexpr bool SL = MODE != MODE_ACC;
        if constexpr (A8) {
            if (nlive == 2) main_loop8<2, SL, J>(st, a.K, wave, ln, acc);
            else if (nlive == 1) main_loop8<1, SL, J>(st, a.K, wave, ln, acc);
            else main_loop8<0, SL, J>(st, a.K, wave, ln, acc);
        } else if constexpr (WIDE) {
            if (nlive == 2) main_loopW<E, 2, SL, J, STREAM>(st, a.K, wave, ln, acc);
            else if (nlive == 1) main_loopW<E, 1, SL, J, STREAM>(st, a.K, wave, ln, acc);
            else main_loopW<E, 0, SL, J, STREAM>(st, a.K, wave, ln, acc);
        } else {
            if (nlive == 2) main_loop<E, 2, SL, J>(st, a.K, wave, ln, acc);
            else if (nlive == 1) main_loop<E, 1, SL, J>(st, a.K, wave, ln, acc);
            else main_loop<E, 0, SL, J>(st, a.K, wave, ln, acc);
        }
        // the next tile's addresses and its routed weights (requested now, used after this tile's stores are out)
        int tmN = 0;
        float wN = 1.f;
        if (have_next) {
            tmN = setup(mn, ln);
            wN = routed_weight(tmN);
        }
        epilogue<E, MODE, J, A8>(a, acc, nlive, s_tok[p], s_wt[p], mc.bid_n, ws, wn, lane, vec_ok, mc.expert_raw - 1);
        if (!have_next) break;
        publish(p ^ 1, tmN, wN);
        lds_only_barrier();   // every wave is done with the ring's stages, and the next tile's slots are in place
        p ^= 1;
        mc = mn;
        nlive = live_of(p);
        cur = nxt;
        nxt += nslot;
        have_next = nxt < hi;
        if (have_next) mn = load_meta(nxt);
        if constexpr (WIDE) ring_fillW<J, STREAM>(st, wave, ln);
        else ring_fill<J>(st, wave, ln);
    }
}

}  // namespace

namespace mi {
namespace moe {

bool dense_applicable(const DenseArgs& a) {
    // MI_MOE_DENSE: 0 = never, 1 = wherever it can run (read at every call, so that one process can compare the kernels)
    const char* env = getenv("MI_MOE_DENSE");
    const int force = env ? atoi(env) : -1;
    if (a.a8) {   // fp8 x fp8: this kernel or none
        if (!a.w8 || a.TILE_M % kRows || a.K % 16 || a.K < 512 || a.N < 1 || (a.silu && (a.N % 2))) return false;
        if (!aligned(a.A, 16) || !aligned(a.B, 16) || a.lda % 16 || a.ldb % 16 || a.sbe % 16 || a.lda < 0 || a.ldb < 0) return false;
        if (cld((int64_t)a.total_tokens, (int64_t)a.replicas) > a.num_a_cols) return false;
        if (a.acc_shift >= 0 && (a.N % 2)) return false;
        const int64_t nb8 = a.silu ? cld((int64_t)a.N / 2, (int64_t)64) : cld((int64_t)a.N, (int64_t)kRows);
        return (cld((int64_t)a.num_blocks * (a.TILE_M / kRows) * nb8, (int64_t)8) + 1) * 8 <= MI_MAX_GRID_DIM;
    }
    if (force == 0 || a.w8) return false;
    if (a.TILE_M % kRows || a.K % 8 || a.K < 256 || a.N < 1) return false;
    if (a.silu && (a.N % 2)) return false;
    if (!aligned(a.A, 16) || !aligned(a.B, 16) || a.lda % 8 || a.ldb % 8 || a.sbe % 8) return false;
    if (a.lda < 0 || a.ldb < 0) return false;
    if (cld((int64_t)a.total_tokens, (int64_t)a.replicas) > a.num_a_cols) return false;   // (a replica without a column of A: the streaming kernel feeds it zeros)
    if (a.acc_shift >= 0 && (a.N % 2)) return false;
    const int64_t n_blocks = a.silu ? cld((int64_t)a.N / 2, (int64_t)64) : cld((int64_t)a.N, (int64_t)kRows);   // (the narrower tile)
    if ((cld((int64_t)a.num_blocks * (a.TILE_M / kRows) * n_blocks, (int64_t)8) + 1) * 8 > MI_MAX_GRID_DIM) return false;
    if (force == 1) return true;
    // dense enough: more than 32 replicas per expert on average (what the streaming kernel's two-tile shape starts at)
    return (int64_t)a.total_tokens >= 32ll * a.num_experts;
}

// Channels per tile: 256 weight rows per workgroup (four MFMA column tiles per wave, three ring stages) halve the LDS
// fragment reads per MFMA -- 0.75 KB against 1 KB, and the LDS pipe (128 bytes per clock and CU) is what bounds the
// K walk of the narrower tile -- and are taken when they still give every workgroup slot of the chip a tile;
// otherwise 128 rows (two column tiles per wave, four stages).  MI_MOE_DENSE_J = 2 | 4 forces one.
static int pick_j(const DenseArgs& a) {
    const char* env = getenv("MI_MOE_DENSE_J");
    const int force = env ? atoi(env) : 0;
    if (a.a8) return 2;
    if (force == 2 || force == 4) return force;
    const int64_t strips4 = a.silu ? cld((int64_t)a.N / 2, (int64_t)128) : cld((int64_t)a.N, (int64_t)256);
    // blocks that hold tokens: at most one partly filled block per expert on top of the full ones
    const int64_t blocks = cld((int64_t)a.total_tokens, (int64_t)kRows) + a.num_experts / 2;
    // (measured, gate / up projection: 256 tokens top-8, 512 such tiles, 62 against 66 us; 1024 top-8 128 / 150; 2048 top-2
    // 100 / 104; 4096 top-2 137 / 160; 8192 top-2 232 / 264.  The down projection has a quarter of the strips and stays
    // on 128 channels up to about 16k replicas: 4096 top-2 93 against 99 us.)
    return blocks * strips4 >= 512 ? 4 : 2;
}

void dense_launch(const DenseArgs& a, hipStream_t s) {
    const int J = pick_j(a);
    const int n_blocks = a.silu ? (int)cld((int64_t)a.N / 2, (int64_t)(32 * J)) : (int)cld((int64_t)a.N, (int64_t)(64 * J));
    const int64_t tiles = (int64_t)a.num_blocks * (a.TILE_M / kRows) * n_blocks;
    // persistent: two workgroups per CU at most (64 or 72 KB of LDS each), a multiple of 8 so that every XCD gets as many
    // Stages of 64 k (one workgroup per CU) with non-temporal weight transfers, for launches in which no weight line is
    // read twice: at most one block per expert.  Measured (us, kernel by kernel and the whole call): 256 tokens top-8 of
    // 32 experts gate / up 60.6 -> 57-59, down 41.8 -> 34-35, cutile_moe 116.5 -> 106.2 (the same with four rotating
    // sets of weights).  With two blocks per expert the streamed weights cost 5-10 % instead, and the wide stages with
    // ordinary transfers gain 3-8 % on the 128-channel tile by the kernels' own durations but lose as much over the
    // whole call (4096 tokens top-2 231 -> 240, 1024 tokens top-8 215 -> 227): one workgroup per CU starts and ends
    // a launch more slowly than two.  MI_MOE_DENSE_WIDE = 0 | 1 and MI_MOE_DENSE_STREAM = 0 | 1 (wide stages only) force
    // the choices.
    const char* env_wide = getenv("MI_MOE_DENSE_WIDE");
    const char* env_stream = getenv("MI_MOE_DENSE_STREAM");
    const bool can_wide = !a.a8 && a.K >= 512;
    // (one block per expert: on average at most 0.8 of a block's slots; weights that would not stay in a cache anyway)
    const bool one_block = (int64_t)a.total_tokens * 10 <= (int64_t)8 * kRows * a.num_experts;
    const bool big_weights = (int64_t)a.num_experts * a.N * a.K * 2 >= (64ll << 20);
    bool stream_w = can_wide && (env_stream ? atoi(env_stream) != 0 : one_block && big_weights);
    const bool wide = can_wide && (env_wide ? atoi(env_wide) != 0 : stream_w);
    if (!wide) stream_w = false;
    const int64_t cap = wide ? 32 : 64;
    const int64_t per_xcd = cld(tiles, (int64_t)8) < cap ? cld(tiles, (int64_t)8) : cap;
    const dim3 grid((unsigned)(per_xcd * 8));
#define LAUNCH1(ET, MODE, JJ, A8, WD, ST) \
    hipLaunchKernelGGL((moe_dense_kernel<ET, MODE, JJ, A8, WD, ST>), grid, dim3(256), 0, s, a, n_blocks)
#define LAUNCH(ET, MODE)                                                           \
    do {                                                                           \
        if (a.a8) LAUNCH1(ET, MODE, 2, true, false, false);                        \
        else if (wide && stream_w && J == 4) LAUNCH1(ET, MODE, 4, false, true, true);   \
        else if (wide && stream_w) LAUNCH1(ET, MODE, 2, false, true, true);        \
        else if (wide && J == 4) LAUNCH1(ET, MODE, 4, false, true, false);         \
        else if (wide) LAUNCH1(ET, MODE, 2, false, true, false);                   \
        else if (J == 4) LAUNCH1(ET, MODE, 4, false, false, false);                \
        else LAUNCH1(ET, MODE, 2, false, false, false);                            \
    } while (0)
    if (a.silu) {
        if (a.bf16) LAUNCH(BF16, MODE_SILU);
        else LAUNCH(F16, MODE_SILU);
        set_variant(a.a8 ? "fused_moe_dense_silu_t128_n64x2_k64_ring4_w8a8" : wide ? (J == 4 ? "fused_moe_dense_silu_t128_n128x2_k64_ring3" : "fused_moe_dense_silu_t128_n64x2_k64_ring4") : J == 4 ? "fused_moe_dense_silu_t128_n128x2_k32_ring3" : "fused_moe_dense_silu_t128_n64x2_k32_ring4");
    } else if (a.acc_shift >= 0) {
        if (a.bf16) LAUNCH(BF16, MODE_ACC);
        else LAUNCH(F16, MODE_ACC);
        set_variant(a.a8 ? "fused_moe_dense_acc_t128_n128_k64_ring4_w8a8" : wide ? (J == 4 ? "fused_moe_dense_acc_t128_n256_k64_ring3" : "fused_moe_dense_acc_t128_n128_k64_ring4") : J == 4 ? "fused_moe_dense_acc_t128_n256_k32_ring3" : "fused_moe_dense_acc_t128_n128_k32_ring4");
    } else {
        if (a.bf16) LAUNCH(BF16, MODE_PLAIN);
        else LAUNCH(F16, MODE_PLAIN);
        set_variant(a.a8 ? "fused_moe_dense_t128_n128_k64_ring4_w8a8" : wide ? (J == 4 ? "fused_moe_dense_t128_n256_k64_ring3" : "fused_moe_dense_t128_n128_k64_ring4") : J == 4 ? "fused_moe_dense_t128_n256_k32_ring3" : "fused_moe_dense_t128_n128_k32_ring4");
    }
#undef LAUNCH
#undef LAUNCH1
}

}  // namespace moe
}  // namespace mi
