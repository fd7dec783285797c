// Fused multi-head attention forward, software-pipelined kernel for head dimension 64:
// stand-in for fmha_kernel of the reference's examples/fmha.jl:20-139 on the shapes its
// benchmark uses (fmha.jl:230-260: D = 64, Sq == Skv, no decode offset).
//
// Work split.  A workgroup is two waves and owns 128 queries of one (batch, head); a wave owns
// two 32-query MFMA column tiles ("streams").  Without a causal mask the streams are adjacent
// tiles.  With it, wave w of workgroup qb takes tiles u = 2*qb + w and NT-1-u, so that every
// wave of the grid has the same number of MFMAs; stream 0 (the early tile) is stored after its
// diagonal, and from then on the long tile takes both streams' slots: two halves per trip ("wide
// steps", see wide_step below), so that the fixed cost of a trip is paid half as often.
//
// K and V travel in halves of 32 keys (4 KB each) through two rings of four LDS slots, filled
// by direct global->LDS loads three steps ahead of their use.  One step handles one half j:
//     raise the running maxima if the maxima of S(j) (taken in the previous step) demand it
//     barrier (publishes the halves issued three steps ago)
//     sixteen issue slots, each one MFMA -- first the ten of S(j+1) = K(j+1) . Q (K fragments already in
//     registers), then O += V(j) . P(j) chunk by chunk as soon as a 16-key chunk of P exists -- and one piece
//     of the weights P(j) = exp2(S(j) - m) (2 exp2, pack, row sum); the step's fixed work rides along a few
//     instructions per slot: the V(j) fragment reads, the requests for K half j+5 and V half j+3, the
//     K(j+2) fragment reads, the row maxima of S(j+1) in stages
//     the last two P.V MFMAs
// The two score buffers swap roles every step (the loops are unrolled by two), so no register
// copies are needed.  The global->LDS loads are issued from inline assembly and waited for with
// explicit vmcnt counts; the compiler sees only the LDS reads.
//
// Online softmax in the exp2 domain (fmha.jl:41,106-127).  The running maximum m of a row is
// only raised when the new maximum exceeds it by more than 8 (a factor 256 in the weights):
// the result is the same function of the inputs, the weights P stay below 2^8 in the storage
// type, and the accumulator rescale all but disappears.  Row sums are taken over the rounded
// weights, i.e. over exactly the values that multiply V (f16; bf16 has no mixed-precision fma, its
// row sums take the weights before rounding).
#include "fmha_common.h"

namespace mi {
namespace fmha {
namespace {

constexpr int kD = 64;            // head dimension
constexpr int kHK = 32;           // keys per half
constexpr int kSlot = kHK * kD;   // elements per ring slot
constexpr int kSlotBytes = kSlot * 2;
constexpr int kPre = 1;           // issue slots of a step that run before its wait and barrier
constexpr float kRaise = 8.0f;    // raise m only when the new maximum exceeds it by this much

#pragma clang diagnostic ignored "-Winline-asm"  // m0 is named as clobbered on purpose

// One 1 KB global->LDS transfer: lane l moves 16 bytes from sbase + voff to lds_base + 16*l.
__device__ __forceinline__ void dma16(unsigned voff, const char* sbase, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(lds_base)
                 : "memory", "m0");
}

__device__ __forceinline__ void fence() { asm volatile("" ::: "memory"); }

// s_waitcnt immediates (gfx9 encoding): lgkmcnt(0) with vmcnt(N)
constexpr int kWaitVm0 = 0x0070, kWaitVm4 = 0x0074, kWaitVm8 = 0x0078, kWaitVm2 = 0x0072, kWaitVm6 = 0x0076,
              kWaitLgkm = 0xc07f;   // lgkmcnt(0) alone

template <int IMM>
__device__ __forceinline__ void wait_and_barrier() {
    __builtin_amdgcn_s_waitcnt(IMM);
    fence();
    __builtin_amdgcn_s_barrier();
    fence();
}

// max(a, b, c) as one instruction (v_maximum3_f32: the IEEE 754-2019 maximum, which propagates NaN).  fmaxf() is
// preceded by a quieting v_max_f32 x, x of every operand the compiler can not prove to be no signalling NaN, and
// MFMA results are such operands; an inline-asm v_max3_f32 makes the compiler put a wait state after every one.
__device__ __forceinline__ float max3(float a, float b, float c) {
    return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}

// max / sum over the lane pair (l, l ^ 32)
__device__ __forceinline__ float xhalf_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return max3(__uint_as_float(r[0]), __uint_as_float(r[1]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// RG: the sequence length is not a multiple of 128.  The grid is that of the next multiple; the halves that exist are
// walked as usual, the last of them re-reads its last row in place of the rows past the end (ragged_offsets), halves
// past it are never requested (the transfers that would fetch them re-send the last one, as at the end of every
// walk), and rows past the end are not stored.  With the causal mask the keys past the end lie above the diagonal of
// every query that exists, so that mask removes them; without it the walk ends with the pair of halves that holds
// the last key, and their scores are masked against the sequence length (MASKN = 2 in half_step).
template <bool RG>
struct LaneT {
    static constexpr bool ragged = RG;
    // wave-uniform
    const char *kptr, *vptr;        // next K / V half to be transferred
    int k_left, v_left;             // halves not yet transferred (the last one is re-sent once they run out)
    int64_t k_half_bytes, v_half_bytes;
    unsigned ks_base, vs_base;      // LDS byte addresses of the rings
    int wave, nh;                   // halves walked by this workgroup
    bool hb0;                       // lane of the lower half-wave (holds k = 0..7 of an MFMA operand)
    // per lane
    unsigned kdma, vdma;            // byte offset of the lane's 16 bytes in transfer `wave` (transfer wave+2: 16 keys on)
    unsigned kfo[4];                // K fragment element offsets inside a slot, per k-step
    unsigned vfo[2];                // V fragment element offsets inside a slot, per d tile
    int lim0;                       // (lane % 32) - 4 * (lane / 32)
    int q0[2];                      // first query of each stream (wave-uniform)
    // RG only
    bool to_end;                    // (wave-uniform) the walk reaches the last half that exists
    unsigned kdma_b, vdma_b;        // offset of the lane's 16 bytes in transfer wave+2, relative to the start of the half
    unsigned k_rg[2], v_rg[2];      // the two offsets for the last half that exists (rows past the end re-read the last row)
    int rag_lim;                    // last key that exists, less the 4 keys the upper half-wave's rows are shifted by
};

// Lane offsets of the two transfers of the last half when rows past `last_row` (0..31) are replaced by that row.
template <bool IS_V>
__device__ __forceinline__ void ragged_offsets(int wave, int lane, int last_row, int64_t half_bytes, unsigned& o0, unsigned& o1) {
    const int key = 8 * wave + (lane >> 3), pos = lane & 7;
    const unsigned pitch = (unsigned)(half_bytes >> 5);   // bytes per key row
    const unsigned sw = 16u * (unsigned)(IS_V ? (pos ^ (2 * (key & 3))) : (pos ^ ((key >> 1) & 7)));
    const int r0 = key < last_row ? key : last_row, r1 = key + 16 < last_row ? key + 16 : last_row;
    o0 = (unsigned)r0 * pitch + sw;
    o1 = (unsigned)r1 * pitch + sw;
}


template <typename E>
struct Acc {
    s16x8 qf[2][4];    // Q fragments, already multiplied by the exp2-domain scale
    s16x8 qm[2];       // a fifth "k step" of the query operand: -(running maximum) at k = 0, zeros elsewhere.  Against
                       // a key operand that is 1 at k = 0 it makes the S MFMAs deliver S - m, so the weights are a
                       // bare exp2 of the accumulator (two MFMAs per step instead of 32 vector fma)
    s16x8 ones;        // that key operand
    f32x16 o[2][2];
    float m[2], l[2];  // running maximum (exp2 domain, a value of the storage type; -inf until the first half) and
                       // sum of the lane's half of the keys
    float thr[2];      // S - m above which m is raised: -inf until the first half, kRaise afterwards
};

// Transfers the next K (V) half into ring slot `slot`.  Past the last half the same half is sent
// again into a slot nobody reads, which keeps the count of outstanding transfers uniform.
// (RG: the selects are wave-uniform conditions on lane offsets -- no branch, the steps keep their layout)
template <bool RG>
__device__ __forceinline__ void issue_k(LaneT<RG>& c, int slot) {
    const unsigned lds = c.ks_base + slot * kSlotBytes + c.wave * 1024;
    if constexpr (RG) {
        const bool last = c.to_end && c.k_left <= 1;
        dma16(last ? c.k_rg[0] : c.kdma, c.kptr, lds);
        dma16(last ? c.k_rg[1] : c.kdma_b, c.kptr, lds + 2048);
    } else {
        dma16(c.kdma, c.kptr, lds);
        dma16(c.kdma, c.kptr + (c.k_half_bytes >> 1), lds + 2048);
    }
    c.k_left -= 1;
    if (c.k_left > 0) c.kptr += c.k_half_bytes;
}
template <bool RG>
__device__ __forceinline__ void issue_v(LaneT<RG>& c, int slot) {
    const unsigned lds = c.vs_base + slot * kSlotBytes + c.wave * 1024;
    if constexpr (RG) {
        const bool last = c.to_end && c.v_left <= 1;
        dma16(last ? c.v_rg[0] : c.vdma, c.vptr, lds);
        dma16(last ? c.v_rg[1] : c.vdma_b, c.vptr, lds + 2048);
    } else {
        dma16(c.vdma, c.vptr, lds);
        dma16(c.vdma, c.vptr + (c.v_half_bytes >> 1), lds + 2048);
    }
    c.v_left -= 1;
    if (c.v_left > 0) c.vptr += c.v_half_bytes;
}

// The same transfers one at a time (PART 0 / 1 of a half), for steps that spread them over their issue slots.
template <int PART, bool RG>
__device__ __forceinline__ void issue_k_part(LaneT<RG>& c, int slot) {
    const unsigned lds = c.ks_base + slot * kSlotBytes + c.wave * 1024;
    const bool last = RG && c.to_end && c.k_left <= 1;
    if (PART == 0) {
        if constexpr (RG) dma16(last ? c.k_rg[0] : c.kdma, c.kptr, lds);
        else dma16(c.kdma, c.kptr, lds);
    } else {
        if constexpr (RG) dma16(last ? c.k_rg[1] : c.kdma_b, c.kptr, lds + 2048);
        else dma16(c.kdma, c.kptr + (c.k_half_bytes >> 1), lds + 2048);
        c.k_left -= 1;
        if (c.k_left > 0) c.kptr += c.k_half_bytes;
    }
}
template <int PART, bool RG>
__device__ __forceinline__ void issue_v_part(LaneT<RG>& c, int slot) {
    const unsigned lds = c.vs_base + slot * kSlotBytes + c.wave * 1024;
    const bool last = RG && c.to_end && c.v_left <= 1;
    if (PART == 0) {
        if constexpr (RG) dma16(last ? c.v_rg[0] : c.vdma, c.vptr, lds);
        else dma16(c.vdma, c.vptr, lds);
    } else {
        if constexpr (RG) dma16(last ? c.v_rg[1] : c.vdma_b, c.vptr, lds + 2048);
        else dma16(c.vdma, c.vptr + (c.v_half_bytes >> 1), lds + 2048);
        c.v_left -= 1;
        if (c.v_left > 0) c.vptr += c.v_half_bytes;
    }
}

template <bool RG>
__device__ __forceinline__ void read_k_frags(const unsigned short* Ks, const LaneT<RG>& c, int slot, s16x8 (&kf)[4]) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) kf[ks] = *reinterpret_cast<const s16x8*>(Ks + slot * kSlot + c.kfo[ks]);
}

// First part of the softmax of one stream's 32x32 score tile: apply the causal mask and return
// the row maximum of the raw scores (before the exp2-domain scale).
template <bool MASK>
__device__ __forceinline__ float masked_row_max(f32x16& s, int lim) {
    if (MASK) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = (8 * (r >> 2) + (r & 3) <= lim) ? s[r] : -INFINITY;
    }
    float mx = max3(s[0], s[1], s[2]);
#pragma unroll
    for (int r = 3; r < 15; r += 2) mx = max3(mx, s[r], s[r + 1]);
    return xhalf_max(max3(mx, s[15], s[15]));
}

// The same in three stages of three to four instructions (eleven with the mask), for steps that spread the row
// maxima over their issue slots: stage 0 and 1 take eight scores each, stage 2 the last one and the other half-wave.
template <bool MASK, int STAGE>
__device__ __forceinline__ void row_max_stage(f32x16& s, int lim, float& mx, float& out) {
    if (MASK && STAGE < 2) {
#pragma unroll
        for (int r = 8 * STAGE; r < 8 * STAGE + 8; ++r) s[r] = (8 * (r >> 2) + (r & 3) <= lim) ? s[r] : -INFINITY;
    }
    if (STAGE == 0) {
        mx = max3(s[0], s[1], s[2]);
        mx = max3(mx, s[3], s[4]);
        mx = max3(mx, s[5], s[6]);
    } else if (STAGE == 1) {
        mx = max3(mx, s[7], s[8]);
        mx = max3(mx, s[9], s[10]);
        mx = max3(mx, s[11], s[12]);
        mx = max3(mx, s[13], s[14]);
    } else {
        out = xhalf_max(max3(mx, s[15], s[15]));
    }
}

// The weights of one score pair (2h, 2h+1), h = 0..7, are made in two stages that the step below
// places in consecutive issue slots, so that no instruction waits for the one just before it:
// stage 1: 2 exp2 of scores that the MFMAs delivered relative to the (possibly stale) running maximum;
// stage 2: round and pack for the P.V MFMAs, add to the row sum (f16: once per 16-key chunk, see Pack<F16>).
__device__ __forceinline__ void exp_stage1(const f32x16& s, int h, float (&p)[2]) {
    p[0] = __builtin_amdgcn_exp2f(s[2 * h]);
    p[1] = __builtin_amdgcn_exp2f(s[2 * h + 1]);
}
template <typename E>
__device__ __forceinline__ void exp_stage2(const float (&p)[2], int h, float& l, unsigned (&pf)[2][4]) {
    const unsigned pk = Pack<E>::pack(p[0], p[1]);
    pf[h >> 2][h & 3] = pk;
    if constexpr (Pack<E>::kChunkSum) {
        if ((h & 3) == 3) l = Pack<E>::sum_chunk(pf[h >> 2], l);   // the chunk is complete
    } else {
        l = Pack<E>::sum2(pk, p[0], p[1], l);
    }
}

// Closes an issue slot: nothing is scheduled across it.
__device__ __forceinline__ void slot_end() {
    __builtin_amdgcn_sched_barrier(0);
}

constexpr int popcount2(int m) { return (m & 1) + ((m >> 1) & 1); }
// k-th stream (0-based) of a non-empty 2-bit stream mask
constexpr int nth_stream(int m, int k) { return (m & 1) ? k : 1; }

// One step.  CUR / NEXT: bit jj set = stream jj takes part in half j / half j+1 (NEXT is a
// subset of CUR).  MASKN: stream whose diagonal may cross half j+1 (-1: none; 2: both streams, against the end of a
// ragged sequence instead of a diagonal).
// On entry cand[jj] holds the raw row maxima of S(j); on exit those of S(j+1).
//
// A wave issues in order, so the body is laid out as issue slots -- one MFMA followed by the
// vector work that fits in its shadow, closed by a scheduling barrier -- instead of leaving
// the interleaving to the compiler:
//   A: one slot per exp piece: [S(j+1) MFMA, then P.V MFMA of a chunk whose weights exist] + the piece (2 exp2,
//      pack, row sum: about the time one MFMA takes);
//   B: the remaining P.V MFMAs, each followed by the row maxima of one stream of S(j+1).
// The K(j+2) fragments are read as soon as the last S MFMA has been issued.
template <typename E, int CUR, int NEXT, int MASKN, bool RG>
__device__ __forceinline__ void half_step(const unsigned short* Ks, const unsigned short* Vs, LaneT<RG>& c, Acc<E>& a,
                                          int j, f32x16 (&s_cur)[2], f32x16 (&s_next)[2], s16x8 (&kf)[4],
                                          float (&cand)[2]) {
    constexpr int nC = popcount2(CUR), nN = popcount2(NEXT);
    constexpr int nQ = 5 * nN;   // S(j+1) MFMAs, k-step major over the NEXT streams; "k step" 0 places -m
    constexpr int nP = 2 * nC;   // P.V MFMAs per 16-key chunk, stream major
    // ---- raise the running maxima if some row outgrew its own by 2^kRaise ---------------------------
    // (Every row sees key 0 in the first half, so a raised maximum is finite.)
    bool raise = false;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
        if ((CUR >> jj) & 1) raise = raise || cand[jj] > a.thr[jj];
    if (__any(raise)) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            if (!((CUR >> jj) & 1)) continue;
            // the scores of this half were computed relative to `base` (0 before the first maximum); the new
            // maximum is rounded to the storage type, in which the MFMA operand carries it
            const float base = a.thr[jj] == -INFINITY ? 0.f : a.m[jj];
            const short mh = E::cvt(fmaxf(a.m[jj], base + cand[jj]));
            const float m_new = E::to_f32(mh);
            const float alpha = __builtin_amdgcn_exp2f(a.m[jj] - m_new);
            const float shift = base - m_new;
            // (the first raise of a stream finds l = 0 and O = 0: nothing to rescale)
            if (!__all(a.thr[jj] == -INFINITY)) {
                a.l[jj] *= alpha;
#pragma unroll
                for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) a.o[jj][dt][r] *= alpha;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) s_cur[jj][r] += shift;
            a.qm[jj][0] = c.hb0 ? (short)(mh ^ (short)0x8000) : (short)0;
            a.m[jj] = m_new;
            a.thr[jj] = kRaise;
        }
    }
    // (The wait for the transfers and for the other wave stands kPre slots further down: the first S MFMAs and exp
    // pieces need registers only, and a wave that arrives early does them while it would otherwise idle.)
    // The rest of a step's fixed work rides in the issue slots below, a few instructions per slot: under two
    // waves per SIMD a slot lasts as long as two MFMAs, and a wave needs less than that for its MFMA and its piece.
    s16x8 vf[2][2];  // V(j) fragments, [16-key chunk][d tile]
    auto vread = [&](int f) {
        const int ch = f >> 1, dt = f & 1;
        const unsigned short* p = Vs + (j & 3) * kSlot + c.vfo[dt] + 16 * ch * kD;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 8 * kD));
        vf[ch][dt] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    auto dma = [&](int d) {   // halves K(j+5) and V(j+3), two transfers each
        if (d == 0) issue_k_part<0>(c, (j + 1) & 3);
        else if (d == 1) issue_k_part<1>(c, (j + 1) & 3);
        else if (d == 2) issue_v_part<0>(c, (j + 3) & 3);
        else issue_v_part<1>(c, (j + 3) & 3);
    };
    unsigned pf[2][2][4];
    slot_end();

    int qi = 0, p0 = 0, p1 = 0, xi = 0, mi = 0;  // next S MFMA, next P.V MFMA of chunk 0 / 1, next exp piece, next maxima
    auto mfma_q = [&]() {
        constexpr int nNd = nN ? nN : 1;  // (never called when NEXT is empty)
        const int ks = qi / nNd, jj = nth_stream(NEXT, qi % nNd);
        s_next[jj] = ks == 0 ? E::mfma32(a.ones, a.qm[jj], f32x16{0}) : E::mfma32(kf[ks - 1], a.qf[jj][ks - 1], s_next[jj]);
        ++qi;
    };
    auto mfma_p = [&](int ch, int k) {
        const int jj = nth_stream(CUR, k / 2), dt = k % 2;
        u32x4 pw = {pf[jj][ch][0], pf[jj][ch][1], pf[jj][ch][2], pf[jj][ch][3]};
        a.o[jj][dt] = E::mfma32(vf[ch][dt], __builtin_bit_cast(s16x8, pw), a.o[jj][dt]);
    };
    // exp pieces run chunk 0 of every stream, then chunk 1: piece x -> (chunk, stream, pair).
    // piece() starts piece xi and finishes piece xi-1.
    float pa[2], pb[2];  // stage-1 results in flight, used alternately
    auto stage1 = [&](int x, float (&p)[2]) {
        const int ch = x / (4 * nC), jj = nth_stream(CUR, (x / 4) % nC), h = 4 * ch + x % 4;
        exp_stage1(s_cur[jj], h, p);
    };
    auto stage2 = [&](int x, const float (&p)[2]) {
        const int ch = x / (4 * nC), jj = nth_stream(CUR, (x / 4) % nC), h = 4 * ch + x % 4;
        exp_stage2<E>(p, h, a.l[jj], pf[jj]);
    };
    auto piece = [&]() {
        if (xi % 2 == 0) {
            if (xi < 8 * nC) stage1(xi, pa);
            if (xi > 0) stage2(xi - 1, pb);
        } else {
            if (xi < 8 * nC) stage1(xi, pb);
            stage2(xi - 1, pa);
        }
        ++xi;
    };
    // row maxima of S(j+1) in stages, stream by stream
    constexpr int nStages = 3 * nN;
    constexpr int kMaxStart = nQ + 1;   // the slot after the one that follows the last S MFMA
    float mx = 0.f;
    auto max_stage = [&]() {
        const int jn = nth_stream(NEXT, mi / 3);
        const int lim = (MASKN == 2 ? c.rag_lim : c.q0[jn] + c.lim0) - kHK * (j + 1);
        if (MASKN == jn || MASKN == 2) {
            if (mi % 3 == 0) row_max_stage<true, 0>(s_next[jn], lim, mx, cand[jn]);
            else if (mi % 3 == 1) row_max_stage<true, 1>(s_next[jn], lim, mx, cand[jn]);
            else row_max_stage<true, 2>(s_next[jn], lim, mx, cand[jn]);
        } else {
            if (mi % 3 == 0) row_max_stage<false, 0>(s_next[jn], lim, mx, cand[jn]);
            else if (mi % 3 == 1) row_max_stage<false, 1>(s_next[jn], lim, mx, cand[jn]);
            else row_max_stage<false, 2>(s_next[jn], lim, mx, cand[jn]);
        }
        ++mi;
    };
    // the K(j+2) fragments are read once every S MFMA has been issued: the old fragments are free then
    bool kread = !NEXT;
    auto after_q = [&]() {
        if (!kread && qi == nQ) {
            read_k_frags(Ks, c, (j + 2) & 3, kf);
            kread = true;
        }
    };
    // A: one MFMA and one exp piece per slot.  First the S MFMAs, then the P.V MFMAs of a chunk as soon as that
    // chunk's weights exist.  Slots kPre..kPre+3 also request one transfer and read one V fragment each (the first P.V MFMA
    // is in slot 5 at the earliest; the transfers are waited for three steps from now, the earlier they leave the
    // better), and from slot kMaxStart on a slot takes a stage of the maxima.
#pragma unroll
    for (int sl = 0; sl < 8 * nC; ++sl) {
        if (qi < nQ) mfma_q();
        else if (p0 < nP && xi > 4 * ((p0 / 2) + 1)) mfma_p(0, p0++);
        else if (p1 < nP && xi > 4 * nC + 4 * (p1 / 2 + 1)) mfma_p(1, p1++);
        after_q();
        if (sl == kPre) wait_and_barrier<kWaitVm8>();
        if (sl >= kPre && sl < kPre + 4) {
            dma(sl - kPre);
            vread(sl - kPre);
        }
        if (sl >= kMaxStart && mi < nStages) max_stage();
        piece();
        slot_end();
    }
    piece();  // finishes the last pair
    // B: the remaining MFMAs, with what is left of the row maxima between them
    after_q();
#pragma unroll
    for (int sl = 0; sl < 2 * nQ + 2 * nP; ++sl) {
        if (qi < nQ) mfma_q();
        else if (p0 < nP) mfma_p(0, p0++);
        else if (p1 < nP) mfma_p(1, p1++);
        else break;
        after_q();
        if (qi == nQ && mi < nStages) max_stage();
        slot_end();
    }
#pragma unroll
    while (mi < nStages) max_stage();
}

// One wide step: the long tile of a wave (stream 1) alone, over the two halves j and j+1.  Once the early
// tile is stored, its score buffers, fragments and issue slots would stand empty for the rest of the walk while
// the fixed cost of a step (barrier, transfers, raise check, fragment reads) stayed the same; instead they take
// the second half, so that a trip has the shape of a two-stream step and the walk takes half as many trips.
// Both halves share the stream's state (m, the accumulators); c0 / c1 are S(j) - m / S(j+1) - m, n0 / n1 receive
// S(j+2) - m / S(j+3) - m, kf[h] holds the K(j+2+h) fragments on entry and the K(j+4+h) fragments on exit,
// cand[h] the row maxima of c_h on entry and of n_h on exit.  Row sums: half j adds to l[1], half j+1 to l[0].
// Ring: a trip waits for everything requested one trip ago (K(j+4), K(j+5), V(j), V(j+1)), then requests
// K(j+6), K(j+7) into the slots whose fragments are in registers and V(j+2), V(j+3) into the slots read one trip
// ago (V(j+2) not in the first wide trip: the narrow steps had requested it already).
template <typename E, bool NEXT, bool MASK, bool RG>
__device__ __forceinline__ void wide_step(const unsigned short* Ks, const unsigned short* Vs, LaneT<RG>& c, Acc<E>& a,
                                          int j, bool first, f32x16& c0, f32x16& c1, f32x16& n0, f32x16& n1,
                                          s16x8 (&kf)[2][4], float (&cand)[2]) {
    constexpr int nQ = NEXT ? 10 : 0;   // S MFMAs, k-step major over the two halves; "k step" 0 places -m
    constexpr int nP = 4;               // P.V MFMAs per 16-key chunk, half major
    {
        const float cm = __builtin_elementwise_maximum(cand[0], cand[1]);
        if (__any(cm > a.thr[1])) {
            const float base = a.thr[1] == -INFINITY ? 0.f : a.m[1];
            const short mh = E::cvt(fmaxf(a.m[1], base + cm));
            const float m_new = E::to_f32(mh);
            const float alpha = __builtin_amdgcn_exp2f(a.m[1] - m_new);
            const float shift = base - m_new;
            a.l[0] *= alpha;
            a.l[1] *= alpha;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) a.o[1][dt][r] *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                c0[r] += shift;
                c1[r] += shift;
            }
            a.qm[1][0] = c.hb0 ? (short)(mh ^ (short)0x8000) : (short)0;
            a.m[1] = m_new;
            a.thr[1] = kRaise;
        }
    }
    // Everything requested one trip ago has landed, and every wave knows.  The first wide trip follows the switch,
    // which has just waited for all it reads before slot 9 and has since stored the early tile and requested K(j+5):
    // it only meets the other wave here (both have read their fragments of the slots about to be refilled) and
    // waits in slot 9, by when stores and request have long returned, for all but this trip's own six transfers.
    // (As in the narrow step, the wait itself stands kPre slots into the trip.)
    // As in the narrow step, the fixed work of the trip rides in the issue slots.
    s16x8 vf[2][2][2];  // [half][16-key chunk][d tile]
    auto vread = [&](int f) {
        const int h = f >> 2, ch = (f >> 1) & 1, dt = f & 1;
        const unsigned short* p = Vs + ((j + h) & 3) * kSlot + c.vfo[dt] + 16 * ch * kD;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 8 * kD));
        vf[h][ch][dt] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    auto dma = [&](int d) {   // K(j+6), K(j+7) (the fragments of j+2, j+3 are in registers), V(j+2), V(j+3)
        if (d == 0) issue_k_part<0>(c, (j + 2) & 3);
        else if (d == 1) issue_k_part<1>(c, (j + 2) & 3);
        else if (d == 2) issue_k_part<0>(c, (j + 3) & 3);
        else if (d == 3) issue_k_part<1>(c, (j + 3) & 3);
        else if (d == 4) { if (!first) issue_v_part<0>(c, (j + 2) & 3); }   // (the narrow steps had requested V(j+2) already)
        else if (d == 5) { if (!first) issue_v_part<1>(c, (j + 2) & 3); }
        else if (d == 6) issue_v_part<0>(c, (j + 3) & 3);
        else issue_v_part<1>(c, (j + 3) & 3);
    };
    unsigned pf[2][2][4];   // [half][chunk][pair]
    slot_end();

    int qi = 0, p0 = 0, p1 = 0, xi = 0;
    auto mfma_q = [&]() {
        const int ks = qi / 2, h = qi % 2;
        f32x16& n = h ? n1 : n0;
        n = ks == 0 ? E::mfma32(a.ones, a.qm[1], f32x16{0}) : E::mfma32(kf[h][ks - 1], a.qf[1][ks - 1], n);
        ++qi;
    };
    auto mfma_p = [&](int ch, int k) {
        const int h = k / 2, dt = k % 2;
        u32x4 pw = {pf[h][ch][0], pf[h][ch][1], pf[h][ch][2], pf[h][ch][3]};
        a.o[1][dt] = E::mfma32(vf[h][ch][dt], __builtin_bit_cast(s16x8, pw), a.o[1][dt]);
    };
    float pa[2], pb[2];
    auto stage1 = [&](int x, float (&p)[2]) {
        const int ch = x / 8, h = (x / 4) % 2, pr = 4 * ch + x % 4;
        exp_stage1(h ? c1 : c0, pr, p);
    };
    auto stage2 = [&](int x, const float (&p)[2]) {
        const int ch = x / 8, h = (x / 4) % 2, pr = 4 * ch + x % 4;
        exp_stage2<E>(p, pr, a.l[1 - h], pf[h]);
    };
    auto piece = [&]() {
        if (xi % 2 == 0) {
            if (xi < 16) stage1(xi, pa);
            if (xi > 0) stage2(xi - 1, pb);
        } else {
            if (xi < 16) stage1(xi, pb);
            stage2(xi - 1, pa);
        }
        ++xi;
    };
    // row maxima of S(j+2), S(j+3) in stages
    constexpr int nStages = NEXT ? 6 : 0;
    int mi = 0;
    float mx = 0.f;
    auto max_stage = [&]() {
        const int h = mi / 3;
        f32x16& n = h ? n1 : n0;
        const int lim = c.q0[1] + c.lim0 - kHK * (j + 2 + h);
        if (mi % 3 == 0) row_max_stage<MASK, 0>(n, lim, mx, cand[h]);
        else if (mi % 3 == 1) row_max_stage<MASK, 1>(n, lim, mx, cand[h]);
        else row_max_stage<MASK, 2>(n, lim, mx, cand[h]);
        ++mi;
    };
    const bool more_k = j + 4 < c.nh;   // (the last trips have no K(j+4), K(j+5) to fetch)
    // Slots 0..7: one transfer each (they are waited for at the head of the next trip: the earlier they leave the
    // better); slots 0..3: two V fragments each (the first P.V MFMA is in slot 5 at the earliest); slots 9, 10: the K(j+4) / K(j+5) fragments, each right after the last S MFMA that read the old
    // ones; from slot 11 on a stage of the maxima.
#pragma unroll
    for (int sl = 0; sl < 16; ++sl) {
        if (qi < nQ) mfma_q();
        else if (p0 < nP && xi > 4 * ((p0 / 2) + 1)) mfma_p(0, p0++);
        else if (p1 < nP && xi > 8 + 4 * (p1 / 2 + 1)) mfma_p(1, p1++);
        if (sl == kPre) {
            if (first) wait_and_barrier<kWaitLgkm>();
            else wait_and_barrier<kWaitVm0>();
        }
        if (sl >= kPre && sl < kPre + 8) dma(sl - kPre);
        if (sl >= kPre && sl < kPre + 4) {
            vread(2 * (sl - kPre));
            vread(2 * (sl - kPre) + 1);
        } else if (sl >= 9 && sl < 11) {
            if (sl == 9 && first) wait_and_barrier<kWaitVm6>();
            if (NEXT && more_k) read_k_frags(Ks, c, (j + 4 + (sl - 9)) & 3, kf[sl - 9]);
        }
        if (sl >= 11 && mi < nStages) max_stage();
        piece();
        slot_end();
    }
    piece();  // finishes the last pair
#pragma unroll
    for (int sl = 0; sl < 2 * nP; ++sl) {
        if (p0 < nP) mfma_p(0, p0++);
        else if (p1 < nP) mfma_p(1, p1++);
        else break;
        if (mi < nStages) max_stage();
        slot_end();
    }
#pragma unroll
    while (mi < nStages) max_stage();
}

// Division of a workgroup id by a launch constant: a multiply-high with floor(2^32 / d) + 1, which is exact while
// x * d < 2^32; the host clears `fast` when the grid is too large for that.  (An integer division is some forty
// instructions, and three of them stand in front of the first load.)
struct Magic {
    unsigned m_nqb, m_h, m_group;
    int fast;
    __device__ __forceinline__ int div(int x, int d, unsigned m) const {
        if (!fast) return x / d;
        return m ? (int)__umulhi((unsigned)x, m) : x;   // (m = 0 stands for d = 1)
    }
    static unsigned of(int d) { return d <= 1 ? 0u : (unsigned)((1ull << 32) / (unsigned)d) + 1u; }
};

template <typename E, bool CAUSAL, bool RG = false>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2, 2))) void fmha_pipe_kernel(
    const unsigned short* __restrict__ Q, Strides qs, const unsigned short* __restrict__ K, Strides ks,
    const unsigned short* __restrict__ V, Strides vs, unsigned short* __restrict__ O, Strides os, int S, int H,
    int group, float scale2, int nqb, int nbh, Magic mg) {
    __shared__ __attribute__((aligned(1024))) unsigned short Ks[4 * kSlot];
    __shared__ __attribute__((aligned(1024))) unsigned short Vs[4 * kSlot];

    const int tid = threadIdx.x, lane = tid & 63, hb = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup ids congruent mod 8 share an XCD: give each XCD whole (batch, head) pairs so
    // that their K / V stay in that XCD's L2.
    int qb, bh;
    {
        const int L = blockIdx.x;
        if (nbh % 8 == 0) {
            const int idx = L >> 3;
            const int q = mg.div(idx, nqb, mg.m_nqb);
            bh = (L & 7) + 8 * q;
            qb = idx - q * nqb;
            // A pair with a late long tile spends more of its walk in wide steps and takes a few per cent longer.
            // An XCD places consecutive workgroups on its 32 CUs in turn, so ids 32 apart share a CU: every
            // second round of 32 takes the pairs in reverse order, and each CU gets both kinds.  (Decided by the
            // first id of the (batch, head) group, so that a group is reversed as a whole: a permutation of its pairs.)
            if (CAUSAL && (((q * nqb) >> 5) & 1)) qb = nqb - 1 - qb;
        } else {
            bh = mg.div(L, nqb, mg.m_nqb);
            qb = L - bh * nqb;
        }
    }
    const int batch = mg.div(bh, H, mg.m_h), head = bh - batch * H, kvh = mg.div(head, group, mg.m_group);
    Q += (int64_t)head * qs.s2 + (int64_t)batch * qs.s3;
    O += (int64_t)head * os.s2 + (int64_t)batch * os.s3;

    const int NT = 4 * nqb;   // 32-query tiles of the grid (RG: of the sequence rounded up to whole workgroups)
    int tq[2];
    if (CAUSAL) {
        tq[0] = 2 * qb + wave;
        tq[1] = NT - 1 - tq[0];
    } else {
        tq[0] = 4 * qb + 2 * wave;
        tq[1] = tq[0] + 1;
    }

    LaneT<RG> c;
    c.kptr = (const char*)(K + (int64_t)kvh * ks.s2 + (int64_t)batch * ks.s3);
    c.vptr = (const char*)(V + (int64_t)kvh * vs.s2 + (int64_t)batch * vs.s3);
    c.k_half_bytes = (int64_t)kHK * ks.s1 * 2;
    c.v_half_bytes = (int64_t)kHK * vs.s1 * 2;
    c.ks_base = (unsigned)(size_t)Ks;
    c.vs_base = (unsigned)(size_t)Vs;
    c.wave = wave;
    // The waves of the second half of the grid land on SIMDs that already host a wave of the first half, and the
    // instruction arbiter serves the older wave first: the younger one ran 20 % longer.  A raised priority evens
    // the two out (they have the same amount of work), which shortens the kernel.
    if (blockIdx.x >= (gridDim.x >> 1)) __builtin_amdgcn_s_setprio(1);
    // (ragged, no causal mask: up to the pair of halves that holds the last key)
    c.nh = CAUSAL ? NT - 2 * qb : RG ? (((S + kHK - 1) / kHK + 1) & ~1) : NT;
    c.k_left = c.v_left = c.nh;
    c.to_end = false;
    int last_row = kHK - 1;
    if constexpr (RG) {
        const int vh = (S + kHK - 1) / kHK;   // halves that exist
        c.to_end = c.nh >= vh;
        if (c.to_end) c.k_left = c.v_left = vh;
        last_row = S - 1 - kHK * (vh - 1);
        c.rag_lim = S - 1 - 4 * hb;
    }
    c.hb0 = hb == 0;
    {
        // transfer `wave` of a half covers keys 8*wave .. 8*wave+7; transfer wave+2 the keys 16 further on,
        // whose swizzle (a function of key % 16 resp. key % 4) is the same.  K: chunk ^ (key / 2) % 8 --
        // rows alternate between the two halves of the banks, so the 16 lanes that the LDS serves
        // together for a 16-byte read (keys k .. k+15 of one chunk column) land on 16 distinct slots.
        const int key = 8 * wave + (lane >> 3), pos = lane & 7;
        c.kdma = (unsigned)(((int64_t)key * ks.s1 + 8 * (pos ^ ((key >> 1) & 7))) * 2);
        c.vdma = (unsigned)(((int64_t)key * vs.s1 + 8 * (pos ^ (2 * (key & 3)))) * 2);
        if constexpr (RG) {
            c.kdma_b = c.kdma + (unsigned)(c.k_half_bytes >> 1);
            c.vdma_b = c.vdma + (unsigned)(c.v_half_bytes >> 1);
            ragged_offsets<false>(wave, lane, last_row, c.k_half_bytes, c.k_rg[0], c.k_rg[1]);
            ragged_offsets<true>(wave, lane, last_row, c.v_half_bytes, c.v_rg[0], c.v_rg[1]);
        }
    }
    c.lim0 = (lane & 31) - 4 * hb;
    c.q0[0] = 32 * tq[0];
    c.q0[1] = 32 * tq[1];
    {
        const int key = lane & 31;
#pragma unroll
        for (int s = 0; s < 4; ++s) c.kfo[s] = key * kD + 8 * ((2 * s + hb) ^ ((key >> 1) & 7));
        const int g = lane >> 4, r = lane & 15;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
            const int row = 4 * (g >> 1) + (r >> 2);
            const int col = 32 * dt + 16 * (g & 1) + 4 * (r & 3);
            c.vfo[dt] = row * kD + 8 * ((col >> 3) ^ (2 * (r >> 2))) + (col & 7);
        }
    }

    // Q first, then the ring fill, in the order of need and spread over the prologue: all the waves of a CU start
    // together, and what they request before their first MFMA passes through the CU's one 64-byte-per-cycle path to
    // the L2 (20 KB per wave would be 2 500 cycles; Q, K(0) and K(1) are 12).  Every load is counted by hand here
    // (the Q loads are inline assembly like the transfers), so that the wave goes on as soon as what it needs next
    // has landed.
    int my_q[2];
    u32x4 qraw[2][4];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
        my_q[jj] = 32 * tq[jj] + (lane & 31);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int row = RG && my_q[jj] >= S ? S - 1 : my_q[jj];   // (queries past the end: any row, never stored)
            const unsigned short* qp = Q + (int64_t)row * qs.s1 + 16 * s + 8 * hb;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qraw[jj][s]) : "v"(qp) : "memory");
        }
    }
    issue_k(c, 0);
    issue_k(c, 1);
    // (the registers are operands of the wait, so nothing that reads them is scheduled above it)
    asm volatile("s_waitcnt vmcnt(4)"
                 : "+v"(qraw[0][0]), "+v"(qraw[0][1]), "+v"(qraw[0][2]), "+v"(qraw[0][3]), "+v"(qraw[1][0]), "+v"(qraw[1][1]),
                   "+v"(qraw[1][2]), "+v"(qraw[1][3])
                 :
                 : "memory");

    Acc<E> a;
    a.ones = s16x8{0};
    a.ones[0] = hb == 0 ? E::cvt(1.0f) : (short)0;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            // Q * (qk_scale / ln 2), rounded once to the storage type: the S MFMAs then deliver exp2-domain
            // scores (fmha.jl:41,106-110 scales the fp32 products instead; the difference is one rounding of Q)
            a.qf[jj][s] = E::scale8(__builtin_bit_cast(s16x8, qraw[jj][s]), scale2);
        }
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) a.o[jj][dt] = f32x16{0};
        a.qm[jj] = s16x8{0};
        a.m[jj] = -INFINITY;
        a.thr[jj] = -INFINITY;
        a.l[jj] = 0.f;
    }

    // ---- prologue: compute S(0), fetch the K(1) fragments -----------------------------------------
    wait_and_barrier<kWaitVm2>();  // K(0) has landed, in every wave's part of the slot
    f32x16 sa[2], sb[2];
    s16x8 kf[4];
    float cand[2];
    read_k_frags(Ks, c, 0, kf);
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) sa[jj] = E::mfma32(kf[s], a.qf[jj][s], s == 0 ? f32x16{0} : sa[jj]);
    issue_k(c, 2);
    issue_v(c, 0);
    wait_and_barrier<kWaitVm4>();   // K(1)
    read_k_frags(Ks, c, 1, kf);
    issue_k(c, 3);
    issue_v(c, 1);
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)  // tile 0 has its diagonal in half 0
        // (only a tile that starts inside half 0 has its diagonal there; q0 is wave-uniform)
        cand[jj] = (CAUSAL && c.q0[jj] < kHK) ? masked_row_max<true>(sa[jj], c.q0[jj] + c.lim0) : masked_row_max<false>(sa[jj], 0);
    wait_and_barrier<kWaitVm8>();  // every wave has read its K(0) fragments: slot 0 is free
    issue_k(c, 0);  // half 4
    issue_v(c, 2);

    // Epilogue of one stream: add the two half-row sums, O / l (approximate reciprocal), round, store.
    auto store_tile = [&](int jj, float lsum) {
        const float inv = __builtin_amdgcn_rcpf(xhalf_sum(lsum));
        if (RG && my_q[jj] >= S) return;
        unsigned short* op = O + (int64_t)my_q[jj] * os.s1;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                s16x4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = E::cvt(a.o[jj][dt][4 * g + e] * inv);
                *reinterpret_cast<s16x4*>(op + 32 * dt + 8 * g + 4 * hb) = w;
            }
    };

    // ---- main loops: two steps per trip, the score buffers swap roles --------------------------------
#define STEP(CUR, NEXT, MASKN, jx, s0, s1) half_step<E, CUR, NEXT, MASKN>(Ks, Vs, c, a, jx, s0, s1, kf, cand)
    const int nh = c.nh;
    int j = 0;
    if (CAUSAL) {
        // Stream 0 takes part in steps 0..n1-1 and has its diagonal in halves n1-2, n1-1 (one per
        // wave); stream 1 runs to the end and has its diagonal in halves nh-2, nh-1.  A half is
        // masked when its row maxima are taken, i.e. one step before it is consumed.
        const int n1 = 2 * qb + 2;
        for (; j < n1 - 4; j += 2) {
            STEP(3, 3, -1, j, sa, sb);
            STEP(3, 3, -1, j + 1, sb, sa);
        }
        for (; j < n1 - 2; j += 2) {  // at most one trip; masking half n1-3 as well is harmless
            STEP(3, 3, 0, j, sa, sb);
            STEP(3, 3, 0, j + 1, sb, sa);
        }
        STEP(3, 3, 0, j, sa, sb);
        STEP(3, 2, 1, j + 1, sb, sa);  // (stream 1's mask only bites when its diagonal is two halves away)
        j += 2;
        // ---- wide steps: the long tile over two halves per trip (always an odd number of trips) ------------
        // S(n1) - m is in sa[1] and the K(n1+1) fragments in kf: compute S(n1+1) - m into sa[0], then fetch
        // the fragments of the next two halves and request the one transfer the wide schedule still lacks.
        s16x8 kw[2][4];
        float wc[2];
        wc[0] = cand[1];
        sa[0] = E::mfma32(a.ones, a.qm[1], f32x16{0});
#pragma unroll
        for (int s = 0; s < 4; ++s) sa[0] = E::mfma32(kf[s], a.qf[1][s], sa[0]);
        {
            const int q_rel = c.q0[1] - kHK * (j + 1);   // first query of the tile relative to the half (wave-uniform)
            wc[1] = q_rel < kHK ? masked_row_max<true>(sa[0], q_rel + c.lim0) : masked_row_max<false>(sa[0], 0);
        }
        // K(j+2) and K(j+3) have landed once only the last narrow step's four transfers (K(j+4), V(j+2)) are out
        wait_and_barrier<kWaitVm4>();
        issue_k(c, (j + 1) & 3);  // half j+5
        // Stream 0 is complete: its registers and issue slots now serve the long tile.  (Stored after the wait above:
        // stores count as outstanding memory operations like the transfers, and are younger than all of them.)
        store_tile(0, a.l[0]);
        a.l[0] = 0.f;
        read_k_frags(Ks, c, (j + 2) & 3, kw[0]);
        read_k_frags(Ks, c, (j + 3) & 3, kw[1]);
#define WIDE(NEXT, MASK, jx, first, s0, s1) wide_step<E, NEXT, MASK>(Ks, Vs, c, a, jx, first, s0[1], s0[0], s1[1], s1[0], kw, wc)
        bool first = true;
        if (j + 2 < nh) {   // three trips or more: an odd number of plain trips, then the one that masks
            for (; j + 6 < nh; j += 4) {
                WIDE(true, false, j, first, sa, sb);
                WIDE(true, false, j + 2, false, sb, sa);
                first = false;
            }
            WIDE(true, false, j, first, sa, sb);
            WIDE(true, true, j + 2, false, sb, sa);
            j += 4;
            first = false;
        }
        WIDE(false, false, j, first, sa, sb);
#undef WIDE
    } else if constexpr (RG) {   // (nh >= 6: at least 129 keys)
        for (; j < nh - 4; j += 2) {
            STEP(3, 3, -1, j, sa, sb);
            STEP(3, 3, -1, j + 1, sb, sa);
        }
        STEP(3, 3, -1, j, sa, sb);
        STEP(3, 3, 2, j + 1, sb, sa);    // S(nh - 2) and S(nh - 1): the halves that may reach past the last key
        STEP(3, 3, 2, j + 2, sa, sb);
        STEP(3, 0, -1, j + 3, sb, sa);
    } else {
        for (; j < nh - 2; j += 2) {
            STEP(3, 3, -1, j, sa, sb);
            STEP(3, 3, -1, j + 1, sb, sa);
        }
        STEP(3, 3, -1, j, sa, sb);
        STEP(3, 0, -1, j + 1, sb, sa);
    }
#undef STEP
    // Transfers issued for halves past the end are still in flight: let them land before the
    // workgroup's LDS can be handed to another workgroup.
    __builtin_amdgcn_s_waitcnt(kWaitVm0);

    if (!CAUSAL) store_tile(0, a.l[0]);
    store_tile(1, CAUSAL ? a.l[0] + a.l[1] : a.l[1]);
}

bool vec16(const mi_tile_array* a) {
    return ((uintptr_t)a->ptr % 16) == 0 && a->strides[1] % 8 == 0 && a->strides[2] % 8 == 0 && a->strides[3] % 8 == 0;
}

template <typename E>
void launch_e(const Problem& p, hipStream_t stream) {
    const mi_tile_array *Q = p.Q, *K = p.K, *V = p.V, *O = p.O;
    Strides qs{Q->strides[1], Q->strides[2], Q->strides[3]}, ks{K->strides[1], K->strides[2], K->strides[3]},
        vs{V->strides[1], V->strides[2], V->strides[3]}, os{O->strides[1], O->strides[2], O->strides[3]};
    const int S = (int)Q->sizes[1];
    const int nqb = (S + 127) / 128, nbh = (int)(Q->sizes[2] * Q->sizes[3]);
    dim3 grid((unsigned)(nqb * nbh)), blk(128);
    Magic mg{Magic::of(nqb), Magic::of(p.H), Magic::of(p.group), 0};
    const int64_t dmax = nqb > p.H ? nqb : p.H;
    mg.fast = (int64_t)grid.x * (dmax > p.group ? dmax : p.group) < (1ll << 32) ? 1 : 0;
    if (p.causal && S % 128 != 0)
        hipLaunchKernelGGL((fmha_pipe_kernel<E, true, true>), grid, blk, 0, stream, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs, (unsigned short*)O->ptr,
                           os, S, p.H, p.group, p.scale2, nqb, nbh, mg);
    else if (S % 128 != 0)
        hipLaunchKernelGGL((fmha_pipe_kernel<E, false, true>), grid, blk, 0, stream, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs, (unsigned short*)O->ptr,
                           os, S, p.H, p.group, p.scale2, nqb, nbh, mg);
    else if (p.causal)
        hipLaunchKernelGGL((fmha_pipe_kernel<E, true>), grid, blk, 0, stream, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs, (unsigned short*)O->ptr,
                           os, S, p.H, p.group, p.scale2, nqb, nbh, mg);
    else
        hipLaunchKernelGGL((fmha_pipe_kernel<E, false>), grid, blk, 0, stream, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs, (unsigned short*)O->ptr,
                           os, S, p.H, p.group, p.scale2, nqb, nbh, mg);
}

}  // namespace

bool pipe_applicable(const Problem& p) {
    const mi_tile_array *Q = p.Q, *K = p.K, *V = p.V, *O = p.O;
    if (Q->sizes[0] != kD || V->sizes[0] != kD) return false;
    const int64_t S = Q->sizes[1];
    if (K->sizes[1] != S || S < 128) return false;
    if (S % 128 != 0 && S < 129) return false;
    if (!(p.scale2 > 0.f)) return false;
    if (p.causal && p.input_pos != 0) return false;
    if (!vec16(Q) || !vec16(K) || !vec16(V) || !vec16(O)) return false;
    if (K->strides[1] >= (1 << 20) || V->strides[1] >= (1 << 20)) return false;
    if (Q->sizes[2] * Q->sizes[3] * ((S + 127) / 128) > MI_MAX_GRID_DIM) return false;
    return true;
}

void pipe_launch(const Problem& p, hipStream_t stream) {
    if (p.bf16) launch_e<BF16>(p, stream);
    else launch_e<F16>(p, stream);
    set_variant(p.Q->sizes[1] % 128 ? "fmha_pipe_d64_q128_kv32_ring4_ragged" : "fmha_pipe_d64_q128_kv32_ring4");
}

}  // namespace fmha
}  // namespace mi

