// Fused multi-head attention forward, software-pipelined kernel for head dimension 64:
// stand-in for fmha_kernel of the reference's examples/fmha.jl:20-139 on the shapes its
// benchmark uses (fmha.jl:230-260: D = 64, Sq == Skv, no decode offset).
//
// Work split.  A workgroup is two waves and owns 128 queries of one (batch, head); a wave owns
// two 32-query MFMA column tiles ("streams").  Without a causal mask the streams are adjacent
// tiles.  With it, wave w of workgroup qb takes tiles u = 2*qb + w and NT-1-u, so that every
// wave of the grid has the same number of MFMAs; stream 0 (the early tile) leaves the loop
// after its diagonal.
//
// K and V travel in halves of 32 keys (4 KB each) through two rings of four LDS slots, filled
// by direct global->LDS loads three steps ahead of their use.  One step handles one half:
//     barrier (publishes the half issued three steps ago)
//     issue loads of K half j+5 and V half j+3
//     S(j+1) = K(j+1) . Q          8 MFMA, K fragments already in registers
//     read K(j+2) and V(j) fragments from LDS
//     softmax of S(j)              VALU, overlaps the MFMAs above
//     O += V(j) . P(j)             8 MFMA
// so the matrix pipe works on the next half's scores while the vector pipe exponentiates this
// half's.  The two score buffers swap roles every step (the loops are unrolled by two), so no
// register copies are needed.  The global->LDS loads are issued from inline assembly and waited
// for with explicit vmcnt counts; the compiler sees only the LDS reads.
//
// Online softmax in the exp2 domain (fmha.jl:41,106-127).  The running maximum m of a row is
// only raised when the new maximum exceeds it by more than 8 (a factor 256 in the weights):
// the result is the same function of the inputs, the weights P stay below 2^8 in the storage
// type, and the accumulator rescale all but disappears.  Row sums are taken over the rounded
// weights, i.e. over exactly the values that multiply V.
#include "fmha_common.h"

namespace mi {
namespace fmha {
namespace {

constexpr int kD = 64;            // head dimension
constexpr int kHK = 32;           // keys per half
constexpr int kSlot = kHK * kD;   // elements per ring slot
constexpr int kSlotBytes = kSlot * 2;
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
constexpr int kWaitVm0 = 0x0070, kWaitVm4 = 0x0074, kWaitVm8 = 0x0078;

template <int IMM>
__device__ __forceinline__ void wait_and_barrier() {
    __builtin_amdgcn_s_waitcnt(IMM);
    fence();
    __builtin_amdgcn_s_barrier();
    fence();
}

// max / sum over the lane pair (l, l ^ 32)
__device__ __forceinline__ float xhalf_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

struct Lane {
    // wave-uniform
    const char *Kg, *Vg;            // first key of this (batch, kv head)
    int64_t k_half_bytes, v_half_bytes;
    unsigned ks_base, vs_base;      // LDS byte addresses of the rings
    int wave, nh;                   // halves walked by this workgroup
    float scale2;
    // per lane
    unsigned kdma[2], vdma[2];      // byte offsets of the lane's 16 bytes in transfers wave, wave+2
    unsigned kfo[4];                // K fragment element offsets inside a slot, per k-step
    unsigned vfo[2];                // V fragment element offsets inside a slot, per d tile
    int lim[2];                     // last visible key of the lane's query minus 4*(lane/32), per stream
};

template <typename E>
struct Acc {
    s16x8 qf[2][4];
    f32x16 o[2][2];
    float m[2], l[2];
};

__device__ __forceinline__ void issue_k(const Lane& c, int h, int slot) {
    const int hc = h < c.nh ? h : c.nh - 1;  // past the end: reload the last half into a free slot
    const char* g = c.Kg + hc * c.k_half_bytes;
    const unsigned lds = c.ks_base + slot * kSlotBytes + c.wave * 1024;
    dma16(c.kdma[0], g, lds);
    dma16(c.kdma[1], g, lds + 2048);
}
__device__ __forceinline__ void issue_v(const Lane& c, int h, int slot) {
    const int hc = h < c.nh ? h : c.nh - 1;
    const char* g = c.Vg + hc * c.v_half_bytes;
    const unsigned lds = c.vs_base + slot * kSlotBytes + c.wave * 1024;
    dma16(c.vdma[0], g, lds);
    dma16(c.vdma[1], g, lds + 2048);
}

__device__ __forceinline__ void read_k_frags(const unsigned short* Ks, const Lane& c, int slot, s16x8 (&kf)[4]) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) kf[ks] = *reinterpret_cast<const s16x8*>(Ks + slot * kSlot + c.kfo[ks]);
}

// First part of the softmax of one stream's 32x32 score tile: apply the causal mask and return
// the row maximum in the exp2 domain.
template <bool MASK>
__device__ __forceinline__ float masked_row_max(f32x16& s, int lim, float scale2) {
    if (MASK) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = (8 * (r >> 2) + (r & 3) <= lim) ? s[r] : -INFINITY;
    }
    float mx = fmaxf(s[0], s[1]);
#pragma unroll
    for (int r = 2; r < 16; r += 2) mx = fmaxf(fmaxf(mx, s[r]), s[r + 1]);
    return xhalf_max(mx) * scale2;
}

// Second part: weights relative to the (possibly stale) running maximum, rounded and packed for
// the P.V MFMAs, and their row sum.
template <typename E>
__device__ __forceinline__ void exp_pack(const f32x16& s, float m, float& l, float scale2, unsigned (&pf)[2][4]) {
    const float nm = -m;
    float lsum = l;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], scale2, nm));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r + 1], scale2, nm));
        const unsigned pk = Pack<E>::pack(p0, p1);
        lsum = Pack<E>::sum2(pk, lsum);
        pf[r >> 3][(r & 7) >> 1] = pk;
    }
    l = lsum;
}

// One step.  CUR / NEXT: bit jj set = stream jj takes part in half j / half j+1.
// MASKJ: stream whose diagonal may cross half j (-1: none).
template <typename E, int CUR, int NEXT, int MASKJ>
__device__ __forceinline__ void half_step(const unsigned short* Ks, const unsigned short* Vs, const Lane& c, Acc<E>& a,
                                          int j, f32x16 (&s_cur)[2], f32x16 (&s_next)[2], s16x8 (&kf)[4]) {
    // ---- row maxima of S(j); raise the running maxima if some row outgrew its own by 2^kRaise ----
    // (Every row sees key 0 in the first half, so a raised maximum is finite.)
    float cand[2];
    bool raise = false;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
        if (!((CUR >> jj) & 1)) continue;
        cand[jj] = MASKJ == jj ? masked_row_max<true>(s_cur[jj], c.lim[jj] - kHK * j, c.scale2)
                               : masked_row_max<false>(s_cur[jj], 0, c.scale2);
        raise = raise || cand[jj] > a.m[jj] + kRaise;
    }
    if (__any(raise)) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            if (!((CUR >> jj) & 1)) continue;
            const float m_new = fmaxf(a.m[jj], cand[jj]);
            const float alpha = __builtin_amdgcn_exp2f(a.m[jj] - m_new);
            a.l[jj] *= alpha;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) a.o[jj][dt][r] *= alpha;
            a.m[jj] = m_new;
        }
    }
    wait_and_barrier<kWaitVm8>();
    issue_k(c, j + 5, (j + 1) & 3);
    issue_v(c, j + 3, (j + 3) & 3);

    // ---- S(j+1) = K(j+1) . Q ------------------------------------------------------------------
    if (NEXT) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
                if ((NEXT >> jj) & 1) s_next[jj] = E::mfma32(kf[ks], a.qf[jj][ks], ks == 0 ? f32x16{0} : s_next[jj]);
    }
    // ---- fragment reads: K(j+2) for the next step, V(j) for this one ----------------------------
    s16x8 kn[4];
    if (NEXT) read_k_frags(Ks, c, (j + 2) & 3, kn);
    s16x8 vf[2][2];  // [16-key chunk][d tile]
    {
        const unsigned short* vb = Vs + (j & 3) * kSlot;
#pragma unroll
        for (int ch = 0; ch < 2; ++ch)
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const unsigned short* p = vb + c.vfo[dt] + 16 * ch * kD;
                s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
                s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 8 * kD));
                vf[ch][dt] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
    }
    // ---- weights of S(j), then O += V(j) . P(j) ---------------------------------------------------
    unsigned pf[2][2][4];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
        if (!((CUR >> jj) & 1)) continue;
        exp_pack<E>(s_cur[jj], a.m[jj], a.l[jj], c.scale2, pf[jj]);
    }
#pragma unroll
    for (int ch = 0; ch < 2; ++ch)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                if (!((CUR >> jj) & 1)) continue;
                u32x4 pw = {pf[jj][ch][0], pf[jj][ch][1], pf[jj][ch][2], pf[jj][ch][3]};
                a.o[jj][dt] = E::mfma32(vf[ch][dt], __builtin_bit_cast(s16x8, pw), a.o[jj][dt]);
            }
    if (NEXT) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) kf[ks] = kn[ks];
    }
}

template <typename E, bool CAUSAL>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2, 2))) void fmha_pipe_kernel(
    const unsigned short* __restrict__ Q, Strides qs, const unsigned short* __restrict__ K, Strides ks,
    const unsigned short* __restrict__ V, Strides vs, unsigned short* __restrict__ O, Strides os, int S, int H,
    int group, float scale2, int nqb, int nbh) {
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
            bh = (L & 7) + 8 * (idx / nqb);
            qb = idx % nqb;
        } else {
            bh = L / nqb;
            qb = L % nqb;
        }
    }
    const int batch = bh / H, head = bh % H, kvh = head / group;
    Q += (int64_t)head * qs.s2 + (int64_t)batch * qs.s3;
    O += (int64_t)head * os.s2 + (int64_t)batch * os.s3;

    const int NT = S / 32;
    int tq[2];
    if (CAUSAL) {
        tq[0] = 2 * qb + wave;
        tq[1] = NT - 1 - tq[0];
    } else {
        tq[0] = 4 * qb + 2 * wave;
        tq[1] = tq[0] + 1;
    }

    Lane c;
    c.Kg = (const char*)(K + (int64_t)kvh * ks.s2 + (int64_t)batch * ks.s3);
    c.Vg = (const char*)(V + (int64_t)kvh * vs.s2 + (int64_t)batch * vs.s3);
    c.k_half_bytes = (int64_t)kHK * ks.s1 * 2;
    c.v_half_bytes = (int64_t)kHK * vs.s1 * 2;
    c.ks_base = (unsigned)(size_t)Ks;
    c.vs_base = (unsigned)(size_t)Vs;
    c.wave = wave;
    c.nh = CAUSAL ? NT - 2 * qb : NT;
    c.scale2 = scale2;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int key = 8 * (wave + 2 * i) + (lane >> 3), pos = lane & 7;
        c.kdma[i] = (unsigned)(((int64_t)key * ks.s1 + 8 * (pos ^ (key & 7))) * 2);
        c.vdma[i] = (unsigned)(((int64_t)key * vs.s1 + 8 * (pos ^ (2 * (key & 3)))) * 2);
    }
    {
        const int key = lane & 31;
#pragma unroll
        for (int s = 0; s < 4; ++s) c.kfo[s] = key * kD + 8 * ((2 * s + hb) ^ (key & 7));
        const int g = lane >> 4, r = lane & 15;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
            const int row = 4 * (g >> 1) + (r >> 2);
            const int col = 32 * dt + 16 * (g & 1) + 4 * (r & 3);
            c.vfo[dt] = row * kD + 8 * ((col >> 3) ^ (2 * (r >> 2))) + (col & 7);
        }
    }

    Acc<E> a;
    int my_q[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
        my_q[jj] = 32 * tq[jj] + (lane & 31);
        c.lim[jj] = my_q[jj] - 4 * hb;
#pragma unroll
        for (int s = 0; s < 4; ++s)
            a.qf[jj][s] = *reinterpret_cast<const s16x8*>(Q + (int64_t)my_q[jj] * qs.s1 + 16 * s + 8 * hb);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) a.o[jj][dt] = f32x16{0};
        a.m[jj] = -INFINITY;
        a.l[jj] = 0.f;
    }

    // ---- prologue: fill the rings, compute S(0), fetch the K(1) fragments -----------------------
    issue_k(c, 0, 0);
    issue_k(c, 1, 1);
    issue_k(c, 2, 2);
    issue_v(c, 0, 0);
    issue_k(c, 3, 3);
    issue_v(c, 1, 1);
    wait_and_barrier<kWaitVm4>();  // K(0..2), V(0) have landed
    f32x16 sa[2], sb[2];
    s16x8 kf[4];
    read_k_frags(Ks, c, 0, kf);
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) sa[jj] = E::mfma32(kf[s], a.qf[jj][s], s == 0 ? f32x16{0} : sa[jj]);
    {
        s16x8 k1[4];
        read_k_frags(Ks, c, 1, k1);
#pragma unroll
        for (int s = 0; s < 4; ++s) kf[s] = k1[s];
    }
    wait_and_barrier<kWaitVm4>();  // every wave has read its K(0) fragments: slot 0 is free
    issue_k(c, 4, 0);
    issue_v(c, 2, 2);

    // ---- main loops: two steps per trip, the score buffers swap roles --------------------------------
    const int nh = c.nh;
    int j = 0;
    if (CAUSAL) {
        const int n1 = 2 * qb + 2;  // steps in which stream 0 takes part; its diagonal is in the last two
        for (; j < n1 - 2; j += 2) {
            half_step<E, 3, 3, -1>(Ks, Vs, c, a, j, sa, sb, kf);
            half_step<E, 3, 3, -1>(Ks, Vs, c, a, j + 1, sb, sa, kf);
        }
        half_step<E, 3, 3, 0>(Ks, Vs, c, a, j, sa, sb, kf);
        half_step<E, 3, 2, 0>(Ks, Vs, c, a, j + 1, sb, sa, kf);
        j += 2;
        for (; j < nh - 2; j += 2) {
            half_step<E, 2, 2, -1>(Ks, Vs, c, a, j, sa, sb, kf);
            half_step<E, 2, 2, -1>(Ks, Vs, c, a, j + 1, sb, sa, kf);
        }
        half_step<E, 2, 2, 1>(Ks, Vs, c, a, j, sa, sb, kf);
        half_step<E, 2, 0, 1>(Ks, Vs, c, a, j + 1, sb, sa, kf);
    } else {
        for (; j < nh - 2; j += 2) {
            half_step<E, 3, 3, -1>(Ks, Vs, c, a, j, sa, sb, kf);
            half_step<E, 3, 3, -1>(Ks, Vs, c, a, j + 1, sb, sa, kf);
        }
        half_step<E, 3, 3, -1>(Ks, Vs, c, a, j, sa, sb, kf);
        half_step<E, 3, 0, -1>(Ks, Vs, c, a, j + 1, sb, sa, kf);
    }
    // Transfers issued for halves past the end are still in flight: let them land before the
    // workgroup's LDS can be handed to another workgroup.
    __builtin_amdgcn_s_waitcnt(kWaitVm0);

    // ---- epilogue: add the two half-row sums, O / l (approximate reciprocal), round, store --------
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
        const float inv = __builtin_amdgcn_rcpf(xhalf_sum(a.l[jj]));
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
    }
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
    const int nqb = S / 128, nbh = (int)(Q->sizes[2] * Q->sizes[3]);
    dim3 grid((unsigned)(nqb * nbh)), blk(128);
    if (p.causal)
        hipLaunchKernelGGL((fmha_pipe_kernel<E, true>), grid, blk, 0, stream, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs, (unsigned short*)O->ptr,
                           os, S, p.H, p.group, p.scale2, nqb, nbh);
    else
        hipLaunchKernelGGL((fmha_pipe_kernel<E, false>), grid, blk, 0, stream, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs, (unsigned short*)O->ptr,
                           os, S, p.H, p.group, p.scale2, nqb, nbh);
}

}  // namespace

bool pipe_applicable(const Problem& p) {
    const mi_tile_array *Q = p.Q, *K = p.K, *V = p.V, *O = p.O;
    if (Q->sizes[0] != kD || V->sizes[0] != kD) return false;
    const int64_t S = Q->sizes[1];
    if (K->sizes[1] != S || S % 128 != 0 || S < 128) return false;
    if (!(p.scale2 > 0.f)) return false;
    if (p.causal && p.input_pos != 0) return false;
    if (!vec16(Q) || !vec16(K) || !vec16(V) || !vec16(O)) return false;
    if (K->strides[1] >= (1 << 20) || V->strides[1] >= (1 << 20)) return false;
    if (Q->sizes[2] * Q->sizes[3] * (S / 128) > 0x7fffffff) return false;
    return true;
}

void pipe_launch(const Problem& p, hipStream_t stream) {
    if (p.bf16) launch_e<BF16>(p, stream);
    else launch_e<F16>(p, stream);
    set_variant("fmha_pipe_d64_q128_kv32_ring4");
}

}  // namespace fmha
}  // namespace mi
