// Fused multi-head attention forward: stand-in for fmha_kernel of the reference's
// examples/fmha.jl:20-139 (FlashAttention-2 style online softmax).
//
// Layout (Julia column-major): Q (D, Sq, H, B), K (D, Skv, KVH, B), V (D, Skv, KVH, B),
// Out (D, Sq, H, B); D is contiguous, so a query / key / value vector is a contiguous run.
//
// Mapping to CDNA4 (fmha_fwd_dma_kernel; fmha_fwd_kernel below is the register-staged
// fallback for inputs that are not 16-byte aligned, one 32-query tile per wave).
// A workgroup owns 128 consecutive queries of one (batch, head): 2 waves x 64 queries for
// D = 64, 4 waves x 32 for D = 128.  A wave's queries are two 32-query MFMA column tiles
// which share every K / V fragment read.  KV is walked in tiles of 64 keys, double-buffered
// in LDS by direct global->LDS loads (XOR swizzle applied on the global-address side).
//   S^T (keys x queries) = K . Q : MFMA 32x32x16, row operand = K rows read as 16-byte
//     D-contiguous fragments from the swizzled LDS tile, column operand = Q fragments
//     held in registers for the whole kernel (lane % 32 = query).
//   online softmax in the exp2 domain, entirely in registers: a query's scores live in the
//     two lanes l and l^32, so the row max needs one cross-lane exchange per tile; the
//     accumulator is rescaled only on tiles where some row max rose; row sums are taken
//     over the rounded P values with v_dot2 and combined across the lane pair at the end.
//   O^T (D x queries) += V . P : the fp32 scores, rounded to the storage type (fmha.jl:124),
//     are already in column-operand layout (lane % 32 = query, 8 keys per lane); the
//     matching row operand is read from the V tile with the LDS transpose read, whose
//     4-consecutive-row granularity matches the accumulator's 4-row groups, so P never
//     moves between lanes.
// Causal balance: with causal masking a wave takes the 32-query tiles u and NT-1-u, so every
// wave walks the same number of KV tiles.  All query tiles of a (batch, head) run on one XCD.
// Causal tile skipping: the KV loop stops at the workgroup's last query, and a wave skips
// tiles that lie wholly above its own last query.  Masking and the ragged KV tail use -Inf
// as in the reference (fmha.jl:92-103).
//
// Few queries against many keys (decode, chunked prefill): B * H * cld(Sq, 128) workgroups leave most of the chip
// idle and each walks the whole KV range alone.  The KV tiles of a workgroup are then dealt to `nsplit` workgroups
// (SPLIT instantiation); each leaves its unnormalised accumulator, running maximum and row sum in a scratch array of
// the library, and fmha_combine_kernel adds the parts with the usual exp2(m_part - m) weights.  A part may start
// above a query's diagonal, so a row can go through tiles without a visible key: its maximum stays -Inf and the
// weights are taken against 0 instead (SAFE), which keeps them at exp2(-Inf) = 0 rather than exp2(-Inf + Inf).
//
// Grouped heads with few queries (`pack` = QUERY_GROUP_SIZE when Sq <= 64): the heads that share a K / V head are
// stacked as rows of one query tile -- row r is query r % Sq of head r / Sq of the group -- so their common keys are
// read once per group instead of once per head.  Positions are no longer monotonic over a tile's rows; the tile-level
// decisions (which key tiles a query tile takes part in, which need the mask) use the group's first and last position.
//
// FLOPs (causal-exact): 4 * B * H * D * Sq*(Sq+1)/2 for Sq == Skv.
#include "fmha_common.h"
#include <stdlib.h>
#include <string.h>

#include "shared_scratch.h"

namespace {

using namespace mi;
using namespace mi::fmha;


typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kQB = 128;  // queries per workgroup
constexpr int kKV = 64;   // keys per LDS tile

// Row operand for P.V from the V tile stored [key][d] (d contiguous, `pitch` elements per
// key): lane l gets column d0 + l%32 and the 8 keys {4h+0..3, 8+4h+0..3} (h = l/32) of the
// 16-key chunk starting at `base` — exactly the keys whose scores the lane holds in
// accumulator registers 8c..8c+7 of a 32x32 S tile.
__device__ __forceinline__ s16x8 lds_read_v_frag(const unsigned short* base, int pitch, int lane) {
    const int g = lane >> 4, r = lane & 15;
    const unsigned short* p = base + (4 * (g >> 1) + (r >> 2)) * pitch + 16 * (g & 1) + 4 * (r & 3);
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 8 * pitch));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}


template <typename E, int D, bool CAUSAL>
__global__ __launch_bounds__(256) void fmha_fwd_kernel(const unsigned short* __restrict__ Q, Strides qs,
                                                       const unsigned short* __restrict__ K, Strides ks,
                                                       const unsigned short* __restrict__ V, Strides vs,
                                                       unsigned short* __restrict__ O, Strides os, int Sq,
                                                       int Skv, int H, int group, float scale2,
                                                       int input_pos, bool vec_ok, int nqb) {
    constexpr int CH = D / 8;             // 16-byte chunks per row
    constexpr int PER_T = kKV * CH / 256;  // chunks per thread per tile
    constexpr int KSTEPS = D / 16;
    constexpr int DT = D / 32;            // 32-wide d tiles of the output
    constexpr int VP = D + 8;             // V tile pitch (elements): rows 4 apart hit distinct banks
    __shared__ __attribute__((aligned(16))) unsigned short Ks[kKV * D];
    __shared__ __attribute__((aligned(16))) unsigned short Vs[kKV * VP];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hb = lane >> 5;
    // one-dimensional grid over (query block, batch * head), query blocks fastest
    const int bh = (int)(blockIdx.x / (unsigned)nqb), qbx = (int)(blockIdx.x % (unsigned)nqb);
    const int qb = CAUSAL ? nqb - 1 - qbx : qbx;  // heavy tiles first
    const int batch = bh / H, head = bh % H, kvh = head / group;
    const int q0 = qb * kQB, qw0 = q0 + wave * 32;
    Q += (int64_t)head * qs.s2 + (int64_t)batch * qs.s3;
    O += (int64_t)head * os.s2 + (int64_t)batch * os.s3;
    K += (int64_t)kvh * ks.s2 + (int64_t)batch * ks.s3;
    V += (int64_t)kvh * vs.s2 + (int64_t)batch * vs.s3;

    // Q fragments: lane holds query qw0 + lane%32, d = 16*s + 8*hb + 0..7 for every k-step s.
    const int my_q = qw0 + (lane & 31);
    s16x8 qf[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
        s16x8 v = {0};
        if (my_q < Sq) {
            const unsigned short* p = Q + (int64_t)my_q * qs.s1 + 16 * s + 8 * hb;
            if (vec_ok) v = *reinterpret_cast<const s16x8*>(p);
            else
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (short)p[e];
        }
        qf[s] = v;
    }

    int kv_end = Skv;
    if (CAUSAL) {
        const int lim = input_pos + q0 + kQB;  // one past the last query position of the group
        kv_end = lim < Skv ? lim : Skv;
        if (kv_end < 0) kv_end = 0;
    }
    const int ntiles = (kv_end + kKV - 1) / kKV;
    const int my_pos = input_pos + my_q;              // this lane's query position
    const int wave_last_pos = input_pos + qw0 + 31;   // last query position of the wave

    f32x16 o[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) o[t] = f32x16{0};
    float m_i = -INFINITY, l_i = 0.f;

    s16x8 kreg[PER_T], vreg[PER_T];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < PER_T; ++i) {
            const int id = tid + 256 * i, key = id / CH, c = id % CH;
            const int gk = t * kKV + key;
            s16x8 a = {0}, b = {0};
            if (gk < Skv) {
                const unsigned short* pk = K + (int64_t)gk * ks.s1 + 8 * c;
                const unsigned short* pv = V + (int64_t)gk * vs.s1 + 8 * c;
                if (vec_ok) {
                    a = *reinterpret_cast<const s16x8*>(pk);
                    b = *reinterpret_cast<const s16x8*>(pv);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) { a[e] = (short)pk[e]; b[e] = (short)pv[e]; }
                }
            }
            kreg[i] = a;
            vreg[i] = b;
        }
    };
    if (ntiles > 0) load_tile(0);

    for (int t = 0; t < ntiles; ++t) {
        __syncthreads();  // every wave has finished reading the previous tile
#pragma unroll
        for (int i = 0; i < PER_T; ++i) {
            const int id = tid + 256 * i, key = id / CH, c = id % CH;
            *reinterpret_cast<s16x8*>(&Ks[key * D + 8 * (c ^ (key & 7))]) = kreg[i];
            *reinterpret_cast<s16x8*>(&Vs[key * VP + 8 * c]) = vreg[i];
        }
        __syncthreads();
        if (t + 1 < ntiles) load_tile(t + 1);  // in flight while this tile is computed

        const int kv0 = t * kKV;
        if (CAUSAL && kv0 > wave_last_pos) continue;  // tile wholly above this wave's queries

        // ---- S^T = K . Q ---------------------------------------------------------------
        f32x16 s[2] = {f32x16{0}, f32x16{0}};
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int key = 32 * kt + (lane & 31);
#pragma unroll
            for (int st = 0; st < KSTEPS; ++st) {
                const int c = 2 * st + hb;
                s16x8 kf = *reinterpret_cast<const s16x8*>(&Ks[key * D + 8 * (c ^ (key & 7))]);
                s[kt] = E::mfma32(kf, qf[st], s[kt]);
            }
        }
        // ---- mask: causal diagonal and ragged KV tail -------------------------------------
        const bool need_mask = (CAUSAL && kv0 + kKV - 1 > input_pos + qw0) || (kv0 + kKV > Skv);
        if (need_mask) {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kv0 + 32 * kt + 8 * (r >> 2) + 4 * hb + (r & 3);
                    const bool ok = key < Skv && (!CAUSAL || key <= my_pos);
                    s[kt][r] = ok ? s[kt][r] : -INFINITY;
                }
        }
        // ---- online softmax (exp2 domain) ----------------------------------------------------
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kt][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_i, mx * scale2);
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
        float rs = 0.f;
        s16x8 pf[2][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(s[kt][r] * scale2 - m_new);
                rs += p;
                pf[kt][r >> 3][r & 7] = E::cvt(p);
            }
        rs += __shfl_xor(rs, 32, 64);
        l_i = l_i * alpha + rs;
        m_i = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
        // ---- O^T += V . P ------------------------------------------------------------------------
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    s16x8 vf = lds_read_v_frag(&Vs[(32 * kt + 16 * c) * VP + 32 * dt], VP, lane);
                    o[dt] = E::mfma32(vf, pf[kt][c], o[dt]);
                }
    }

    // ---- epilogue: O / l (approximate reciprocal, fmha.jl:132-134), round, store -------------
    if (my_q < Sq) {
        const float inv = __builtin_amdgcn_rcpf(l_i);
        unsigned short* op = O + (int64_t)my_q * os.s1;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                s16x4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = E::cvt(o[dt][4 * g + e] * inv);
                unsigned short* dst = op + 32 * dt + 8 * g + 4 * hb;
                if (vec_ok) *reinterpret_cast<s16x4*>(dst) = w;
                else
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[e] = (unsigned short)w[e];
            }
    }
}

// ---- main kernel: direct global->LDS K/V tiles, double-buffered, 64 queries per wave ----------
// Used when every row is 16-byte aligned.  A workgroup owns 128 queries of one (batch, head):
// for D = 64 two waves of 64 queries (two 32-query MFMA column tiles each, so every K / V
// fragment read from LDS feeds two MFMAs), for D = 128 four waves of 32 queries.  K and V tiles
// of 64 keys travel global -> LDS with global_load_lds (no staging registers) into two stages;
// the transfer of tile t+1 is issued right after the barrier that publishes tile t.
//   K tile [key][d]: 16-byte chunk c of row `key` at position c ^ ksw(key).  A 16-byte fragment read is served a
//     quarter-wave (16 consecutive keys) at a time and has to spread those over all 64 banks: with rows of 128 bytes
//     (D = 64) a row covers half the banks and two neighbouring keys differ in the half, so ksw = (key >> 1) & 7
//     gives the eight key pairs eight different chunk positions; with rows of 256 bytes (D = 128) every row starts
//     on bank 0 and ksw = key & 15 gives the sixteen keys sixteen positions.  (key & 7 put keys k and k + 8 of a
//     quarter-wave on the same banks: two passes per read.)
//   V tile [key][d]: chunk c at position c ^ ((D/32) * (key & 3)), which spreads the 4 rows x 32
//     bytes of a transpose-read group over distinct banks.
// Softmax bookkeeping per lane: running max m (shared by lanes l and l^32 after one exchange
// per tile), running sum l of the lane's own half of the keys (the halves are added once at
// the end), taken over the scores AFTER rounding to the storage type, i.e. over exactly the
// weights that multiply V.  The accumulator is rescaled only on tiles where some row's max
// actually rose.  Workgroups are numbered so that all query tiles of one (batch, head) run
// on the same XCD and share its K/V in that XCD's L2.

template <int D>
__device__ __forceinline__ int ksw(int key) {
    return D == 64 ? (key >> 1) & 7 : key & 15;
}

// AUX: the instruction's cache policy bits (0 = default, 2 = non-temporal: the line is the first to leave the L2 and
// takes no room in the memory-side cache).
template <int AUX = 0>
__device__ __forceinline__ void gload_lds16(const void* g, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, AUX);
}

template <int D, int NW>
struct DmaLane {
    static constexpr int TPW = (D / 8) / NW;  // 1 KB transfers per wave per tile, for K and for V
    unsigned koff[TPW], voff[TPW];            // byte offsets of the lane's chunk, relative to the tile's first key
};

template <typename E, int D, int JT, bool CAUSAL>
struct FmhaDma {
    static constexpr int NW = 4 / JT;          // waves per workgroup (128 queries)
    static constexpr int KSTEPS = D / 16, DT = D / 32, CH = D / 8;
    static constexpr int TPW = (D / 8) / NW;
    static constexpr int TILE = kKV * D;       // elements per K or V stage

    struct State {
        s16x8 qf[JT][KSTEPS];
        f32x16 o[JT][DT];
        float m[JT], l[JT];
        unsigned kfo[KSTEPS];  // K fragment element offsets per k-step (+ 32*kt*D)
        unsigned vfo[DT];      // V fragment element offsets per d tile (+ (32*kt + 16*c)*D, + 8*D for the high half)
        int my_pos[JT];     // position of this lane's query in column tile j
        int first_pos[JT];  // position of the first query of column tile j
    };

    template <int AUX>
    static __device__ __forceinline__ void issue_as(const char* Kg, const char* Vg, unsigned short* Ks,
                                                    unsigned short* Vs, int wave, const DmaLane<D, NW>& dl) {
#pragma unroll
        for (int i = 0; i < TPW; ++i) gload_lds16<AUX>(Kg + dl.koff[i], Ks + (wave + NW * i) * 512);
#pragma unroll
        for (int i = 0; i < TPW; ++i) gload_lds16<AUX>(Vg + dl.voff[i], Vs + (wave + NW * i) * 512);
    }
    // stream: every key is read by this workgroup alone and the keys of the launch do not fit the memory-side cache
    // (a KV cache walked once per new token): non-temporal transfers (the host decides, see the launch).
    static __device__ __forceinline__ void issue(const char* Kg, const char* Vg, unsigned short* Ks,
                                                 unsigned short* Vs, int wave, const DmaLane<D, NW>& dl, bool stream) {
        if (stream) issue_as<2>(Kg, Vg, Ks, Vs, wave, dl);
        else issue_as<0>(Kg, Vg, Ks, Vs, wave, dl);
    }

    // JM: bit j set = column tile j takes part in this KV tile (a causal wave drops its early
    // query tile once the keys pass that tile's diagonal).
    template <int JM, bool SAFE = false>
    static __device__ __forceinline__ void compute(const unsigned short* Ks, const unsigned short* Vs, State& st,
                                                   int kv0, int Skv, float scale2, int lane) {
        const int hb = lane >> 5;
        // ---- S^T = K . Q ---------------------------------------------------------------
        f32x16 s[JT][2];
#pragma unroll
        for (int j = 0; j < JT; ++j) s[j][0] = s[j][1] = f32x16{0};
#define ACT(j) ((JM >> (j)) & 1)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                s16x8 kf = *reinterpret_cast<const s16x8*>(Ks + st.kfo[ks] + 32 * kt * D);
#pragma unroll
                for (int j = 0; j < JT; ++j)
                    if (ACT(j)) s[j][kt] = E::mfma32(kf, st.qf[j][ks], s[j][kt]);
            }
        // ---- mask (causal diagonal, ragged KV tail) ------------------------------------------
#pragma unroll
        for (int j = 0; j < JT; ++j) {
            if (!ACT(j)) continue;
            const bool need_mask = (CAUSAL && kv0 + kKV - 1 > st.first_pos[j]) || (kv0 + kKV > Skv);
            if (need_mask) {
                // last visible key, relative to this lane's first key of the tile
                int lim = Skv - 1;
                if (CAUSAL && st.my_pos[j] < lim) lim = st.my_pos[j];
                lim -= kv0 + 4 * hb;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        s[j][kt][r] = (32 * kt + 8 * (r >> 2) + (r & 3) <= lim) ? s[j][kt][r] : -INFINITY;
            }
        }
        // ---- online softmax ---------------------------------------------------------------------
        unsigned pf[JT][2][2][4];  // [j][kt][16-key chunk][4 dwords = 8 packed values]
#pragma unroll
        for (int j = 0; j < JT; ++j) {
            if (!ACT(j)) continue;
            float mx = fmaxf(s[j][0][0], s[j][1][0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s[j][0][r]), s[j][1][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(st.m[j], mx * scale2);
            if (__any(m_new > st.m[j])) {  // some row's max rose: rescale the wave's accumulators
                // (SAFE: a row that has not seen a key yet keeps l = 0 and o = 0)
                const float alpha = __builtin_amdgcn_exp2f(st.m[j] - (SAFE && m_new == -INFINITY ? 0.f : m_new));
                st.l[j] *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) st.o[j][dt][r] *= alpha;
                st.m[j] = m_new;
            }
            const float mj = SAFE && st.m[j] == -INFINITY ? 0.f : st.m[j];
            float lsum = st.l[j];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(s[j][kt][r] * scale2 - mj);
                    const float p1 = __builtin_amdgcn_exp2f(s[j][kt][r + 1] * scale2 - mj);
                    const unsigned pk = Pack<E>::pack(p0, p1);
                    lsum = Pack<E>::sum2(pk, p0, p1, lsum);
                    pf[j][kt][r >> 3][(r & 7) >> 1] = pk;
                }
            st.l[j] = lsum;
        }
        // ---- O^T += V . P ------------------------------------------------------------------------
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const unsigned short* p = Vs + st.vfo[dt] + (32 * kt + 16 * c) * D;
                    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
                    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 8 * D));
                    s16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                    for (int j = 0; j < JT; ++j) {
                        if (!ACT(j)) continue;
                        u32x4 pw = {pf[j][kt][c][0], pf[j][kt][c][1], pf[j][kt][c][2], pf[j][kt][c][3]};
                        st.o[j][dt] = E::mfma32(vf, __builtin_bit_cast(s16x8, pw), st.o[j][dt]);
                    }
                }
#undef ACT
    }
};

__device__ __forceinline__ void tile_barrier() {
    // own LDS reads done, own transfers landed; gfx9 s_waitcnt encoding of vmcnt(0) lgkmcnt(0)
    __builtin_amdgcn_s_waitcnt(0x0070);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Query tiles of 32 are dealt to the waves as follows.  Non-causal: wave w of workgroup qb
// takes the JT adjacent tiles starting at JT*(NW*qb + w).  Causal (JT == 2): the work of a
// tile grows with its index, so a wave takes one early and one late tile, u and NT-1-u with
// u = 2*qb + w; every wave then has the same number of MFMAs, and the two waves of a workgroup
// need the same KV range.  The early tile simply drops out of the KV loop after its diagonal.
constexpr int kFuseParts = 8;      // most parts that the last-arriving part adds up itself
constexpr int kFuseRows = 64;      // most rows per (batch, head) for that
constexpr int kFusePairs = 65536;  // most (query block, batch * head) pairs for that
constexpr int kPartPad = 4;   // a part's row: D accumulator values, running maximum, row sum, two unused (16-byte rows)

template <typename E, int D, int JT, bool CAUSAL, bool SPLIT = false>
__global__ __launch_bounds__(128 * 2 / JT) __attribute__((amdgpu_waves_per_eu(2, 2))) void fmha_fwd_dma_kernel(
    const unsigned short* __restrict__ Q, Strides qs, const unsigned short* __restrict__ K, Strides ks,
    const unsigned short* __restrict__ V, Strides vs, unsigned short* __restrict__ O, Strides os, int Sq, int Skv,
    int H, int group, float scale2, int input_pos, int nqb, int nbh, int pack, int kv_stream, int nsplit = 1,
    float* __restrict__ part = nullptr, int* __restrict__ arrivals = nullptr) {
    using F = FmhaDma<E, D, JT, CAUSAL>;
    constexpr int NW = F::NW, KSTEPS = F::KSTEPS, DT = F::DT, CH = F::CH, TPW = F::TPW;
    constexpr bool PAIRED = CAUSAL && JT == 2;
    __shared__ __attribute__((aligned(1024))) unsigned short Ks0[F::TILE], Ks1[F::TILE], Vs0[F::TILE], Vs1[F::TILE];

    const int tid = threadIdx.x, lane = tid & 63, hb = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup -> (query block, batch*head): ids congruent mod 8 share an XCD; give each XCD
    // whole (batch, head) pairs so their K/V stay in that XCD's L2.  Low block index = most work.
    int qb, bh, sp = 0;
    {
        int L = blockIdx.x;
        if (SPLIT) {   // the parts of one (query block, batch * head) are nqb * nbh workgroup ids apart
            sp = L / (nqb * nbh);
            L -= sp * (nqb * nbh);
        }
        if (nbh % 8 == 0) {
            const int idx = L >> 3;
            bh = (L & 7) + 8 * (idx / nqb);
            qb = idx % nqb;
        } else {
            bh = L / nqb;
            qb = L % nqb;
        }
        if (CAUSAL && !PAIRED) qb = nqb - 1 - qb;
    }
    // (pack > 1: bh counts (batch, K / V head) pairs, H is their number per batch, and a row carries its head)
    const int batch = bh / H, hrem = bh % H;
    const int head = pack > 1 ? hrem * group : hrem, kvh = pack > 1 ? hrem : hrem / group;
    const int R = Sq * pack;   // query rows of this (batch, head) or (batch, head group)
    Q += (int64_t)head * qs.s2 + (int64_t)batch * qs.s3;
    if (!SPLIT) O += (int64_t)head * os.s2 + (int64_t)batch * os.s3;
    const char* Kg = (const char*)(K + (int64_t)kvh * ks.s2 + (int64_t)batch * ks.s3);
    const char* Vg = (const char*)(V + (int64_t)kvh * vs.s2 + (int64_t)batch * vs.s3);

    const int NT = (R + 31) / 32;  // query tiles of 32
    int tq[JT];                     // this wave's query tiles (wave-uniform); -1 = none
    int wg_last_tile;               // highest query tile of the workgroup (bounds the causal KV loop)
    if (PAIRED) {
        const int u = 2 * qb + wave;
        const int hi = NT - 1 - u;
        tq[0] = (u < hi) ? u : -1;
        tq[JT - 1] = (u <= hi) ? hi : -1;
        wg_last_tile = NT - 1 - 2 * qb;
    } else {
#pragma unroll
        for (int j = 0; j < JT; ++j) {
            const int t = JT * (NW * qb + wave) + j;
            tq[j] = t < NT ? t : -1;
        }
        wg_last_tile = JT * NW * (qb + 1) - 1;
        if (wg_last_tile > NT - 1) wg_last_tile = NT - 1;
    }

    typename F::State st;
    int my_q[JT], last_pos[JT];   // my_q: the lane's row, R = none
    int64_t q_off[JT], o_off[JT];  // element offsets of the row in Q and in Out
#pragma unroll
    for (int j = 0; j < JT; ++j) {
        my_q[j] = tq[j] >= 0 ? 32 * tq[j] + (lane & 31) : R;
        int qi = my_q[j], hq = 0;   // query index and head within the group
        if (pack > 1) {
            hq = my_q[j] / Sq;
            qi = my_q[j] - hq * Sq;
        }
        q_off[j] = (int64_t)qi * qs.s1 + (int64_t)hq * qs.s2;
        o_off[j] = (int64_t)qi * os.s1 + (int64_t)hq * os.s2;
        st.my_pos[j] = input_pos + qi;
        st.first_pos[j] = pack > 1 ? input_pos : input_pos + 32 * tq[j];
        last_pos[j] = tq[j] < 0 ? -1 : pack > 1 ? input_pos + Sq - 1 : st.first_pos[j] + 31;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            s16x8 v = {0};
            if (my_q[j] < R) v = *reinterpret_cast<const s16x8*>(Q + q_off[j] + 16 * s + 8 * hb);
            st.qf[j][s] = v;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) st.o[j][dt] = f32x16{0};
        st.m[j] = -INFINITY;
        st.l[j] = 0.f;
    }
    {
        const int key = lane & 31;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) st.kfo[s] = key * D + 8 * ((2 * s + hb) ^ ksw<D>(key));
        const int g = lane >> 4, r = lane & 15;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int row = 4 * (g >> 1) + (r >> 2);
            const int col = 32 * dt + 16 * (g & 1) + 4 * (r & 3);
            st.vfo[dt] = row * D + 8 * ((col >> 3) ^ ((D / 32) * (r >> 2))) + (col & 7);
        }
    }
    DmaLane<D, NW> dl;
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        const int t = wave + NW * i;  // transfer index: rows (512/D)*t ... of the tile
        const int key = (512 / D) * t + lane / CH, pos = lane % CH;
        dl.koff[i] = (unsigned)(((int64_t)key * ks.s1 + 8 * (pos ^ ksw<D>(key))) * 2);
        dl.voff[i] = (unsigned)(((int64_t)key * vs.s1 + 8 * (pos ^ ((D / 32) * (key & 3)))) * 2);
    }

    int kv_end = Skv;
    if (CAUSAL) {
        const int lim = input_pos + (pack > 1 ? Sq : 32 * (wg_last_tile + 1));  // one past the workgroup's last query position
        kv_end = lim < Skv ? lim : Skv;
        if (kv_end < 0) kv_end = 0;
    }
    const int ntiles = (kv_end + kKV - 1) / kKV;
    int t_begin = 0, t_end = ntiles;
    if (SPLIT) {
        t_begin = (int)((int64_t)ntiles * sp / nsplit);
        t_end = (int)((int64_t)ntiles * (sp + 1) / nsplit);
    }
    const int64_t k_tile_bytes = (int64_t)kKV * ks.s1 * 2, v_tile_bytes = (int64_t)kKV * vs.s1 * 2;

    // Rows past the end of K / V in the last tile are never dereferenced: their lanes re-read
    // the last valid row (the masked scores make the values irrelevant, and finite).
    auto issue_tile = [&](int t, unsigned short* Ksx, unsigned short* Vsx) {
        if ((t + 1) * kKV <= Skv) {
            F::issue(Kg + t * k_tile_bytes, Vg + t * v_tile_bytes, Ksx, Vsx, wave, dl, kv_stream != 0);
        } else {
            DmaLane<D, NW> cl;
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                const int tr = wave + NW * i;
                int key = (512 / D) * tr + lane / CH;
                const int pos = lane % CH;
                const int swk = ksw<D>(key), swv = key & 3;
                if (t * kKV + key >= Skv) key = Skv - 1 - t * kKV;
                cl.koff[i] = (unsigned)(((int64_t)key * ks.s1 + 8 * (pos ^ swk)) * 2);
                cl.voff[i] = (unsigned)(((int64_t)key * vs.s1 + 8 * (pos ^ ((D / 32) * swv))) * 2);
            }
            F::issue(Kg + t * k_tile_bytes, Vg + t * v_tile_bytes, Ksx, Vsx, wave, cl, kv_stream != 0);
        }
    };
    // Which of the wave's column tiles still see keys of the tile starting at kv0.
    auto run_tile = [&](const unsigned short* Ksx, const unsigned short* Vsx, int kv0) {
        if (JT == 2) {
            const bool a0 = tq[0] >= 0 && (!CAUSAL || kv0 <= last_pos[0]);
            const bool a1 = tq[JT - 1] >= 0 && (!CAUSAL || kv0 <= last_pos[JT - 1]);
            if (a0 && a1) F::template compute<3, SPLIT>(Ksx, Vsx, st, kv0, Skv, scale2, lane);
            else if (a1) F::template compute<2, SPLIT>(Ksx, Vsx, st, kv0, Skv, scale2, lane);
            else if (a0) F::template compute<1, SPLIT>(Ksx, Vsx, st, kv0, Skv, scale2, lane);
        } else {
            if (tq[0] >= 0 && (!CAUSAL || kv0 <= last_pos[0])) F::template compute<1, SPLIT>(Ksx, Vsx, st, kv0, Skv, scale2, lane);
        }
    };

    if (t_begin < t_end) issue_tile(t_begin, Ks0, Vs0);
    for (int t = t_begin; t < t_end; t += 2) {
        tile_barrier();  // tile t has landed for every wave; every wave is done with the other stage
        if (t + 1 < t_end) issue_tile(t + 1, Ks1, Vs1);
        run_tile(Ks0, Vs0, t * kKV);
        if (t + 1 < t_end) {
            tile_barrier();
            if (t + 2 < t_end) issue_tile(t + 2, Ks0, Vs0);
            run_tile(Ks1, Vs1, (t + 1) * kKV);
        }
    }

    if constexpr (SPLIT) {
        // ---- this part's unnormalised accumulator, maximum and row sum -> scratch ---------------
#pragma unroll
        for (int j = 0; j < JT; ++j) {
            const float l_tot = st.l[j] + __shfl_xor(st.l[j], 32, 64);
            if (my_q[j] < R) {
                float* pr = part + (((int64_t)sp * nbh + bh) * R + my_q[j]) * (D + kPartPad);
                if (arrivals) {
                    // (device-scope stores: written through to where the part that adds them up, on whatever XCD it
                    // runs, reads them from -- no cache maintenance is needed on either side)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int g = 0; g < 4; ++g)
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                __hip_atomic_store(pr + 32 * dt + 8 * g + 4 * hb + e, st.o[j][dt][4 * g + e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (hb == 0) {
                        __hip_atomic_store(pr + D, st.m[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(pr + D + 1, l_tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    continue;
                }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        f32x4 w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = st.o[j][dt][4 * g + e];
                        *reinterpret_cast<f32x4*>(pr + 32 * dt + 8 * g + 4 * hb) = w;
                    }
                if (hb == 0) *reinterpret_cast<f32x2*>(pr + D) = f32x2{st.m[j], l_tot};
            }
        }
        if (!arrivals) return;   // the parts are added by a launch of their own
        // ---- the part that arrives last adds the parts (few rows and few parts: decode) ----------
        // Every part writes its results with device-scope stores, waits until they have been performed, and then
        // takes a ticket of its (query block, batch * head); the holder of the last ticket knows that all the others
        // have published theirs.  The counter is left at zero for the next launch.  (Fences are avoided on purpose: a
        // device-scope fence writes back and invalidates the whole L2 of the XCD, and one per workgroup made the
        // launch twice as long.)
        __shared__ int s_last;
        const int pair = (int)blockIdx.x - sp * (nqb * nbh);
        __builtin_amdgcn_s_waitcnt(0x0070);   // this wave's stores have been performed (vmcnt(0), lgkmcnt(0))
        __syncthreads();                      // ... and so have the other waves'
        if (tid == 0) {
            const int ticket = __hip_atomic_fetch_add(arrivals + pair, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = ticket == nsplit - 1;
            if (s_last) __hip_atomic_store(arrivals + pair, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!s_last) return;
        {
            constexpr int CPRW = D / 4, NTH = 128 * 2 / JT, RPP = NTH / CPRW;   // threads per row, rows per pass
            const int c = tid % CPRW;
            const int64_t part_stride = (int64_t)nbh * R * (D + kPartPad);
            for (int row = tid / CPRW; row < R; row += RPP) {
                const float* p0 = part + ((int64_t)bh * R + row) * (D + kPartPad);
                // one pass with every part's loads in flight together (at most kFuseParts parts); device-scope loads
                f32x2 ml[kFuseParts];
                f32x4 o[kFuseParts];
#pragma unroll
                for (int q = 0; q < kFuseParts; ++q) {
                    const float* pr = p0 + (q < nsplit ? q : 0) * part_stride;
#pragma unroll
                    for (int e = 0; e < 2; ++e) ml[q][e] = __hip_atomic_load(pr + D + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[q][e] = __hip_atomic_load(pr + 4 * c + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                float m = -INFINITY;
#pragma unroll
                for (int q = 0; q < kFuseParts; ++q) m = q < nsplit ? fmaxf(m, ml[q][0]) : m;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                float l = 0.f;
#pragma unroll
                for (int q = 0; q < kFuseParts; ++q) {
                    // (a part without a visible key for this row is left out, as in the combine kernel: same sums)
                    const bool seen = q < nsplit && ml[q][0] != -INFINITY;
                    const float w = seen ? __builtin_amdgcn_exp2f(ml[q][0] - m) : 0.f;
                    l += seen ? w * ml[q][1] : 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] += seen ? w * o[q][e] : 0.f;
                }
                const float inv = __builtin_amdgcn_rcpf(l);
                const int hq = row / Sq, q = row - hq * Sq;   // head within a stacked group, query
                s16x4 out;
#pragma unroll
                for (int e = 0; e < 4; ++e) out[e] = E::cvt(acc[e] * inv);
                *reinterpret_cast<s16x4*>(O + (int64_t)(head + hq) * os.s2 + (int64_t)batch * os.s3 + (int64_t)q * os.s1 + 4 * c) = out;
            }
        }
        return;
    }

    // ---- epilogue: add the two half-row sums, O / l (approximate reciprocal), round, store -----
#pragma unroll
    for (int j = 0; j < JT; ++j) {
        const float l_tot = st.l[j] + __shfl_xor(st.l[j], 32, 64);
        if (my_q[j] < R) {
            const float inv = __builtin_amdgcn_rcpf(l_tot);
            unsigned short* op = O + o_off[j];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    s16x4 w;
#pragma unroll
                    for (int e = 0; e < 4; ++e) w[e] = E::cvt(st.o[j][dt][4 * g + e] * inv);
                    *reinterpret_cast<s16x4*>(op + 32 * dt + 8 * g + 4 * hb) = w;
                }
        }
    }
}

// Adds the parts of a split launch.  Four adjacent channels of one query row belong to PL threads, which take the
// parts pl, pl + PL, ... and meet in LDS (with one thread per row and 64 parts the two dependent passes over the
// parts took 49 us for 32 rows).
template <typename E, int D, int PL>
__global__ __launch_bounds__(256) void fmha_combine_kernel(const float* __restrict__ part, int nsplit, int64_t rows,
                                                           unsigned short* __restrict__ O, Strides os, int Sq, int H,
                                                           int pack) {
    constexpr int CPRW = D / 4, TPR = CPRW * PL, RPB = 256 / TPR;
    static_assert(TPR <= 256 && 256 % TPR == 0, "the threads of a row stay inside the workgroup");
    __shared__ float s_max[PL > 1 ? 256 : 1];
    __shared__ float s_acc[PL > 1 ? 256 : 1][5];
    const int tid = threadIdx.x, c = tid % CPRW, pl = (tid / CPRW) % PL, rl = tid / TPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + rl;
    const bool live = row < rows;
    const float* p0 = part + (live ? row : 0) * (D + kPartPad);
    const int64_t part_stride = rows * (D + kPartPad);
    float m = -INFINITY;
    if (live) {
#pragma unroll 4
        for (int sp = pl; sp < nsplit; sp += PL) m = fmaxf(m, p0[sp * part_stride + D]);
    }
    if (PL > 1) {
        s_max[tid] = m;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PL; ++i) m = fmaxf(m, s_max[rl * TPR + i * CPRW + c]);
    }
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float l = 0.f;
    if (live) {
        // (a part without a visible key for this row is left out by selects, not by a branch, so that the loads of
        // the parts can all be in flight together)
#pragma unroll 4
        for (int sp = pl; sp < nsplit; sp += PL) {
            const float* pr = p0 + sp * part_stride;
            const f32x2 ml = *reinterpret_cast<const f32x2*>(pr + D);
            const f32x4 o = *reinterpret_cast<const f32x4*>(pr + 4 * c);
            const bool seen = ml[0] != -INFINITY;
            const float w = seen ? __builtin_amdgcn_exp2f(ml[0] - m) : 0.f;
            l += seen ? w * ml[1] : 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += seen ? w * o[e] : 0.f;
        }
    }
    if (PL > 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s_acc[tid][e] = acc[e];
        s_acc[tid][4] = l;
        __syncthreads();
        if (pl != 0) return;
#pragma unroll
        for (int i = 1; i < PL; ++i) {
            const float* o = s_acc[rl * TPR + i * CPRW + c];
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += o[e];
            l += o[4];
        }
    }
    if (!live) return;
    const float inv = __builtin_amdgcn_rcpf(l);
    // a row is (query, head within the group when the group's heads are stacked, head or head group, batch)
    const int R = Sq * pack;
    const int64_t bh = row / R;
    const int r = (int)(row - bh * R), hq = r / Sq, q = r - hq * Sq;
    const int64_t batch = bh / H, head = (bh - batch * H) * pack + hq;
    s16x4 out;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = E::cvt(acc[e] * inv);
    *reinterpret_cast<s16x4*>(O + head * os.s2 + batch * os.s3 + (int64_t)q * os.s1 + 4 * c) = out;
}

// Scratch of the split launches (see shared_scratch.h for how its users are ordered).
constexpr int64_t kPartFloats = 16 * 1024 * 1024;   // 64 MiB
static __device__ __align__(256) float fmha_part_scratch[kPartFloats];
// Arrival counters of the parts of a (query block, batch * head) pair; zero between launches (the part that arrives
// last resets its counter).  Held under the same lease as the part array.
static __device__ __align__(256) int fmha_part_arrivals[kFusePairs];
SharedScratch g_part[16];

// Number of parts for the launch, 0 = no split.
int pick_parts(int64_t wgs, int64_t rows, int D, int Sq, int Skv, bool causal, int input_pos) {
    static const int force = [] { const char* e = getenv("MI_FMHA_SPLIT"); return e ? atoi(e) : -1; }();   // 0 = never, n = n parts
    if (force == 0 || wgs >= 1024) return 0;   // (four workgroups of two or four waves fill a CU)
    int64_t keys = Skv;   // keys the busiest workgroup walks
    if (causal && (int64_t)input_pos + Sq < keys) keys = (int64_t)input_pos + Sq;
    const int64_t tiles = (keys + kKV - 1) / kKV;
    // Measured, 8 x 16 heads: one query against 4096 keys 28 us with 512 workgroups in all, 33 us with 1024 (64 us unsplit);
    // 128 queries against 4096 keys 46 us with 1024, 64 us with 384 (104 us unsplit).
    const int64_t target = Sq <= 32 ? 512 : 1024;
    int64_t parts = force > 0 ? force : (target + wgs - 1) / wgs;
    if (parts > tiles / 4) parts = tiles / 4;                              // at least four tiles (256 keys) per part
    if (parts > 64) parts = 64;
    while (parts >= 2 && parts * rows * (D + kPartPad) > kPartFloats) --parts;
    return parts >= 2 ? (int)parts : 0;
}

bool vec16(const mi_tile_array* a) {
    return aligned(a->ptr, 16) && a->strides[1] % 8 == 0 && a->strides[2] % 8 == 0 && a->strides[3] % 8 == 0;
}

template <typename E, int D>
void launch(dim3 grid, hipStream_t s, bool causal, const mi_tile_array* Q, const mi_tile_array* K,
            const mi_tile_array* V, const mi_tile_array* O, int H, int group, float scale2, int input_pos,
            bool vec_ok) {
    Strides qs{Q->strides[1], Q->strides[2], Q->strides[3]}, ks{K->strides[1], K->strides[2], K->strides[3]},
        vs{V->strides[1], V->strides[2], V->strides[3]}, os{O->strides[1], O->strides[2], O->strides[3]};
    const int Sq = (int)Q->sizes[1], Skv = (int)K->sizes[1];
    if (vec_ok && K->strides[1] < (1 << 24) && V->strides[1] < (1 << 24)) {
        constexpr int JT = D == 64 ? 2 : 1;
        // few queries and grouped heads: the heads of a group are stacked in one query tile
        const int pack = group > 1 && Sq <= 64 ? group : 1;
        const int Hb = H / pack;                                   // heads, or head groups, per batch
        const int nqb = pack > 1 ? (Sq * pack + kQB - 1) / kQB : (int)grid.x, nbh = (int)grid.y / pack;
        dim3 g1((unsigned)(nqb * nbh)), blk(128 * 2 / JT);
        const int64_t rows = (int64_t)nbh * Sq * pack;
        // Keys that one query block walks alone and that are well beyond what the memory-side cache (256 MB) holds are
        // streamed.  Measured with the same buffers launch after launch, 16-bit keys of 64 elements: 134 MB 26.8 us
        // cached / 28.8 streamed, 268 MB 47.3 / 49.7, 537 MB 96.0 / 82.2 (5.6 -> 6.5 TB/s), 32 x 16 heads x 4096 keys
        // unsplit 91.8 / 78.0 (6.9 TB/s); 134 MB in six rotating sets 30.8 / 28.6.  A caller that knows its cache will not
        // be read again before it has left the memory-side cache anyway sets MI_FMHA_KV_STREAM = 1 (0 = never; read at
        // every call).
        const char* env_kv = getenv("MI_FMHA_KV_STREAM");
        const int64_t kv_bytes = 2 * (int64_t)(grid.y / group) * Skv * D * 2;
        const int kv_stream = nqb == 1 && (env_kv ? atoi(env_kv) != 0 : kv_bytes > (320ll << 20)) ? 1 : 0;
        if (const int parts = pick_parts((int64_t)nqb * nbh, rows, D, Sq, Skv, causal, input_pos)) {
            ScratchLease lease;   // ends behind the combine launch
            if (float* scratch = (float*)lease.acquire(g_part, HIP_SYMBOL(fmha_part_scratch), s)) {
                dim3 gs((unsigned)(nqb * nbh * parts));
                // Few rows and few parts (one new token per sequence): the part that arrives last adds the parts
                // itself, and the launch of the combine kernel (4 to 5 us behind a 23 us kernel) goes away.  The
                // arrival counters are a static array as well; its address is looked up under the lease.
                int* arrivals = nullptr;
                static const bool fuse_on = [] { const char* e = getenv("MI_FMHA_FUSE_COMBINE"); return !e || atoi(e) != 0; }();   // 0: always the combine kernel
                if (fuse_on && parts <= kFuseParts && (int64_t)Sq * pack <= kFuseRows && nqb == 1 && nbh <= kFusePairs) {
                    static int* arr_ptr[16];
                    int dev = 0;
                    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 16) {
                        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;   // (no lookup inside a capture: an eager call has to have made it)
                        if (!arr_ptr[dev] && hipStreamIsCapturing(s, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone &&
                            hipGetSymbolAddress((void**)&arr_ptr[dev], HIP_SYMBOL(fmha_part_arrivals)) != hipSuccess) {
                            arr_ptr[dev] = nullptr;
                            (void)hipGetLastError();
                        }
                        arrivals = arr_ptr[dev];
                    }
                }
                if (causal)
                    hipLaunchKernelGGL((fmha_fwd_dma_kernel<E, D, JT, true, true>), gs, blk, 0, s, (const unsigned short*)Q->ptr, qs,
                                       (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs,
                                       (unsigned short*)O->ptr, os, Sq, Skv, Hb, group, scale2, input_pos, nqb, nbh, pack, kv_stream, parts, scratch, arrivals);
                else
                    hipLaunchKernelGGL((fmha_fwd_dma_kernel<E, D, JT, false, true>), gs, blk, 0, s, (const unsigned short*)Q->ptr, qs,
                                       (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs,
                                       (unsigned short*)O->ptr, os, Sq, Skv, Hb, group, scale2, input_pos, nqb, nbh, pack, kv_stream, parts, scratch, arrivals);
                if (arrivals) {
                    set_variant(pack > 1 ? (D == 64 ? "fmha_dma_q128_kv64_d64_w64q_grouped_splitkv_fused" : "fmha_dma_q128_kv64_d128_w32q_grouped_splitkv_fused")
                                         : (D == 64 ? "fmha_dma_q128_kv64_d64_w64q_splitkv_fused" : "fmha_dma_q128_kv64_d128_w32q_splitkv_fused"));
                    return;
                }
                constexpr int PLMAX = 256 / (D / 4) < 16 ? 256 / (D / 4) : 16;
#define COMBINE(PL)                                                                                                              \
    hipLaunchKernelGGL((fmha_combine_kernel<E, D, PL>), dim3((unsigned)((rows * (D / 4) * PL + 255) / 256)), dim3(256), 0, s, scratch, \
                       parts, rows, (unsigned short*)O->ptr, os, Sq, Hb, pack)
                if (parts <= 4) COMBINE(1);
                else if (parts <= 16) COMBINE(4);
                else COMBINE(PLMAX);
#undef COMBINE
                set_variant(pack > 1 ? (D == 64 ? "fmha_dma_q128_kv64_d64_w64q_grouped_splitkv" : "fmha_dma_q128_kv64_d128_w32q_grouped_splitkv")
                                     : (D == 64 ? "fmha_dma_q128_kv64_d64_w64q_splitkv" : "fmha_dma_q128_kv64_d128_w32q_splitkv"));
                return;
            }
        }
        if (causal)
            hipLaunchKernelGGL((fmha_fwd_dma_kernel<E, D, JT, true>), g1, blk, 0, s, (const unsigned short*)Q->ptr, qs,
                               (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs,
                               (unsigned short*)O->ptr, os, Sq, Skv, Hb, group, scale2, input_pos, nqb, nbh, pack, kv_stream);
        else
            hipLaunchKernelGGL((fmha_fwd_dma_kernel<E, D, JT, false>), g1, blk, 0, s, (const unsigned short*)Q->ptr, qs,
                               (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs,
                               (unsigned short*)O->ptr, os, Sq, Skv, Hb, group, scale2, input_pos, nqb, nbh, pack, kv_stream);
        set_variant(pack > 1 ? (D == 64 ? "fmha_dma_q128_kv64_d64_w64q_grouped" : "fmha_dma_q128_kv64_d128_w32q_grouped")
                             : (D == 64 ? "fmha_dma_q128_kv64_d64_w64q" : "fmha_dma_q128_kv64_d128_w32q"));
        return;
    }
    const dim3 g2((unsigned)(grid.x * grid.y));
    if (causal)
        hipLaunchKernelGGL((fmha_fwd_kernel<E, D, true>), g2, dim3(256), 0, s, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs,
                           (unsigned short*)O->ptr, os, Sq, Skv, H, group, scale2, input_pos, vec_ok, (int)grid.x);
    else
        hipLaunchKernelGGL((fmha_fwd_kernel<E, D, false>), g2, dim3(256), 0, s, (const unsigned short*)Q->ptr, qs,
                           (const unsigned short*)K->ptr, ks, (const unsigned short*)V->ptr, vs,
                           (unsigned short*)O->ptr, os, Sq, Skv, H, group, scale2, input_pos, vec_ok, (int)grid.x);
    set_variant(D == 64 ? "fmha_regstage_q128_kv64_d64" : "fmha_regstage_q128_kv64_d128");
}

}  // namespace

extern "C" int mi_fmha_kernel(const mi_tile_array* Q, const mi_tile_array* K, const mi_tile_array* V,
                              const mi_tile_array* Out, float qk_scale, int32_t input_pos, int TILE_D, int H,
                              int TILE_M, int TILE_N, int QUERY_GROUP_SIZE, int CAUSAL, int EVEN_K, void* stream) {
    MI_CHECK(check_array(Q, 4));
    MI_CHECK(check_array(K, 4));
    MI_CHECK(check_array(V, 4));
    MI_CHECK(check_array(Out, 4));
    const int dt = Q->dtype;
    if (dt != MI_F16 && dt != MI_BF16) return MI_E_DTYPE;
    if (K->dtype != dt || V->dtype != dt || Out->dtype != dt) return MI_E_DTYPE;
    if (!is_pow2(TILE_D) || !is_pow2(TILE_M) || !is_pow2(TILE_N)) return MI_E_TILE;
    if (QUERY_GROUP_SIZE < 1 || H < 1) return MI_E_ARG;
    const int64_t D = Q->sizes[0], Sq = Q->sizes[1], Hq = Q->sizes[2], B = Q->sizes[3];
    const int64_t Skv = K->sizes[1], KVH = K->sizes[2];
    if (K->sizes[0] != D || V->sizes[0] != D || Out->sizes[0] != D || TILE_D != D) return MI_E_SHAPE;
    if (Hq != H || KVH * QUERY_GROUP_SIZE != H || V->sizes[1] != Skv || V->sizes[2] != KVH) return MI_E_SHAPE;
    if (K->sizes[3] != B || V->sizes[3] != B || Out->sizes[3] != B || Out->sizes[1] != Sq || Out->sizes[2] != H)
        return MI_E_SHAPE;
    if ((EVEN_K != 0) != (Skv % TILE_N == 0)) return MI_E_ARG;  // fmha.jl:153
    if (input_pos < 0) return MI_E_ARG;
    if (D != 64 && D != 128) return MI_E_UNSUPPORTED;
    for (const mi_tile_array* a : {Q, K, V, Out})
        if (a->strides[0] != 1) return MI_E_STRIDE;
    if (Sq > 0x3fffffff || Skv > 0x3fffffff) return MI_E_SHAPE;
    // the reference's grid is (cld(Sq, TILE_M), B * H) (fmha.jl:163-165), each below 2^24; the kernels here
    // use a one-dimensional grid over both
    if (cld(Sq, (int64_t)TILE_M) > MI_MAX_GRID_DIM || B * H > MI_MAX_GRID_DIM ||
        cld(Sq, (int64_t)kQB) * B * H > MI_MAX_GRID_DIM)   // (query block, head) pairs share one grid dimension
        return MI_E_GRID;
    if (Sq == 0 || B == 0) return MI_OK;
    if (Skv == 0) return MI_E_SHAPE;
    const bool vec_ok = vec16(Q) && vec16(K) && vec16(V) && vec16(Out);
    const float scale2 = qk_scale * 1.4426950408889634f;  // fmha.jl:41: fold 1/log(2) for exp2
    dim3 grid((unsigned)cld(Sq, (int64_t)kQB), (unsigned)(B * H));
    hipStream_t s = (hipStream_t)stream;
    // A decode offset that already exposes every key to the first query makes the mask a no-op.
    const bool causal = CAUSAL != 0 && input_pos < Skv - 1;
    {
        // MI_FMHA_KERNEL=dma keeps the double-buffered kernel below for every shape (comparison runs).
        static const bool no_pipe = [] {
            const char* e = getenv("MI_FMHA_KERNEL");
            return e && strcmp(e, "dma") == 0;
        }();
        fmha::Problem pr{Q, K, V, Out, H, QUERY_GROUP_SIZE, scale2, input_pos, causal, dt == MI_BF16};
        if (!no_pipe && fmha::pipe_applicable(pr)) {
            fmha::pipe_launch(pr, s);
            return launch_status();
        }
    }
    if (dt == MI_F16) {
        if (D == 64) launch<F16, 64>(grid, s, causal, Q, K, V, Out, H, QUERY_GROUP_SIZE, scale2, input_pos, vec_ok);
        else launch<F16, 128>(grid, s, causal, Q, K, V, Out, H, QUERY_GROUP_SIZE, scale2, input_pos, vec_ok);
    } else {
        if (D == 64) launch<BF16, 64>(grid, s, causal, Q, K, V, Out, H, QUERY_GROUP_SIZE, scale2, input_pos, vec_ok);
        else launch<BF16, 128>(grid, s, causal, Q, K, V, Out, H, QUERY_GROUP_SIZE, scale2, input_pos, vec_ok);
    }
    return launch_status();
}
