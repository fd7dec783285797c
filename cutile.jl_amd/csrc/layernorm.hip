// LayerNorm forward and backward: stand-ins for layer_norm_fwd (examples/layernorm.jl:27-68),
// layer_norm_bwd_dx_partial_dwdb (:118-171) and layer_norm_bwd_dwdb (:186-205).
//
// Arrays are (N, M) fp32 with the normalised dimension N contiguous; "row" below means the
// N contiguous elements that belong to one m.
//
// Forward: one workgroup per row, the row held in registers, so X is read once and Y
// written once (algorithmic traffic 2*M*N*4 + small vectors) instead of the reference's
// three passes.  Mean and variance are still two separate passes over the cached row
// (mean first, then the sum of squared deviations), biased variance, rstd = 1/sqrt(var+eps).
//
// Backward: workgroup (g, s) walks the rows m with m mod GROUP_SIZE_M == g in S interleaved
// splits, keeps the row's X and DY in registers (read once), writes DX, and accumulates its
// rows' dW/dB contributions in registers.  At the end it adds them into slot g of the
// caller's zero-filled DW/DB partial buffers: a plain read-add-write when one workgroup
// owns the slot (S == 1), device-scope float atomics otherwise.  No spin-lock: workgroups of
// one grid have no forward-progress guarantee relative to each other on this hardware.
#include "common.h"
#include <type_traits>
#include <math.h>
#include <stdlib.h>

namespace {

using namespace mi;

typedef float f32x4 __attribute__((ext_vector_type(4)));

// w * dy as a value of its own.  The backward kernels form this product twice, once for the row sums and once for dX;
// left to the compiler, the second one may be fused into the subtraction that follows (an unrounded product minus a
// sum of rounded ones), and a row of one element then gets the product's rounding error times rstd instead of 0.
__device__ __forceinline__ float rounded_product(float a, float b) {
    float p = a * b;
    asm volatile("" : "+v"(p));
    return p;
}

// Block all-reduce (sum) of two floats at once.
template <int NWAVES>
__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
    a = wave_reduce(a, SumOp{});
    b = wave_reduce(b, SumOp{});
    if constexpr (NWAVES == 1) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { red[wave] = a; red[NWAVES + wave] = b; }
    __syncthreads();
    float ra = (lane < NWAVES) ? red[lane] : 0.f;
    float rb = (lane < NWAVES) ? red[NWAVES + lane] : 0.f;
#pragma unroll
    for (int off = NWAVES / 2; off >= 1; off >>= 1) {
        ra += __shfl_xor(ra, off, 64);
        rb += __shfl_xor(rb, off, 64);
    }
    a = __shfl(ra, 0, 64);
    b = __shfl(rb, 0, 64);
    __syncthreads();
}

// Load / store the lane's VPT 4-element groups of one row.  Out-of-range elements load 0.
// ALIGNED: 16-byte aligned rows of a multiple of 4 elements, so a group is wholly inside the row or
// wholly outside and there is no element-wise tail (whose second code path would keep twice the
// registers alive).  Otherwise the groups inside the row move as unaligned vectors and the one across its end
// element by element.
template <int BLOCK, int VPT, bool ALIGNED, bool NT>
__device__ __forceinline__ void load_row(const float* __restrict__ p, int N, float (&r)[VPT][4]) {
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const int e0 = (threadIdx.x + v * BLOCK) * 4;
        if constexpr (ALIGNED) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (e0 < N) t = ld_global<NT>(reinterpret_cast<const f32x4*>(p + e0));
#pragma unroll
            for (int q = 0; q < 4; ++q) r[v][q] = t[q];
        } else if (e0 + 4 <= N) {
            // rows that start anywhere: global memory takes a 16-byte access at a 4-byte aligned address, in one
            // instruction (element by element these rows moved at a third of the aligned rate)
            f32x4 t;
            __builtin_memcpy(&t, p + e0, sizeof(t));
#pragma unroll
            for (int q = 0; q < 4; ++q) r[v][q] = t[q];
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) r[v][q] = (e0 + q < N) ? p[e0 + q] : 0.f;
        }
    }
}
template <int BLOCK, int VPT, bool ALIGNED, bool NT>
__device__ __forceinline__ void store_row(float* __restrict__ p, int N, const float (&r)[VPT][4]) {
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const int e0 = (threadIdx.x + v * BLOCK) * 4;
        if constexpr (ALIGNED) {
            f32x4 t;
#pragma unroll
            for (int q = 0; q < 4; ++q) t[q] = r[v][q];
            if (e0 < N) st_global<true>(t, reinterpret_cast<f32x4*>(p + e0));
        } else if (e0 + 4 <= N) {
            f32x4 t;
#pragma unroll
            for (int q = 0; q < 4; ++q) t[q] = r[v][q];
            __builtin_memcpy(p + e0, &t, sizeof(t));
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (e0 + q < N) p[e0 + q] = r[v][q];
        }
    }
}

// ---- forward ---------------------------------------------------------------------------
template <int BLOCK, int VPT, bool ALIGNED, bool STREAM>
__global__ __launch_bounds__(BLOCK) void ln_fwd_kernel(const float* __restrict__ X, int64_t ldx,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ B,
                                                       float* __restrict__ Y, int64_t ldy,
                                                       float* __restrict__ Mean,
                                                       float* __restrict__ Rstd, float eps, int N,
                                                       int64_t M) {
    constexpr int NW = BLOCK / 64;
    __shared__ float red[NW > 1 ? NW : 1];
    const float invN = 1.0f / (float)N;
    for (int64_t m = blockIdx.x; m < M; m += gridDim.x) {
        // (eight vectors per lane: W and B are asked for after the reductions, half a row at a time -- with the row
        // they would be 96 registers of a lane's 128)
        constexpr bool LATE_WB = VPT >= 8;
        constexpr int WV = LATE_WB ? VPT / 2 : VPT;
        float x[VPT][4], w[WV][4], b[WV][4];
        load_row<BLOCK, VPT, ALIGNED, STREAM>(X + m * ldx, N, x);
        // W and B come from L2; asked for now, they arrive while the row is being reduced
        if constexpr (!LATE_WB) {
            load_row<BLOCK, VPT, ALIGNED, false>(W, N, w);
            load_row<BLOCK, VPT, ALIGNED, false>(B, N, b);
        }
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) s += x[v][q];
        const float mean = block_reduce<NW>(s, red, SumOp{}, 0.f) / (float)N;
        float sq = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int e0 = (threadIdx.x + v * BLOCK) * 4;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float d = (e0 + q < N) ? x[v][q] - mean : 0.f;
                sq += d * d;
            }
        }
        const float var = block_reduce<NW>(sq, red, SumOp{}, 0.f) / (float)N;
        const float rstd = 1.0f / sqrtf(var + eps);
        if (threadIdx.x == 0) {
            Mean[m] = mean;
            Rstd[m] = rstd;
        }
        if constexpr (!LATE_WB) {
#pragma unroll
            for (int v = 0; v < VPT; ++v)
#pragma unroll
                for (int q = 0; q < 4; ++q) x[v][q] = ((x[v][q] - mean) * rstd) * w[v][q] + b[v][q];
        } else {
            const float *Wp = W, *Bp = B;
            asm volatile("" : "+s"(Wp), "+s"(Bp));   // (opaque per row: the loads stay here instead of being hoisted out of the row loop into registers)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                // (the second half of the row: the same lanes, WV vectors further on)
                load_row<BLOCK, WV, ALIGNED, false>(Wp + half * WV * BLOCK * 4, N - half * WV * BLOCK * 4, w);
                load_row<BLOCK, WV, ALIGNED, false>(Bp + half * WV * BLOCK * 4, N - half * WV * BLOCK * 4, b);
#pragma unroll
                for (int v = 0; v < WV; ++v)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        x[half * WV + v][q] = ((x[half * WV + v][q] - mean) * rstd) * w[v][q] + b[v][q];
            }
        }
        store_row<BLOCK, VPT, ALIGNED, STREAM>(Y + m * ldy, N, x);
    }
    (void)invN;
}

// Workgroup barrier that waits for the wave's LDS accesses only (lgkmcnt(0), vmcnt and expcnt at
// their maxima): unlike __syncthreads() it leaves global loads and stores in flight.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Forward by persistent workgroups with one row of look-ahead: a workgroup walks the rows m0, m0 +
// gridDim.x, ..., keeps W and B in registers for all of them and requests the next row before it
// reduces the current one (two register sets take turns).  With one row per workgroup lifetime a CU
// has nothing in flight between a workgroup's last load and its successor's first, which costs a
// fifth of the rate when X comes from HBM rather than from the memory-side cache.
// 16-byte aligned rows of a multiple of 4 elements; loads are unpredicated (a vector past the end
// re-reads the last one of the row and counts as zeros).
template <int BLOCK, int VPT, bool STREAM>
__global__ __launch_bounds__(BLOCK) void ln_fwd_pipe_kernel(const float* __restrict__ X, int64_t ldx,
                                                            const float* __restrict__ W,
                                                            const float* __restrict__ B,
                                                            float* __restrict__ Y, int64_t ldy,
                                                            float* __restrict__ Mean,
                                                            float* __restrict__ Rstd, float eps, int N,
                                                            int64_t M) {
    constexpr int NW = BLOCK / 64;
    __shared__ float red[2][NW];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int col[VPT];
    bool valid[VPT];
    f32x4 w[VPT], b[VPT];
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const int e = (threadIdx.x + v * BLOCK) * 4;
        valid[v] = e < N;
        col[v] = valid[v] ? e : N - 4;
        w[v] = *reinterpret_cast<const f32x4*>(W + col[v]);
        b[v] = *reinterpret_cast<const f32x4*>(B + col[v]);
    }
    f32x4 buf[2][VPT];
    const int64_t step = gridDim.x, m0 = blockIdx.x;
    const int64_t trips = (M - m0 + step - 1) / step;
    auto fetch = [&](f32x4 (&bx)[VPT], int64_t m) {
        const float* p = X + m * ldx;
#pragma unroll
        for (int v = 0; v < VPT; ++v) bx[v] = ld_global<STREAM>(reinterpret_cast<const f32x4*>(p + col[v]));
    };
    auto trip = [&](f32x4 (&cur)[VPT], f32x4 (&nxt)[VPT], int64_t it) {
        const int64_t m = m0 + it * step;
        float x[VPT][4];
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) x[v][q] = valid[v] ? cur[v][q] : 0.f;
        if (it + 1 < trips) fetch(nxt, m + step);
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) s += x[v][q];
        s = wave_reduce(s, SumOp{});
        if constexpr (NW > 1) {
            if (lane == 0) red[0][wave] = s;
            lds_barrier();
            s = red[0][0];
#pragma unroll
            for (int k = 1; k < NW; ++k) s += red[0][k];
        }
        const float mean = s / (float)N;
        float sq = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float d = valid[v] ? x[v][q] - mean : 0.f;
                sq += d * d;
            }
        sq = wave_reduce(sq, SumOp{});
        if constexpr (NW > 1) {
            if (lane == 0) red[1][wave] = sq;
            lds_barrier();   // (also keeps the next trip's write of red[0] behind this trip's reads of it)
            sq = red[1][0];
#pragma unroll
            for (int k = 1; k < NW; ++k) sq += red[1][k];
        }
        const float var = sq / (float)N;
        const float rstd = 1.0f / sqrtf(var + eps);
        if (threadIdx.x == 0) {
            Mean[m] = mean;
            Rstd[m] = rstd;
        }
        float* yp = Y + m * ldy;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            f32x4 t;
#pragma unroll
            for (int q = 0; q < 4; ++q) t[q] = ((x[v][q] - mean) * rstd) * w[v][q] + b[v][q];
            if (valid[v]) st_global<true>(t, reinterpret_cast<f32x4*>(yp + col[v]));
        }
    };
    if (trips > 0) fetch(buf[0], m0);
    for (int64_t it = 0; it < trips; it += 2) {
        trip(buf[0], buf[1], it);
        if (it + 1 < trips) trip(buf[1], buf[0], it + 1);
    }
}

// Forward for rows longer than the register-cached variants hold: three passes, the second
// and third re-reading the row (served by L2 for rows up to a few MB).  VEC: every row, W and B are
// 16-byte aligned and N is a multiple of 4 (16-byte accesses, four per lane in flight).
template <int BLOCK, bool VEC>
__global__ __launch_bounds__(BLOCK) void ln_fwd_3pass_kernel(const float* __restrict__ X, int64_t ldx,
                                                             const float* __restrict__ W,
                                                             const float* __restrict__ B,
                                                             float* __restrict__ Y, int64_t ldy,
                                                             float* __restrict__ Mean,
                                                             float* __restrict__ Rstd, float eps,
                                                             int64_t N, int64_t M) {
    constexpr int NW = BLOCK / 64;
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ float red[NW];
    const int64_t nvec = VEC ? N / 4 : 0;
    for (int64_t m = blockIdx.x; m < M; m += gridDim.x) {
        const float* x = X + m * ldx;
        float s = 0.f;
#pragma unroll 4
        for (int64_t v = threadIdx.x; v < nvec; v += BLOCK) {
            const f4 r = *reinterpret_cast<const f4*>(x + 4 * v);
            s += (r[0] + r[1]) + (r[2] + r[3]);
        }
        for (int64_t e = 4 * nvec + threadIdx.x; e < N; e += BLOCK) s += x[e];
        const float mean = block_reduce<NW>(s, red, SumOp{}, 0.f) / (float)N;
        float sq = 0.f;
#pragma unroll 4
        for (int64_t v = threadIdx.x; v < nvec; v += BLOCK) {
            const f4 r = *reinterpret_cast<const f4*>(x + 4 * v);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float d = r[q] - mean;
                sq += d * d;
            }
        }
        for (int64_t e = 4 * nvec + threadIdx.x; e < N; e += BLOCK) {
            const float d = x[e] - mean;
            sq += d * d;
        }
        const float var = block_reduce<NW>(sq, red, SumOp{}, 0.f) / (float)N;
        const float rstd = 1.0f / sqrtf(var + eps);
        if (threadIdx.x == 0) {
            Mean[m] = mean;
            Rstd[m] = rstd;
        }
        float* y = Y + m * ldy;
#pragma unroll 2
        for (int64_t v = threadIdx.x; v < nvec; v += BLOCK) {
            const f4 r = *reinterpret_cast<const f4*>(x + 4 * v);
            const f4 w = *reinterpret_cast<const f4*>(W + 4 * v), bb = *reinterpret_cast<const f4*>(B + 4 * v);
            f4 o;
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = ((r[q] - mean) * rstd) * w[q] + bb[q];
            st_global<true>(o, reinterpret_cast<f4*>(y + 4 * v));
        }
        for (int64_t e = 4 * nvec + threadIdx.x; e < N; e += BLOCK) y[e] = ((x[e] - mean) * rstd) * W[e] + B[e];
    }
}

// ---- backward: dX + partial dW/dB ------------------------------------------------------
template <int BLOCK, int VPT, bool ALIGNED, bool STREAM>
__global__ __launch_bounds__(BLOCK) void ln_bwd_kernel(float* __restrict__ DX, int64_t lddx,
                                                       const float* __restrict__ DY, int64_t lddy,
                                                       float* __restrict__ DW, int64_t lddw,
                                                       float* __restrict__ DB, int64_t lddb,
                                                       const float* __restrict__ X, int64_t ldx,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ Mean,
                                                       const float* __restrict__ Rstd, int N,
                                                       int64_t M, int G, int S) {
    constexpr int NW = BLOCK / 64;
    __shared__ float red[2 * NW];
    __shared__ float stage[BLOCK * VPT * 4];
    const int g = blockIdx.x % G, s = blockIdx.x / G;
    float w[VPT][4], dw[VPT][4], db[VPT][4];
    load_row<BLOCK, VPT, ALIGNED, false>(W, N, w);
#pragma unroll
    for (int v = 0; v < VPT; ++v)
#pragma unroll
        for (int q = 0; q < 4; ++q) dw[v][q] = db[v][q] = 0.f;

    for (int64_t m = g + (int64_t)G * s; m < M; m += (int64_t)G * S) {
        float x[VPT][4], dy[VPT][4];
        load_row<BLOCK, VPT, ALIGNED, STREAM>(X + m * ldx, N, x);
        load_row<BLOCK, VPT, ALIGNED, STREAM>(DY + m * lddy, N, dy);
        const float mean = Mean[m], rstd = Rstd[m];
        float c1 = 0.f, c2 = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int e0 = (threadIdx.x + v * BLOCK) * 4;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bool in = e0 + q < N;
                const float xhat = in ? (x[v][q] - mean) * rstd : 0.f;
                const float wdy = in ? w[v][q] * dy[v][q] : 0.f;
                x[v][q] = xhat;
                c1 += xhat * wdy;
                c2 += wdy;
            }
        }
        block_sum2<NW>(c1, c2, red);
        c1 /= (float)N;
        c2 /= (float)N;
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float xhat = x[v][q], wdy = rounded_product(w[v][q], dy[v][q]);
                dw[v][q] += dy[v][q] * xhat;
                db[v][q] += dy[v][q];
                x[v][q] = (wdy - (xhat * c1 + c2)) * rstd;
            }
        store_row<BLOCK, VPT, ALIGNED, STREAM>(DX + m * lddx, N, x);
    }
    // Flush through LDS so that consecutive lanes add to consecutive addresses: a float atomic
    // instruction then covers 256 contiguous bytes instead of 64 scattered words (memory-side
    // float atomics are the scarce resource here, not bandwidth).
    float* dwp = DW + (int64_t)g * lddw;
    float* dbp = DB + (int64_t)g * lddb;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) stage[(threadIdx.x + v * BLOCK) * 4 + q] = pass == 0 ? dw[v][q] : db[v][q];
        __syncthreads();
        float* dst = pass == 0 ? dwp : dbp;
        for (int c = threadIdx.x; c < N; c += BLOCK) {
            if (S == 1) dst[c] += stage[c];
            else unsafeAtomicAdd(dst + c, stage[c]);
        }
        __syncthreads();
    }
}

// Backward with RG row groups of 256 lanes per workgroup (rows of up to 4096 elements, 16-byte
// aligned): the groups walk different rows of the same partial slot and add their dW/dB
// partials in LDS before the flush, which divides the number of memory-side float atomics --
// the scarce resource of this kernel -- by RG at the same number of rows in flight.
// Workgroup (g, s): group h handles rows m = g + G*(RG*s + h), stepping by RG*G*S.
template <int BLOCK, int VPT, bool STREAM, int RG>
__global__ __launch_bounds__(BLOCK * RG) void ln_bwd_rg_kernel(float* __restrict__ DX, int64_t lddx,
                                                         const float* __restrict__ DY, int64_t lddy,
                                                         float* __restrict__ DW, int64_t lddw,
                                                         float* __restrict__ DB, int64_t lddb,
                                                         const float* __restrict__ X, int64_t ldx,
                                                         const float* __restrict__ W,
                                                         const float* __restrict__ Mean,
                                                         const float* __restrict__ Rstd, int N,
                                                         int64_t M, int G, int S) {
    constexpr int NW = BLOCK / 64;
    static_assert(NW == 1 || NW == 4 || NW == 8, "the cross-wave sums are written out for 4 and 8 waves");
    __shared__ float red[RG][2 * NW];
    __shared__ float stage[BLOCK * VPT * 4];
    const int g = blockIdx.x % G, s = blockIdx.x / G;
    const int h = threadIdx.x / BLOCK, lt = threadIdx.x % BLOCK, lane = lt & 63, wave = lt >> 6;
    auto vec = [&](int v) { return (lt + v * BLOCK) * 4; };
    float w[VPT][4], dw[VPT][4], db[VPT][4];
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const f32x4 t = vec(v) < N ? *reinterpret_cast<const f32x4*>(W + vec(v)) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            w[v][q] = t[q];
            dw[v][q] = db[v][q] = 0.f;
        }
    }
    const int64_t step = (int64_t)RG * G * S, m0 = g + (int64_t)G * (RG * s + h);
    const int64_t trips = (M - (g + (int64_t)G * RG * s) + step - 1) / step;  // of group 0; later groups may idle in the last
    // The rows of the next two trips are requested before the current one is reduced: the reductions
    // meet at barriers, which no load crosses on its own, and a workgroup would otherwise have
    // nothing in flight for half of every trip.  Two register sets take turns.
    // (Unpredicated: a row past the end re-reads the last row and a column past the end the last
    // vector of the row, and the values are discarded where they are used.  A predicated load
    // would have to be waited for at once to be merged with its default.)
    f32x4 bx[2][VPT], by[2][VPT];
    float bmean[2] = {0.f, 0.f}, brstd[2] = {0.f, 0.f};
    auto fetch = [&](auto set, int64_t m) {
        constexpr int B = decltype(set)::value;
        const int64_t mc = m < M ? m : M - 1;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int col = vec(v) < N ? vec(v) : N - 4;   // N % 4 == 0 here
            bx[B][v] = ld_global<STREAM>(reinterpret_cast<const f32x4*>(X + mc * ldx + col));
            by[B][v] = ld_global<STREAM>(reinterpret_cast<const f32x4*>(DY + mc * lddy + col));
        }
        bmean[B] = Mean[mc];
        brstd[B] = Rstd[mc];
    };
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;
    if (trips > 0) fetch(Set0{}, m0);
    if (trips > 1) fetch(Set1{}, m0 + step);
    auto trip = [&](auto set, int64_t it) {
        constexpr int B = decltype(set)::value;
        const int64_t m = m0 + it * step;
        const bool live = m < M;  // uniform per group; both groups keep meeting at the barriers
        float x[VPT][4], dy[VPT][4];
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                x[v][q] = bx[B][v][q];
                dy[v][q] = (live && vec(v) < N) ? by[B][v][q] : 0.f;
            }
        const float mean = bmean[B], rstd = live ? brstd[B] : 0.f;
        if (it + 2 < trips) fetch(set, m + 2 * step);
        float c1 = 0.f, c2 = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const bool in = live && vec(v) < N;  // N % 4 == 0 here
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float xhat = in ? (x[v][q] - mean) * rstd : 0.f;
                const float wdy = rounded_product(w[v][q], dy[v][q]);
                x[v][q] = xhat;
                c1 += xhat * wdy;
                c2 += wdy;
            }
        }
        c1 = wave_reduce(c1, SumOp{});
        c2 = wave_reduce(c2, SumOp{});
        if constexpr (NW > 1) {   // (a one-wave group is done after the shuffles)
            if (lane == 0) {
                red[h][wave] = c1;
                red[h][NW + wave] = c2;
            }
            lds_barrier();
            c1 = (red[h][0] + red[h][1]) + (red[h][2] + red[h][3]);
            c2 = (red[h][NW] + red[h][NW + 1]) + (red[h][NW + 2] + red[h][NW + 3]);
            if constexpr (NW == 8) {
                c1 += (red[h][4] + red[h][5]) + (red[h][6] + red[h][7]);
                c2 += (red[h][NW + 4] + red[h][NW + 5]) + (red[h][NW + 6] + red[h][NW + 7]);
            }
            lds_barrier();
        }
        c1 /= (float)N;
        c2 /= (float)N;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            f32x4 t;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float xhat = x[v][q], wdy = rounded_product(w[v][q], dy[v][q]);
                dw[v][q] += dy[v][q] * xhat;
                db[v][q] += dy[v][q];
                t[q] = (wdy - (xhat * c1 + c2)) * rstd;
            }
            if (live && vec(v) < N) st_global<true>(t, reinterpret_cast<f32x4*>(DX + m * lddx + vec(v)));
        }
    };
    for (int64_t it = 0; it < trips; it += 2) {
        trip(Set0{}, it);
        if (it + 1 < trips) trip(Set1{}, it + 1);
    }
    // the groups add their partials in LDS, one after the other; then everybody flushes with
    // coalesced atomics
    float* dwp = DW + (int64_t)g * lddw;
    float* dbp = DB + (int64_t)g * lddb;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int turn = 0; turn < RG; ++turn) {
            if (h == turn) {
#pragma unroll
                for (int v = 0; v < VPT; ++v)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float val = pass == 0 ? dw[v][q] : db[v][q];
                        if (turn == 0) stage[vec(v) + q] = val;
                        else stage[vec(v) + q] += val;
                    }
            }
            __syncthreads();
        }
        float* dst = pass == 0 ? dwp : dbp;
        for (int c = threadIdx.x; c < N; c += BLOCK * RG) {
            if (S == 1) dst[c] += stage[c];
            else unsafeAtomicAdd(dst + c, stage[c]);
        }
        __syncthreads();
    }
}

// Backward for rows of 8192 to 16384 elements (16-byte aligned): 1024 lanes, four vectors of every array per lane.
// W, dW, dB and the row at hand are 80 registers of a lane's 128; a second row in registers for look-ahead does not
// fit (it spilled), and without look-ahead the kernel ran at 3.1-3.5 TB/s.  The row in flight therefore lands in LDS:
// every lane requests its own four vectors of X and of dY with global->LDS transfers (no staging registers), copies
// them to registers once they have landed, and at once requests the next row into the same places.  A lane reads back
// only what its own wave's transfers wrote, so the prefetch needs no barrier; the two barriers of a trip belong to the
// row sums, and they wait for LDS accesses only, so the transfers stay in flight across them.  128 KB of LDS: one
// workgroup per CU with a whole row (128 KB) in flight.
// Workgroup (g, s) walks the rows m = g + G*s, stepping by G*S, of partial slot g.
constexpr int kWideLanes = 1024, kWideVpt = 4, kWideFloats = kWideLanes * kWideVpt * 4;
__global__ __launch_bounds__(kWideLanes) void ln_bwd_wide_kernel(float* __restrict__ DX, int64_t lddx,
                                                                 const float* __restrict__ DY, int64_t lddy,
                                                                 float* __restrict__ DW, int64_t lddw,
                                                                 float* __restrict__ DB, int64_t lddb,
                                                                 const float* __restrict__ X, int64_t ldx,
                                                                 const float* __restrict__ W,
                                                                 const float* __restrict__ Mean,
                                                                 const float* __restrict__ Rstd, int N,
                                                                 int64_t M, int G, int S) {
    constexpr int NW = kWideLanes / 64, VPT = kWideVpt;
    __shared__ __attribute__((aligned(1024))) float xs[kWideFloats], ys[kWideFloats];
    __shared__ float red[2][2 * NW];   // (two sets: a trip's sums are read while the next trip's are not yet written)
    const int g = blockIdx.x % G, s = blockIdx.x / G;
    const int lt = threadIdx.x, lane = lt & 63;
    const int wave = __builtin_amdgcn_readfirstlane(lt >> 6);
    auto vec = [&](int v) { return (lt + v * kWideLanes) * 4; };
    float w[VPT][4], dw[VPT][4], db[VPT][4];
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const f32x4 t = vec(v) < N ? *reinterpret_cast<const f32x4*>(W + vec(v)) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            w[v][q] = t[q];
            dw[v][q] = db[v][q] = 0.f;
        }
    }
    // (unpredicated: a vector past the end of the row re-reads the row's last vector and is discarded where it is used)
    auto request = [&](int64_t m) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int col = vec(v) < N ? vec(v) : N - 4;   // N % 4 == 0 here
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(X + m * ldx + col),
                                             (__attribute__((address_space(3))) void*)(xs + (wave * 64 + v * kWideLanes) * 4), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(DY + m * lddy + col),
                                             (__attribute__((address_space(3))) void*)(ys + (wave * 64 + v * kWideLanes) * 4), 16, 0, 0);
        }
    };
    const int64_t step = (int64_t)G * S, m0 = g + (int64_t)G * s;
    if (m0 < M) request(m0);
    int set = 0;
    for (int64_t m = m0; m < M; m += step) {
        const float mean = Mean[m], rstd = Rstd[m];
        // this wave's transfers (and the previous trip's stores) are done: vmcnt(0); expcnt and lgkmcnt untouched
        __builtin_amdgcn_s_waitcnt(0x0f70);
        asm volatile("" ::: "memory");
        float x[VPT][4], dy[VPT][4];
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const f32x4 tx = *reinterpret_cast<const f32x4*>(xs + vec(v)), ty = *reinterpret_cast<const f32x4*>(ys + vec(v));
            const bool in = vec(v) < N;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                x[v][q] = tx[q];
                dy[v][q] = in ? ty[q] : 0.f;
            }
        }
        // the copies have left LDS before the next row is asked into their places
        __builtin_amdgcn_s_waitcnt(0xc07f);
        asm volatile("" ::: "memory");
        if (m + step < M) request(m + step);
        float c1 = 0.f, c2 = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const bool in = vec(v) < N;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float xhat = in ? (x[v][q] - mean) * rstd : 0.f;
                const float wdy = rounded_product(w[v][q], dy[v][q]);
                x[v][q] = xhat;
                c1 += xhat * wdy;
                c2 += wdy;
            }
        }
        c1 = wave_reduce(c1, SumOp{});
        c2 = wave_reduce(c2, SumOp{});
        if (lane == 0) {
            red[set][wave] = c1;
            red[set][NW + wave] = c2;
        }
        lds_barrier();
        c1 = c2 = 0.f;
#pragma unroll
        for (int i = 0; i < NW; i += 4) {
            c1 += (red[set][i] + red[set][i + 1]) + (red[set][i + 2] + red[set][i + 3]);
            c2 += (red[set][NW + i] + red[set][NW + i + 1]) + (red[set][NW + i + 2] + red[set][NW + i + 3]);
        }
        set ^= 1;   // (the next trip writes the other set; the barrier of that trip keeps the one after it behind these reads)
        c1 /= (float)N;
        c2 /= (float)N;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            f32x4 t;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float xhat = x[v][q], wdy = rounded_product(w[v][q], dy[v][q]);
                dw[v][q] += dy[v][q] * xhat;
                db[v][q] += dy[v][q];
                t[q] = (wdy - (xhat * c1 + c2)) * rstd;
            }
            if (vec(v) < N) st_global<true>(t, reinterpret_cast<f32x4*>(DX + m * lddx + vec(v)));
        }
    }
    // flush through LDS (the row buffer is free now) with coalesced atomics, as the other backward kernels do
    float* dwp = DW + (int64_t)g * lddw;
    float* dbp = DB + (int64_t)g * lddb;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) xs[vec(v) + q] = pass == 0 ? dw[v][q] : db[v][q];
        __syncthreads();
        float* dst = pass == 0 ? dwp : dbp;
        for (int c = lt; c < N; c += kWideLanes) {
            if (S == 1) dst[c] += xs[c];
            else unsafeAtomicAdd(dst + c, xs[c]);
        }
    }
}

// Backward for rows of 16385 to 32768 elements (16-byte aligned): 512 lanes, sixteen vectors of the row per lane.  dW
// and dB of the lane's 64 columns stay in registers for all the rows of the workgroup (128 of the 256 registers that
// eight waves per CU leave a lane; with 1024 lanes and 128 registers the kernel spilled) and are flushed
// once; the row itself does not fit beside them, so it is walked twice -- once for the two row sums, once for dX and
// the partials, the second time out of the caches -- two vectors of each array at a time.  (The kernel for still
// longer rows adds every element of every row to the partial slots with an atomic of its own: 1.2-1.6 TB/s at 32768.)
// Loads are unpredicated (a vector past the end of the row re-reads the row's last vector and is masked where it is
// used): behind a branch each, the compiler could not order them and spilled 140 registers.
__global__ __launch_bounds__(512) void ln_bwd_two_pass_kernel(float* __restrict__ DX, int64_t lddx,
                                                               const float* __restrict__ DY, int64_t lddy,
                                                               float* __restrict__ DW, int64_t lddw,
                                                               float* __restrict__ DB, int64_t lddb,
                                                               const float* __restrict__ X, int64_t ldx,
                                                               const float* __restrict__ W,
                                                               const float* __restrict__ Mean,
                                                               const float* __restrict__ Rstd, int N,
                                                               int64_t M, int G, int S) {
    constexpr int BLOCK = 512, NW = BLOCK / 64, VPT = 16, HV = 2;
    __shared__ float red[2 * NW];
    __shared__ __attribute__((aligned(16))) float stage[BLOCK * VPT * 4];   // 128 KB: the flush of dW, then of dB
    const int g = blockIdx.x % G, s = blockIdx.x / G;
    float dw[VPT][4], db[VPT][4];
#pragma unroll
    for (int v = 0; v < VPT; ++v)
#pragma unroll
        for (int q = 0; q < 4; ++q) dw[v][q] = db[v][q] = 0.f;
    auto e0_of = [&](int v) { return ((int)threadIdx.x + v * BLOCK) * 4; };
    // Vector v of a lane lies v * BLOCK * 16 bytes behind vector 0: that part of the address is the same for the whole
    // workgroup and goes into the scalar base of the load, the lane's own part is one 32-bit offset for all vectors and
    // arrays (an address pair per vector and array was 128 registers).  A lane past the end of the row in a vector that
    // others still have re-reads the row's last vector; vectors that lie past the end for everybody are skipped.
    const unsigned lane_bytes = threadIdx.x * 16u;
    auto ldv = [&](const float* row, int v) {
        const int left = N - v * BLOCK * 4;                         // elements of the row from this vector's first lane on (> 0)
        const unsigned off = lane_bytes < (unsigned)left * 4u ? lane_bytes : (unsigned)left * 4u - 16u;
        return *reinterpret_cast<const f32x4*>(reinterpret_cast<const char*>(row + v * BLOCK * 4) + off);
    };
    const int nv = (N + BLOCK * 4 - 1) / (BLOCK * 4);               // vectors that hold elements of the row for some lane
    for (int64_t m = g + (int64_t)G * s; m < M; m += (int64_t)G * S) {
        const float* xr = X + m * ldx;
        const float* dyr = DY + m * lddy;
        const float* Wr = W;
        asm volatile("" : "+s"(Wr));   // (opaque per row: W is loaded where it is used, not hoisted out of the row loop into registers)
        const float mean = Mean[m], rstd = Rstd[m];
        float c1 = 0.f, c2 = 0.f;
#pragma unroll
        for (int h = 0; h < VPT / HV; ++h) {
            __builtin_amdgcn_sched_barrier(0);
            if (h * HV >= nv) break;   // (the same for the whole workgroup)
            f32x4 x[HV], dy[HV], w[HV];
#pragma unroll
            for (int u = 0; u < HV; ++u) {
                const int v = h * HV + u < nv ? h * HV + u : nv - 1;
                x[u] = ldv(xr, v);
                dy[u] = ldv(dyr, v);
                w[u] = ldv(Wr, v);
            }
#pragma unroll
            for (int u = 0; u < HV; ++u) {
                const bool in = e0_of(h * HV + u) < N;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float xhat = in ? (x[u][q] - mean) * rstd : 0.f;
                    const float wdy = in ? w[u][q] * dy[u][q] : 0.f;
                    c1 += xhat * wdy;
                    c2 += wdy;
                }
            }
        }
        block_sum2<NW>(c1, c2, red);
        c1 /= (float)N;
        c2 /= (float)N;
        // (opaque again: the second walk loads anew -- as the same loads from the same unwritten addresses the
        // compiler would keep the first walk's values alive instead, in scratch memory)
        asm volatile("" : "+s"(xr), "+s"(dyr), "+s"(Wr));
        float* dxr = DX + m * lddx;
#pragma unroll
        for (int h = 0; h < VPT / HV; ++h) {
            __builtin_amdgcn_sched_barrier(0);
            if (h * HV >= nv) break;
            f32x4 x[HV], dy[HV], w[HV];
#pragma unroll
            for (int u = 0; u < HV; ++u) {
                const int v = h * HV + u < nv ? h * HV + u : nv - 1;
                x[u] = ldv(xr, v);
                dy[u] = ldv(dyr, v);
                w[u] = ldv(Wr, v);
            }
#pragma unroll
            for (int u = 0; u < HV; ++u) {
                const int v = h * HV + u;
                const bool in = e0_of(v) < N;
                f32x4 t;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float dyq = in ? dy[u][q] : 0.f;
                    const float xhat = in ? (x[u][q] - mean) * rstd : 0.f;
                    const float wdy = rounded_product(w[u][q], dyq);
                    dw[v][q] += dyq * xhat;
                    db[v][q] += dyq;
                    t[q] = (wdy - (xhat * c1 + c2)) * rstd;
                }
                if (in) st_global<true>(t, reinterpret_cast<f32x4*>(reinterpret_cast<char*>(dxr + v * BLOCK * 4) + lane_bytes));
            }
        }
    }
    float* dwp = DW + (int64_t)g * lddw;
    float* dbp = DB + (int64_t)g * lddb;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < VPT; ++v)
#pragma unroll
            for (int q = 0; q < 4; ++q) stage[e0_of(v) + q] = pass == 0 ? dw[v][q] : db[v][q];
        __syncthreads();
        float* dst = pass == 0 ? dwp : dbp;
        for (int c = threadIdx.x; c < N; c += BLOCK) {
            if (S == 1) dst[c] += stage[c];
            else unsafeAtomicAdd(dst + c, stage[c]);
        }
    }
}

// Backward for rows longer than the register-cached variants hold.
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void ln_bwd_long_kernel(float* __restrict__ DX, int64_t lddx,
                                                            const float* __restrict__ DY, int64_t lddy,
                                                            float* __restrict__ DW, int64_t lddw,
                                                            float* __restrict__ DB, int64_t lddb,
                                                            const float* __restrict__ X, int64_t ldx,
                                                            const float* __restrict__ W,
                                                            const float* __restrict__ Mean,
                                                            const float* __restrict__ Rstd,
                                                            int64_t N, int64_t M, int G) {
    constexpr int NW = BLOCK / 64;
    __shared__ float red[2 * NW];
    for (int64_t m = blockIdx.x; m < M; m += gridDim.x) {
        const float* x = X + m * ldx;
        const float* dy = DY + m * lddy;
        const float mean = Mean[m], rstd = Rstd[m];
        float c1 = 0.f, c2 = 0.f;
        for (int64_t e = threadIdx.x; e < N; e += BLOCK) {
            const float xhat = (x[e] - mean) * rstd, wdy = rounded_product(W[e], dy[e]);
            c1 += xhat * wdy;
            c2 += wdy;
        }
        block_sum2<NW>(c1, c2, red);
        c1 /= (float)N;
        c2 /= (float)N;
        float* dwp = DW + (m % G) * lddw;
        float* dbp = DB + (m % G) * lddb;
        float* dx = DX + m * lddx;
        for (int64_t e = threadIdx.x; e < N; e += BLOCK) {
            const float xhat = (x[e] - mean) * rstd, wdy = rounded_product(W[e], dy[e]);
            dx[e] = (wdy - (xhat * c1 + c2)) * rstd;
            unsafeAtomicAdd(dwp + e, dy[e] * xhat);
            unsafeAtomicAdd(dbp + e, dy[e]);
        }
    }
}

// ---- backward: final reduction over the partial slots -----------------------------------
// 64 consecutive n per workgroup; its 16 waves split the slots (independent loads, one round
// trip for GROUP_SIZE_M <= 64), LDS combines them in a fixed order.
// CLEAR: every slot is set to zero once it has been read (the library's own slot array, which
// the next call then finds ready for its atomic adds).
template <bool CLEAR>
__global__ __launch_bounds__(1024) void ln_dwdb_kernel(float* __restrict__ DW, int64_t lddw,
                                                       float* __restrict__ DB, int64_t lddb,
                                                       float* __restrict__ FDW, float* __restrict__ FDB,
                                                       int64_t N, int G) {
    __shared__ float part[2][16][64];
    const int lane = threadIdx.x & 63, wq = threadIdx.x >> 6;
    const int64_t n = (int64_t)blockIdx.x * 64 + lane;
    float a = 0.f, b = 0.f;
    if (n < N) {
#pragma unroll 4
        for (int g = wq; g < G; g += 16) {
            a += DW[n + g * lddw];
            b += DB[n + g * lddb];
        }
        if (CLEAR) {
            for (int g = wq; g < G; g += 16) {
                DW[n + g * lddw] = 0.f;
                DB[n + g * lddb] = 0.f;
            }
        }
    }
    part[0][wq][lane] = a;
    part[1][wq][lane] = b;
    __syncthreads();
    if (wq < 2 && n < N) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 16; ++k) t += part[wq][k][lane];
        (wq == 0 ? FDW : FDB)[n] = t;
    }
}

// ---- static scratch of the allocation-free backward ---------------------------------------
// Partial dW / dB slots of mi_layer_norm_bwd_static: kScratchFloats floats for DW followed by as many
// for DB (4 MiB in all).  Host code never uses the array's name as an address: the device address
// is looked up once per device (scratch_ptr) and passed to the kernels like any other buffer.
constexpr int64_t kScratchFloats = 512 * 1024;
static __device__ __align__(256) float scratch[2 * kScratchFloats];

constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices];
bool g_scratch_known[kMaxDevices];
bool g_scratch_dirty[kMaxDevices];   // a call is under way, or one ended before its final kernel was launched

// Device address of `scratch` on the current device; positive hipError_t on failure.  The lookup
// (hipGetSymbolAddress may load the code object and is not a stream operation) happens once per
// device and never while `stream` is being captured: the forward and the three-step backward do
// it on their first eager call as well, so a capture that holds the static backward finds the
// address known whenever any LayerNorm entry point has run eagerly on the device before.
int scratch_ptr(float** out, hipStream_t stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return MI_E_UNSUPPORTED;
    if (!__atomic_load_n(&g_scratch_known[dev], __ATOMIC_ACQUIRE)) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return MI_E_UNSUPPORTED;   // first use on this device inside a capture: call once eagerly before
        }
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return MI_E_NULL;
        g_scratch_ptr[dev] = p;   // every thread that gets here stores the same address
        __atomic_store_n(&g_scratch_known[dev], true, __ATOMIC_RELEASE);
    }
    if (out) *out = g_scratch_ptr[dev];
    return MI_OK;
}

// Called by the other LayerNorm entry points: makes the address known while no capture is on.
void scratch_warm(void* stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    if (dev >= 0 && dev < kMaxDevices && !__atomic_load_n(&g_scratch_known[dev], __ATOMIC_ACQUIRE) &&
        scratch_ptr(nullptr, (hipStream_t)stream) > 0)
        (void)hipGetLastError();
}

// Zero fill as a kernel (a memset node would not survive stream capture and replay on this runtime).
__global__ __launch_bounds__(256) void fill_zero_kernel(f32x4* __restrict__ a, f32x4* __restrict__ b, int64_t nvec) {
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        a[i] = z;
        b[i] = z;
    }
}

int check_f32(const mi_tile_array* a, int ndim) {
    MI_CHECK(check_array(a, ndim));
    if (a->dtype != MI_F32) return MI_E_DTYPE;
    for (int i = 0; i < ndim; ++i)
        if (i == 0 && a->sizes[0] > 1 && a->strides[0] != 1) return MI_E_STRIDE;
    return MI_OK;
}

bool rows_vec_ok(const mi_tile_array* a) {
    return aligned(a->ptr, 16) && (a->ndim < 2 || a->sizes[1] <= 1 || a->strides[1] % 4 == 0);
}

constexpr int kMaxRegsN = 256 * 16 * 4;

// Persistent look-ahead forward: used when every workgroup gets at least two rows.
template <bool ST>
bool launch_fwd_pipe(int vecs, hipStream_t s, const float* X, int64_t ldx, const float* W, const float* B,
                     float* Y, int64_t ldy, float* Mean, float* Rstd, float eps, int N, int64_t M) {
    static const int wpc = [] { const char* e = getenv("MI_LN_FWD_WPC"); return e ? atoi(e) : 0; }();   // workgroups per CU (tuning; < 0: off)
    if (wpc < 0 || vecs > 4096) return false;
    const int block = vecs <= 256 ? 64 : vecs <= 1024 ? 256 : vecs <= 2048 ? 512 : 1024;
    // (256-lane workgroups: six per CU measured best, 80 % of the HBM rate on resident input and 64 % on cold
    // input against 78 % and 60 % for one row per workgroup lifetime)
    const int64_t cap = 256 * (int64_t)(wpc > 0 ? wpc : block == 256 ? 6 : 2048 / block);
    if (M < 2 * cap) return false;
    dim3 grid((unsigned)cap);
#define PIPE(BL, VP)                                                                               \
    hipLaunchKernelGGL((ln_fwd_pipe_kernel<BL, VP, ST>), grid, dim3(BL), 0, s, X, ldx, W, B, Y, ldy, \
                       Mean, Rstd, eps, N, M)
    if (vecs <= 64) { PIPE(64, 1); set_variant("ln_fwd_pipe_b64_v1"); }
    else if (vecs <= 128) { PIPE(64, 2); set_variant("ln_fwd_pipe_b64_v2"); }
    else if (vecs <= 256) { PIPE(64, 4); set_variant("ln_fwd_pipe_b64_v4"); }
    else if (vecs <= 512) { PIPE(256, 2); set_variant("ln_fwd_pipe_b256_v2"); }
    else if (vecs <= 1024) { PIPE(256, 4); set_variant("ln_fwd_pipe_b256_v4"); }
    else if (vecs <= 2048) { PIPE(512, 4); set_variant("ln_fwd_pipe_b512_v4"); }
    else { PIPE(1024, 4); set_variant("ln_fwd_pipe_b1024_v4"); }
#undef PIPE
    return true;
}

template <bool AL, bool ST>
void launch_fwd(int vecs, dim3 grid, hipStream_t s, const float* X, int64_t ldx, const float* W,
                const float* B, float* Y, int64_t ldy, float* Mean, float* Rstd, float eps, int N,
                int64_t M) {
    if constexpr (AL) {
        if (launch_fwd_pipe<ST>(vecs, s, X, ldx, W, B, Y, ldy, Mean, Rstd, eps, N, M)) return;
    }
#define FWD(BL, VP)                                                                              \
    hipLaunchKernelGGL((ln_fwd_kernel<BL, VP, AL, ST>), grid, dim3(BL), 0, s, X, ldx, W, B, Y, ldy, \
                       Mean, Rstd, eps, N, M)
    if (vecs <= 64) { FWD(64, 1); set_variant("ln_fwd_regs_b64_v1"); }
    else if (vecs <= 128) { FWD(64, 2); set_variant("ln_fwd_regs_b64_v2"); }
    else if (vecs <= 256) { FWD(64, 4); set_variant("ln_fwd_regs_b64_v4"); }   // one wave per row: no barriers (5.4 -> 6.3 TB/s at N = 1024)
    else if (vecs <= 512) { FWD(256, 2); set_variant("ln_fwd_regs_b256_v2"); }
    else if (vecs <= 1024) { FWD(256, 4); set_variant("ln_fwd_regs_b256_v4"); }
    else if (vecs <= 2048) { FWD(512, 4); set_variant("ln_fwd_regs_b512_v4"); }      // longer rows: more lanes, not more
    else if (vecs <= 4096) { FWD(1024, 4); set_variant("ln_fwd_regs_b1024_v4"); }    // registers per lane
    else { FWD(1024, 8); set_variant("ln_fwd_regs_b1024_v8"); }   // up to 32768 elements: x, W and B are 96 of a lane's 128 registers

#undef FWD
}

template <bool AL, bool ST>
void launch_bwd(int vecs, dim3 grid, hipStream_t s, float* DX, int64_t lddx, const float* DY,
                int64_t lddy, float* DW, int64_t lddw, float* DB, int64_t lddb, const float* X,
                int64_t ldx, const float* W, const float* Mean, const float* Rstd, int N, int64_t M,
                int G, int S) {
#define BWD(BL, VP)                                                                            \
    hipLaunchKernelGGL((ln_bwd_kernel<BL, VP, AL, ST>), grid, dim3(BL), 0, s, DX, lddx, DY, lddy, \
                       DW, lddw, DB, lddb, X, ldx, W, Mean, Rstd, N, M, G, S)
    if (vecs <= 64) { BWD(64, 1); set_variant("ln_bwd_regs_b64_v1"); }
    else if (vecs <= 256) { BWD(256, 1); set_variant("ln_bwd_regs_b256_v1"); }
    else if (vecs <= 512) { BWD(256, 2); set_variant("ln_bwd_regs_b256_v2"); }
    else if (vecs <= 1024) { BWD(256, 4); set_variant("ln_bwd_regs_b256_v4"); }
    else if (vecs <= 2048) { BWD(512, 4); set_variant("ln_bwd_regs_b512_v4"); }
    else { BWD(1024, 4); set_variant("ln_bwd_regs_b1024_v4"); }
#undef BWD
}

}  // namespace

extern "C" int mi_layer_norm_fwd(const mi_tile_array* X, const mi_tile_array* W,
                                 const mi_tile_array* B, const mi_tile_array* Y,
                                 const mi_tile_array* Mean, const mi_tile_array* Rstd, float eps,
                                 int TILE_N, void* stream) {
    scratch_warm(stream);
    MI_CHECK(check_f32(X, 2));
    MI_CHECK(check_f32(Y, 2));
    MI_CHECK(check_f32(W, 1));
    MI_CHECK(check_f32(B, 1));
    MI_CHECK(check_f32(Mean, 1));
    MI_CHECK(check_f32(Rstd, 1));
    if (!is_pow2(TILE_N)) return MI_E_TILE;
    const int64_t N = X->sizes[0], M = X->sizes[1];
    if (!same_shape(X, Y) || W->sizes[0] != N || B->sizes[0] != N || Mean->sizes[0] != M ||
        Rstd->sizes[0] != M)
        return MI_E_SHAPE;
    if ((M > 1 && (Mean->strides[0] != 1 || Rstd->strides[0] != 1))) return MI_E_STRIDE;
    if (M > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (M == 0) return MI_OK;
    if (N == 0) return MI_E_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const float* x = (const float*)X->ptr;
    float* y = (float*)Y->ptr;
    dim3 grid((unsigned)M);
    if (N > 2 * kMaxRegsN) {
        const bool vec = N % 4 == 0 && rows_vec_ok(X) && rows_vec_ok(Y) && rows_vec_ok(W) && rows_vec_ok(B);
        const bool wide = M < 1024;   // few rows: 1024 lanes each
#define GO(BL, VEC)                                                                                           \
    hipLaunchKernelGGL((ln_fwd_3pass_kernel<BL, VEC>), grid, dim3(BL), 0, s, x, X->strides[1], (const float*)W->ptr, \
                       (const float*)B->ptr, y, Y->strides[1], (float*)Mean->ptr, (float*)Rstd->ptr, eps, N, M)
        if (wide && vec) GO(1024, true);
        else if (wide) GO(1024, false);
        else if (vec) GO(256, true);
        else GO(256, false);
#undef GO
        set_variant(wide ? (vec ? "ln_fwd_3pass_b1024_v4" : "ln_fwd_3pass_b1024") : (vec ? "ln_fwd_3pass_b256_v4" : "ln_fwd_3pass_b256"));
        return launch_status();
    }
    const bool al = N % 4 == 0 && rows_vec_ok(X) && rows_vec_ok(Y) && rows_vec_ok(W) && rows_vec_ok(B);
    const int vecs = (int)cld(N, 4);
#define ARGS                                                                                      \
    vecs, grid, s, x, X->strides[1], (const float*)W->ptr, (const float*)B->ptr, y, Y->strides[1], \
        (float*)Mean->ptr, (float*)Rstd->ptr, eps, (int)N, M
    if (!al) launch_fwd<false, false>(ARGS);
    else if (stream_hint(2 * M * N * (int64_t)sizeof(float))) launch_fwd<true, true>(ARGS);
    else launch_fwd<true, false>(ARGS);
#undef ARGS
    return launch_status();
}

extern "C" int mi_layer_norm_bwd_dx_partial_dwdb(
    const mi_tile_array* DX, const mi_tile_array* DY, const mi_tile_array* DW, const mi_tile_array* DB,
    const mi_tile_array* X, const mi_tile_array* W, const mi_tile_array* Mean,
    const mi_tile_array* Rstd, const mi_tile_array* Locks, int GROUP_SIZE_M, int TILE_N,
    void* stream) {
    scratch_warm(stream);
    MI_CHECK(check_f32(DX, 2));
    MI_CHECK(check_f32(DY, 2));
    MI_CHECK(check_f32(DW, 2));
    MI_CHECK(check_f32(DB, 2));
    MI_CHECK(check_f32(X, 2));
    MI_CHECK(check_f32(W, 1));
    MI_CHECK(check_f32(Mean, 1));
    MI_CHECK(check_f32(Rstd, 1));
    if (Locks) {
        MI_CHECK(check_array(Locks, 1));
        if (Locks->dtype != MI_I64) return MI_E_DTYPE;
        if (Locks->sizes[0] < GROUP_SIZE_M) return MI_E_SHAPE;
    }
    if (GROUP_SIZE_M < 1) return MI_E_ARG;
    if (!is_pow2(TILE_N)) return MI_E_TILE;
    const int64_t N = X->sizes[0], M = X->sizes[1];
    const int G = GROUP_SIZE_M;
    if (!same_shape(X, DX) || !same_shape(X, DY) || W->sizes[0] != N || Mean->sizes[0] != M ||
        Rstd->sizes[0] != M || DW->sizes[0] != N || DB->sizes[0] != N || DW->sizes[1] < G ||
        DB->sizes[1] < G)
        return MI_E_SHAPE;
    if ((M > 1 && (Mean->strides[0] != 1 || Rstd->strides[0] != 1))) return MI_E_STRIDE;
    if (M > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (M == 0) return MI_OK;
    if (N == 0) return MI_E_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    if (N > kMaxRegsN && N <= 2 * kMaxRegsN && G <= 256 && N % 4 == 0 && rows_vec_ok(X) && rows_vec_ok(DX) && rows_vec_ok(DY) &&
        rows_vec_ok(W)) {
        // one workgroup of 512 lanes per CU (128 KB of LDS for the flush)
        const int64_t rows_per_slot = cld(M, (int64_t)G);
        int64_t Sw = cld((int64_t)256, (int64_t)G);
        if (Sw > rows_per_slot) Sw = rows_per_slot;
        if (Sw < 1) Sw = 1;
        hipLaunchKernelGGL(ln_bwd_two_pass_kernel, dim3((unsigned)(G * Sw)), dim3(512), 0, s, (float*)DX->ptr,
                           DX->strides[1], (const float*)DY->ptr, DY->strides[1], (float*)DW->ptr, DW->strides[1],
                           (float*)DB->ptr, DB->strides[1], (const float*)X->ptr, X->strides[1], (const float*)W->ptr,
                           (const float*)Mean->ptr, (const float*)Rstd->ptr, (int)N, M, G, (int)Sw);
        set_variant("ln_bwd_two_pass_b512_v16");
        return launch_status();
    }
    if (N > kMaxRegsN) {
        hipLaunchKernelGGL((ln_bwd_long_kernel<256>), dim3((unsigned)M), dim3(256), 0, s,
                           (float*)DX->ptr, DX->strides[1], (const float*)DY->ptr, DY->strides[1],
                           (float*)DW->ptr, DW->strides[1], (float*)DB->ptr, DB->strides[1],
                           (const float*)X->ptr, X->strides[1], (const float*)W->ptr,
                           (const float*)Mean->ptr, (const float*)Rstd->ptr, N, M, G);
        set_variant("ln_bwd_long_b256");
        return launch_status();
    }
    // Splits per slot: about two workgroups per CU (measured optimum on MI355X: more
    // workgroups cost more atomics, fewer leave HBM idle), and at least ~4 rows per workgroup
    // so the register partials amortise the flush.
    const int64_t rows_per_slot = cld(M, (int64_t)G);
    int64_t S = cld((int64_t)512, (int64_t)G);
    if (S > cld(rows_per_slot, (int64_t)4)) S = cld(rows_per_slot, (int64_t)4);
    if (S < 1) S = 1;
    if (const char* env = getenv("MI_LN_BWD_SPLITS")) {  // tuning override: workgroups per partial slot
        const long v = atol(env);
        if (v >= 1 && v <= rows_per_slot) S = v;
    }
    const bool al = N % 4 == 0 && rows_vec_ok(X) && rows_vec_ok(DX) && rows_vec_ok(DY) && rows_vec_ok(W);
    const int vecs = (int)cld(N, 4);
    dim3 grid((unsigned)(G * S));
#define ARGS                                                                                   \
    vecs, grid, s, (float*)DX->ptr, DX->strides[1], (const float*)DY->ptr, DY->strides[1],     \
        (float*)DW->ptr, DW->strides[1], (float*)DB->ptr, DB->strides[1], (const float*)X->ptr, \
        X->strides[1], (const float*)W->ptr, (const float*)Mean->ptr, (const float*)Rstd->ptr,  \
        (int)N, M, G, (int)S
    const bool stream_in = stream_hint(3 * M * N * (int64_t)sizeof(float));
    static const bool one_group = [] { const char* e = getenv("MI_LN_BWD_RG"); return e && e[0] == '1'; }();
    if (al && N % 4 == 0 && vecs <= 2048 && !one_group) {
        // Row groups with two rows of look-ahead.  Up to 4096 elements a group is 256 lanes and two
        // groups share a workgroup (same rows in flight, half the atomics; four groups measured no
        // better); up to 8192 elements one group of 512 lanes.
        // Up to 512 elements a group is a single wave (no barriers in the walk) and eight groups
        // share a workgroup; there the chip wants four times as many groups in flight, since a
        // group's rows are that much shorter.
        const int rg = vecs <= 128 ? 8 : vecs <= 1024 ? 2 : 1;
        if ((vecs <= 128 || vecs > 1024) && !getenv("MI_LN_BWD_SPLITS")) {
            // (and a 512-lane group fills a CU by itself: one workgroup per CU, half the flushes)
            S = cld((int64_t)(vecs <= 128 ? 2048 : 256), (int64_t)G);
            if (S > cld(rows_per_slot, (int64_t)4)) S = cld(rows_per_slot, (int64_t)4);
            if (S < 1) S = 1;
        }
        const int S2 = (int)cld(S, (int64_t)rg);
        dim3 grid2((unsigned)(G * S2));
#define RGK(BL, VP, ST, R)                                                                                      \
    hipLaunchKernelGGL((ln_bwd_rg_kernel<BL, VP, ST, R>), grid2, dim3(BL * R), 0, s, (float*)DX->ptr, DX->strides[1], \
                       (const float*)DY->ptr, DY->strides[1], (float*)DW->ptr, DW->strides[1], (float*)DB->ptr, \
                       DB->strides[1], (const float*)X->ptr, X->strides[1], (const float*)W->ptr,               \
                       (const float*)Mean->ptr, (const float*)Rstd->ptr, (int)N, M, G, S2)
#define RGS(BL, VP, R)                 \
    do {                               \
        if (stream_in) RGK(BL, VP, true, R); \
        else RGK(BL, VP, false, R);    \
    } while (0)
        if (vecs <= 64) { RGS(64, 1, 8); set_variant("ln_bwd_regs_b512_v1_rg8"); }
        else if (vecs <= 128) { RGS(64, 2, 8); set_variant("ln_bwd_regs_b512_v2_rg8"); }
        else if (vecs <= 256) { RGS(256, 1, 2); set_variant("ln_bwd_regs_b512_v1_rg2"); }
        else if (vecs <= 512) { RGS(256, 2, 2); set_variant("ln_bwd_regs_b512_v2_rg2"); }
        else if (vecs <= 1024) { RGS(256, 4, 2); set_variant("ln_bwd_regs_b512_v4_rg2"); }
        else { RGS(512, 4, 1); set_variant("ln_bwd_regs_b512_v4_rg1"); }
#undef RGS
#undef RGK
    } else if (al && vecs > 2048 && vecs <= kWideFloats / 4 && !one_group && G <= 256) {
        // one workgroup of 1024 lanes per CU
        int64_t Sw = cld((int64_t)256, (int64_t)G);
        if (Sw > rows_per_slot) Sw = rows_per_slot;
        if (Sw < 1) Sw = 1;
        hipLaunchKernelGGL(ln_bwd_wide_kernel, dim3((unsigned)(G * Sw)), dim3(kWideLanes), 0, s, (float*)DX->ptr, DX->strides[1],
                           (const float*)DY->ptr, DY->strides[1], (float*)DW->ptr, DW->strides[1], (float*)DB->ptr,
                           DB->strides[1], (const float*)X->ptr, X->strides[1], (const float*)W->ptr,
                           (const float*)Mean->ptr, (const float*)Rstd->ptr, (int)N, M, G, (int)Sw);
        set_variant("ln_bwd_wide_b1024_v4_lds_lookahead");
    } else if (!al) launch_bwd<false, false>(ARGS);
    else if (stream_in) launch_bwd<true, true>(ARGS);
    else launch_bwd<true, false>(ARGS);
#undef ARGS
    return launch_status();
}

static int dwdb_impl(const mi_tile_array* DW, const mi_tile_array* DB, const mi_tile_array* FINAL_DW,
                     const mi_tile_array* FINAL_DB, int TILE_M, int TILE_N, bool clear, void* stream) {
    MI_CHECK(check_f32(DW, 2));
    MI_CHECK(check_f32(DB, 2));
    MI_CHECK(check_f32(FINAL_DW, 1));
    MI_CHECK(check_f32(FINAL_DB, 1));
    if (!is_pow2(TILE_M) || !is_pow2(TILE_N)) return MI_E_TILE;
    const int64_t N = DW->sizes[0], G = DW->sizes[1];
    if (!same_shape(DW, DB) || FINAL_DW->sizes[0] != N || FINAL_DB->sizes[0] != N) return MI_E_SHAPE;
    if (N > 1 && (FINAL_DW->strides[0] != 1 || FINAL_DB->strides[0] != 1)) return MI_E_STRIDE;
    if (cld(N, (int64_t)TILE_N) > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (N == 0) return MI_OK;
    if (G > 0x7fffffff) return MI_E_SHAPE;
    const dim3 grid((unsigned)cld(N, (int64_t)64));
    if (clear)
        hipLaunchKernelGGL(ln_dwdb_kernel<true>, grid, dim3(1024), 0, (hipStream_t)stream, (float*)DW->ptr, DW->strides[1],
                           (float*)DB->ptr, DB->strides[1], (float*)FINAL_DW->ptr, (float*)FINAL_DB->ptr, N, (int)G);
    else
        hipLaunchKernelGGL(ln_dwdb_kernel<false>, grid, dim3(1024), 0, (hipStream_t)stream, (float*)DW->ptr, DW->strides[1],
                           (float*)DB->ptr, DB->strides[1], (float*)FINAL_DW->ptr, (float*)FINAL_DB->ptr, N, (int)G);
    set_variant(clear ? "ln_dwdb_b1024_clear" : "ln_dwdb_b1024");
    return launch_status();
}

extern "C" int mi_layer_norm_bwd_dwdb(const mi_tile_array* DW, const mi_tile_array* DB,
                                      const mi_tile_array* FINAL_DW, const mi_tile_array* FINAL_DB,
                                      int TILE_M, int TILE_N, void* stream) {
    return dwdb_impl(DW, DB, FINAL_DW, FINAL_DB, TILE_M, TILE_N, false, stream);
}

// Backward in one call with the partial slots in the library's static scratch:
// layer_norm_bwd_dx_partial_dwdb and layer_norm_bwd_dwdb (layernorm.jl:245-251 issues a zero fill and
// the same two steps on buffers its caller allocated, layernorm.jl:226-228; here the final kernel
// leaves the slots zeroed for the next call, so the fill is not a launch).  Calls nothing that allocates.
extern "C" int mi_layer_norm_bwd_static(const mi_tile_array* DX, const mi_tile_array* DY,
                                        const mi_tile_array* X, const mi_tile_array* W,
                                        const mi_tile_array* Mean, const mi_tile_array* Rstd,
                                        const mi_tile_array* FINAL_DW, const mi_tile_array* FINAL_DB,
                                        int GROUP_SIZE_M, int TILE_M, int TILE_N, void* stream) {
    MI_CHECK(check_f32(X, 2));
    MI_CHECK(check_f32(FINAL_DW, 1));
    MI_CHECK(check_f32(FINAL_DB, 1));
    if (GROUP_SIZE_M < 1) return MI_E_ARG;
    const int64_t N = X->sizes[0], G = GROUP_SIZE_M;
    if (FINAL_DW->sizes[0] != N || FINAL_DB->sizes[0] != N) return MI_E_SHAPE;
    // rows of the slot matrices are padded to whole 16-byte vectors
    const int64_t ld = (N + 3) / 4 * 4;
    if (ld * G > kScratchFloats) return MI_E_SCRATCH;
    float* base = nullptr;
    MI_CHECK(scratch_ptr(&base, (hipStream_t)stream));
    mi_tile_array dw = {}, db = {};
    dw.ptr = base;
    db.ptr = base + kScratchFloats;
    for (mi_tile_array* a : {&dw, &db}) {
        a->dtype = MI_F32;
        a->ndim = 2;
        a->sizes[0] = N;
        a->sizes[1] = G;
        a->strides[0] = 1;
        a->strides[1] = ld;
    }
    if (N == 0) return MI_OK;
    // The array is all zero when the library is loaded, and the final kernel of every call puts back the zeros where it
    // has read sums: a call normally finds its slots ready and is two launches.  Only after a call that did not get
    // as far as its final kernel (a failed launch) is the whole array filled first.
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (__atomic_exchange_n(&g_scratch_dirty[dev], true, __ATOMIC_ACQ_REL)) {
        const int64_t nvec = kScratchFloats / 4;
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, (hipStream_t)stream, (f32x4*)base,
                           (f32x4*)(base + kScratchFloats), nvec);
        MI_CHECK(launch_status());
    }
    MI_CHECK(mi_layer_norm_bwd_dx_partial_dwdb(DX, DY, &dw, &db, X, W, Mean, Rstd, nullptr, GROUP_SIZE_M,
                                               TILE_N, stream));
    MI_CHECK(dwdb_impl(&dw, &db, FINAL_DW, FINAL_DB, TILE_M, TILE_N, true, stream));
    __atomic_store_n(&g_scratch_dirty[dev], false, __ATOMIC_RELEASE);
    return MI_OK;
}
