// Matrix multiplication: stand-ins for matmul_kernel (examples/matmul.jl:28-60) and
// batch_matmul_kernel (examples/batchmatmul.jl:15-56) of the reference.
//
// C(M,N) = A(M,K) * B(K,N), all column-major (first index contiguous), fp32 accumulation.
// In memory A is "M-contiguous" (row k of A^T holds M consecutive values) and B is
// "K-contiguous" (column n of B holds K consecutive values).  CDNA4 MFMA wants, for both
// operands, the K values of one row/column packed in a lane; B has that shape already, A is
// brought to it with the LDS transpose read ds_read_b64_tr_b16.  The MFMA's row operand
// carries n and its column operand (lane % 32) carries m, so that the 32 lanes of a
// half-wave hold 32 consecutive m of one column of C and every store is a full 128-byte
// line.
//
// Kernels:
//   gemm16_generic   f16/bf16, 64x64x32 workgroup tile, any shape / stride / alignment
//                    (ragged edges are zero-padded on load and clipped on store, as
//                    ct.load(padding_mode=Zero) / ct.store do).
//   gemm16_mid       f16/bf16, 128x128x32 workgroup tile with a register look-ahead of one K step, any
//                    shape; used for larger problems that gemm16_big does not take (rows that are
//                    not 16-byte aligned, K below 256).
//   gemm16_big       (gemm_big.hip) f16/bf16, 256x256 workgroup tile, 4 waves of 128x128 (or 256x128 /
//                    128x128 tiles for problems with few tiles), K step 32 through a ring of four LDS
//                    stages filled by direct global->LDS loads, XOR-swizzled LDS layouts; used when M
//                    and K are multiples of 8, K >= 256, everything is 16-byte aligned and there are
//                    at least 16 tiles of 128x128 (ragged edges in M, N and K are handled on the way in).
//   gemm32           fp32 via v_mfma_f32_32x32x2_f32 (gfx950 has no TF32-class MFMA;
//                    the reference rounds fp32 operands to TF32, matmul.jl:49-52), 128x128x16 tile,
//                    any shape; gemm32_big (gemm32_big.hip), the fp32 sibling of gemm16_big, takes
//                    the problems whose rows are 16-byte aligned (M, K multiples of 4, K >= 128).
//
// The (tm, tn, tk) tile constants of the reference only fix the block->data mapping and
// the L2 swizzle; results do not depend on them, and the physical tiling above is chosen
// for CDNA4.  FLOP count: 2*M*N*K per batch.
#include <cstdio>

#include "gemm_common.h"
#include "gemm_direct.h"

namespace {

using namespace mi;
using namespace mi::gemm;

// 16 bytes from an address that is aligned for its elements only.  Global memory takes unaligned vector accesses (a
// row of a dense matrix whose leading dimension is odd starts anywhere): one instruction either way, where eight
// 2-byte loads per lane ran a 4095^3 problem at a tenth of the aligned rate.
template <typename V, typename T>
__device__ __forceinline__ V ld16(const T* p) {
    V v;
    __builtin_memcpy(&v, p, sizeof(V));
    return v;
}

// A vector of NE elements of a row at p of which only the first `valid` belong to the matrix (the row ends there; valid
// may be <= 0 or >= NE); `room` elements from p on lie inside the array (up to the end of its last row).  Where the
// whole vector is readable it is read whole and the elements past the row's end -- the start of the next row, or the
// parent's padding -- are zeroed in registers; only at the end of the last row does the tail go element by element.
// (Element-wise tails on every row made the workgroups on the matrix edge five times slower than the others, and a
// launch waited for them.)
template <typename V, int NE, typename T>
__device__ __forceinline__ V ld_edge(const T* p, int64_t valid, int64_t room) {
    V v = {0};
    if (valid <= 0) return v;
    if (room >= NE) {
        v = ld16<V>(p);
#pragma unroll
        for (int q = 1; q < NE; ++q)
            if (q >= valid) v[q] = 0;
    } else {
#pragma unroll
        for (int q = 0; q < NE; ++q)
            if (q < valid) v[q] = p[q];
    }
    return v;
}

// ---- generic 16-bit kernel ---------------------------------------------------------------
// Workgroup tile 64(m) x 64(n), K step 32, 4 waves as 2x2 of 32x32.
constexpr int GT = 64, GK = 32, GA_PITCH = GT + 8, GB_PITCH = GK + 8;

template <typename E, typename OutT>
__global__ __launch_bounds__(256) void gemm16_generic(
    const unsigned short* __restrict__ A, int64_t lda, int64_t sa, const unsigned short* __restrict__ B,
    int64_t ldb, int64_t sb, OutT* __restrict__ C, int64_t ldc, int64_t sc, int M, int N, int K,
    int tiles_m, int tiles_mn) {
    __shared__ __attribute__((aligned(16))) unsigned short As[GK * GA_PITCH];  // [k][m]
    __shared__ __attribute__((aligned(16))) unsigned short Bs[GT * GB_PITCH];  // [n][k]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bz = blockIdx.x / (unsigned)tiles_mn, L = blockIdx.x - bz * tiles_mn;   // (tile, batch entry), tiles fastest
    const int bm = L % tiles_m, bn = L / tiles_m;
    const int64_t m0 = (int64_t)bm * GT, n0 = (int64_t)bn * GT;
    A += (int64_t)bz * sa;
    B += (int64_t)bz * sb;
    C += (int64_t)bz * sc;
    const int wm = (wave & 1) * 32, wn = (wave >> 1) * 32;

    const int ak = tid >> 3, am = (tid & 7) * 8;  // A tile: row k, 8 consecutive m
    const int bnn = tid >> 2, bk = (tid & 3) * 8;  // B tile: column n, 8 consecutive k
    f32x16 acc = {0};

    for (int k0 = 0; k0 < K; k0 += GK) {
        s16x8 va = {0}, vb = {0};
        {
            const int64_t gm = m0 + am;
            const int gk = k0 + ak;
            if (gk < K) {
                const int64_t o = gm + (int64_t)gk * lda;
                va = ld_edge<s16x8, 8>((const short*)A + o, M - gm, (int64_t)(K - 1) * lda + M - o);
            }
            const int64_t gn = n0 + bnn;
            const int gk2 = k0 + bk;
            if (gn < N) {
                const int64_t o = gk2 + gn * ldb;
                vb = ld_edge<s16x8, 8>((const short*)B + o, K - gk2, (int64_t)(N - 1) * ldb + K - o);
            }
        }
        __syncthreads();  // previous iteration's fragment reads are done
        *reinterpret_cast<s16x8*>(&As[ak * GA_PITCH + am]) = va;
        *reinterpret_cast<s16x8*>(&Bs[bnn * GB_PITCH + bk]) = vb;
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < GK / 16; ++ks) {
            s16x8 fn = *reinterpret_cast<const s16x8*>(&Bs[(wn + (lane & 31)) * GB_PITCH + ks * 16 + 8 * (lane >> 5)]);
            s16x8 fm = lds_read_tr_k16(&As[(ks * 16) * GA_PITCH + wm], GA_PITCH, lane);
            acc = E::mfma32(fn, fm, acc);
        }
    }
    const int64_t gm = m0 + wm + (lane & 31);
    if (gm < M) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t gn = n0 + wn + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (gn < N) C[gm + gn * ldc] = cvt_out<E, OutT>(acc[r]);
        }
    }
}

// ---- 128 x 128 16-bit kernel ----------------------------------------------------------------
// Workgroup tile 128(m) x 128(n), K step 32, 4 waves as 2x2 of 64x64 (four 32x32x16 MFMAs per 16
// k, one LDS fragment read per MFMA).  The next K step's operands are requested into registers
// before the current step's MFMAs and cross the workgroup barriers in flight (the barriers wait
// for LDS accesses only).  Any shape: workgroups whose tile is interior load without predicates (16 bytes
// per lane, aligned or not); the others zero-pad, element by element where a vector crosses the edge.
constexpr int MT = 128, MA_PITCH = MT + 8, MB_PITCH = GK + 8;

__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0); vmcnt and expcnt at their maxima
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <typename E, typename OutT>
__global__ __launch_bounds__(256) void gemm16_mid(
    const unsigned short* __restrict__ A, int64_t lda, int64_t sa, const unsigned short* __restrict__ B,
    int64_t ldb, int64_t sb, OutT* __restrict__ C, int64_t ldc, int64_t sc, int M, int N, int K,
    int tiles_m, int tiles_mn) {
    __shared__ __attribute__((aligned(16))) unsigned short As[GK * MA_PITCH];  // [k][m]
    __shared__ __attribute__((aligned(16))) unsigned short Bs[MT * MB_PITCH];  // [n][k]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bz = blockIdx.x / (unsigned)tiles_mn, L = blockIdx.x - bz * tiles_mn;   // (tile, batch entry), tiles fastest
    const int bm = L % tiles_m, bn = L / tiles_m;
    const int64_t m0 = (int64_t)bm * MT, n0 = (int64_t)bn * MT;
    A += (int64_t)bz * sa;
    B += (int64_t)bz * sb;
    C += (int64_t)bz * sc;
    const int wm = (wave & 1) * 64, wn = (wave >> 1) * 64;
    const int ak = tid >> 4, am = (tid & 15) * 8;   // A tile: rows k = ak and ak + 16, 8 consecutive m
    const int bnn = tid >> 2, bk = (tid & 3) * 8;   // B tile: columns n = bnn and bnn + 64, 8 consecutive k
    // Workgroups on the M or N edge load like the others wherever that reads existing memory: a row of B past the
    // last one is replaced by the last one, a vector of A past the end of its row reads on into the next row; what they
    // bring only reaches elements of C that are never stored.  Left to the element-wise path: the K steps in which
    // such a vector of A would pass the end of the array (the last rows), and a last K step that is not whole.
    const int64_t over_m = m0 + MT - M;   // > 0: elements by which the tile's rows overrun the matrix
    const int64_t bn_row[2] = {n0 + bnn < N ? n0 + bnn : N - 1, n0 + bnn + 64 < N ? n0 + bnn + 64 : N - 1};

    f32x16 acc[2][2] = {};
    s16x8 va[2], vb[2];
    int validA = 8, validB = 8;   // elements of the staged vectors that belong to the matrix
    auto gload = [&](int k0) {
        if (k0 + GK <= K && (over_m <= 0 || (lda >= 0 && (int64_t)(K - k0 - GK) * lda >= over_m))) {   // same for the whole workgroup
            validA = validB = 8;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                va[h] = ld16<s16x8>(A + m0 + am + (int64_t)(k0 + ak + 16 * h) * lda);
                vb[h] = ld16<s16x8>(B + k0 + bk + bn_row[h] * ldb);
            }
            return;
        }
        // Edge: whole vectors wherever they are readable; what lies past the end of a row is zeroed when the vector
        // goes to LDS, a K step later (zeroing it here would wait for the load here, and the edge workgroups, with no
        // look-ahead left, ran five times longer than the others).
        const int64_t gm = m0 + am;
        const int gk2 = k0 + bk;
        validA = M - gm < 8 ? (M - gm > 0 ? (int)(M - gm) : 0) : 8;
        validB = K - gk2 < 8 ? (K - gk2 > 0 ? K - gk2 : 0) : 8;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            va[h] = vb[h] = s16x8{0};
            const int gk = k0 + ak + 16 * h;
            if (gk < K && validA > 0) {
                const int64_t o = gm + (int64_t)gk * lda;
                if ((int64_t)(K - 1) * lda + M - o >= 8) va[h] = ld16<s16x8>(A + o);
                else va[h] = ld_edge<s16x8, 8>((const short*)A + o, validA, 0);
            }
            const int64_t gn = n0 + bnn + 64 * h;
            if (gn < N && validB > 0) {
                const int64_t o = gk2 + gn * ldb;
                if ((int64_t)(N - 1) * ldb + K - o >= 8) vb[h] = ld16<s16x8>(B + o);
                else vb[h] = ld_edge<s16x8, 8>((const short*)B + o, validB, 0);
            }
        }
    };
    auto keep = [](s16x8 v, int valid) {
#pragma unroll
        for (int q = 1; q < 8; ++q)
            if (q >= valid) v[q] = 0;
        return v;
    };
    gload(0);
    for (int k0 = 0; k0 < K; k0 += GK) {
        lds_barrier();  // previous iteration's fragment reads are done
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<s16x8*>(&As[(ak + 16 * h) * MA_PITCH + am]) = validA < 8 ? keep(va[h], validA) : va[h];
            *reinterpret_cast<s16x8*>(&Bs[(bnn + 64 * h) * MB_PITCH + bk]) = validB < 8 ? keep(vb[h], validB) : vb[h];
        }
        lds_barrier();
        if (k0 + GK < K) gload(k0 + GK);
#pragma unroll
        for (int ks = 0; ks < GK / 16; ++ks) {
            s16x8 fn[2], fm[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fn[i] = *reinterpret_cast<const s16x8*>(&Bs[(wn + 32 * i + (lane & 31)) * MB_PITCH + ks * 16 + 8 * (lane >> 5)]);
                fm[i] = lds_read_tr_k16(&As[(ks * 16) * MA_PITCH + wm + 32 * i], MA_PITCH, lane);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = E::mfma32(fn[j], fm[i], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t gm = m0 + wm + 32 * i + (lane & 31);
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t gn = n0 + wn + 32 * j + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gn < N) C[gm + gn * ldc] = cvt_out<E, OutT>(acc[i][j][r]);
            }
    }
}

// ---- fp32 kernel ---------------------------------------------------------------------------
// Workgroup tile 128(m) x 128(n), K step 16, 4 waves as 2x2 of 64x64 (2x2 MFMA 32x32x2).
// Pitch 160 floats: consecutive rows are 32 banks apart, so the two half-waves of a fragment read
// (rows kk and kk + 1, 32 consecutive floats each) cover the 64 banks once.
constexpr int FT = 128, FK = 16, F_PITCH = FT + 32;

__global__ __launch_bounds__(256) void gemm32_kernel(const float* __restrict__ A, int64_t lda, int64_t sa,
                                                     const float* __restrict__ B, int64_t ldb, int64_t sb,
                                                     float* __restrict__ C, int64_t ldc, int64_t sc, int M,
                                                     int N, int K, int tiles_m, int tiles_mn) {
    __shared__ __attribute__((aligned(16))) float As[FK * F_PITCH];  // [k][m]
    __shared__ __attribute__((aligned(16))) float Bs[FK * F_PITCH];  // [k][n]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bz = blockIdx.x / (unsigned)tiles_mn, L = blockIdx.x - bz * tiles_mn;   // (tile, batch entry), tiles fastest
    const int bm = L % tiles_m, bn = L / tiles_m;
    const int64_t m0 = (int64_t)bm * FT, n0 = (int64_t)bn * FT;
    A += (int64_t)bz * sa;
    B += (int64_t)bz * sb;
    C += (int64_t)bz * sc;
    const int wm = (wave & 1) * 64, wn = (wave >> 1) * 64;
    const int ak = tid >> 4, am = (tid & 15) * 4;  // A tile: row k, m = am .. am+3 and 64 + am .. 64 + am+3
    const int bnn = tid & 127, bk = (tid >> 7) * 8;  // B tile: column n, 8 consecutive k; a wave's 64 lanes
                                                     // transpose into 64 consecutive floats of one row
    f32x16 acc[2][2] = {};

    for (int k0 = 0; k0 < K; k0 += FK) {
        float va[8], vb[8];
        {
            const int64_t gm = m0 + am;
            const int gk = k0 + ak;
            f32x4 t0 = {0}, t1 = {0};
            if (gk < K) {
                const int64_t o = gm + (int64_t)gk * lda, room = (int64_t)(K - 1) * lda + M - o;
                t0 = ld_edge<f32x4, 4>(A + o, M - gm, room);
                t1 = ld_edge<f32x4, 4>(A + o + 64, M - gm - 64, room - 64);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) { va[q] = t0[q]; va[4 + q] = t1[q]; }
            const int64_t gn = n0 + bnn;
            const int gk2 = k0 + bk;
            t0 = t1 = f32x4{0};
            if (gn < N) {
                const int64_t o = gk2 + gn * ldb, room = (int64_t)(N - 1) * ldb + K - o;
                t0 = ld_edge<f32x4, 4>(B + o, K - gk2, room);
                t1 = ld_edge<f32x4, 4>(B + o + 4, K - gk2 - 4, room - 4);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) { vb[q] = t0[q]; vb[4 + q] = t1[q]; }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 2; ++q)   // 16 lanes x 16 bytes = one contiguous 256-byte run per store
            *reinterpret_cast<f32x4*>(&As[ak * F_PITCH + am + 64 * q]) = f32x4{va[4 * q], va[4 * q + 1], va[4 * q + 2], va[4 * q + 3]};
#pragma unroll
        for (int q = 0; q < 8; ++q) Bs[(bk + q) * F_PITCH + bnn] = vb[q];
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < FK; kk += 2) {
            float fm[2], fn[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fm[i] = As[(kk + (lane >> 5)) * F_PITCH + wm + 32 * i + (lane & 31)];
                fn[i] = Bs[(kk + (lane >> 5)) * F_PITCH + wn + 32 * i + (lane & 31)];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fn[j], fm[i], acc[i][j], 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t gm = m0 + wm + 32 * i + (lane & 31);
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t gn = n0 + wn + 32 * j + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gn < N) C[gm + gn * ldc] = acc[i][j][r];
            }
    }
}

// ---- host side -------------------------------------------------------------------------------

int validate(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C, int ndim, int tm,
             int tn, int tk, Problem* p) {
    MI_CHECK(check_array(A, ndim));
    MI_CHECK(check_array(B, ndim));
    MI_CHECK(check_array(C, ndim));
    if (A->dtype != B->dtype) return MI_E_DTYPE;
    const bool fp8 = A->dtype == MI_F8E4M3FN || A->dtype == MI_F8E5M2;
    if (A->dtype != MI_F16 && A->dtype != MI_BF16 && A->dtype != MI_F32 && !fp8) return MI_E_DTYPE;
    // fp8 operands accumulate in fp32 and store f32, f16 or bf16 (the accumulator types the reference
    // allows are f16 and f32: ext/DLFP8TypesExt.jl:15-19)
    if (fp8 ? (C->dtype != MI_F32 && C->dtype != MI_F16 && C->dtype != MI_BF16)
            : (C->dtype != A->dtype && C->dtype != MI_F32))
        return MI_E_DTYPE;
    if (!is_pow2(tm) || !is_pow2(tn) || !is_pow2(tk)) return MI_E_TILE;
    const int64_t M = A->sizes[0], K = A->sizes[1], N = B->sizes[1];
    if (B->sizes[0] != K || C->sizes[0] != M || C->sizes[1] != N) return MI_E_SHAPE;
    int64_t batch = 1;
    if (ndim == 3) {
        batch = A->sizes[2];
        if (B->sizes[2] != batch || C->sizes[2] != batch) return MI_E_SHAPE;
        if (batch > MI_MAX_GRID_DIM) return MI_E_GRID;   // the reference's grid is (cld(M,tm), cld(N,tn), Batch), batchmatmul.jl:78-80
    }
    if (M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return MI_E_SHAPE;
    // the kernels number (tile, batch entry) pairs in one grid dimension of 256-lane workgroups, and a launch takes
    // fewer than 2^32 lanes per dimension; their smallest tile is 64 x 64
    if (cld(M, (int64_t)64) * cld(N, (int64_t)64) * batch > MI_MAX_GRID_DIM) return MI_E_GRID;
    if (cld(M, (int64_t)tm) > MI_MAX_GRID_DIM || cld(N, (int64_t)tn) > MI_MAX_GRID_DIM ||
        cld(M, (int64_t)tm) * cld(N, (int64_t)tn) > MI_MAX_GRID_DIM)
        return MI_E_GRID;
    if ((M > 1 && (A->strides[0] != 1 || C->strides[0] != 1)) || (K > 1 && B->strides[0] != 1))
        return MI_E_STRIDE;
    p->A = A->ptr; p->B = B->ptr; p->C = C->ptr;
    p->lda = A->strides[1]; p->ldb = B->strides[1]; p->ldc = C->strides[1];
    p->sa = ndim == 3 ? A->strides[2] : 0;
    p->sb = ndim == 3 ? B->strides[2] : 0;
    p->sc = ndim == 3 ? C->strides[2] : 0;
    p->M = (int)M; p->N = (int)N; p->K = (int)K; p->batch = (int)batch;
    p->in_dtype = A->dtype; p->out_dtype = C->dtype;
    return MI_OK;
}

template <typename E, typename OutT>
void launch_mid16(const Problem& p, hipStream_t s) {
    const int tiles_m = (int)cld((int64_t)p.M, (int64_t)MT), tiles_n = (int)cld((int64_t)p.N, (int64_t)MT);
    hipLaunchKernelGGL((gemm16_mid<E, OutT>), dim3((unsigned)(tiles_m * tiles_n * p.batch)), dim3(256), 0,
                       s, (const unsigned short*)p.A, p.lda, p.sa, (const unsigned short*)p.B, p.ldb, p.sb,
                       (OutT*)p.C, p.ldc, p.sc, p.M, p.N, p.K, tiles_m, tiles_m * tiles_n);
}

template <typename E, typename OutT>
void launch_generic16(const Problem& p, hipStream_t s) {
    const int tiles_m = (int)cld((int64_t)p.M, (int64_t)GT), tiles_n = (int)cld((int64_t)p.N, (int64_t)GT);
    hipLaunchKernelGGL((gemm16_generic<E, OutT>), dim3((unsigned)(tiles_m * tiles_n * p.batch)),
                       dim3(256), 0, s, (const unsigned short*)p.A, p.lda, p.sa, (const unsigned short*)p.B,
                       p.ldb, p.sb, (OutT*)p.C, p.ldc, p.sc, p.M, p.N, p.K, tiles_m, tiles_m * tiles_n);
}

int run(const Problem& p, hipStream_t s, bool may_split = true);

// A 16-bit or fp32 product whose tiles are whole rounds of the chip plus a thin strip -- 4097 x 4096 is 16 x 16 tiles of
// 256 x 256 and one more row of sixteen, which costs a second round -- is launched as the product without its last row
// and / or column of tiles plus those as one or two small products of their own (disjoint parts of C, one stream, no
// dependency).  Estimates in us, from what was measured at 4096^3 and scaled with K: the tile choices' own figures for
// the whole and the main part, a strip as its launches plus its K walk.  A split has to promise 10 %.  Measured (us,
// K = 4096 unless given):
//   f16   4096 x 4128 166 -> 131, 4352 x 4096 165 -> 137, 4097 x 4097 220 -> 182, 4097 x 4096 x 4100 247 -> 202,
//         4096 x 8448 287 -> 248, 8200 x 8192 558 -> 499 (4096^3: 123); left alone: 4400 x 4096 x 1024 (56; 66 split)
//   f32   4097 x 4096 1287 -> 1071, 4352 x 4096 1284 -> 1051, 4096 x 4100 x 2048 640 -> 504 (4096^3: 954)
// Not for fp8, where a second, nearly empty round costs little (4352 x 4096 92 against 59 + 36), and not to take rows
// off an M that is not a multiple of a chunk: what slows those products is the leading dimension, which a part keeps
// (f16 4095 x 4096 166 -> 174, e4m3 4100 x 4100 144 -> 169).  MI_GEMM_EDGE_SPLIT=0 switches it off.
bool edge_split(const Problem& p, hipStream_t s, int* status) {
    static const bool on = [] { const char* e = getenv("MI_GEMM_EDGE_SPLIT"); return !e || atoi(e) != 0; }();
    if (!on || p.batch != 1 || p.K < 1024 || p.M < 512 || p.N < 512) return false;
    const bool f16 = p.in_dtype == MI_F16 || p.in_dtype == MI_BF16, f32 = p.in_dtype == MI_F32;
    if (f16 ? !big16_applicable(p) : f32 ? !big32_applicable(p) : true) return false;
    const double ks = p.K / 4096.0;
    const int align = f16 ? 8 : 4;   // rows of A per 16-byte chunk
    // the whole product or a main part (us)
    auto whole = [&](const Problem& q) {
        if (f16) {
            int64_t c = 0;
            (void)pick_direct_tile(q, &c);
            return c * 1.37 * ks;
        }
        return big32_cost(q) * 59.0 * ks;
    };
    // a strip of r rows or columns by itself (us): f16 splits it over K (two launches, 10 us) unless K is off the chunks;
    // f32 walks K in one launch of small tiles
    auto strip = [&](int64_t r, int64_t other) {
        if (f16) return p.K % 8 ? 6.0 + 22.0 * ks : 10.0 + 9.5 * ks * (double)(r * other) / (256.0 * 4096.0);
        return 4.0 + 62.0 * ks * (other > 8192 ? other / 8192.0 : 1.0);
    };
    const double full = whole(p);
    if (full < (f16 ? 137.0 : 1100.0) * ks) return false;   // (less than about two rounds: the estimates are too coarse)
    const int rM = p.M % 256 ? p.M % 256 : 256, rN = p.N % 256 ? p.N % 256 : 256;
    // candidates: rows kept = all | up to the last tile row; columns kept = all | up to the last tile column
    const int keepM[2] = {p.M, p.M >= 768 ? p.M - rM : p.M};
    const int keepN[2] = {p.N, p.N >= 768 ? p.N - rN : p.N};
    int bm = p.M, bn = p.N;
    double best = full;
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 2; ++j) {
            const int m = keepM[i], n = keepN[j];
            if ((m == p.M && n == p.N) || m < 512 || n < 256) continue;
            Problem q = p;
            q.M = m;
            q.N = n;
            double t = whole(q);
            if (m < p.M) t += strip(p.M - m, p.N);
            if (n < p.N) t += strip(p.N - n, m);
            if (t < best) {
                best = t;
                bm = m;
                bn = n;
            }
        }
    if (best > 0.9 * full) return false;
    const int64_t esz = f32 ? 4 : 2, csz = p.out_dtype == MI_F32 ? 4 : 2;
    Problem main = p;
    main.M = bm;
    main.N = bn;
    int st = run(main, s, false);
    static thread_local char name[96];
    snprintf(name, sizeof name, "%s+edge_strips", last_variant_name());
    if (st == MI_OK && bm < p.M) {   // rows M' .. M - 1 of every column
        // (at least a chunk of rows, which is what the direct-to-LDS kernels take: a thinner strip starts inside the main
        // part and writes those rows of C a second time, behind the main launch on the same stream)
        const int rows = p.M - bm < align ? align : p.M - bm;
        Problem e = p;
        e.M = rows;
        e.A = (const char*)p.A + (int64_t)(p.M - rows) * esz;
        e.C = (char*)p.C + (int64_t)(p.M - rows) * csz;
        st = run(e, s, false);
    }
    if (st == MI_OK && bn < p.N) {   // columns N' .. N - 1 of the rows above that strip
        Problem e = p;
        e.M = bm;
        e.N = p.N - bn;
        e.B = (const char*)p.B + (int64_t)bn * p.ldb * esz;
        e.C = (char*)p.C + (int64_t)bn * p.ldc * csz;
        st = run(e, s, false);
    }
    set_variant(name);
    *status = st;
    return true;
}

int run(const Problem& p, hipStream_t s, bool may_split) {
    if (p.M == 0 || p.N == 0 || p.batch == 0) return MI_OK;
    if (may_split) {
        int st = MI_OK;
        if (edge_split(p, s, &st)) return st;
    }
    static const int force = [] { const char* e = getenv("MI_GEMM_KERNEL"); return e ? atoi(e) : 0; }();   // 1 generic, 2 mid, 3 big
    if (p.in_dtype == MI_F8E4M3FN || p.in_dtype == MI_F8E5M2) {
        fp8_launch(p, s);
        return launch_status();
    }
    if (p.in_dtype == MI_F32) {
        if (big32_applicable(p) && force != 1) {   // 16-byte aligned rows: the direct-to-LDS kernel
            big32_launch(p, s);
            return launch_status();
        }
        const int tiles_m = (int)cld((int64_t)p.M, (int64_t)FT), tiles_n = (int)cld((int64_t)p.N, (int64_t)FT);
        hipLaunchKernelGGL(gemm32_kernel, dim3((unsigned)(tiles_m * tiles_n * p.batch)), dim3(256), 0, s,
                           (const float*)p.A, p.lda, p.sa, (const float*)p.B, p.ldb, p.sb, (float*)p.C, p.ldc, p.sc,
                           p.M, p.N, p.K, tiles_m, tiles_m * tiles_n);
        set_variant("gemm32_128x128x16_mfma32x32x2");
        return launch_status();
    }
    const bool f32out = p.out_dtype == MI_F32;
    const int64_t tiles_mid = (int64_t)cld((int64_t)p.M, (int64_t)MT) * cld((int64_t)p.N, (int64_t)MT) * p.batch;
    // The direct-to-LDS kernel wherever it applies (16-byte aligned rows, K >= 256: with a shorter K the
    // problem is bound by the stores of C and smaller workgroups in several rounds overlap them better;
    // it picks its own tile size);
    // the register-staged 128x128 kernel for other shapes whose tiles give at least half the CUs work;
    // the 64x64 kernel for what is left (small problems).
    if (big16_applicable(p) && (force == 3 || force == 0)) {
        big16_launch(p, s);
        return launch_status();
    }
    if (force == 2 || (force == 0 && tiles_mid >= 128)) {
        if (p.in_dtype == MI_F16) {
            if (f32out) launch_mid16<F16, float>(p, s);
            else launch_mid16<F16, unsigned short>(p, s);
        } else {
            if (f32out) launch_mid16<BF16, float>(p, s);
            else launch_mid16<BF16, unsigned short>(p, s);
        }
        set_variant("gemm16_mid_128x128x32");
        return launch_status();
    }
    if (p.in_dtype == MI_F16) {
        if (f32out) launch_generic16<F16, float>(p, s);
        else launch_generic16<F16, unsigned short>(p, s);
    } else {
        if (f32out) launch_generic16<BF16, float>(p, s);
        else launch_generic16<BF16, unsigned short>(p, s);
    }
    set_variant("gemm16_generic_64x64x32");
    return launch_status();
}

}  // namespace

extern "C" int mi_matmul_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C, int tm,
                                int tn, int tk, void* stream) {
    Problem p;
    MI_CHECK(validate(A, B, C, 2, tm, tn, tk, &p));
    return run(p, (hipStream_t)stream);
}

extern "C" int mi_batch_matmul_kernel(const mi_tile_array* A, const mi_tile_array* B, const mi_tile_array* C,
                                      int tm, int tn, int tk, void* stream) {
    Problem p;
    MI_CHECK(validate(A, B, C, 3, tm, tn, tk, &p));
    return run(p, (hipStream_t)stream);
}
