// Pieces shared by the two direct-to-LDS GEMM kernels (gemm_big.hip: 16-bit operands, gemm32_big.hip: fp32).
#pragma once
#include <cstdlib>

#include "gemm_common.h"

namespace mi {
namespace gemm {

// sched_group_barrier masks
#define SG_MFMA 0x008
#define SG_VMEM 0x010
#define SG_DSRD 0x100

__device__ __forceinline__ void gload_lds16(const void* g, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

template <int VMCNT>
__device__ __forceinline__ void stage_barrier() {
    // My reads of the current stage are done (lgkmcnt(0)) and my transfers into the next stage
    // have landed (vmcnt leaves only the VMCNT youngest transfers in flight); then meet the
    // other waves.  The wait is the builtin, not inline asm, so that the compiler's own
    // wait-count bookkeeping sees it and does not add a full vmcnt(0) drain before the
    // following LDS reads.  gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14].
    constexpr int imm = (VMCNT & 15) | (7 << 4) | (0 << 8) | ((VMCNT >> 4) << 14);
    __builtin_amdgcn_s_waitcnt(imm);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

inline int64_t tiles_of(const Problem& p, int btm, int btn) {
    return (int64_t)((p.M + btm - 1) / btm) * ((p.N + btn - 1) / btn) * p.batch;
}

// Tile size: whichever needs least time by "rounds of workgroups x time of a round".  Measured time of
// one K step of a round (us): 256x256 0.63 (a quarter of the CUs busy) to 0.93 (all busy: the clock
// drops); 256x128 0.42 to 0.51; 128x128 0.33 with one workgroup per CU, 0.58 when CUs hold two.
// f16 examples (us, 256x256 / 256x128 / 128x128): 1024^3 23 / 15 / 10, 2048^3 40 / 27 / 21,
// 2560^3 51 / 37 / 46, 4096 x 2048 x 4096 77 / 65 / 74, 3072^3 64 / 83 / 77, 4096^3 119 / 128 / 144.
// `cost` (optional): the estimate for the tile chosen, in units of about 1 % of the 4096^3 product's time per 4096 of K.
inline int pick_direct_tile(const Problem& p, int64_t* cost = nullptr) {
    static const int force = [] { const char* e = getenv("MI_GEMM_BIG_TILE"); return e ? atoi(e) : 0; }();   // 44, 42 or 22
    const int64_t t44 = tiles_of(p, 256, 256), t42 = tiles_of(p, 256, 128), t22 = tiles_of(p, 128, 128);
    const int64_t c44 = (t44 + 255) / 256 * 90, c42 = (t42 + 255) / 256 * 50;
    const int64_t c22 = t22 <= 256 ? 33 : (t22 + 511) / 512 * 60;
    const int t = c22 <= c42 && c22 <= c44 ? 22 : c42 <= c44 ? 42 : 44;
    if (cost) *cost = t == 22 ? c22 : t == 42 ? c42 : c44;
    if (force == 44 || force == 42 || force == 22) return force;
    return t;
}

}  // namespace gemm
}  // namespace mi
