// Entry points whose kernels are not written yet.
#include "common.h"
extern "C" int mi_matmul_kernel(const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, int, int, int, void*) { return MI_E_UNSUPPORTED; }
extern "C" int mi_batch_matmul_kernel(const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, int, int, int, void*) { return MI_E_UNSUPPORTED; }
extern "C" int mi_fmha_kernel(const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, float, int32_t, int, int, int, int, int, int, int, void*) { return MI_E_UNSUPPORTED; }
extern "C" int mi_fused_moe_kernel(const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, int, int, int, int, int, const mi_tile_array*, void*) { return MI_E_UNSUPPORTED; }
extern "C" int mi_silu_and_mul_kernel(const mi_tile_array*, const mi_tile_array*, const mi_tile_array*, int, void*) { return MI_E_UNSUPPORTED; }
extern "C" int mi_moe_sum_topk(const mi_tile_array*, const mi_tile_array*, void*) { return MI_E_UNSUPPORTED; }
