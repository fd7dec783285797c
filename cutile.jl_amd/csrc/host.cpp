// Host-only entry points of libmi355tile: version / error strings, the variant record, and
// the two integer host helpers of the reference's examples (swizzle_2d, moe_align_tile_size).
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

#include "common.h"

namespace mi {
static thread_local const char* g_variant = "";
void set_variant(const char* name) { g_variant = name; }
const char* last_variant_name() { return g_variant; }

static std::atomic<int> g_scratch_under_capture{[] {
    const char* e = getenv("MI_SCRATCH_UNDER_CAPTURE");
    return e && e[0] == '1' ? 1 : 0;
}()};
bool scratch_under_capture() { return g_scratch_under_capture.load(std::memory_order_relaxed) != 0; }
}  // namespace mi

extern "C" int mi_scratch_under_capture(int allow) {
    return mi::g_scratch_under_capture.exchange(allow ? 1 : 0, std::memory_order_relaxed);
}

extern "C" int mi_version(void) { return MI355TILE_VERSION; }

extern "C" const char* mi_last_variant(void) { return mi::g_variant; }

extern "C" const char* mi_strerror(int code) {
    switch (code) {
        case MI_OK: return "success";
        case MI_E_NULL: return "a required pointer is NULL";
        case MI_E_DTYPE: return "unsupported or mismatching element type";
        case MI_E_RANK: return "wrong number of dimensions";
        case MI_E_SHAPE: return "array sizes do not agree";
        case MI_E_STRIDE: return "unsupported layout (dimension 1 must be contiguous)";
        case MI_E_TILE: return "tile constant must be a positive power of two supported by the kernel";
        case MI_E_GRID: return "grid dimension exceeds the 24-bit limit";
        case MI_E_ALIGN: return "pointer is not aligned to its element size";
        case MI_E_ARG: return "invalid scalar argument";
        case MI_E_UNSUPPORTED: return "configuration not supported";
        case MI_E_SCRATCH: return "problem exceeds the library's static scratch buffer";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

// Floor division / ceil division on int32 with Julia's semantics for the non-negative
// operands that occur here.
static inline int32_t cld32(int32_t a, int32_t b) { return (a + b - 1) / b; }

// Reference: examples/matmul.jl:13-24 (duplicated at examples/moe.jl:20-31).
extern "C" void mi_swizzle_2d(int32_t M, int32_t N, int32_t tm, int32_t tn, int32_t group_size_m,
                              int32_t bid, int32_t* bid_m, int32_t* bid_n) {
    const int32_t num_bid_m = cld32(M, tm);
    const int32_t num_bid_n = cld32(N, tn);
    const int32_t num_bid_in_group = group_size_m * num_bid_n;
    const int32_t bid0 = bid - 1;
    const int32_t group_id = bid0 / num_bid_in_group;
    const int32_t first_bid_m = group_id * group_size_m;
    const int32_t gsm = std::min(num_bid_m - first_bid_m, group_size_m);
    if (bid_m) *bid_m = first_bid_m + bid0 % gsm + 1;
    if (bid_n) *bid_n = (bid0 % num_bid_in_group) / gsm + 1;
}

// Reference: examples/moe.jl:142-183.  A counting sort reproduces the stable sortperm by
// expert id over the slot-fastest flattening of topk_ids.
extern "C" int mi_moe_align_tile_size(const int64_t* topk_ids, int64_t num_tokens, int64_t topk,
                                      int tile_m, int num_experts, int32_t* sorted_token_ids_out,
                                      int32_t* sorted_expert_ids_out, int64_t* total_blocks_out) {
    if (num_tokens < 0 || topk < 0 || num_experts < 1) return MI_E_ARG;
    if (!mi::is_pow2(tile_m)) return MI_E_TILE;
    const int64_t total = num_tokens * topk;
    if (total > 0 && !topk_ids) return MI_E_NULL;
    if (total + 1 > 0x7fffffffLL) return MI_E_SHAPE;
    std::vector<int64_t> counts(num_experts, 0);
    // flat index f (0-based) = token*topk + slot; topk_ids is column-major (num_tokens, topk)
    for (int64_t t = 0; t < num_tokens; ++t)
        for (int64_t k = 0; k < topk; ++k) {
            const int64_t e = topk_ids[t + k * num_tokens];
            if (e < 1 || e > num_experts) return MI_E_ARG;
            counts[e - 1]++;
        }
    std::vector<int64_t> block_start(num_experts + 1, 0);
    for (int e = 0; e < num_experts; ++e)
        block_start[e + 1] = block_start[e] + mi::cld(counts[e], (int64_t)tile_m);
    const int64_t total_blocks = block_start[num_experts];
    if (total_blocks_out) *total_blocks_out = total_blocks;
    if (!sorted_token_ids_out || !sorted_expert_ids_out) return MI_OK;
    std::fill(sorted_token_ids_out, sorted_token_ids_out + total_blocks * tile_m, (int32_t)(total + 1));
    for (int e = 0; e < num_experts; ++e)
        for (int64_t b = block_start[e]; b < block_start[e + 1]; ++b)
            sorted_expert_ids_out[b] = (int32_t)(e + 1);
    std::vector<int64_t> cursor(num_experts);
    for (int e = 0; e < num_experts; ++e) cursor[e] = block_start[e] * tile_m;
    for (int64_t t = 0; t < num_tokens; ++t)
        for (int64_t k = 0; k < topk; ++k) {
            const int64_t e = topk_ids[t + k * num_tokens] - 1;
            sorted_token_ids_out[cursor[e]++] = (int32_t)(t * topk + k + 1);
        }
    return MI_OK;
}
