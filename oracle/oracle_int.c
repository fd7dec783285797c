/* CPU oracle, integer / byte-level part, in plain C.  TEST INFRASTRUCTURE ONLY: loaded by
 * tests/ to cross-check the numpy restatement (oracle/cutile_oracle.py) and the library's
 * host helpers; never linked into or called from the product.
 *
 * Each function restates the reference lines it cites with scalar loops. */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int32_t cld32(int32_t a, int32_t b) { return (a + b - 1) / b; }

/* examples/matmul.jl:13-24 (duplicate: examples/moe.jl:20-31). 1-based in, 1-based out. */
void oracle_swizzle_2d(int32_t M, int32_t N, int32_t tm, int32_t tn, int32_t group_size_m,
                       int32_t bid, int32_t* bid_m, int32_t* bid_n) {
    int32_t num_bid_m = cld32(M, tm);
    int32_t num_bid_n = cld32(N, tn);
    int32_t num_bid_in_group = group_size_m * num_bid_n;
    int32_t bid0 = bid - 1;
    int32_t group_id = bid0 / num_bid_in_group;
    int32_t first_bid_m = group_id * group_size_m;
    int32_t gsm = num_bid_m - first_bid_m;
    if (gsm > group_size_m) gsm = group_size_m;
    *bid_m = first_bid_m + bid0 % gsm + 1;
    *bid_n = (bid0 % num_bid_in_group) / gsm + 1;
}

/* examples/moe.jl:142-183.  topk_ids: column-major (num_tokens, topk), 1-based expert ids.
 * The stable sort is done literally (insertion into per-expert lists in flat order, which
 * is what a stable sort by expert id yields).  Outputs must hold
 * tile_m * sum_e cld(count_e, tile_m) and sum_e cld(count_e, tile_m) entries.
 * Returns the number of blocks, or -1 on a bad expert id. */
int64_t oracle_moe_align_tile_size(const int64_t* topk_ids, int64_t num_tokens, int64_t topk,
                                   int32_t tile_m, int32_t num_experts, int32_t* sorted_token_ids,
                                   int32_t* sorted_expert_ids) {
    int64_t total = num_tokens * topk;
    int64_t* flat = (int64_t*)malloc(sizeof(int64_t) * (size_t)(total > 0 ? total : 1));
    int64_t* counts = (int64_t*)calloc((size_t)num_experts, sizeof(int64_t));
    /* vec(permutedims(topk_ids)): slot varies fastest within each token (moe.jl:146-148) */
    for (int64_t t = 0; t < num_tokens; ++t)
        for (int64_t k = 0; k < topk; ++k) flat[t * topk + k] = topk_ids[t + k * num_tokens];
    for (int64_t f = 0; f < total; ++f) {
        if (flat[f] < 1 || flat[f] > num_experts) { free(flat); free(counts); return -1; }
        counts[flat[f] - 1]++;
    }
    int64_t total_blocks = 0;
    for (int32_t e = 0; e < num_experts; ++e) total_blocks += (counts[e] + tile_m - 1) / tile_m;
    if (sorted_token_ids && sorted_expert_ids) {
        for (int64_t i = 0; i < total_blocks * tile_m; ++i) sorted_token_ids[i] = (int32_t)(total + 1);
        int64_t cur_block = 0;
        for (int32_t e = 1; e <= num_experts; ++e) {
            int64_t bc = (counts[e - 1] + tile_m - 1) / tile_m;
            for (int64_t i = 0; i < bc; ++i) sorted_expert_ids[cur_block + i] = e;
            int64_t pos = cur_block * tile_m;
            for (int64_t f = 0; f < total; ++f) /* ascending flat order == stable */
                if (flat[f] == e) sorted_token_ids[pos++] = (int32_t)(f + 1);
            cur_block += bc;
        }
    }
    free(flat);
    free(counts);
    return total_blocks;
}

/* OCP FP8 E4M3FN (the type behind Float8_E4M3FN, ext/DLFP8TypesExt.jl:7-9): sign, 4-bit
 * exponent with bias 7, 3-bit mantissa, no infinities, S.1111.111 = NaN, max finite 448. */
float oracle_e4m3fn_decode(uint8_t c) {
    int s = c >> 7, e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if (e == 15 && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf((float)(8 + m), e - 10);
    return s ? -v : v;
}

/* Round to nearest even by exhaustive search over the 127 non-negative finite codes:
 * slow, obviously correct.  Magnitudes that round past 448 (>= 464) give NaN (0x7F). */
uint8_t oracle_e4m3fn_encode(float x) {
    uint8_t sign = signbit(x) ? 0x80 : 0;
    if (isnan(x)) return (uint8_t)(sign | 0x7F);
    double a = fabs((double)x);
    if (a >= 464.0) return (uint8_t)(sign | 0x7F);
    int best = 0;
    double best_err = INFINITY;
    for (int c = 0; c < 0x7F; ++c) {
        double err = fabs((double)oracle_e4m3fn_decode((uint8_t)c) - a);
        if (err < best_err) {
            best = c;
            best_err = err;
        } else if (err == best_err && (c & 1) == 0) {
            best = c; /* tie: the code with an even mantissa */
        }
    }
    return (uint8_t)(sign | best);
}
