// kq_gemm_plan.h — which form of the bf16 dequant-GEMM serves a shape.  Host arithmetic only (no device call), so
// that the choice can be checked on a machine without a GPU (bpk_gemm_plan).
#pragma once
#include <cstdint>

#include "kq_format.h"

namespace kq {

enum GemmForm : int {
    GEMM_FORM_SMALL = 0,             // 128 x 128 tiles, two workgroups per CU
    GEMM_FORM_WHOLE = 1,             // 256 x 256 tiles, one workgroup per tile, in rounds over the CUs
    GEMM_FORM_SHARES = 2,            // the walk over the (256-tile, k step) units cut into equal shares, one per CU
    GEMM_FORM_HALF = 3,              // 256 tokens x 128 weight rows per workgroup, whole tiles
    GEMM_FORM_ROUNDS_THEN_HALF = 4,  // the full rounds of 256-tiles, then the last round's weight rows as 256 x 128 tiles
    GEMM_FORM_192 = 5,               // 256 tokens x 192 weight rows per workgroup, whole tiles
};

struct GemmPlan {
    int form;
    uint32_t share;        // k steps per workgroup of the 256-tile walk (forms 1, 2, 4)
    uint32_t rows_first;   // form 4: weight rows of the first launch
};

// Priced in microseconds with figures measured on the Llama-3-8B matrices at M = 256 .. 2048: (a) 256-tiles, one
// workgroup per tile, in rounds over the CUs; (b) the walk over all (tile, k step) units of the 256-tiles cut into
// equal shares, one per CU, where every run over part of a tile costs a workspace slot (256 KB written, read back
// by the sum kernel); (c) 128-tiles, two workgroups per CU; (d) 256 x 128 tiles, whole, in rounds over the CUs.  A k
// step of a 256-tile takes tk, of a 128-tile tk128, of a 256 x 128 tile tk_h; a 256-tile's epilogue te.
// tile: 0 automatic, 128 / 256 force (c) / (a or b), 129 forces (d), 192 the 256 x 192 tile; split: 0 automatic, 1 whole tiles, 2 equal shares.
inline GemmPlan plan_gemm_bf16(int type, uint32_t M, uint32_t N, uint32_t K, uint32_t cus, int tile, int split)
{
    const bool q4 = type == KQ_TYPE_Q4_K, q5 = type == KQ_TYPE_Q5_K;
    const uint32_t nk = K / 64u;
    const uint64_t big = (uint64_t)((M + 255u) / 256u) * ((N + 255u) / 256u);
    const uint64_t small = (uint64_t)((M + 127u) / 128u) * ((N + 127u) / 128u);
    const float tk = q4 ? 1.7f : q5 ? 1.9f : 2.2f, tk128 = q4 ? 1.4f : q5 ? 1.6f : 2.0f, te = 12.0f, t_slot = 0.1f, t_sum = 5.0f;
    const uint32_t one_per_cu = (uint32_t)((big * nk + cus - 1u) / cus);   // equal shares over all CUs
    const uint64_t runs = (big * nk + one_per_cu - 1u) / one_per_cu;
    const float t_whole = (float)((big + cus - 1u) / cus) * ((float)nk * tk + te);
    const float t_shares = (float)one_per_cu * tk + te * (1.0f + (float)one_per_cu / (float)nk)
                           + t_slot * (float)(one_per_cu < nk ? runs : 2u * (runs - 1u)) + t_sum;
    const float t_small = (float)((small + 2u * cus - 1u) / (2u * cus)) * ((float)nk * tk128 + 0.25f * te);
    bool use_big = t_small > (t_whole < t_shares ? t_whole : t_shares);
    uint32_t share = t_shares < t_whole ? one_per_cu : nk;
    // (d): a k step 1.08 us (Q4_K) / 1.3 us (Q6_K), an epilogue 8 us, and three quarters of that while half of the
    // CUs or more have no tile.  Measured: 4096 x 4096 Q4_K at M = 2048 87 against 106 us for the cheapest of
    // (a)..(c) inside a pass over a layer set (77 against 96-100 us launched back to back), at M = 1024 57 against
    // 62 us; 4096 x 14336 Q6_K at M = 2048 269 against 267 us for equal shares inside the pass (259 against 270 back
    // to back), at M = 1024 183 against 147 us: priced so that the Q6_K matrix keeps its equal shares.
    const uint64_t half = (uint64_t)((M + 255u) / 256u) * ((N + 127u) / 128u);
    const float tk_h = q4 ? 1.08f : q5 ? 1.15f : 1.3f;
    const float t_half = (float)((half + cus - 1u) / cus) * ((float)nk * tk_h + 8.0f) * (2u * half <= cus ? 0.75f : 1.0f);
    const float t_ab = t_whole < t_shares ? t_whole : t_shares;
    const float t_best = t_small < t_ab ? t_small : t_ab;
    bool use_half = t_half < t_best;
    if (tile == 192) return GemmPlan{GEMM_FORM_192, 0u, 0u};
    if (tile == 256) { use_big = true; use_half = false; }
    if (tile == 128) { use_big = false; use_half = false; }
    if (tile == 129) use_half = true;
    if (split != 0) use_half = use_half && tile == 129;   // a forced split means the 256-tile walk
    // (e) 256 x 192 tiles where they fill one round over the CUs better than anything above: a k step 1.45 us
    // (Q4_K) / 1.6 us (Q6_K).  Measured at M = 2048: 6144 x 4096 Q4_K 105 against 108-119 us for 192 whole 256-tiles,
    // Q5_K 110 against 121-127, Q6_K 113 against 115-118; over several rounds it loses (128256 x 4096 Q6_K 2605
    // against 2461 us, 28672 x 4096 Q4_K 480 against 445), so it is only priced for a single round.
    const uint64_t n192 = (uint64_t)((M + 255u) / 256u) * ((N + 191u) / 192u);
    const float t_192 = (float)nk * (q4 ? 1.45f : q5 ? 1.55f : 1.6f) + te;
    if (tile == 0 && split == 0 && n192 <= cus && 4u * n192 > 3u * cus && t_192 < (use_half ? t_half : t_best))
        return GemmPlan{GEMM_FORM_192, 0u, 0u};
    if (use_half) return GemmPlan{GEMM_FORM_HALF, 0u, 0u};
    if (split == 1) share = nk;
    if (split == 2) share = one_per_cu;              // forced: any number of runs per tile
    share = (share + 3u) & ~3u;                      // the k loop takes whole superblocks (nk is a multiple of 4)
    // Whole 256-tiles whose last round over the CUs is at most half full (gate|up at M = 2048: 896 tiles = 3.5
    // rounds): the last round's tiles, a block of weight rows over all tokens, run as 256 x 128 tiles in a second
    // launch — twice as many, so they fill the CUs — behind the full rounds.
    if (use_big && share == nk && tile == 0 && split == 0) {
        const uint32_t m_tiles = (M + 255u) / 256u, n_tiles = (N + 255u) / 256u;
        const uint32_t rounds = (uint32_t)(big / cus), rest = (uint32_t)(big % cus);
        if (rounds >= 1u && rest > 0u && 2u * rest <= cus && rest % m_tiles == 0u) {
            const float t_two = (float)rounds * ((float)nk * tk + te) + ((float)nk * tk_h + 8.0f) + 3.0f;
            if (t_two < t_whole) return GemmPlan{GEMM_FORM_ROUNDS_THEN_HALF, nk, (n_tiles - rest / m_tiles) * 256u};
        }
    }
    if (use_big) return GemmPlan{share % nk == 0u ? GEMM_FORM_WHOLE : GEMM_FORM_SHARES, share, 0u};
    return GemmPlan{GEMM_FORM_SMALL, 0u, 0u};
}

}  // namespace kq
