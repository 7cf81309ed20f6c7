// Device code of the router top-k shared by the stand-alone route kernel and the fused route + pack kernel.
#pragma once
#include "common.h"

namespace dmoe {

// Monotone u32 key of an f32 for "ascending stable argsort, NaN last, -0 == +0".
// Never returns 0, so 0 can mark an entry that was already taken.
__device__ __forceinline__ uint32_t f32_sort_key(float c) {
    if (c != c) return 0xffffffffu;
    if (c == 0.0f) return 0x80000000u;
    uint32_t b = __float_as_uint(c);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// A (key, index) pair as one 64-bit number: pairs compare like (key, then index), so the HIGHER index wins among
// equal scores - what "take the last K columns of a stable ascending argsort" selects.
__device__ __forceinline__ uint64_t route_pair(uint32_t key, uint32_t idx) { return ((uint64_t)key << 32) | idx; }

// pair <- the larger of this lane's pair and the pair of the lane the DPP control selects (no branches)
template <int CTRL>
__device__ __forceinline__ void route_pair_step(uint64_t &p) {
    const uint32_t lo = (uint32_t)p, hi = (uint32_t)(p >> 32);
    const uint32_t olo = (uint32_t)__builtin_amdgcn_update_dpp((int)lo, (int)lo, CTRL, 0xf, 0xf, false);
    const uint32_t ohi = (uint32_t)__builtin_amdgcn_update_dpp((int)hi, (int)hi, CTRL, 0xf, 0xf, false);
    const uint64_t o = ((uint64_t)ohi << 32) | olo;
    p = o > p ? o : p;
}

// One wavefront routes NT tokens at once (`s[j]` = the E scores of token j). Lane l keeps the keys of experts
// l, l + 64, ... (EPL of them, E <= 64 * EPL) of every token in registers. The K winners are found by K rounds of a
// wave-wide maximum over (key, index) pairs; round r fills column K-1-r, so the columns come out in ascending
// score order. The NT tokens' reductions are independent chains that overlap. Lane j < K returns column j of
// every token. Straight-line code: selects instead of branches.
template <int NT, int EPL>
__device__ __forceinline__ void route_tokens(const float *const (&s)[NT], const float *__restrict__ bias,
                                             const uint8_t *__restrict__ resident, int E, int K, int normalize,
                                             int apply_scale, float route_scale, int lane, uint32_t (&my_idx)[NT],
                                             float (&w)[NT]) {
    uint32_t key[NT][EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int e = lane + 64 * i;
        const bool in = e < E;
        const int ec = in ? e : 0; // loads stay in bounds and unconditional
        const float b = bias ? bias[ec] : 0.0f;
        const float m = resident ? (resident[ec] ? 0.0f : -1e9f) : 0.0f;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            float c = s[j][ec];
            if (bias) c = c + b;
            if (resident) c = c + m;
            key[j][i] = in ? f32_sort_key(c) : 0u; // 0 never wins: real keys are never 0
        }
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) my_idx[j] = 0;
    for (int it = 0; it < K; ++it) {
        uint64_t best[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            best[j] = 0;
#pragma unroll
            for (int i = 0; i < EPL; ++i) {
                const uint64_t p = route_pair(key[j][i], (uint32_t)(lane + 64 * i));
                best[j] = p > best[j] ? p : best[j];
            }
        }
        // wave-wide maximum: four cross-lane steps inside each row of 16 lanes (after them every lane holds its
        // row's maximum), then the four rows through scalar registers. The pairs are totally ordered, so the shape
        // of the reduction tree does not matter.
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            route_pair_step<0xB1>(best[j]);  // lane ^ 1 (quad_perm 1,0,3,2)
            route_pair_step<0x4E>(best[j]);  // lane ^ 2 (quad_perm 2,3,0,1)
            route_pair_step<0x141>(best[j]); // the other quad of each eight lanes (row_half_mirror)
            route_pair_step<0x140>(best[j]); // the other half of the row (row_mirror)
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            uint64_t top = 0;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)best[j], 16 * r);
                const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(best[j] >> 32), 16 * r);
                const uint64_t p = ((uint64_t)hi << 32) | lo;
                top = p > top ? p : top;
            }
            const uint32_t bi = (uint32_t)top; // the winner's expert index, uniform
#pragma unroll
            for (int i = 0; i < EPL; ++i) key[j][i] = (bi == (uint32_t)(lane + 64 * i)) ? 0u : key[j][i]; // taken
            my_idx[j] = (lane == K - 1 - it) ? bi : my_idx[j];
        }
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const float got = s[j][my_idx[j]];
        const float my_w = (lane < K) ? got : 0.0f;
        float sum = 0.0f;
        for (int c = 0; c < K; ++c) sum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), c)); // left to right, like a row reduction
        float v = my_w;
        if (normalize) v = v / (sum + 1e-20f);
        if (apply_scale) v = v * route_scale;
        w[j] = v;
    }
}

// The same selection for ONE token whose E scores are already in registers (lane l holds experts l, l + 64, ... in
// `sc`), for kernels that have just computed the scores: no round trip through memory. Same arithmetic, same tie rule
// and same summation order as route_tokens, so both give the same bits. Lane j < K returns column j.
template <int EPL>
__device__ __forceinline__ void route_from_registers(const float (&sc)[EPL], const float *__restrict__ bias,
                                                     const uint8_t *__restrict__ resident, int E, int K, int normalize,
                                                     int apply_scale, float route_scale, int lane, uint32_t &my_idx,
                                                     float &w) {
    uint32_t key[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int e = lane + 64 * i;
        const bool in = e < E;
        const int ec = in ? e : 0;
        float c = sc[i];
        if (bias) c = c + bias[ec];
        if (resident) c = c + (resident[ec] ? 0.0f : -1e9f);
        key[i] = in ? f32_sort_key(c) : 0u;
    }
    my_idx = 0;
    float my_score = 0.0f;
    for (int it = 0; it < K; ++it) {
        uint64_t best = 0;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const uint64_t p = route_pair(key[i], (uint32_t)(lane + 64 * i));
            best = p > best ? p : best;
        }
        route_pair_step<0xB1>(best);
        route_pair_step<0x4E>(best);
        route_pair_step<0x141>(best);
        route_pair_step<0x140>(best);
        uint64_t top = 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)best, 16 * r);
            const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(best >> 32), 16 * r);
            const uint64_t p = ((uint64_t)hi << 32) | lo;
            top = p > top ? p : top;
        }
        const uint32_t bi = (uint32_t)top; // the winner's expert index, uniform
        // the winner's unbiased score sits in register bi / 64 of lane bi % 64
        float mine = 0.0f;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const bool hit = bi == (uint32_t)(lane + 64 * i);
            mine = hit ? sc[i] : mine;
            key[i] = hit ? 0u : key[i]; // taken
        }
        const float won = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), (int)(bi & 63u)));
        const bool col = lane == K - 1 - it;
        my_idx = col ? bi : my_idx;
        my_score = col ? won : my_score;
    }
    const float my_w = (lane < K) ? my_score : 0.0f;
    float sum = 0.0f;
    for (int c = 0; c < K; ++c) sum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), c)); // left to right
    float v = my_w;
    if (normalize) v = v / (sum + 1e-20f);
    if (apply_scale) v = v * route_scale;
    w = v;
}

} // namespace dmoe
