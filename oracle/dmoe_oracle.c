/*
 * CPU oracle for the quantized MoE expert-FFN path — TEST INFRASTRUCTURE ONLY.
 * See dmoe_oracle.h for what this is, who may call it, and the list of MLX
 * behaviours that are assumed rather than observed (u1..u6).
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference tree: src/moe_router.zig, src/models/deepseek_v4.zig, ...).
 */
#include "dmoe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ bf16 -- */

uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest, ties to even */
    return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline float rbf(float f) { return orc_bf16_to_f32(orc_f32_to_bf16(f)); }

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------- argsort ---- */

/* Total order used for argsort (u1): a precedes b if a < b, NaN after everything,
 * -0 == +0; equal keys keep their input order (the sort below is stable). */
static inline int f32_less(float a, float b) {
    if (isnan(a)) return 0;
    if (isnan(b)) return 1;
    return a < b;
}

/* stable merge sort of indices by f32 key; parity unpinned vs MLX (u1) */
static void argsort_f32(const float *key, int n, uint32_t *out, uint32_t *tmp) {
    for (int i = 0; i < n; i++) out[i] = (uint32_t)i;
    for (int w = 1; w < n; w *= 2) {
        for (int lo = 0; lo < n; lo += 2 * w) {
            int mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            int i = lo, j = mid, k = lo;
            while (i < mid && j < hi) {
                /* take from the right run only if strictly smaller: stability */
                if (f32_less(key[out[j]], key[out[i]])) tmp[k++] = out[j++];
                else tmp[k++] = out[i++];
            }
            while (i < mid) tmp[k++] = out[i++];
            while (j < hi) tmp[k++] = out[j++];
        }
        memcpy(out, tmp, (size_t)n * sizeof(uint32_t));
    }
}

/* stable merge sort of indices by u32 key; parity unpinned vs MLX (u1) */
static void argsort_u32(const uint32_t *key, size_t n, uint32_t *out, uint32_t *tmp) {
    for (size_t i = 0; i < n; i++) out[i] = (uint32_t)i;
    for (size_t w = 1; w < n; w *= 2) {
        for (size_t lo = 0; lo < n; lo += 2 * w) {
            size_t mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            size_t i = lo, j = mid, k = lo;
            while (i < mid && j < hi) {
                if (key[out[j]] < key[out[i]]) tmp[k++] = out[j++];
                else tmp[k++] = out[i++];
            }
            while (i < mid) tmp[k++] = out[i++];
            while (j < hi) tmp[k++] = out[j++];
        }
        memcpy(out, tmp, n * sizeof(uint32_t));
    }
}

/* ---------------------------------------------------------------- route --- */

/* moe_router.zig:55-103. argsort ascending over E (:61), slice columns [E-K, E)
 * (:66-74), take_along_axis (:78), optional w / (sum_k w + 1e-20) (:82-90).
 * Column order is ascending score, largest last. */
void orc_topk_route(const float *scores, int T, int E, int K, int normalize,
                    uint32_t *idx_out, float *w_out) {
    uint32_t *ord = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)E * 2);
    for (int t = 0; t < T; t++) {
        const float *s = scores + (size_t)t * E;
        argsort_f32(s, E, ord, ord + E);
        float sum = 0.0f;
        for (int j = 0; j < K; j++) {
            uint32_t e = ord[E - K + j];
            idx_out[(size_t)t * K + j] = e;
            w_out[(size_t)t * K + j] = s[e];
            sum += s[e]; /* reduce over the last axis, left to right */
        }
        if (normalize) {
            float denom = sum + 1e-20f;
            for (int j = 0; j < K; j++) w_out[(size_t)t * K + j] /= denom;
        }
    }
    free(ord);
}

/* deepseek_v4.zig:567-585: softmax | sigmoid | sqrt(log(1 + exp(x))) in f32.
 * Uses libm; results are compared to a tolerance, never bit for bit. */
void orc_gate_scores(const float *logits, int T, int E, int func, float *out) {
    for (int t = 0; t < T; t++) {
        const float *x = logits + (size_t)t * E;
        float *o = out + (size_t)t * E;
        if (func == ORC_SCORE_SOFTMAX) {
            float mx = x[0];
            for (int e = 1; e < E; e++) mx = x[e] > mx ? x[e] : mx;
            float sum = 0.0f;
            for (int e = 0; e < E; e++) { o[e] = expf(x[e] - mx); sum += o[e]; }
            for (int e = 0; e < E; e++) o[e] /= sum;
        } else if (func == ORC_SCORE_SIGMOID) {
            for (int e = 0; e < E; e++) o[e] = 1.0f / (1.0f + expf(-x[e]));
        } else if (func == ORC_SCORE_SQRTSOFTPLUS) {
            /* the reference's literal form, overflow for large x included (:575-583) */
            for (int e = 0; e < E; e++) o[e] = sqrtf(logf(1.0f + expf(x[e])));
        } else {
            /* the stable softplus of the Python model the reference follows (logaddexp(x, 0) = max + log1p(exp(-|x|));
             * docs/en/deepseek-v4/remaining-deviations.md:10 lists the literal form above as a deviation from it) */
            for (int e = 0; e < E; e++) o[e] = sqrtf(fmaxf(x[e], 0.0f) + log1pf(expf(-fabsf(x[e]))));
        }
    }
}

/* ---- router matmul and scoring with a fixed arithmetic (u7) ---------------------------------- */

/* deepseek_v4.zig:556-565. Products of two bf16 numbers are exact in f32; what is not
 * fixed by the reference is the order of the f32 additions. The order used here: the
 * reduction dimension is cut into segments of 128 elements, each segment is summed
 * left to right starting from 0, and the segment sums are added left to right. The
 * result is rounded to bf16 (the matmul's output dtype) and widened to f32 (:563). */
#define ORC_GATE_SEG 128
void orc_gate_logits(const uint16_t *x, const uint16_t *wg, int T, int D, int E, float *out) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < T; t++) {
        const uint16_t *xr = x + (size_t)t * D;
        for (int e = 0; e < E; e++) {
            const uint16_t *wr = wg + (size_t)e * D;
            float total = 0.0f;
            for (int k0 = 0; k0 < D; k0 += ORC_GATE_SEG) {
                int k1 = k0 + ORC_GATE_SEG < D ? k0 + ORC_GATE_SEG : D;
                float part = 0.0f;
                for (int k = k0; k < k1; k++) part = fmaf(orc_bf16_to_f32(xr[k]), orc_bf16_to_f32(wr[k]), part);
                total = total + part;
            }
            out[(size_t)t * E + e] = orc_bf16_to_f32(orc_f32_to_bf16(total));
        }
    }
}

static float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* exp(x) in f32 from IEEE operations only (Cody-Waite reduction by ln 2 in two parts, the
 * degree-5 polynomial of the Cephes expf, scaling by two exact powers of two). Inputs below
 * -87 give 0 (no denormal results), above 88.72 give +inf; NaN passes through. */
float orc_det_expf(float x) {
    if (x != x) return x;
    if (x > 88.72283935546875f) return bits_to_f32(0x7f800000u);
    if (x < -87.0f) return 0.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500E-4f;
    p = fmaf(p, r, 1.3981999507E-3f);
    p = fmaf(p, r, 8.3334519073E-3f);
    p = fmaf(p, r, 4.1665795894E-2f);
    p = fmaf(p, r, 1.6666665459E-1f);
    p = fmaf(p, r, 5.0000001201E-1f);
    float y = fmaf(p, r * r, r) + 1.0f;
    int ni = (int)n, k1 = ni / 2, k2 = ni - k1;
    y = y * bits_to_f32((uint32_t)(k1 + 127) << 23);
    return y * bits_to_f32((uint32_t)(k2 + 127) << 23);
}

/* log(x) in f32 for normal x > 0 (the Cephes logf: mantissa in [sqrt(1/2), sqrt(2)), degree-8
 * polynomial, exponent added back in two parts); +inf -> +inf, 0 -> -inf, negative or NaN -> NaN. */
float orc_det_logf(float x) {
    if (x != x || x < 0.0f) return bits_to_f32(0x7fc00000u);
    if (x == 0.0f) return bits_to_f32(0xff800000u);
    uint32_t u = f32_to_bits(x);
    if (u == 0x7f800000u) return x;
    int e = (int)((u >> 23) & 0xffu) - 126;
    float m = bits_to_f32((u & 0x007fffffu) | 0x3f000000u); /* [0.5, 1) */
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
    float z = m * m;
    float y = 7.0376836292E-2f;
    y = fmaf(y, m, -1.1514610310E-1f);
    y = fmaf(y, m, 1.1676998740E-1f);
    y = fmaf(y, m, -1.2420140846E-1f);
    y = fmaf(y, m, 1.4249322787E-1f);
    y = fmaf(y, m, -1.6668057665E-1f);
    y = fmaf(y, m, 2.0000714765E-1f);
    y = fmaf(y, m, -2.4999993993E-1f);
    y = fmaf(y, m, 3.3333331174E-1f);
    y = (y * m) * z;
    float fe = (float)e;
    y = fmaf(fe, -2.12194440e-4f, y);
    y = fmaf(-0.5f, z, y);
    float r = m + y;
    return fmaf(fe, 0.693359375f, r);
}

/* softplus(x) = max(x, 0) + log1p(exp(-|x|)) in f32 from the two routines above. log1p(u) for u in [0, 1] is
 * log(w) * (u / (w - 1)) with w = 1 + u rounded (the quotient undoes the rounding of w to first order), and u itself
 * where w rounds to 1. No overflow for large x (the result is x), no loss of the small results for very negative x
 * (the result is exp(x)). NaN passes through. Not part of the reference's Zig (which has the literal
 * log(1 + exp(x)), deepseek_v4.zig:575-583); it is the form of the Python model that
 * docs/en/deepseek-v4/remaining-deviations.md:10 names as the target. */
float orc_det_softplusf(float x) {
    float u = orc_det_expf(-fabsf(x));
    float w = 1.0f + u;
    float l = w == 1.0f ? u : orc_det_logf(w) * (u / (w - 1.0f));
    return (x > 0.0f ? x : 0.0f) + l;
}

/* deepseek_v4.zig:567-585, op by op, with orc_det_expf / orc_det_logf in place of MLX's exp / log.
 * softmax (:569): exp(x - max) / sum, the sum taken as 64 strided partial sums (element e goes to
 * partial e mod 64, in increasing e) that are then folded by halves (p[i] += p[i + 32], 16, .. 1). */
void orc_gate_scores_det(const float *logits, int T, int E, int func, float *out) {
    for (int t = 0; t < T; t++) {
        const float *x = logits + (size_t)t * E;
        float *o = out + (size_t)t * E;
        if (func == ORC_SCORE_SOFTMAX) {
            float mx = x[0];
            for (int e = 1; e < E; e++) mx = x[e] > mx ? x[e] : mx;
            float part[64];
            for (int i = 0; i < 64; i++) part[i] = 0.0f;
            for (int e = 0; e < E; e++) {
                o[e] = orc_det_expf(x[e] - mx);
                part[e & 63] = part[e & 63] + o[e];
            }
            for (int off = 32; off >= 1; off >>= 1)
                for (int i = 0; i < off; i++) part[i] = part[i] + part[i + off];
            for (int e = 0; e < E; e++) o[e] = o[e] / part[0];
        } else if (func == ORC_SCORE_SIGMOID) {
            for (int e = 0; e < E; e++) o[e] = 1.0f / (1.0f + orc_det_expf(-x[e]));
        } else if (func == ORC_SCORE_SQRTSOFTPLUS) {
            for (int e = 0; e < E; e++) o[e] = sqrtf(orc_det_logf(1.0f + orc_det_expf(x[e])));
        } else {
            for (int e = 0; e < E; e++) o[e] = sqrtf(orc_det_softplusf(x[e]));
        }
    }
}

/* deepseek_v4.zig:589-678. choice = scores + bias[E] (:593-599), then
 * + (resident ? 0 : -1e9) (:601-615); indices = last K of the ascending argsort of
 * choice (:654 -> :383-396); weights gathered from the UNBIASED scores (:589,:658);
 * if renorm: w / (sum_k w + 1e-20) (:663-672); then * route_scale (:676-678). */
void orc_gate_route(const float *scores, const float *bias, const uint8_t *resident,
                    int T, int E, int K, int renorm, float route_scale,
                    uint32_t *idx_out, float *w_out) {
    float *choice = (float *)malloc(sizeof(float) * (size_t)E);
    uint32_t *ord = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)E * 2);
    for (int t = 0; t < T; t++) {
        const float *s = scores + (size_t)t * E;
        for (int e = 0; e < E; e++) {
            float c = s[e];
            if (bias) c = c + bias[e];
            if (resident) c = c + (resident[e] ? 0.0f : -1e9f);
            choice[e] = c;
        }
        argsort_f32(choice, E, ord, ord + E);
        float sum = 0.0f;
        for (int j = 0; j < K; j++) {
            uint32_t e = ord[E - K + j];
            idx_out[(size_t)t * K + j] = e;
            w_out[(size_t)t * K + j] = s[e];
            sum += s[e];
        }
        float denom = sum + 1e-20f;
        for (int j = 0; j < K; j++) {
            float w = w_out[(size_t)t * K + j];
            if (renorm) w = w / denom;
            w_out[(size_t)t * K + j] = w * route_scale;
        }
    }
    free(choice);
    free(ord);
}

/* ------------------------------------------------ remap / mask / dedup ---- */

/* deepseek_v4.zig:619-636 (mlx_take_axis(tid2eid, ids, 0) -> [T,K]) followed by the common tail
 * :655-678 (gatherScores on the unbiased scores, w / (sum_k w + 1e-20) unless softmax, * scale). */
void orc_gate_hash_route(const float *scores, const int32_t *tid2eid, const uint32_t *ids, int T, int E,
                         int K, int renorm, float route_scale, uint32_t *idx_out, float *w_out) {
    for (int t = 0; t < T; t++) {
        float sum = 0.0f;
        for (int j = 0; j < K; j++) {
            uint32_t e = (uint32_t)tid2eid[(size_t)ids[t] * K + j];
            idx_out[(size_t)t * K + j] = e;
            w_out[(size_t)t * K + j] = scores[(size_t)t * E + e];
            sum += w_out[(size_t)t * K + j];
        }
        for (int j = 0; j < K; j++) {
            float v = w_out[(size_t)t * K + j];
            if (renorm) v = v / (sum + 1e-20f);
            w_out[(size_t)t * K + j] = v * route_scale;
        }
    }
}

/* The step after the MoE layer in DSV4TransformerBlock.forward (deepseek_v4.zig:2652-2654, 2674).
 * hc_mult == 0: ops.add(after_attn, ffn_out) (:2674), bf16 + bf16 rounded once.
 * hc_mult  > 0: mhcPost (:2450-2499): everything widened to f32 (:2468-2473),
 *   out[t,i,:] = x[t,:] * post_mix[t,i] + sum_j comb[t,j,i] * residual[t,j,:]   (comb transposed, :2481-2490)
 *   rounded to the dtype of x (:2498). The f32 matmul's accumulation order is MLX's and unknown (u8): this
 *   restatement takes j ascending, one fused multiply-add per term starting from comb[t,0,i] * residual[t,0,:],
 *   then adds term1 = x * post_mix with one rounding. Parity unpinned vs MLX in the last f32 bit only. */
void orc_block_post(const uint16_t *x, const uint16_t *residual, const float *post_mix, const float *comb_mix,
                    int T, int D, int hc_mult, uint16_t *out) {
    if (hc_mult == 0) {
        for (size_t i = 0; i < (size_t)T * D; i++)
            out[i] = orc_f32_to_bf16(orc_bf16_to_f32(residual[i]) + orc_bf16_to_f32(x[i]));
        return;
    }
    const int m = hc_mult;
    for (int t = 0; t < T; t++)
        for (int i = 0; i < m; i++) {
            const float post = post_mix[(size_t)t * m + i];
            for (int d = 0; d < D; d++) {
                const uint16_t *res = residual + (size_t)t * m * D + d;
                float term2 = comb_mix[((size_t)t * m + 0) * m + i] * orc_bf16_to_f32(res[0]);
                for (int j = 1; j < m; j++)
                    term2 = fmaf(comb_mix[((size_t)t * m + j) * m + i], orc_bf16_to_f32(res[(size_t)j * D]), term2);
                const float term1 = orc_bf16_to_f32(x[(size_t)t * D + d]) * post;
                out[((size_t)t * m + i) * D + d] = orc_f32_to_bf16(term1 + term2);
            }
        }
}

/* mlx_take(remap, indices) then astype(u32): deepseek_v4.zig:1035-1039,
 * expert_preload.zig:200-206, expert_stream.zig:522-529 (host loop) */
void orc_remap(const int32_t *remap, const uint32_t *idx, size_t n, uint32_t *out) {
    for (size_t i = 0; i < n; i++) out[i] = (uint32_t)remap[idx[i]];
}

/* Zig's @round: half away from zero, computed in f32 */
static inline float zig_roundf(float x) { return roundf(x); }

/* deepseek_v4_loader.zig:272-293 (SmeltConfig.buildMask), f32 arithmetic as there */
int orc_smelt_mask(int n_experts, float load_fraction, int strategy, int enabled,
                   uint8_t *mask) {
    memset(mask, 0, (size_t)n_experts);
    if (!enabled || load_fraction >= 1.0f) {
        memset(mask, 1, (size_t)n_experts);
        return n_experts;
    }
    float nf = zig_roundf(load_fraction * (float)n_experts);
    long n_load = (long)nf;
    if (n_load < 1) n_load = 1;
    if (strategy == ORC_SMELT_FIRST) {
        for (long i = 0; i < n_load; i++) mask[i] = 1;
    } else {
        /* n_load == 1 divides by zero in the reference: step = inf, 0*inf = NaN
         * for i = 0; treat that single pick as expert 0 */
        float step = (float)(n_experts - 1) / (float)(n_load - 1);
        for (long i = 0; i < n_load; i++) {
            float p = zig_roundf(step * (float)i);
            long idx = (n_load == 1) ? 0 : (long)p;
            if (idx > n_experts - 1) idx = n_experts - 1;
            mask[idx] = 1;
        }
    }
    int cnt = 0;
    for (int i = 0; i < n_experts; i++) cnt += mask[i];
    return cnt;
}

/* deepseek_v4_loader.zig:2151-2168: running slot index over the mask, unloaded -> 0 */
void orc_build_remap(const uint8_t *mask, int n_experts, int32_t *remap) {
    int32_t s = 0;
    for (int e = 0; e < n_experts; e++) {
        if (mask[e]) remap[e] = s++;
        else remap[e] = 0;
    }
}

/* expert_preload.zig:141-160: remap[eid]=slot (default 0); cache_bias 0 / -1000 */
void orc_preload_remap(const uint32_t *ids, int n_ids, int n_total, int32_t *remap,
                       float *cache_bias) {
    for (int e = 0; e < n_total; e++) { remap[e] = 0; if (cache_bias) cache_bias[e] = -1000.0f; }
    for (int s = 0; s < n_ids; s++) { remap[ids[s]] = s; if (cache_bias) cache_bias[ids[s]] = 0.0f; }
}

/* expert_stream.zig:449-465 (set union, ascending sort) and :510-515 (remap) */
int orc_dedup(const uint32_t *idx, size_t n, int n_experts, uint32_t *unique_out,
              int32_t *remap_out) {
    uint8_t *seen = (uint8_t *)calloc((size_t)n_experts, 1);
    for (size_t i = 0; i < n; i++) seen[idx[i]] = 1;
    int u = 0;
    for (int e = 0; e < n_experts; e++) {
        if (remap_out) remap_out[e] = 0;
        if (seen[e]) {
            if (remap_out) remap_out[e] = u;
            unique_out[u++] = (uint32_t)e;
        }
    }
    free(seen);
    return u;
}

/* ----------------------------------------------------------------- pack --- */

/* deepseek_v4.zig:749-784. order = argsort(flat_indices) (:753), inv_order =
 * argsort(order) (:758), token = order / K (:765-772), si = idx[order] (:777-779).
 * counts / offsets are what the sort implies: bincount and its exclusive scan.
 * Permutation values are parity unpinned vs MLX (u1: stability). */
void orc_pack(const uint32_t *idx, int T, int K, int E, uint32_t *order, uint32_t *inv,
              uint32_t *token, uint32_t *sorted_e, uint32_t *counts, uint32_t *offsets) {
    size_t n = (size_t)T * K;
    uint32_t *tmp = (uint32_t *)malloc(sizeof(uint32_t) * (n ? n : 1));
    argsort_u32(idx, n, order, tmp);
    if (inv) argsort_u32(order, n, inv, tmp);
    for (size_t i = 0; i < n; i++) {
        if (token) token[i] = order[i] / (uint32_t)K;
        if (sorted_e) sorted_e[i] = idx[order[i]];
    }
    if (counts) {
        memset(counts, 0, sizeof(uint32_t) * (size_t)E);
        for (size_t i = 0; i < n; i++) counts[idx[i]]++;
        if (offsets) {
            uint32_t run = 0;
            for (int e = 0; e < E; e++) { offsets[e] = run; run += counts[e]; }
            offsets[E] = run;
        }
    }
    free(tmp);
}

/* moe_router.zig:111-132: [T,D] -> [T,1,D] -> broadcast [T,K,D] -> [T*K,D] */
void orc_expand_tokens(const float *x, int T, int D, int K, float *out) {
    for (int t = 0; t < T; t++)
        for (int k = 0; k < K; k++)
            memcpy(out + ((size_t)t * K + k) * D, x + (size_t)t * D, sizeof(float) * (size_t)D);
}

/* moe_router.zig:139-164: [T*K,D] -> [T,K,D]; * w[T,K,1]; sum over axis 1 */
void orc_reduce_experts(const float *eo, const float *w, int T, int K, int D, float *out) {
    for (int t = 0; t < T; t++)
        for (int d = 0; d < D; d++) {
            float acc = 0.0f;
            for (int k = 0; k < K; k++)
                acc += eo[((size_t)t * K + k) * D + d] * w[(size_t)t * K + k];
            out[(size_t)t * D + d] = acc;
        }
}

/* -------------------------------------------------------------- dequant --- */

/* E2M1 code points, deepseek_v4_loader.zig:861-863 */
static const float kE2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

/* E8M0 -> 2^(s-127); deepseek_v4_loader.zig:841-856 states it as exp((s-127) ln 2),
 * the exact power of two is what that approximates. 255 is NaN (OCP MX). */
static inline float e8m0_to_f32(uint8_t s) {
    if (s == 255) return NAN;
    return ldexpf(1.0f, (int)s - 127);
}

/* OCP FP8 E4M3FN (u6) */
static inline float e4m3_to_f32(uint8_t v) {
    int sign = v >> 7, e = (v >> 3) & 15, m = v & 7;
    float r;
    if (e == 15 && m == 7) r = NAN;
    else if (e == 0) r = ldexpf((float)m, -9);           /* m/8 * 2^-6 */
    else r = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return sign ? -r : r;
}

static inline size_t qmat_words_per_row(const orc_qmat *m) {
    if (m->mode == ORC_FP8_ROW) return (size_t)m->cols; /* bytes */
    return (size_t)m->cols * (size_t)m->bits / 32;
}

/* Value (row, col) of matrix `mi`, in f32 before any rounding to bf16.
 * affine: element i of a row sits at bits [bits*(i % (32/bits)), +bits) of word
 * i / (32/bits) (low bits first; byte-level statement of the same order at
 * deepseek_v4_loader.zig:870-882; packed shape [out, in*bits/32] at
 * llama_loader.zig:270-276); value = q*scale + bias in f32 (u3).
 * mxfp4: LUT[nibble] * 2^(s-127), one E8M0 per 32 values (loader :859-920).
 * fp8row: e4m3(byte) * row_scale in f32. */
float orc_dequant_value(const orc_qmat *m, int mi, int row, int col) {
    size_t r = (size_t)mi * m->rows + row;
    if (m->mode == ORC_NONE) /* unquantized bf16 weights: dispatchGatherMm's float arm, deepseek_v4.zig:978 */
        return orc_bf16_to_f32(((const uint16_t *)m->w)[r * m->cols + col]);
    if (m->mode == ORC_FP8_ROW) {
        const uint8_t *w = (const uint8_t *)m->w;
        const float *sc = (const float *)m->scales;
        return e4m3_to_f32(w[r * m->cols + col]) * sc[r];
    }
    const uint32_t *w = (const uint32_t *)m->w;
    int per = 32 / m->bits;
    uint32_t word = w[r * qmat_words_per_row(m) + (size_t)(col / per)];
    uint32_t q = (word >> (m->bits * (col % per))) & ((1u << m->bits) - 1u);
    size_t g = r * (size_t)(m->cols / m->group) + (size_t)(col / m->group);
    if (m->mode == ORC_MXFP4) {
        const uint8_t *sc = (const uint8_t *)m->scales;
        return kE2M1[q] * e8m0_to_f32(sc[g]);
    }
    const uint16_t *sc = (const uint16_t *)m->scales;
    const uint16_t *bi = (const uint16_t *)m->biases;
    float s = orc_bf16_to_f32(sc[g]);
    float b = bi ? orc_bf16_to_f32(bi[g]) : 0.0f;
    float t = (float)q * s; /* exact: <= 8 x 8 significant bits */
    return t + b;           /* one f32 rounding */
}

/* fill one dequantized row in f32 */
static void dequant_row_f32(const orc_qmat *m, int mi, int row, float *out) {
    for (int c = 0; c < m->cols; c++) out[c] = orc_dequant_value(m, mi, row, c);
}

/* mlx_dequantize(..., dtype=bf16), deepseek_v4_loader.zig:129,1298; rounding order
 * parity unpinned vs MLX (u3) for affine; exact for mxfp4 */
void orc_dequantize(const orc_qmat *m, int mi, uint16_t *out) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < m->rows; r++)
        for (int c = 0; c < m->cols; c++)
            out[(size_t)r * m->cols + c] = orc_f32_to_bf16(orc_dequant_value(m, mi, r, c));
}

/* dequantFp8, deepseek_v4_loader.zig:922-990: w u8 [rows, cols] (E4M3FN, fromFp8 -> bf16 is exact), scale
 * [ceil(rows/block), ceil(cols/block)] through scaleToFloat (:839-856: f32 as it is, u8 as E8M0), weight viewed as
 * [m/bs, bs, n/bs, bs] times scale[:, None, :, None] in f32 (:957-970), then astype(bf16) (:981-984). The padding to
 * whole blocks (:936-955) and the truncation (:979-982) do not change any value. */
void orc_dequant_fp8_block(const uint8_t *w, const void *scale, int scale_is_e8m0, int rows, int cols, int block,
                           uint16_t *out) {
    int scale_cols = (cols + block - 1) / block;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            size_t si = (size_t)(r / block) * scale_cols + (size_t)(c / block);
            float sc = scale_is_e8m0 ? e8m0_to_f32(((const uint8_t *)scale)[si]) : ((const float *)scale)[si];
            out[(size_t)r * cols + c] = orc_f32_to_bf16(e4m3_to_f32(w[(size_t)r * cols + c]) * sc);
        }
}

/* the same values in f32, before the rounding to bf16 */
void orc_dequantize_f32(const orc_qmat *m, int mi, float *out) {
    for (int r = 0; r < m->rows; r++) dequant_row_f32(m, mi, r, out + (size_t)r * m->cols);
}

/* ------------------------------------------------------------ gather_qmm -- */

/* f32 dot product with 16 interleaved partial sums (fixed order, vectorisable) */
static inline float dot_f32(const float *a, const float *b, int n) {
    float acc[16];
    for (int j = 0; j < 16; j++) acc[j] = 0.0f;
    int k = 0;
    for (; k + 16 <= n; k += 16)
        for (int j = 0; j < 16; j++) acc[j] += a[k + j] * b[k + j];
    for (; k < n; k++) acc[k & 15] += a[k] * b[k];
    for (int w = 8; w >= 1; w /= 2)
        for (int j = 0; j < w; j++) acc[j] += acc[j + w];
    return acc[0];
}

/* rows of x gathered to f32 [R, cols] */
static float *rows_to_f32(const void *x, int x_is_f32, const uint32_t *lhs, int R, int cols) {
    float *xf = (float *)malloc(sizeof(float) * (size_t)(R ? R : 1) * cols);
    for (int r = 0; r < R; r++) {
        size_t src = lhs ? lhs[r] : (size_t)r;
        for (int c = 0; c < cols; c++)
            xf[(size_t)r * cols + c] = x_is_f32 ? ((const float *)x)[src * cols + c]
                                                 : orc_bf16_to_f32(((const uint16_t *)x)[src * cols + c]);
    }
    return xf;
}

/* gatherQmm(x, w, scales, biases, lhs=null|lhs, rhs, transpose=true, cfg, sorted):
 * call shape deepseek_v4.zig:976, expert_preload.zig:265; y[r] = x[r] . dq(W[rhs[r]])^T.
 * Accumulates in f32 (u4). Output rounded to bf16 when x is bf16 (u4).
 * Rows are visited grouped by expert so each weight row is dequantized once; the
 * result does not depend on that order. */
void orc_gather_qmm(const void *x, int x_is_f32, const orc_qmat *m, const uint32_t *lhs,
                    const uint32_t *rhs, int R, float *out) {
    int cols = m->cols, rows = m->rows;
    float *xf = rows_to_f32(x, x_is_f32, lhs, R, cols);
    /* group row ids by expert */
    uint32_t *ord = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)(R ? R : 1) * 2);
    argsort_u32(rhs, (size_t)R, ord, ord + R);
    int seg = 0;
    while (seg < R) {
        int end = seg;
        uint32_t e = rhs[ord[seg]];
        while (end < R && rhs[ord[end]] == e) end++;
#pragma omp parallel
        {
            float *wrow = (float *)malloc(sizeof(float) * (size_t)cols);
#pragma omp for schedule(static)
            for (int n = 0; n < rows; n++) {
                dequant_row_f32(m, (int)e, n, wrow);
                for (int i = seg; i < end; i++) {
                    uint32_t r = ord[i];
                    float y = dot_f32(xf + (size_t)r * cols, wrow, cols);
                    out[(size_t)r * rows + n] = x_is_f32 ? y : rbf(y);
                }
            }
            free(wrow);
        }
        seg = end;
    }
    free(ord);
    free(xf);
}

/* ------------------------------------------------------------ MoE layer --- */

static inline float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

/* limitedSwiGLU, deepseek_v4.zig:947-966 (routed) / :500-513 (shared), on bf16
 * operands: every MLX op rounds its result to bf16. The gate is clamped from above
 * only; up is clamped on both sides; limit <= 0 disables the clamp. */
/* deepseek_v4.zig:947-966; bf16 flow for every limit, see (u9) in the header: parity unpinned vs MLX */
static inline float limited_swiglu_bf16(float g, float u, float limit) {
    if (limit > 0.0f) {
        g = g < limit ? g : limit;   /* minimum(gate, L)       */
        u = u > -limit ? u : -limit; /* maximum(up, -L)        */
        u = u < limit ? u : limit;   /* minimum(.., L)         */
    }
    float sg = rbf(sigmoidf_(g));
    float silu = rbf(g * sg);
    return rbf(silu * u);
}

/* DSV4MoE.forward after the gate, deepseek_v4.zig:1017-1052, with
 * DSV4SwitchGLU.forward (:721-848, score before down) or forwardNoScores +
 * weighted sum (:855-945 and expert_stream.zig:575-580, score after down), and
 * DSV4Expert.forward for the shared expert (:489-517). The sort/unsort pair
 * (:749-784, :809) only permutes rows and is not materialised. dtype flow (u4,u5):
 * gate/up/activation bf16; score-before: act*score f32 -> down in f32;
 * score-after: down bf16, *score -> f32; sum over k left to right in f32;
 * + shared (bf16) -> f32. */
void orc_moe_forward(const orc_layer *L, const uint16_t *x, const uint32_t *idx,
                     const float *w, float *out, float *h_out) {
    int T = L->T, D = L->D, F = L->F, K = L->K;
    size_t R = (size_t)T * K;
    uint32_t *lhs = (uint32_t *)malloc(sizeof(uint32_t) * (R ? R : 1));
    for (size_t r = 0; r < R; r++) lhs[r] = (uint32_t)(r / (size_t)K);
    float *g = (float *)malloc(sizeof(float) * (R ? R : 1) * F);
    float *u = (float *)malloc(sizeof(float) * (R ? R : 1) * F);
    float *y = (float *)malloc(sizeof(float) * (R ? R : 1) * D);
    orc_gather_qmm(x, 0, &L->up, lhs, idx, (int)R, u);   /* :787 */
    orc_gather_qmm(x, 0, &L->gate, lhs, idx, (int)R, g); /* :789 */
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < R; r++)
        for (int f = 0; f < F; f++) {
            float a = limited_swiglu_bf16(g[r * F + f], u[r * F + f], L->swiglu_limit);
            if (h_out) h_out[r * F + f] = a;
            if (L->score_before_down) a = a * w[r]; /* :796-801, f32 */
            g[r * F + f] = a;
        }
    if (L->score_before_down) {
        orc_gather_qmm(g, 1, &L->down, NULL, idx, (int)R, y); /* :805, f32 in/out */
    } else {
        uint16_t *hb = (uint16_t *)malloc(sizeof(uint16_t) * (R ? R : 1) * F);
        for (size_t i = 0; i < R * (size_t)F; i++) hb[i] = orc_f32_to_bf16(g[i]);
        orc_gather_qmm(hb, 0, &L->down, NULL, idx, (int)R, y); /* bf16 out */
        free(hb);
    }
    for (int t = 0; t < T; t++)
        for (int d = 0; d < D; d++) {
            float acc = 0.0f;
            for (int k = 0; k < K; k++) {
                size_t r = (size_t)t * K + k;
                float v = y[r * D + d];
                if (!L->score_before_down) v = v * w[r]; /* expert_stream.zig:575-577 */
                acc += v;                                /* sum(axis=-2) */
            }
            out[(size_t)t * D + d] = acc;
        }
    if (L->has_shared) {
        float *sg = (float *)malloc(sizeof(float) * (size_t)T * F);
        float *su = (float *)malloc(sizeof(float) * (size_t)T * F);
        float *sy = (float *)malloc(sizeof(float) * (size_t)T * D);
        uint32_t *zero = (uint32_t *)calloc((size_t)(T ? T : 1), sizeof(uint32_t));
        uint16_t *hb = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)T * F);
        orc_gather_qmm(x, 0, &L->sh_gate, NULL, zero, T, sg); /* :495 */
        orc_gather_qmm(x, 0, &L->sh_up, NULL, zero, T, su);   /* :497 */
        for (size_t i = 0; i < (size_t)T * F; i++)
            hb[i] = orc_f32_to_bf16(limited_swiglu_bf16(sg[i], su[i], L->shared_swiglu_limit));
        orc_gather_qmm(hb, 0, &L->sh_down, NULL, zero, T, sy); /* :516 */
        for (size_t i = 0; i < (size_t)T * D; i++) out[i] = out[i] + sy[i]; /* :1051 */
        free(sg); free(su); free(sy); free(zero); free(hb);
    }
    free(lhs); free(g); free(u); free(y);
}

/* ---------------------------------------------------------- batch build --- */

/* batch_builder.zig:128-166: concatenate per-request tokens (prefill requests
 * first, then decode ones, as the caller orders them: :104-111), positions
 * base_pos + j, and the running offsets of each request in the flat batch. */
void orc_batch_concat(const uint32_t *const *req_tokens, const int *lens,
                      const int *base_pos, int n_req, uint32_t *tokens_out,
                      int32_t *pos_out, int32_t *req_offsets_out) {
    int off = 0;
    for (int i = 0; i < n_req; i++) {
        req_offsets_out[i] = off;
        for (int j = 0; j < lens[i]; j++) {
            tokens_out[off + j] = req_tokens[i][j];
            pos_out[off + j] = base_pos[i] + j;
        }
        off += lens[i];
    }
    req_offsets_out[n_req] = off;
}

/* batch_builder.zig:140-177: all -inf, then 0 where col <= row inside a request */
void orc_batch_mask(const int *lens, int n_req, float *mask) {
    int T = 0;
    for (int i = 0; i < n_req; i++) T += lens[i];
    for (size_t i = 0; i < (size_t)T * T; i++) mask[i] = -INFINITY;
    int off = 0;
    for (int i = 0; i < n_req; i++) {
        for (int r = 0; r < lens[i]; r++)
            for (int c = 0; c <= r; c++) mask[(size_t)(off + r) * T + (off + c)] = 0.0f;
        off += lens[i];
    }
}
