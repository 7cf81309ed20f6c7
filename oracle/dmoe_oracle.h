/*
 * CPU oracle for the quantized MoE expert-FFN path — TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the op sequence that zouyee/dmlx runs through
 * MLX for one MoE layer. It exists so that the HIP path can be checked against
 * something that follows the reference line by line. Nothing in the product
 * (the HIP library, its host layer) may link, load or call it; only tests, the
 * smoke check and the benchmark's CPU-baseline leg do.
 *
 * The arithmetic of argsort / take / quantize / dequantize / gather_qmm lives in
 * MLX (reached through zouyee/mlx-zig v0.0.2 -> mlx-c), which is NOT part of the
 * reference tree. The behaviours below are therefore ASSUMED, not observed
 * ("parity unpinned" against real MLX; pinned only against the reference's own
 * test vectors, closed forms and library routines, see tests/):
 *   (u1) argsort is stable: ties keep ascending index order, so the "last k" slice
 *        prefers the HIGHER index among equal scores; NaN sorts last.
 *   (u2) quantize's scale/bias rule is not used here at all: callers hand over
 *        packed words + scales (+ biases) and both sides consume the same bytes.
 *   (u3) affine dequantize computes q*scale + bias in f32 and rounds once to bf16.
 *   (u4) gather_qmm / quantized_matmul accumulate in f32; output dtype = x dtype.
 *   (u5) bf16 (activations) x f32 (scores) promotes to f32.
 *   (u6) FP8 is OCP E4M3FN (no infinities, 0x7f/0xff are NaN).
 *   (u7) the router matmul (bf16 x bf16 -> bf16) accumulates in f32 and rounds once;
 *        the accumulation ORDER and the rounding of exp / log inside the scoring
 *        function are MLX's and unknown. orc_gate_logits / orc_gate_scores_det fix
 *        one order and one explicit polynomial exp / log (stated at their
 *        definitions) so that a GPU implementation of the same arithmetic can be
 *        compared bit for bit; against libm they agree to a few ulp (tests).
 *   (u8) the f32 matmul inside mhcPost sums its hc_mult terms in MLX's order, unknown;
 *        orc_block_post takes them in ascending order with fused multiply-adds.
 *   (u9) limitedSwiGLU with limit > 0 clamps against f32 scalar ARRAYS (ops.scalarF32,
 *        deepseek_v4.zig:948-955): if MLX promotes bf16 (+) f32-array to f32 as (u5) assumes for
 *        the score multiply, the activation and everything after it would be f32 for limit > 0 and
 *        bf16 only for limit = 0. The oracle keeps ONE flow for both: sigmoid, silu and the product
 *        are each rounded to bf16, as the limit = 0 branch does on bf16 arrays. It therefore rounds
 *        at least as often as either reading of the reference; how far the kernels are from the
 *        exact value is bounded separately against float64 (tests/test_gpu_accuracy_margin.py).
 * Functions whose results depend on one of (u1), (u3)..(u6), (u9) are marked
 * "parity unpinned vs MLX" at their definition.
 *
 * All matrices are dense row-major. bf16 values travel as uint16_t.
 */
#ifndef DMOE_ORACLE_H
#define DMOE_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_AFFINE = 0, ORC_MXFP4 = 1, ORC_FP8_ROW = 2, ORC_NONE = 3 };
enum { ORC_SCORE_SOFTMAX = 0, ORC_SCORE_SIGMOID = 1, ORC_SCORE_SQRTSOFTPLUS = 2, ORC_SCORE_SQRTSOFTPLUS_STABLE = 3 };
enum { ORC_SMELT_UNIFORM = 0, ORC_SMELT_FIRST = 1 };

/* One quantized matrix stack [n_mats, rows, cols] in MLX layout.
 * affine : w u32 [n, rows, cols*bits/32], scales/biases bf16 [n, rows, cols/group]
 * mxfp4  : w u32 [n, rows, cols/8], scales u8 (E8M0) [n, rows, cols/32], biases NULL
 * fp8row : w u8  [n, rows, cols] (E4M3FN), scales f32 [n, rows], biases NULL
 * none   : w bf16 [n, rows, cols] as it is (the unquantized arm, ops.gatherMm), scales/biases NULL */
typedef struct {
    const void *w;
    const void *scales;
    const void *biases;
    int rows, cols;
    int mode, bits, group;
} orc_qmat;

uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);

/* moe_router.zig:55-103 */
void orc_topk_route(const float *scores, int T, int E, int K, int normalize,
                    uint32_t *idx_out, float *w_out);
/* deepseek_v4.zig:567-585 */
void orc_gate_scores(const float *logits, int T, int E, int func, float *scores_out);
/* deepseek_v4.zig:556-565: logits = (x @ Wg^T) in bf16, then astype(f32).
 * x bf16 [T,D], wg bf16 [E,D] -> logits f32 [T,E] (every value representable in bf16). */
void orc_gate_logits(const uint16_t *x, const uint16_t *wg, int T, int D, int E, float *logits_out);
/* deepseek_v4.zig:567-585 with exp / log evaluated by explicit f32 polynomials (u7) */
void orc_gate_scores_det(const float *logits, int T, int E, int func, float *scores_out);
float orc_det_expf(float x);
float orc_det_logf(float x);
float orc_det_softplusf(float x);
/* deepseek_v4.zig:589-678 (selection on biased/masked scores, weights from the
 * unbiased ones, renorm when not softmax, * route_scale) */
void orc_gate_route(const float *scores, const float *bias, const uint8_t *resident,
                    int T, int E, int K, int renorm, float route_scale,
                    uint32_t *idx_out, float *w_out);
/* hash layers, deepseek_v4.zig:619-636 + :655-678: indices = tid2eid[input_ids], weights from the
 * unbiased scores, renorm when not softmax, * route_scale */
/* residual add / mhcPost after the layer (deepseek_v4.zig:2450-2499, 2652-2654, 2674); x bf16 [T,D];
 * hc_mult == 0: residual, out bf16 [T,D]; else residual, out bf16 [T,hc_mult,D], post_mix f32 [T,hc_mult],
 * comb_mix f32 [T,hc_mult,hc_mult] */
void orc_block_post(const uint16_t *x, const uint16_t *residual, const float *post_mix, const float *comb_mix,
                    int T, int D, int hc_mult, uint16_t *out);
void orc_gate_hash_route(const float *scores, const int32_t *tid2eid, const uint32_t *ids, int T, int E,
                         int K, int renorm, float route_scale, uint32_t *idx_out, float *w_out);
/* mlx_take(remap, indices): deepseek_v4.zig:1037, expert_preload.zig:202 */
void orc_remap(const int32_t *remap, const uint32_t *idx, size_t n, uint32_t *out);
/* deepseek_v4_loader.zig:272-293; returns the number of resident experts */
int orc_smelt_mask(int n_experts, float load_fraction, int strategy, int enabled,
                   uint8_t *mask_out);
/* deepseek_v4_loader.zig:2151-2168 */
void orc_build_remap(const uint8_t *mask, int n_experts, int32_t *remap_out);
/* expert_preload.zig:141-160 */
void orc_preload_remap(const uint32_t *expert_ids, int n_ids, int n_total,
                       int32_t *remap_out, float *cache_bias_out);
/* expert_stream.zig:449-515: sorted unique ids + remap[e]=slot (default 0);
 * returns n_unique */
int orc_dedup(const uint32_t *idx, size_t n, int n_experts, uint32_t *unique_out,
              int32_t *remap_out);
/* deepseek_v4.zig:749-784: order=argsort(flat idx), inv=argsort(order),
 * token=order/K, sorted_e=idx[order]; plus bincount and its exclusive scan */
void orc_pack(const uint32_t *idx, int T, int K, int E, uint32_t *order, uint32_t *inv,
              uint32_t *token, uint32_t *sorted_e, uint32_t *counts, uint32_t *offsets);
/* moe_router.zig:111-132 / :139-164 (f32) */
void orc_expand_tokens(const float *x, int T, int D, int K, float *out);
void orc_reduce_experts(const float *expert_outs, const float *w, int T, int K, int D,
                        float *out);

/* dequantize -> bf16 [rows, cols] of matrix `mat_index` of the stack */
void orc_dequantize(const orc_qmat *m, int mat_index, uint16_t *out_bf16);
void orc_dequant_fp8_block(const uint8_t *w, const void *scale, int scale_is_e8m0, int rows, int cols, int block,
                           uint16_t *out);
/* whole matrix / single value in f32, before the bf16 rounding */
void orc_dequantize_f32(const orc_qmat *m, int mat_index, float *out_f32);
float orc_dequant_value(const orc_qmat *m, int mat_index, int row, int col);

/* y[r, :] = x[lhs?lhs[r]:r, :] . dequant(W[rhs[r]])^T, f32 accumulate.
 * x is bf16 when x_is_f32 == 0 (then y is rounded to bf16 and widened back),
 * f32 otherwise. out is f32 [R, rows]. */
void orc_gather_qmm(const void *x, int x_is_f32, const orc_qmat *m, const uint32_t *lhs,
                    const uint32_t *rhs, int R, float *out);

typedef struct {
    int T, D, F, K, E;          /* E = number of resident expert slots           */
    orc_qmat gate, up, down;    /* stacks of E matrices                          */
    float swiglu_limit;         /* deepseek_v4.zig:947-966                       */
    int score_before_down;      /* 1: DSV4SwitchGLU.forward (:796-806)
                                   0: provider paths (expert_stream.zig:575-580) */
    int has_shared;             /* DSV4Expert (:489-517), swiglu_limit_shared    */
    orc_qmat sh_gate, sh_up, sh_down;
    float shared_swiglu_limit;
} orc_layer;

/* DSV4MoE.forward after the gate (deepseek_v4.zig:1030-1052): routed experts on
 * slot indices idx[T,K] with weights w[T,K], plus the shared expert. x bf16 [T,D],
 * out f32 [T,D] (the dtype the reference's promotion rules give). h_out (optional,
 * f32 [T*K, F], flat row r = t*K+k) receives the SwiGLU activations. */
void orc_moe_forward(const orc_layer *L, const uint16_t *x, const uint32_t *idx,
                     const float *w, float *out, float *h_out);

/* batch_builder.zig:90-214 without the O(T^2) mask: concatenated ids, positions and
 * request offsets. lens[i] tokens starting at position base_pos[i]. */
void orc_batch_concat(const uint32_t *const *req_tokens, const int *lens,
                      const int *base_pos, int n_req, uint32_t *tokens_out,
                      int32_t *pos_out, int32_t *req_offsets_out);
/* batch_builder.zig:140-177: block-diagonal causal mask, 0 / -inf, [T,T] */
void orc_batch_mask(const int *lens, int n_req, float *mask_out);

int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
