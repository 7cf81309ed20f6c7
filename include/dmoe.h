/*
 * dmoe — MI355X (gfx950) implementation of dmlx's quantized MoE expert-FFN path.
 *
 * C ABI of libdmoe.so. Conventions follow the mlx-c call style the reference binds
 * (out-parameters first, inputs next, stream last, `int` return code, 0 = ok; see
 * e.g. moe_router.zig:61,78 and deepseek_v4.zig:1037 in the reference):
 *   - every pointer named `d_*` is DEVICE memory (HIP), dense row-major, owned by
 *     the caller; inputs are borrowed for the duration of the call, outputs are
 *     written in place. Nullable arguments say so.
 *   - bf16 tensors are passed as `uint16_t*` bit patterns.
 *   - all work is enqueued on the given stream and returns without waiting;
 *     `dmoe_stream_synchronize` is the only wait. A stream with ctx == NULL is the
 *     default HIP stream.
 *   - a non-zero return code means nothing useful was enqueued; the message is
 *     available (per thread) from `dmoe_last_error()`. The reference maps any
 *     non-zero mlx-c code to one Zig error after logging the message; a binding
 *     does the same here.
 *   - calls that share one `dmoe_workspace` must be ordered on one stream.
 *
 * Each entry point names the reference interface it replaces (file:line in the
 * reference tree).
 */
#ifndef DMOE_H
#define DMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DMOE_VERSION 100 /* 0.1.0 */

typedef enum {
    DMOE_OK = 0,
    DMOE_ERR_INVALID = 1,     /* bad argument / unsupported shape            */
    DMOE_ERR_HIP = 2,         /* a HIP runtime call failed                   */
    DMOE_ERR_UNSUPPORTED = 3, /* valid request this build does not implement */
    DMOE_ERR_NO_DEVICE = 4,   /* no gfx950 device visible                    */
    DMOE_ERR_TIMEOUT = 5      /* a bounded wait inside a kernel gave up (see dmoe_workspace_check) */
} dmoe_status;

/* quantization mode; the reference passes it as the C strings "affine"/"mxfp4"
 * (deepseek_v4.zig:974, deepseek_v4_loader.zig:129) */
typedef enum {
    DMOE_QUANT_AFFINE = 0, /* bits 4|8, group 32|64|128, bf16 scales + bf16 biases (biases nullable = 0) */
    DMOE_QUANT_MXFP4 = 1,  /* E2M1 nibbles, one E8M0 byte per 32 values, no biases                      */
    DMOE_QUANT_FP8_ROW = 2, /* E4M3FN bytes, one f32 scale per output row, no biases                    */
    DMOE_QUANT_NONE = 3     /* unquantized bf16 [n_mats, rows, cols]; bits 16, no scales, no biases: the float
                               arm of dispatchGatherMm / ops.gatherMm (deepseek_v4.zig:969-979)           */
} dmoe_quant_mode;

typedef struct dmoe_stream_ { void *ctx; } dmoe_stream;           /* ctx = hipStream_t */
typedef struct dmoe_workspace_ { void *ctx; } dmoe_workspace;     /* grow-only device scratch */
typedef struct dmoe_layer_ { void *ctx; } dmoe_layer;             /* resident expert weights of one MoE layer */
typedef struct dmoe_gate_ { void *ctx; } dmoe_gate;               /* resident router of one MoE layer */
typedef struct dmoe_resident_weight_ { void *ctx; } dmoe_resident_weight; /* one weight stack in the kernels' layout */

/* "affine" -> DMOE_QUANT_AFFINE, "mxfp4" -> DMOE_QUANT_MXFP4, "fp8" -> DMOE_QUANT_FP8_ROW,
 * "none" | "bf16" -> DMOE_QUANT_NONE; -1 if unknown */
int dmoe_quant_mode_from_string(const char *name);

/* ---- runtime ------------------------------------------------------------------ */

int dmoe_version(void);
const char *dmoe_last_error(void);              /* thread-local, never NULL */
/* replaces c.initErrorHandler() + default GPU stream set-up (src/tests.zig:66-68, main.zig:479-480):
 * selects the device, checks it is gfx950. device < 0 keeps the current device. */
int dmoe_init(int device);

int dmoe_stream_create(dmoe_stream *out);
int dmoe_stream_destroy(dmoe_stream s);
int dmoe_stream_synchronize(dmoe_stream s);     /* replaces Array.eval() as the host-visible sync point */

/* device memory for host languages that do not link HIP themselves (what Array.fromData /
 * dataSlice do in the reference: copies in and out of device arrays) */
int dmoe_malloc(void **out_d_ptr, size_t bytes);
int dmoe_free(void *d_ptr);
int dmoe_copy_to_device(void *d_dst, const void *h_src, size_t bytes, dmoe_stream s);
int dmoe_copy_to_host(void *h_dst, const void *d_src, size_t bytes, dmoe_stream s);   /* waits for the copy */

int dmoe_workspace_create(dmoe_workspace *out, size_t initial_bytes);
int dmoe_workspace_destroy(dmoe_workspace ws);
/* bytes currently reserved; growth happens inside calls (it synchronizes the device) */
int dmoe_workspace_reserved(size_t *out_bytes, dmoe_workspace ws);
/* Waits for stream s, then reports what the kernels launched with this workspace since the last check could not
 * report through a return code. Plays the role of c.check(rc) after Array.eval() in the reference
 * (moe_router.zig:68,74), where a failed lazy graph surfaces at the sync point: the outputs of dmoe_moe_forward,
 * dmoe_moe_layer_forward, dmoe_switch_glu_forward_no_scores, dmoe_gather_qmm* and dmoe_pack are valid once a check
 * that follows them returns DMOE_OK. Both conditions are cleared by the call that reports them.
 *   DMOE_ERR_TIMEOUT  a bounded wait gave up. At decode sizes the gate/up and the down projection share one launch:
 *                     a down workgroup waits for its own tile's gate/up workgroups and gives up after the workspace's
 *                     poll limit (~16 ms), so that the launch ends whatever happens. That a waiting workgroup's
 *                     producers are running or done rests on the hardware starting workgroups in index order, which
 *                     holds on gfx950 but is not promised by the programming model. After this error the workspace
 *                     runs the two projections as two launches in a row (dmoe_workspace_set_paired_launch(ws, 0)),
 *                     which wait for nothing; the outputs since the last check must be discarded and recomputed.
 *   DMOE_ERR_INVALID  an expert id outside the layer's [0, n_experts) reached the packing step. Such a row is computed
 *                     as the last expert so that every access stays in bounds; the outputs must be discarded. */
int dmoe_workspace_check(dmoe_workspace ws, dmoe_stream s);
/* polls (~0.25 us each) a waiting workgroup makes before it gives up; default 65536. For tests of the give-up path. */
int dmoe_workspace_set_wait_limit(dmoe_workspace ws, unsigned polls);
/* 1 (default): decode-sized calls of more than 64 expert rows (T * K, plus T when the shared expert rides along) run
 * gate/up and down in one launch, as described at dmoe_workspace_check; smaller ones take two launches, which is faster
 * there. 0: always two launches in a row (same results, a few per cent slower at 64 tokens, no waits inside kernels).
 * No counterpart in the reference. */
int dmoe_workspace_set_paired_launch(dmoe_workspace ws, int enabled);

/* Per-stage device timing of the layer forward calls made with this workspace (HIP events recorded on the
 * call's stream around each stage). Off by default. While on, prefill-sized calls keep their launches in a row on
 * one stream (so that a stage's time covers all of its tiles), and a forward call waits for the device once 64 calls'
 * events are unread: use it for measurement runs. No counterpart in the reference, which logs host wall time per
 * token step (expert_stream.zig:587-610). */
enum {
    DMOE_STAGE_ROUTE = 0,        /* dmoe_gate_route inside dmoe_moe_layer_forward */
    DMOE_STAGE_PACK = 1,         /* remap + counting sort                         */
    DMOE_STAGE_GATE_UP = 2,      /* grouped gate/up GEMM + SwiGLU                 */
    DMOE_STAGE_DOWN = 3,         /* grouped down GEMM                             */
    DMOE_STAGE_SHARED = 4,       /* shared expert (both GEMMs)                    */
    DMOE_STAGE_COMBINE = 5,      /* weighted sum over k + shared add              */
    /* prefill-sized calls on packed 4-bit weights split each grouped GEMM into two launches on one tile list: the
     * matrix-core kernel takes the tiles above 8 rows (stages 2 and 3), the weight-streaming kernel the rest: */
    DMOE_STAGE_GATE_UP_SMALL = 6,
    DMOE_STAGE_DOWN_SMALL = 7,
    DMOE_STAGE_COUNT = 8
};
int dmoe_workspace_set_stage_timing(dmoe_workspace ws, int enabled);
/* total milliseconds and number of samples per stage since timing was enabled; arrays of DMOE_STAGE_COUNT */
int dmoe_workspace_read_stage_times(float *h_out_total_ms, int *h_out_samples, dmoe_workspace ws);

/* ---- router ------------------------------------------------------------------- */

/* MoERouter.topkRoute (moe_router.zig:55-103): per token, the K largest of E scores.
 * Columns are in ASCENDING score order (the reference slices the last K columns of an
 * ascending argsort); among equal scores the higher expert index wins. Weights are the
 * selected scores, divided by (sum_k + 1e-20) when `normalize` != 0.
 *   d_out_indices u32 [T,K], d_out_weights f32 [T,K], d_scores f32 [T,E]; 1 <= K <= E <= 1024 */
int dmoe_topk_route(uint32_t *d_out_indices, float *d_out_weights, const float *d_scores,
                    int T, int E, int K, int normalize, dmoe_stream s);

/* DSV4Gate.forward from the scores on (deepseek_v4.zig:589-678): selection on
 * scores + bias[E] (+ -1e9 where resident_mask[e] == 0), weights gathered from the
 * unbiased scores, divided by (sum_k + 1e-20) when `renorm` != 0 (the reference does so
 * for every scoring function except softmax, :663), then * route_scale (:676-678).
 *   d_bias f32 [E] nullable; d_resident_mask u8 [E] nullable (Smelt mask, :601-615) */
int dmoe_gate_route(uint32_t *d_out_indices, float *d_out_weights, const float *d_scores,
                    const float *d_bias, const uint8_t *d_resident_mask,
                    int T, int E, int K, int renorm, float route_scale, dmoe_stream s);

/* mlx_take(remap, indices).astype(u32) (deepseek_v4.zig:1035-1039, expert_preload.zig:200-206):
 * d_out[i] = (u32) d_remap[d_indices[i]], n elements, every index < n_total. */
int dmoe_remap_indices(uint32_t *d_out, const int32_t *d_remap, const uint32_t *d_indices,
                       size_t n, int n_total, dmoe_stream s);

/* MoERouter.expandTokens (moe_router.zig:111-132): out[t*K+k, :] = x[t, :]; elem_size in bytes (2 or 4) */
int dmoe_expand_tokens(void *d_out, const void *d_x, int T, int D, int K, int elem_size, dmoe_stream s);

/* MoERouter.reduceExperts (moe_router.zig:139-164): out[t,:] = sum_k w[t,k] * expert_outs[t*K+k,:], f32,
 * summed over k left to right. expert_outs is f32 (outs_are_bf16 == 0) or bf16. */
int dmoe_reduce_experts(float *d_out, const void *d_expert_outs, int outs_are_bf16, const float *d_weights,
                        int T, int K, int D, dmoe_stream s);

/* SmeltConfig.buildMask (deepseek_v4_loader.zig:272-293), host side: h_out_mask u8 [n_experts];
 * strategy 0 = uniform, 1 = first. Returns the number of resident experts in *out_n_resident. */
int dmoe_smelt_build_mask(uint8_t *h_out_mask, int *out_n_resident, int n_experts, float load_fraction,
                          int strategy, int enabled);
/* expert_remap construction (deepseek_v4_loader.zig:2151-2168), host side: running slot index over the
 * mask, non-resident experts map to slot 0. */
int dmoe_build_remap(int32_t *h_out_remap, const uint8_t *h_mask, int n_experts);
/* ExpertPreloadProvider.init remap + cache bias (expert_preload.zig:141-160), host side:
 * remap[ids[s]] = s (others 0); cache_bias 0 for loaded ids, -1000 otherwise (nullable). */
int dmoe_preload_remap(int32_t *h_out_remap, float *h_out_cache_bias, const uint32_t *h_expert_ids,
                       int n_ids, int n_total);

/* ---- packing (token -> expert segments) --------------------------------------------- */

/* The sort block of DSV4SwitchGLU.forward (deepseek_v4.zig:749-784) as one stable counting sort:
 *   order[p]     = flat index (t*K+k) of the p-th row when rows are grouped by expert, ties in
 *                  ascending flat index                                (argsort(flat_indices), :753)
 *   inv_order[i] = position of flat index i                            (argsort(order), :758)
 *   token[p]     = order[p] / K                                        (:765-772)
 *   sorted_expert[p] = indices[order[p]]                               (:777-779)
 *   counts[e], offsets[e] = rows of expert e and their exclusive scan; offsets[E] = T*K
 * plus what expert_stream.zig:449-465 derives on the host: live_experts = ascending ids with
 * counts > 0 and *n_live their number (d_out_n_live is a device u32).
 * Any output pointer except d_out_order may be NULL. indices < E <= 1024. */
int dmoe_pack(uint32_t *d_out_order, uint32_t *d_out_inv_order, uint32_t *d_out_token,
              uint32_t *d_out_sorted_expert, uint32_t *d_out_counts, uint32_t *d_out_offsets,
              uint32_t *d_out_live_experts, uint32_t *d_out_n_live,
              const uint32_t *d_indices, int T, int K, int E, dmoe_workspace ws, dmoe_stream s);

/* ---- quantized weights ------------------------------------------------------------------ */

/* one stack [n_mats, rows, cols] of quantized matrices in MLX layout (out-features = rows):
 *   affine : w u32 [n, rows, cols*bits/32]; scales, biases bf16 [n, rows, cols/group_size]
 *   mxfp4  : w u32 [n, rows, cols/8];       scales u8 [n, rows, cols/32]; biases NULL
 *   fp8row : w u8  [n, rows, cols];         scales f32 [n, rows];         biases NULL
 *   none   : w bf16 [n, rows, cols] (rows % 4 == 0, cols % 8 == 0); scales, biases NULL
 * (QuantizedWeight / QuantConfig of mlx-zig as used at deepseek_v4.zig:474-481, :971-976) */
typedef struct {
    const void *w;
    const void *scales; /* NULL for DMOE_QUANT_NONE */
    const void *biases; /* nullable */
    int n_mats, rows, cols;
    int mode;           /* dmoe_quant_mode */
    int bits;           /* 4 | 8 (affine), 4 (mxfp4), 8 (fp8row), 16 (none) */
    int group_size;     /* 32 | 64 | 128 (affine), 32 (mxfp4), ignored (fp8row, none) */
} dmoe_qweight;

/* mlx_dequantize(..., dtype = bf16) (deepseek_v4_loader.zig:129): d_out bf16 [rows, cols] of matrix
 * `mat_index`; value = q*scale + bias evaluated in f32 and rounded once to bf16 (affine),
 * E2M1 * 2^(s-127) (mxfp4, exact), e4m3 * row_scale rounded to bf16 (fp8row). Device pointers in `qw`. */
int dmoe_dequantize(uint16_t *d_out, const dmoe_qweight *qw, int mat_index, dmoe_stream s);

/* dequantFp8 (deepseek_v4_loader.zig:922-990) with scaleToFloat (:839-856): FP8 E4M3FN bytes [rows, cols] with one
 * scale per block_size x block_size tile, d_scale [ceil(rows / block_size), ceil(cols / block_size)] as f32, or as
 * E8M0 bytes (scale_is_e8m0 != 0: 2^(s-127), the value the reference's exp((s-127) ln 2) stands for; 255 is NaN)
 * -> d_out bf16 [rows, cols] = bf16(f32(fp8) * scale), one rounding. rows and cols need not be multiples of the block
 * (the reference pads and truncates; the values are the same). The FP4 counterpart, dequantFp4 (:859-920), is
 * dmoe_dequantize on a DMOE_QUANT_MXFP4 matrix (low nibble first, one E8M0 byte per 32 values). */
int dmoe_dequant_fp8_block(uint16_t *d_out, const uint8_t *d_weight, const void *d_scale, int scale_is_e8m0,
                           int rows, int cols, int block_size, dmoe_stream s);

/* quantize_mod.gatherQmm(x, w, scales, biases, lhs_indices, rhs_indices, transpose = true, cfg, sorted)
 * (call shape deepseek_v4.zig:976, expert_preload.zig:265; mlx.core.gather_qmm):
 *   out[r, :] = x[lhs ? lhs[r] : r, :] . dequant(W[rhs[r]])^T     r < R
 * x bf16 [*, cols], out bf16 [R, rows], f32 accumulation. d_lhs_indices nullable. `sorted` != 0 promises
 * non-decreasing rhs_indices (as the reference's sorted=true); the result is the same either way.
 * With qw->mode == DMOE_QUANT_NONE (bf16 weights [n_mats, rows, cols], bits 16, no scales) this is
 * ops.gatherMm(x, w^T, null, rhs_indices, sorted) of the unquantized arm (deepseek_v4.zig:978): pass the
 * [E, out, in] weight itself, not its transposed view. */
int dmoe_gather_qmm(uint16_t *d_out, const uint16_t *d_x, const dmoe_qweight *qw,
                    const uint32_t *d_lhs_indices, const uint32_t *d_rhs_indices, int R, int sorted,
                    dmoe_workspace ws, dmoe_stream s);

/* Opt-in for callers that keep the gatherQmm call surface unchanged (borrowed MLX-layout arrays on every call): with
 * the cache on, dmoe_gather_qmm makes the re-ordered resident copy of a stack the first time it sees it on this
 * workspace (one pass over the stack, the call waits for it) and streams that copy from then on, as
 * dmoe_gather_qmm_resident does. A stack is recognised by its three pointers, shape and format: the caller promises
 * that the arrays behind cached pointers neither change nor are freed while the cache is on. Costs the stack's size
 * in HBM again. enabled = 0 (the default) drops every copy; so does dmoe_workspace_destroy. Same results either way.
 * No counterpart in the reference (its QuantizedWeight arrays live as long as the model).
 *
 * An allocator that recycles addresses can hand a freed stack's pointers to a NEW stack of the same shape; the cache
 * cannot tell the two apart and would serve the old copy. A caller that frees or rewrites a stack while the cache is
 * on calls dmoe_workspace_weight_cache_invalidate with that stack's descriptor first (qw = null drops every copy; it
 * waits for the device, since kernels in flight may still read a copy). The copies are capped by bytes
 * (dmoe_workspace_set_weight_cache_limit, default 32 GiB, 0 = no cap): a new stack that would exceed the cap pushes
 * out the least recently used copies, which costs one wait for the device. dmoe_workspace_weight_cache_stats reports
 * what is held. */
int dmoe_workspace_set_weight_cache(dmoe_workspace ws, int enabled);
int dmoe_workspace_weight_cache_invalidate(dmoe_workspace ws, const dmoe_qweight *qw);
int dmoe_workspace_set_weight_cache_limit(dmoe_workspace ws, size_t max_bytes);
int dmoe_workspace_weight_cache_stats(size_t *out_bytes, int *out_stacks, dmoe_workspace ws);

/* The same call on a stack that was made resident once: mlx-zig's QuantizedWeight is a long-lived object (the w /
 * scales / biases Arrays of DSV4SwitchGLU live as long as the model, deepseek_v4.zig:687-717), and its counterpart
 * here is a copy in HBM re-ordered into the layout the kernels stream (rows in blocks of 32, one contiguous KiB per
 * wavefront and reduction step). dmoe_gather_qmm on the MLX layout gives the same bits; at decode sizes the
 * resident stack streams about 1.3 times faster (the MLX layout needs whole cache lines turned through LDS, and
 * scales / biases fetched apart), and shapes whose scale rows are not whole 16-byte blocks several times faster. `weight_source` as in dmoe_layer_desc
 * (the stack is always copied: it is re-ordered). Shapes that cannot be re-ordered (rows not a multiple of 32) stay
 * in the MLX layout inside the handle. */
int dmoe_resident_weight_create(dmoe_resident_weight *out, const dmoe_qweight *qw, int weight_source, dmoe_stream s);
int dmoe_resident_weight_destroy(dmoe_resident_weight w);
int dmoe_gather_qmm_resident(uint16_t *d_out, const uint16_t *d_x, dmoe_resident_weight w,
                             const uint32_t *d_lhs_indices, const uint32_t *d_rhs_indices, int R, int sorted,
                             dmoe_workspace ws, dmoe_stream s);

/* ---- resident MoE layer -------------------------------------------------------------------- */

typedef enum {
    DMOE_WEIGHTS_COPY_FROM_HOST = 0,   /* pointers in the descriptor are host memory; copied to HBM   */
    DMOE_WEIGHTS_COPY_FROM_DEVICE = 1, /* device memory; copied, caller may free its copy afterwards  */
    DMOE_WEIGHTS_BORROW_DEVICE = 2     /* device memory used in place; must outlive the layer         */
} dmoe_weight_source;

/* DSV4SwitchGLU fields (deepseek_v4.zig:687-705) + DSV4Expert fields for the shared expert (:442-457)
 * + DSV4MoE.expert_remap (:991-993). Replaces LayerExpertMeta + the SSD/LFU expert cache of
 * expert_stream.zig / expert_cache.zig: all `n_mats` expert slots stay resident in HBM. */
typedef struct {
    int hidden;                 /* D */
    int ffn;                    /* F (routed experts)                         */
    int top_k;                  /* K                                          */
    dmoe_qweight gate, up, down;/* gate/up: rows=F, cols=D; down: rows=D, cols=F; n_mats = resident slots */
    float swiglu_limit;         /* limitedSwiGLU clamp, 0 = none (:947-966)   */
    int score_before_down;      /* 1 = DSV4SwitchGLU.forward (:796-806); 0 = provider paths
                                   (expert_stream.zig:575-580, expert_preload.zig:283-289). With 1 the product
                                   activation * score is rounded to bf16 before the down projection (the
                                   reference keeps it in f32 after promoting bf16 x f32, :801): one more bf16
                                   rounding of that operand, inside the 1e-2 output tolerance */
    int has_shared;             /* shared expert (DSV4Expert, :489-517), n_mats = 1, rows/cols as above with its own F */
    dmoe_qweight shared_gate, shared_up, shared_down;
    float shared_swiglu_limit;  /* the reference builds the shared expert with 0 (deepseek_v4_loader.zig:1893) */
    const int32_t *remap;       /* nullable HOST i32 [n_experts_total]: router id -> slot (:1035-1039) */
    int n_experts_total;        /* length of remap; ignored when remap is NULL */
    int weight_source;          /* dmoe_weight_source */
} dmoe_layer_desc;

int dmoe_layer_create(dmoe_layer *out, const dmoe_layer_desc *desc, dmoe_stream s);
int dmoe_layer_destroy(dmoe_layer layer);

/* One-time resident upload of a layer's experts from MLX-format safetensors files: what
 * model_registry.zig:255-329 prepares for on-demand reads (TensorIndex + LayerExpertMeta +
 * ExpertStreamProvider.initWithStrategy(..., quantized, group_size, bits, mode, swiglu_limit, ...)) done once,
 * into HBM. Tensor names as there (:264-269):
 *   model.layers.{layer_idx}.ffn.switch_mlp.{gate,up,down}_proj.{weight,scales,biases}   U32 / BF16|U8 / BF16
 *   model.layers.{layer_idx}.ffn.shared_experts.{gate,up,down}_proj.{...}                 (when load_shared)
 * Shapes [E, rows, cols*bits/32] and [E, rows, cols/group]; D, F and E are read from them. */
typedef struct {
    int top_k;
    const char *mode;            /* "affine" | "mxfp4" (the reference passes "mxfp4", 32, 4; :318-321) | "none":
                                    float checkpoint, weights BF16 [E, rows, cols], no scales */
    int group_size, bits;
    float swiglu_limit;
    int score_before_down;
    int load_shared;             /* also load the shared expert when the files hold one */
    const char *shared_mode;     /* NULL: decided by the file as the reference's loader does
                                    (deepseek_v4_loader.zig:1890-1892): biases present -> "affine", scales only ->
                                    "mxfp4" with group 32, neither -> "none" */
    int shared_group_size, shared_bits; /* 0: the routed experts' values */
    float shared_swiglu_limit;
    const uint8_t *resident_mask;/* nullable HOST u8 [n_experts_total]: Smelt, only experts with 1 are uploaded, in
                                    increasing id order; the router-id -> slot remap is built like
                                    deepseek_v4_loader.zig:2151-2168 (unloaded -> 0) */
    int n_experts_total;         /* length of resident_mask = experts in the file */
} dmoe_safetensors_opts;

int dmoe_layer_create_from_safetensors(dmoe_layer *out, const char *const *paths, int n_paths, int layer_idx,
                                       const dmoe_safetensors_opts *opts, dmoe_stream s);

/* shape of a resident layer: D, F, resident expert slots, K (any out pointer may be NULL) */
int dmoe_layer_dims(int *out_hidden, int *out_ffn, int *out_n_slots, int *out_top_k, dmoe_layer layer);

/* ExpertProvider.VTable.forward(ptr, layer_idx, flat_x, indices, scores) (expert_provider.zig:21) ==
 * ExpertStreamProvider.streamForward (expert_stream.zig:245-261) == the provider arm of DSV4MoE.forward
 * (deepseek_v4.zig:1030-1047), plus the shared expert and the final add (:1021, :1050-1052) when the layer
 * has one: remap -> pack -> grouped gate/up + limited SwiGLU -> grouped down -> weighted sum over k.
 *   d_out bf16 [T,D]; d_x bf16 [T,D]; d_indices u32 [T,K] router expert ids; d_scores f32 [T,K] */
int dmoe_moe_forward(uint16_t *d_out, dmoe_layer layer, const uint16_t *d_x, const uint32_t *d_indices,
                     const float *d_scores, int T, dmoe_workspace ws, dmoe_stream s);

/* DSV4SwitchGLU.forwardNoScores (deepseek_v4.zig:855-945): expert outputs without score weighting,
 * d_out bf16 [T,K,D] in (t,k) order; indices are slot ids (no remap applied, no shared expert). */
int dmoe_switch_glu_forward_no_scores(uint16_t *d_out, dmoe_layer layer, const uint16_t *d_x,
                                      const uint32_t *d_slot_indices, int T, dmoe_workspace ws, dmoe_stream s);

/* DSV4MoE.forward from the gate scores on (deepseek_v4.zig:1021-1052): dmoe_gate_route followed by
 * dmoe_moe_forward. d_scores f32 [T,E_total]; d_bias, d_resident_mask nullable as in dmoe_gate_route.
 * d_out_indices / d_out_weights (nullable) receive the routing for inspection. */
int dmoe_moe_layer_forward(uint16_t *d_out, uint32_t *d_out_indices, float *d_out_weights, dmoe_layer layer,
                           const uint16_t *d_x, const float *d_scores, const float *d_bias,
                           const uint8_t *d_resident_mask, int T, int E_total, int renorm, float route_scale,
                           dmoe_workspace ws, dmoe_stream s);

/* dmoe_moe_layer_forward for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments without the
 * workspace: all intermediate buffers live in a 16 MiB device array that is part of the library (one per GPU, held
 * until the process ends), so the call makes no hipMalloc / hipFree and creates no stream or event. Differences from
 * dmoe_moe_layer_forward:
 *   - a batch whose buffers do not fit is rejected with DMOE_ERR_INVALID and a message naming the size (at D = 4096,
 *     F = 2048, K = 6 with a folded shared expert: up to 194 tokens);
 *   - gate/up and down always run as two launches and a shared expert of another format runs after them on the same
 *     stream, so nothing waits inside a kernel; results are bit-identical;
 *   - there is no dmoe_workspace_check for this entry point and none is needed: the two conditions that check reports
 *     cannot arise here. No kernel waits (see above), and the expert ids reach the packing step from the call's own
 *     routing - a top-k over E_total scores, mapped through the remap that dmoe_layer_create validated - so they are
 *     always inside the layer's range (the reference's remap gives the same guarantee, expert_preload.zig:141-149).
 *     The flag words the packing kernels would count bad ids in sit in the static array and are never read;
 *   - every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race.
 * The array's address and every kernel's launch attributes are set up by dmoe_init on the device it selects, else by
 * the first call on a device (do not make that first call under stream capture). After that a call does no host-side
 * set-up and can be captured into a HIP graph from any thread. */
int dmoe_moe_layer_forward_static(uint16_t *d_out, uint32_t *d_out_indices, float *d_out_weights, dmoe_layer layer,
                                  const uint16_t *d_x, const float *d_scores, const float *d_bias,
                                  const uint8_t *d_resident_mask, int T, int E_total, int renorm, float route_scale,
                                  dmoe_stream s);

/* ---- router (gate) from the hidden states on ------------------------------------------------ */

/* DSV4Config.ScoringFunc (deepseek_v4.zig:82-86) */
typedef enum {
    DMOE_SCORE_SOFTMAX = 0,
    DMOE_SCORE_SIGMOID = 1,
    DMOE_SCORE_SQRTSOFTPLUS = 2, /* sqrt(log(1 + exp(x))), the reference's default (:48), literally as it computes it
                                  * (:575-583): +inf from x = 88.73 on */
    /* Not in the reference's enum: the same score through the overflow-free softplus max(x, 0) + log1p(exp(-|x|)) of
     * the Python model the reference follows (its docs/en/deepseek-v4/remaining-deviations.md:10 lists the literal form
     * as an open deviation from that). Equal to the literal form to rounding wherever that one is finite and above
     * 1e-3; a caller opts in, the default stays the reference's arithmetic. */
    DMOE_SCORE_SQRTSOFTPLUS_STABLE = 3
} dmoe_scoring_func;

/* DSV4Gate fields (deepseek_v4.zig:521-535). Pointers are host or device memory as `weight_source` says
 * (DMOE_WEIGHTS_COPY_FROM_HOST / _FROM_DEVICE; the weight is re-ordered, so it is always copied). */
typedef struct {
    const void *weight;           /* bf16 [n_experts, dim] (:523)                                  */
    const float *bias;            /* nullable f32 [n_experts]: selection bias (:524, :593-599)     */
    const uint8_t *resident_mask; /* nullable u8 [n_experts]: Smelt mask, 1 = resident (:531-535)  */
    int n_experts, dim, top_k;
    int scoring_func;             /* dmoe_scoring_func */
    float route_scale;            /* :528 */
    int is_hash;                  /* hash routing layer (:529): experts come from tid2eid[input_ids] (:619-636) */
    const int32_t *tid2eid;       /* i32 [vocab_size, top_k] when is_hash, else ignored (:525)    */
    int vocab_size;
    int weight_source;            /* dmoe_weight_source */
} dmoe_gate_desc;

int dmoe_gate_create(dmoe_gate *out, const dmoe_gate_desc *desc, dmoe_stream s);
int dmoe_gate_destroy(dmoe_gate gate);

/* DSV4Gate.forward(hidden_states, input_ids, stream) (deepseek_v4.zig:546-681): logits = (x @ W^T) in bf16
 * widened to f32, scoring function, then dmoe_gate_route with the gate's bias, mask, top_k and route scale
 * (renormalised unless the scoring function is softmax). Returns (weights, indices) like the reference.
 *   d_out_indices u32 [T,K]; d_out_weights f32 [T,K]; d_out_scores nullable f32 [T,n_experts]: the
 *   unbiased scores, for inspection; d_x bf16 [T,dim], 16-byte aligned; d_input_ids nullable u32 [T]: on a
 *   hash gate the indices are tid2eid[input_ids] and only the weights come from the scores (:619-636); a hash
 *   gate called without ids selects by top-k like the reference (:618-622).
 * The order of the f32 additions in the matmul and the evaluation of exp / log are fixed by this library
 * (segments of 128 reduction elements summed left to right; polynomial exp / log), so the selected experts
 * do not depend on tile shapes or library versions; MLX's own choices are not observable from the reference. */
int dmoe_gate_forward(uint32_t *d_out_indices, float *d_out_weights, float *d_out_scores, dmoe_gate gate,
                      const uint16_t *d_x, const uint32_t *d_input_ids, int T, dmoe_workspace ws, dmoe_stream s);

/* ---- the step after the layer ------------------------------------------------------------------ */

/* What DSV4TransformerBlock.forward does with the layer's output (deepseek_v4.zig:2652-2654, 2674).
 *   hc_mult == 0: ops.add(after_attn, ffn_out) (:2674): d_out bf16 [T,D] = d_residual [T,D] + d_ffn_out [T,D];
 *                 the mixes are ignored (may be null).
 *   hc_mult  > 0: DSV4HyperConn.post = mhcPost (:2450-2499, :2585-2588): d_residual and d_out are bf16
 *                 [T,hc_mult,D], d_post_mix f32 [T,hc_mult] (the reference's [B,S,hc_mult,1]), d_comb_mix f32
 *                 [T,hc_mult,hc_mult]; out[t,i,:] = x[t,:] * post_mix[t,i] + sum_j comb_mix[t,j,i] * residual[t,j,:]
 *                 in f32 (terms in ascending j, fused multiply-adds), rounded once to bf16. hc_mult <= 8.
 * d_out may alias d_residual only when hc_mult == 0. Pointers 16-byte aligned, D a multiple of 8. */
int dmoe_block_post(uint16_t *d_out, const uint16_t *d_ffn_out, const uint16_t *d_residual,
                    const float *d_post_mix, const float *d_comb_mix, int T, int D, int hc_mult, dmoe_stream s);

/* ---- continuous-batch assembly ---------------------------------------------------------------- */

/* batch_builder.build (batch_builder.zig:90-214) with the per-token work on the device. The caller walks its
 * requests (prefill requests first, then decode ones, :104-111), concatenates their tokens
 * (getRequestTokens, :47-83) and passes per request the token count and the position of its first token
 * (:146-153). Outputs, each nullable:
 *   d_out_tokens u32 [T]           batched_tokens (a copy of h_tokens)
 *   d_out_positions i32 [T]        position_ids: base_pos[r] + index within request r
 *   d_out_mask f32 [T,T]           attention_mask: 0 where row and column belong to the same request and
 *                                  column <= row, -inf elsewhere (:140-177); 16-byte aligned, T <= 65535
 *   d_out_request_of_token u32 [T] request index of every token (no counterpart in the reference; the
 *                                  per-request view of a packed batch)
 * Host inputs are read before the call returns. T = sum of h_seq_lens; T == 0 is the empty batch. */
int dmoe_batch_build(uint32_t *d_out_tokens, int32_t *d_out_positions, float *d_out_mask,
                     uint32_t *d_out_request_of_token, const uint32_t *h_tokens, const int32_t *h_seq_lens,
                     const int32_t *h_base_pos, int n_requests, int T, dmoe_workspace ws, dmoe_stream s);

/* Inspection of the last dmoe_moe_forward / dmoe_switch_glu_forward_no_scores on this workspace:
 * the SwiGLU activations in flat (t*K+k) row order, bf16 [T*K, F]. For parity tests. */
int dmoe_debug_last_activations(uint16_t *d_out, dmoe_layer layer, int T, dmoe_workspace ws, dmoe_stream s);

/* dmoe_dequantize through the decoder that the prefill kernels run in registers between their matrix instructions
 * (same arguments, same result layout). For parity tests: the fused decode must give the bits of dmoe_dequantize,
 * i.e. of mlx_dequantize as called at deepseek_v4_loader.zig:129, for every scale and bias. */
int dmoe_debug_dequantize_fused(uint16_t *d_out, const dmoe_qweight *qw, int mat_index, dmoe_stream s);

/* Calibration for the benchmark (no counterpart in the reference): ONE launch of a loop of bf16 matrix instructions
 * (v_mfma_f32_32x32x16_bf16) on operands held in registers, 512 workgroups of 4 wavefronts, `iters` iterations of 32
 * instructions per wavefront: DMOE_MFMA_LOOP_FLOP_PER_ITER floating-point operations per iteration and launch. What
 * the matrix cores sustain with nothing else running depends on the operand values (power), so the caller chooses them:
 * d_operands = DMOE_MFMA_LOOP_OPERANDS bf16 values (24 fragments x 256 lanes x 8), d_out = DMOE_MFMA_LOOP_OUT floats
 * (one checksum per lane, so that the loop is not removed). The caller times the launch. */
#define DMOE_MFMA_LOOP_OPERANDS 49152
#define DMOE_MFMA_LOOP_OUT 131072
#define DMOE_MFMA_LOOP_FLOP_PER_ITER 2147483648.0 /* 512 x 4 wavefronts x 32 instructions x 2*32*32*16 */
int dmoe_debug_mfma_loop(float *d_out, const uint16_t *d_operands, int iters, dmoe_stream s);

/* Calibration for the benchmark (no counterpart in the reference): ONE launch of a kernel that only reads. `workgroups`
 * workgroups of 4 wavefronts; every wavefront streams a private contiguous part of d_src [bytes] with 16-byte loads,
 * eight per lane in flight, with the streaming hint of the decode kernel's weight loads, and stores one checksum word
 * into d_sink [4 * workgroups]. Whole 8 KiB chunks per wavefront only: *out_bytes_read gets the bytes one launch reads
 * (<= bytes). The caller times the launch; a source larger than the 256 MiB memory-side cache measures HBM. */
int dmoe_debug_read_stream(size_t *out_bytes_read, uint32_t *d_sink, const void *d_src, size_t bytes, int workgroups,
                           dmoe_stream s);

#ifdef __cplusplus
}
#endif
#endif /* DMOE_H */
