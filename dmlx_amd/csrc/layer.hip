// Resident MoE layer: weights held in HBM, and the forward pass
//   pack (slot map of Smelt layers applied as the ids are read) -> grouped gate/up + limited SwiGLU -> grouped down ->
//   weighted sum over k (+ shared).
// Also dmoe_gather_qmm, the leaf operator, built from the same pack + grouped-GEMM kernels.
#include <string.h>

#include <algorithm>
#include <mutex>
#include <new>
#include <vector>

#include "common.h"

namespace dmoe {

struct QOwned {
    dmoe_qweight q;        // device pointers (MLX layout) while the layer is being built
    void *own[5] = {nullptr, nullptr, nullptr, nullptr, nullptr}; // w, scales, biases (MLX layout); packed w, packed meta
    QView view;            // what the kernels read: the packed layout whenever the shape allows it
};

struct Layer {
    int D = 0, F = 0, K = 0, E = 0, Fs = 0;
    QOwned gate, up, down, sgate, sup, sdown;
    bool has_shared = false;
    // the shared expert's packed weights also sit behind the routed experts' as matrix E of the same buffers: at
    // decode sizes it then rides in the routed launches as an always-on expert (no side stream, no fork / join)
    bool shared_folded = false;
    float swiglu_limit = 0.0f, shared_swiglu_limit = 0.0f;
    bool score_before_down = false;
    int32_t *remap = nullptr; // device
    int n_total = 0;
    int device = 0;
};

static void free_owned(QOwned &o) {
    for (void *&p : o.own) {
        if (p) (void)hipFree(p);
        p = nullptr;
    }
}

static void free_layer(Layer *L) {
    free_owned(L->gate);
    free_owned(L->up);
    free_owned(L->down);
    free_owned(L->sgate);
    free_owned(L->sup);
    free_owned(L->sdown);
    if (L->remap) (void)hipFree(L->remap);
    delete L;
}

// `spare_mats`: room for that many more matrices behind the stack in the packed buffers
static int adopt(QOwned *dst, const dmoe_qweight *src, int source, const char *name, hipStream_t st, int spare_mats = 0) {
    dst->q = *src;
    if (source != DMOE_WEIGHTS_BORROW_DEVICE) {
        DMOE_REQUIRE(src->w && (src->scales || src->mode == DMOE_QUANT_NONE), "%s: weight / scales pointer is null", name);
        // validate the shape before sizing any copy
        QView probe;
        dmoe_qweight tmp = *src;
        // make_qview checks pointer alignment; host pointers need not be aligned, device copies will be
        tmp.w = (const void *)(uintptr_t)16;
        DMOE_TRY(make_qview(&probe, &tmp, name));
        const void *in[3] = {src->w, src->scales, src->biases};
        size_t bytes[3] = {qweight_w_bytes(src), qweight_s_bytes(src), qweight_b_bytes(src)};
        hipMemcpyKind kind = source == DMOE_WEIGHTS_COPY_FROM_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
        for (int i = 0; i < 3; ++i) {
            if (!in[i] || !bytes[i]) continue;
            DMOE_HIP(hipMalloc(&dst->own[i], bytes[i]));
            DMOE_HIP(hipMemcpyAsync(dst->own[i], in[i], bytes[i], kind, st));
        }
        dst->q.w = dst->own[0];
        dst->q.scales = dst->own[1];
        dst->q.biases = dst->own[2];
    }
    DMOE_TRY(make_qview(&dst->view, &dst->q, name));
    if (!can_pack(dst->view)) return DMOE_OK; // odd shapes stay in the MLX layout (slower addressing, same results)
    // resident layout: re-order once so that every wavefront streams its 32 weight rows linearly
    const size_t wb = packed_w_bytes(dst->view), mb = packed_meta_bytes(dst->view);
    const size_t n_mats = (size_t)dst->view.n_mats;
    DMOE_HIP(hipMalloc(&dst->own[3], wb + wb / n_mats * (size_t)spare_mats));
    if (mb) DMOE_HIP(hipMalloc(&dst->own[4], mb + mb / n_mats * (size_t)spare_mats));
    DMOE_TRY(launch_repack(dst->own[3], dst->own[4], dst->view, st));
    DMOE_HIP(hipStreamSynchronize(st));
    // the MLX-layout copies are no longer needed (fp8 keeps its per-row scales)
    const bool keep_scales = dst->view.mode == DMOE_QUANT_FP8_ROW;
    for (int i = 0; i < 3; ++i) {
        if (i == 1 && keep_scales) continue;
        if (dst->own[i]) DMOE_HIP(hipFree(dst->own[i]));
        dst->own[i] = nullptr;
    }
    dst->view.packed = true;
    dst->view.w = (const uint8_t *)dst->own[3];
    dst->view.meta = (const uint8_t *)dst->own[4];
    dst->view.m_mat = mb / (size_t)dst->view.n_mats;
    if (!keep_scales) dst->view.scales = nullptr;
    dst->view.biases = nullptr;
    return DMOE_OK;
}

// Copies the shared expert's packed weights behind the routed experts' (matrix index E of the routed buffers), when
// the two have the same shape and format. Needs the spare matrix adopt() left room for.
static bool same_packed_format(const QView &a, const QView &b) {
    return a.packed && b.packed && a.rows == b.rows && a.cols == b.cols && a.mode == b.mode && a.bits == b.bits &&
           a.group == b.group && a.mode != DMOE_QUANT_FP8_ROW;
}
static int fold_shared(Layer *L, hipStream_t st) {
    QOwned *routed[3] = {&L->gate, &L->up, &L->down}, *shared[3] = {&L->sgate, &L->sup, &L->sdown};
    for (int i = 0; i < 3; ++i)
        if (!same_packed_format(routed[i]->view, shared[i]->view)) return DMOE_OK;
    for (int i = 0; i < 3; ++i) {
        const QView &r = routed[i]->view, &s = shared[i]->view;
        DMOE_HIP(hipMemcpyAsync((uint8_t *)routed[i]->own[3] + (size_t)L->E * r.w_mat, s.w, s.w_mat, hipMemcpyDeviceToDevice, st));
        if (r.m_mat)
            DMOE_HIP(hipMemcpyAsync((uint8_t *)routed[i]->own[4] + (size_t)L->E * r.m_mat, s.meta, s.m_mat, hipMemcpyDeviceToDevice, st));
    }
    DMOE_HIP(hipStreamSynchronize(st));
    L->shared_folded = true;
    return DMOE_OK;
}

// ---- small kernels ----------------------------------------------------------------------------------

__global__ void compose_rows_kernel(uint32_t *__restrict__ out, const uint32_t *__restrict__ lhs,
                                    const uint32_t *__restrict__ order, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = lhs[order[i]];
}

// out[dst[p], :] = in[p, :], 16 bytes per thread
__global__ void scatter_rows_kernel(uint4 *__restrict__ out, const uint4 *__restrict__ in,
                                    const uint32_t *__restrict__ dst, size_t row_vecs, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    size_t p = i / row_vecs, c = i - p * row_vecs;
    out[(size_t)dst[p] * row_vecs + c] = in[i];
}

// out[t, :] = sum_k (w ? w[t,k] : 1) * y[t*K+k, :] + (shared ? shared[t, :] : 0); 8 columns per thread
__global__ void combine_kernel(uint16_t *__restrict__ out, const uint16_t *__restrict__ y,
                               const float *__restrict__ w, const uint16_t *__restrict__ shared, int T, int K,
                               int D) {
    const size_t vec_per_row = (size_t)D / 8;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * vec_per_row) return;
    size_t t = i / vec_per_row, c = i - t * vec_per_row;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
    for (int k = 0; k < K; ++k) {
        size_t r = t * (size_t)K + k;
        float wk = w ? w[r] : 1.0f;
        uint4 q = *(const uint4 *)(y + r * (size_t)D + c * 8);
        uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] += bf16_bits_to_f32(u[j] & 0xffffu) * wk;
            acc[2 * j + 1] += bf16_bits_to_f32(u[j] >> 16) * wk;
        }
    }
    if (shared) {
        uint4 q = *(const uint4 *)(shared + t * (size_t)D + c * 8);
        uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] += bf16_bits_to_f32(u[j] & 0xffffu);
            acc[2 * j + 1] += bf16_bits_to_f32(u[j] >> 16);
        }
    }
    uint4 o = make_uint4(pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]), pack_bf16x2(acc[4], acc[5]),
                         pack_bf16x2(acc[6], acc[7]));
    *(uint4 *)(out + t * (size_t)D + c * 8) = o;
}

// ---- forward -------------------------------------------------------------------------------------------

// At or below this many rows per expert on average the skinny (weight-streaming) kernel runs every tile. Measured on one
// projection [128, 2048, 4096] with every expert live (TB/s of weight bytes, whole call): at 12 and 16 rows per expert
// the weight-streaming kernel gives 4.1 / 4.0 against the matrix-core kernel's 3.5 / 3.6 (4-bit affine), 4.5 / 4.3 against
// 4.4 / 4.3 (MXFP4), 5.3 / 5.3 against 5.2 / 5.2 (8-bit); at 24 and 32 rows the matrix-core kernel is level or ahead.
constexpr int kSkinnyAvgRows = 16;
// Up to this many sorted rows (hence tiles) in a decode step the weight-streaming launch leaves most of the chip's
// workgroup slots empty (32 workgroups per tile, 512 slots): each tile's reduction is then split over twice the
// workgroups (GemmArgs::ksplit), on tiles of one row block.
constexpr int kSplitMaxTiles = 8;
constexpr int kSplitTileM = 8;
#ifndef DMOE_PAIR_MIN_ROWS
#define DMOE_PAIR_MIN_ROWS 64
#endif
constexpr int kPairMinRows = DMOE_PAIR_MIN_ROWS; // decode steps above this many sorted rows run gate/up and down in one launch
constexpr int kSharedSkinnyRows = 64;

static bool few_rows(size_t rows, int n_experts) { return rows <= (size_t)kSkinnyAvgRows * (size_t)n_experts; }
static bool use_small_path(size_t rows, int n_experts, const QView &b) {
    return qgemm_skinny_supports(b) && few_rows(rows, n_experts);
}
struct FwdLayout {
    size_t order, inv, token, sorted_e, counts, offsets, live, n_live, tiles, n_tiles, tile_done, scratch;
    size_t h, y, sh_h, sh_y, total;
    int max_tiles, tile_m;
    bool small;
    bool ksplit; // a handful of tiles of at most 8 rows: the weight-streaming kernel splits each tile's reduction in two
    bool fold; // the shared expert rides in the routed launches: T more sorted rows behind the T*K routed ones
};

static FwdLayout forward_layout(const Layer *L, int T, bool with_shared = true) {
    FwdLayout f;
    Bump b;
    size_t n = (size_t)T * L->K;
    f.small = use_small_path(n, L->E, L->gate.view) && qgemm_skinny_supports(L->down.view);
    // one tile list serves both GEMMs: the smaller of their tile sizes
    f.tile_m = f.small ? std::min(qgemm_skinny_tile_m(L->gate.view), qgemm_skinny_tile_m(L->down.view))
                       : std::min(qgemm_mfma_tile_m(L->gate.view), qgemm_mfma_tile_m(L->down.view));
    f.fold = with_shared && f.small && L->shared_folded;
    const size_t rows = n + (f.fold ? (size_t)T : 0); // sorted rows of the GEMMs
    // single-stream decode: at most kSplitMaxTiles tiles even if every row goes to another expert
    f.ksplit = f.small && rows <= (size_t)kSplitMaxTiles && qgemm_skinny_ksplit_ok(L->gate.view) &&
               qgemm_skinny_ksplit_ok(L->up.view) && qgemm_skinny_ksplit_ok(L->down.view) &&
               (!f.fold || (qgemm_skinny_ksplit_ok(L->sgate.view) && qgemm_skinny_ksplit_ok(L->sup.view) &&
                            qgemm_skinny_ksplit_ok(L->sdown.view)));
    if (f.ksplit) f.tile_m = kSplitTileM;
    f.max_tiles = pack_max_tiles(n, L->E, f.tile_m) + (f.fold ? ceil_div(T, f.tile_m) : 0);
    f.order = b.take(rows * 4);
    f.inv = b.take(n * 4);
    f.token = b.take(rows * 4);
    f.sorted_e = b.take(rows * 4);
    f.counts = b.take((size_t)L->E * 4);
    f.offsets = b.take((size_t)(L->E + 1) * 4);
    f.live = b.take((size_t)L->E * 4);
    f.n_live = b.take(4);
    f.tiles = b.take((size_t)(f.max_tiles > 0 ? f.max_tiles : 1) * sizeof(Tile));
    f.n_tiles = b.take(4);
    f.tile_done = b.take((size_t)(f.max_tiles > 0 ? f.max_tiles : 1) * 4);
    f.scratch = b.take(pack_scratch_bytes(n, L->E));
    f.h = b.take(rows * (size_t)L->F * 2);
    f.y = b.take(rows * (size_t)L->D * 2);
    f.sh_h = b.take(L->has_shared && !f.fold ? (size_t)T * L->Fs * 2 : 0);
    f.sh_y = b.take(L->has_shared && !f.fold ? (size_t)T * L->D * 2 : 0);
    f.total = b.off;
    return f;
}

// Prefill-sized calls: the matrix-core kernel takes the tiles above `small_rows` rows, and the weight-streaming kernel
// the rest of the same list right behind it (a tile of a few rows is bound by reading its expert's weights, and the
// large-tile kernel spends a whole pass of its LDS pipeline on it). small_rows = 0: everything on the matrix-core kernel.
constexpr int kPrefillSmallRows = 8;
static int prefill_small_rows(const QView &b0, const QView &b1) {
    if (!qgemm_skinny_supports(b0) || !qgemm_skinny_supports(b1)) return 0;
    // measured: pays with the kernel of the packed 4-bit formats (8k-token ragged prefill: gate/up 1.757 -> 1.715 ms, down
    // unchanged), not with the 8-bit kernel (2080-token mixed batch: +1 %)
    if (!qgemm_wide_supports(b0) || !qgemm_wide_supports(b1)) return 0;
    const auto four_bit = [](const QView &b) { return b.mode == DMOE_QUANT_MXFP4 || (b.mode == DMOE_QUANT_AFFINE && b.bits == 4); };
    if (!four_bit(b0) || !four_bit(b1)) return 0;
    // threshold measured on the same prefill: 8 rows 2.62 ms, 16 rows 2.63, 32 rows 2.64, 4 rows 2.67, no split 2.70
    return std::min(kPrefillSmallRows, std::min(qgemm_skinny_tile_m(b0), qgemm_skinny_tile_m(b1)));
}
// `few` = few rows per expert (only read for unquantized weights; the quantized formats have `small`)
static int run_gemm(const GemmArgs &g, bool small, hipStream_t st, int small_rows = 0, bool few = false) {
    if (g.b0.mode == DMOE_QUANT_NONE) {
        if (small) return launch_qgemm_skinny(g, st); // few rows per expert on resident weights: the weight-streaming kernel
        // prefill sizes on resident weights: the matrix-core kernel with activations through LDS
        const bool wide = !few && qgemm_wide_bf16_supports(g.b0) && (!g.gate_up || qgemm_wide_bf16_supports(g.b1)) &&
                          g.tile_m % 32 == 0 && g.tile_m <= kMfmaWideTileM;
        return wide ? launch_qgemm_wide(g, st) : launch_gemm_bf16(g, st);
    }
    if (small) return launch_qgemm_skinny(g, st);
    if (small_rows <= 0 || !g.tiles) return launch_qgemm_mfma(g, st);
    GemmArgs big = g, rest = g;
    big.min_rows = small_rows + 1;
    rest.max_rows = small_rows;
    DMOE_TRY(launch_qgemm_mfma(big, st));
    return launch_qgemm_skinny(rest, st);
}

// routed experts on slot ids: fills ws->y ([T*K, D] bf16 in flat (t,k) order) or `y_out` when given
static int routed_forward(const Layer *L, Workspace *w, const FwdLayout &f, const uint16_t *d_x,
                          const uint32_t *d_ids, bool remap, const float *d_scores, int T, uint16_t *y_out,
                          hipStream_t st, const RouteArgs *route = nullptr) {
    size_t n = (size_t)T * L->K;
    PackOut po;
    po.order = at<uint32_t>(w, f.order);
    po.inv = at<uint32_t>(w, f.inv);
    po.token = at<uint32_t>(w, f.token);
    po.sorted_e = at<uint32_t>(w, f.sorted_e);
    po.counts = at<uint32_t>(w, f.counts);
    po.offsets = at<uint32_t>(w, f.offsets);
    po.live = at<uint32_t>(w, f.live);
    po.n_live = at<uint32_t>(w, f.n_live);
    po.tiles = at<Tile>(w, f.tiles);
    po.n_tiles = at<uint32_t>(w, f.n_tiles);
    if (f.fold) {
        po.dense_rows = (uint32_t)T;
        po.dense_expert = (uint32_t)L->E;
    }
    // per-tile completion counters of the paired gate/up + down launch, zeroed with the tile list
    po.tile_done = at<uint32_t>(w, f.tile_done);
    po.n_done = (uint32_t)f.max_tiles;
    po.bad_ids = w->flags + 1;
    if (remap) { // global expert ids -> resident slots, inside the packing kernels
        po.remap = L->remap;
        po.n_remap = (uint32_t)L->n_total;
    }
    if (route) DMOE_TRY(launch_route_pack_tiny(po, *route, L->E, f.tile_m, st)); // the selection has not run yet: one launch for both
    else DMOE_TRY(launch_pack(po, d_ids, n, L->K, L->E, f.tile_m, at<void>(w, f.scratch), st));
    DMOE_TRY(stage_end(w, DMOE_STAGE_PACK, st));

    GemmArgs gu;
    gu.b0 = L->gate.view;
    gu.b1 = L->up.view;
    gu.gate_up = true;
    gu.a = d_x;
    gu.a_rows = po.token;
    gu.out = at<uint16_t>(w, f.h);
    gu.ldo = L->F;
    gu.tiles = po.tiles;
    gu.n_tiles = po.n_tiles;
    gu.max_tiles = f.max_tiles;
    gu.tile_m = f.tile_m;
    gu.ksplit = f.ksplit ? 1 : 0;
    gu.swiglu_limit = L->swiglu_limit;
    gu.swiglu_limit_dense = L->shared_swiglu_limit;
    if (L->score_before_down && d_scores) {
        gu.row_scale = d_scores;
        gu.row_scale_idx = po.order;
        gu.row_scale_rows = (uint32_t)n; // the folded shared expert's rows carry no routing weight
    }
    GemmArgs dn;
    dn.b0 = L->down.view;
    dn.a = at<uint16_t>(w, f.h);
    dn.out = y_out ? y_out : at<uint16_t>(w, f.y);
    dn.ldo = L->D;
    dn.out_rows = po.order; // unsort while storing (deepseek_v4.zig:809)
    dn.tiles = po.tiles;
    dn.n_tiles = po.n_tiles;
    dn.max_tiles = f.max_tiles;
    dn.tile_m = f.tile_m;
    dn.ksplit = f.ksplit ? 1 : 0;

    // Decode sizes: both GEMMs in one launch; a down workgroup waits for its own tile's gate/up workgroups only, so
    // the down projection fills the chip while the last gate/up workgroups drain (timed as the gate/up stage).
    gu.tile_done = po.tile_done;
    dn.spin_limit = w->spin_limit;
    dn.wait_expired = w->flags;
    // (Up to kPairMinRows sorted rows the two projections run as two launches: with so few tiles nearly every gate/up
    // workgroup is resident from the start, no down workgroup can begin before they end, and what the single launch
    // adds is the hand-over through memory - stores acknowledged, counter, poll - of 6-8 us per step.)
    if (f.small && w->paired && n + (f.fold ? (size_t)T : 0) > (size_t)kPairMinRows && qgemm_skinny_pair_supports(gu, dn)) {
        DMOE_TRY(stage_begin(w, DMOE_STAGE_GATE_UP, st));
        DMOE_TRY(launch_qgemm_skinny_pair(gu, dn, st));
        DMOE_TRY(stage_end(w, DMOE_STAGE_GATE_UP, st));
        return DMOE_OK;
    }
    const int small_rows = f.small ? 0 : prefill_small_rows(L->gate.view, L->down.view);
    if (small_rows > 0 && !w->timer.enabled && w->paired && !w->fixed) {
        // Prefill: the small tiles' two GEMMs (one paired launch) depend on the tile list only. They go to the side
        // stream and fill the tails of the two matrix-core launches, which take the large tiles on `st`. (With stage
        // timing on, the launches stay in a row on `st` so that every stage's time covers all of its tiles.)
        GemmArgs gu_small = gu, dn_small = dn, gu_big = gu, dn_big = dn;
        gu_small.max_rows = dn_small.max_rows = small_rows;
        gu_big.min_rows = dn_big.min_rows = small_rows + 1;
        if (qgemm_skinny_pair_supports(gu_small, dn_small)) {
            DMOE_TRY(side_stream_ready(w));
            DMOE_HIP(hipEventRecord(w->packed, st));
            DMOE_HIP(hipStreamWaitEvent(w->side, w->packed, 0));
            DMOE_TRY(launch_qgemm_skinny_pair(gu_small, dn_small, w->side));
            DMOE_HIP(hipEventRecord(w->small_done, w->side));
            DMOE_TRY(launch_qgemm_mfma(gu_big, st));
            DMOE_TRY(launch_qgemm_mfma(dn_big, st));
            DMOE_HIP(hipStreamWaitEvent(st, w->small_done, 0));
            return DMOE_OK;
        }
    }
    if (small_rows > 0) { // stage timing on, or no paired launch / no side stream: the four launches in a row, each its own stage
        GemmArgs gu_small = gu, dn_small = dn, gu_big = gu, dn_big = dn;
        gu_small.max_rows = dn_small.max_rows = small_rows;
        gu_big.min_rows = dn_big.min_rows = small_rows + 1;
        DMOE_TRY(stage_begin(w, DMOE_STAGE_GATE_UP, st));
        DMOE_TRY(launch_qgemm_mfma(gu_big, st));
        DMOE_TRY(stage_end(w, DMOE_STAGE_GATE_UP, st));
        DMOE_TRY(stage_begin(w, DMOE_STAGE_GATE_UP_SMALL, st));
        DMOE_TRY(launch_qgemm_skinny(gu_small, st));
        DMOE_TRY(stage_end(w, DMOE_STAGE_GATE_UP_SMALL, st));
        DMOE_TRY(stage_begin(w, DMOE_STAGE_DOWN, st));
        DMOE_TRY(launch_qgemm_mfma(dn_big, st));
        DMOE_TRY(stage_end(w, DMOE_STAGE_DOWN, st));
        DMOE_TRY(stage_begin(w, DMOE_STAGE_DOWN_SMALL, st));
        DMOE_TRY(launch_qgemm_skinny(dn_small, st));
        DMOE_TRY(stage_end(w, DMOE_STAGE_DOWN_SMALL, st));
        return DMOE_OK;
    }
    DMOE_TRY(stage_begin(w, DMOE_STAGE_GATE_UP, st));
    const bool few = few_rows(n, L->E);
    DMOE_TRY(run_gemm(gu, f.small, st, 0, few));
    DMOE_TRY(stage_end(w, DMOE_STAGE_GATE_UP, st));
    DMOE_TRY(stage_begin(w, DMOE_STAGE_DOWN, st));
    DMOE_TRY(run_gemm(dn, f.small, st, 0, few));
    DMOE_TRY(stage_end(w, DMOE_STAGE_DOWN, st));
    return DMOE_OK;
}

static int shared_forward(const Layer *L, Workspace *w, const FwdLayout &f, const uint16_t *d_x, int T,
                          hipStream_t st) {
    // up to 64 rows the dense expert is streamed by the skinny kernel in 8-row tiles (many workgroups per
    // block of weight rows); above that the big-tile kernel amortises the dequantization
    const bool small = T <= kSharedSkinnyRows && qgemm_skinny_supports(L->sgate.view) && qgemm_skinny_supports(L->sdown.view);
    const int tile_m = small ? kSkinnyDenseTileM : std::min(qgemm_mfma_tile_m(L->sgate.view), qgemm_mfma_tile_m(L->sdown.view));
    GemmArgs gu;
    gu.b0 = L->sgate.view;
    gu.b1 = L->sup.view;
    gu.gate_up = true;
    gu.a = d_x;
    gu.out = at<uint16_t>(w, f.sh_h);
    gu.ldo = L->Fs;
    gu.dense_rows = T;
    gu.max_tiles = ceil_div(T, tile_m);
    gu.tile_m = tile_m;
    gu.swiglu_limit = L->shared_swiglu_limit;
    DMOE_TRY(run_gemm(gu, small, st, 0, T <= kSharedSkinnyRows));
    GemmArgs dn;
    dn.b0 = L->sdown.view;
    dn.a = at<uint16_t>(w, f.sh_h);
    dn.out = at<uint16_t>(w, f.sh_y);
    dn.ldo = L->D;
    dn.dense_rows = T;
    dn.max_tiles = ceil_div(T, tile_m);
    dn.tile_m = tile_m;
    DMOE_TRY(run_gemm(dn, small, st, 0, T <= kSharedSkinnyRows));
    return DMOE_OK;
}

// ---- per-workspace cache of resident copies for dmoe_gather_qmm --------------------------------------------
struct CachedStack {
    dmoe_qweight key; // the caller's stack as passed (pointers, shape, format)
    QOwned owned;     // its re-ordered copy
    size_t bytes = 0; // device bytes held by the copy
    uint64_t last_use = 0;
};
struct WeightCache {
    std::vector<CachedStack *> items;
    size_t bytes = 0;
    uint64_t clock = 0;
};
static bool same_stack(const dmoe_qweight &a, const dmoe_qweight &b) {
    return a.w == b.w && a.scales == b.scales && a.biases == b.biases && a.n_mats == b.n_mats && a.rows == b.rows &&
           a.cols == b.cols && a.mode == b.mode && a.bits == b.bits && a.group_size == b.group_size;
}
static void drop_item(WeightCache *c, size_t i) {
    CachedStack *it = c->items[i];
    c->bytes -= it->bytes;
    free_owned(it->owned);
    delete it;
    c->items.erase(c->items.begin() + (long)i);
}
void weight_cache_clear(Workspace *w) {
    WeightCache *c = (WeightCache *)w->weight_cache;
    if (!c) return;
    while (!c->items.empty()) drop_item(c, c->items.size() - 1);
    delete c;
    w->weight_cache = nullptr;
}
// drops the copy of `qw` (null: every copy); kernels in flight may still read a copy, so the device is waited for
int weight_cache_invalidate(Workspace *w, const dmoe_qweight *qw) {
    WeightCache *c = (WeightCache *)w->weight_cache;
    if (!c || c->items.empty()) return DMOE_OK;
    DMOE_HIP(hipDeviceSynchronize());
    for (size_t i = c->items.size(); i-- > 0;)
        if (!qw || same_stack(c->items[i]->key, *qw)) drop_item(c, i);
    return DMOE_OK;
}
// the cached resident view of `qw`, made on first sight (one re-ordering pass, waits for it)
static int weight_cache_find_or_add(Workspace *w, const dmoe_qweight *qw, const QView **out, hipStream_t st) {
    if (!w->weight_cache) w->weight_cache = new (std::nothrow) WeightCache();
    WeightCache *c = (WeightCache *)w->weight_cache;
    DMOE_REQUIRE(c != nullptr, "gather_qmm: out of host memory");
    for (CachedStack *it : c->items)
        if (same_stack(it->key, *qw)) {
            it->last_use = ++c->clock;
            *out = &it->owned.view;
            return DMOE_OK;
        }
    CachedStack *it = new (std::nothrow) CachedStack();
    DMOE_REQUIRE(it != nullptr, "gather_qmm: out of host memory");
    it->key = *qw;
    int rc = adopt(&it->owned, qw, DMOE_WEIGHTS_BORROW_DEVICE, "gather_qmm (cached stack)", st);
    if (rc != DMOE_OK) {
        free_owned(it->owned);
        delete it;
        return rc;
    }
    it->bytes = it->owned.view.packed ? packed_w_bytes(it->owned.view) + packed_meta_bytes(it->owned.view) : 0;
    // over the byte limit: the least recently used copies go first (never the new one). Their kernels may still run.
    if (w->cache_limit_bytes && c->bytes + it->bytes > w->cache_limit_bytes && !c->items.empty()) {
        hipError_t e = hipDeviceSynchronize();
        if (e != hipSuccess) {
            free_owned(it->owned);
            delete it;
            return hip_fail(e, "hipDeviceSynchronize");
        }
        while (!c->items.empty() && c->bytes + it->bytes > w->cache_limit_bytes) {
            size_t oldest = 0;
            for (size_t i = 1; i < c->items.size(); ++i)
                if (c->items[i]->last_use < c->items[oldest]->last_use) oldest = i;
            drop_item(c, oldest);
        }
    }
    it->last_use = ++c->clock;
    c->bytes += it->bytes;
    c->items.push_back(it);
    *out = &it->owned.view;
    return DMOE_OK;
}
int weight_cache_stats(Workspace *w, size_t *out_bytes, int *out_stacks) {
    WeightCache *c = (WeightCache *)w->weight_cache;
    if (out_bytes) *out_bytes = c ? c->bytes : 0;
    if (out_stacks) *out_stacks = c ? (int)c->items.size() : 0;
    return DMOE_OK;
}

// ---- static device scratch of the allocation-free entry point ---------------------------------------------
// One array per GPU, part of the library's code object (held by every GPU the library runs on until the process
// ends). In host code `scratch` is only a handle for hipGetSymbolAddress: the device address is looked up once per
// device and everything below uses that pointer.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
constexpr size_t kStaticFlagBytes = 256;   // the workspace's flag words sit in front of the bump area
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kStaticMaxDevices = 64;
static Workspace g_static_ws[kStaticMaxDevices];
static bool g_static_ready[kStaticMaxDevices];
static std::mutex g_static_mutex;

int static_workspace(Workspace **out) {
    int dev = 0;
    DMOE_HIP(hipGetDevice(&dev));
    DMOE_REQUIRE(dev >= 0 && dev < kStaticMaxDevices, "static scratch: device index %d is out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_mutex);
    Workspace &w = g_static_ws[dev];
    if (!g_static_ready[dev]) {
        void *ptr = nullptr;
        DMOE_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))); // this device's copy (the current device)
        DMOE_REQUIRE(ptr != nullptr && ((uintptr_t)ptr % 256) == 0, "static scratch: bad device address %p", ptr);
        w.flags = (uint32_t *)ptr; // never read back on this path (no bounded waits; bad ids stay clamped)
        w.base = (unsigned char *)ptr + kStaticFlagBytes;
        w.bytes = kStaticScratchBytes - kStaticFlagBytes;
        w.device = dev;
        w.fixed = true;   // never grows, never creates a stream or an event
        w.paired = false; // gate/up and down as two launches: nothing waits inside a kernel, nothing to check later
        g_static_ready[dev] = true;
    }
    *out = &w;
    return DMOE_OK;
}

} // namespace dmoe

using namespace dmoe;

extern "C" {

int dmoe_layer_create(dmoe_layer *out, const dmoe_layer_desc *d, dmoe_stream s) {
    DMOE_REQUIRE(out && d, "layer_create: null argument");
    out->ctx = nullptr;
    DMOE_REQUIRE(d->hidden > 0 && d->ffn > 0 && d->top_k > 0, "layer_create: bad dims D=%d F=%d K=%d", d->hidden,
                 d->ffn, d->top_k);
    DMOE_REQUIRE(d->weight_source >= 0 && d->weight_source <= 2, "layer_create: bad weight_source %d",
                 d->weight_source);
    DMOE_REQUIRE(d->hidden % 8 == 0 && d->ffn % 8 == 0, "layer_create: D and F must be multiples of 8");
    DMOE_REQUIRE(d->gate.rows == d->ffn && d->gate.cols == d->hidden && d->up.rows == d->ffn &&
                     d->up.cols == d->hidden && d->down.rows == d->hidden && d->down.cols == d->ffn,
                 "layer_create: projection shapes do not match D=%d F=%d", d->hidden, d->ffn);
    DMOE_REQUIRE(d->gate.n_mats == d->up.n_mats && d->gate.n_mats == d->down.n_mats && d->gate.n_mats >= 1 &&
                     d->gate.n_mats <= 1024,
                 "layer_create: expert counts differ or are out of range");
    Layer *L = new (std::nothrow) Layer();
    DMOE_REQUIRE(L != nullptr, "layer_create: out of host memory");
    hipStream_t st = to_hip(s);
    int rc = DMOE_OK;
    do {
        if (hipGetDevice(&L->device) != hipSuccess) { rc = hip_fail(hipGetLastError(), "hipGetDevice"); break; }
        L->D = d->hidden;
        L->F = d->ffn;
        L->K = d->top_k;
        L->E = d->gate.n_mats;
        L->swiglu_limit = d->swiglu_limit;
        L->score_before_down = d->score_before_down != 0;
        const int spare = d->has_shared ? 1 : 0; // room for the shared expert behind the routed ones (fold_shared)
        if ((rc = adopt(&L->gate, &d->gate, d->weight_source, "gate_proj", st, spare))) break;
        if ((rc = adopt(&L->up, &d->up, d->weight_source, "up_proj", st, spare))) break;
        if ((rc = adopt(&L->down, &d->down, d->weight_source, "down_proj", st, spare))) break;
        if (d->has_shared) {
            L->has_shared = true;
            L->Fs = d->shared_gate.rows;
            L->shared_swiglu_limit = d->shared_swiglu_limit;
            if (d->shared_gate.n_mats != 1 || d->shared_up.n_mats != 1 || d->shared_down.n_mats != 1 ||
                d->shared_gate.cols != L->D || d->shared_up.cols != L->D || d->shared_up.rows != L->Fs ||
                d->shared_down.rows != L->D || d->shared_down.cols != L->Fs || L->Fs % 8 != 0) {
                set_error("layer_create: shared expert shapes do not match D=%d", L->D);
                rc = DMOE_ERR_INVALID;
                break;
            }
            if ((rc = adopt(&L->sgate, &d->shared_gate, d->weight_source, "shared gate_proj", st))) break;
            if ((rc = adopt(&L->sup, &d->shared_up, d->weight_source, "shared up_proj", st))) break;
            if ((rc = adopt(&L->sdown, &d->shared_down, d->weight_source, "shared down_proj", st))) break;
            if (L->Fs == L->F && (rc = fold_shared(L, st))) break;
        }
        if (d->remap) {
            if (d->n_experts_total < 1) { set_error("layer_create: n_experts_total must be >= 1 with a remap"); rc = DMOE_ERR_INVALID; break; }
            for (int i = 0; i < d->n_experts_total; ++i)
                if (d->remap[i] < 0 || d->remap[i] >= L->E) {
                    set_error("layer_create: remap[%d] = %d is not a slot in [0,%d)", i, d->remap[i], L->E);
                    rc = DMOE_ERR_INVALID;
                    break;
                }
            if (rc) break;
            L->n_total = d->n_experts_total;
            hipError_t e = hipMalloc((void **)&L->remap, sizeof(int32_t) * (size_t)L->n_total);
            if (e == hipSuccess)
                e = hipMemcpyAsync(L->remap, d->remap, sizeof(int32_t) * (size_t)L->n_total, hipMemcpyHostToDevice, st);
            if (e != hipSuccess) { rc = hip_fail(e, "remap upload"); break; }
        }
        // host sources may be pageable and may be released by the caller right after this call
        hipError_t e = hipStreamSynchronize(st);
        if (e != hipSuccess) { rc = hip_fail(e, "hipStreamSynchronize"); break; }
    } while (0);
    if (rc != DMOE_OK) {
        free_layer(L);
        return rc;
    }
    out->ctx = L;
    return DMOE_OK;
}

int dmoe_layer_dims(int *out_hidden, int *out_ffn, int *out_n_slots, int *out_top_k, dmoe_layer layer) {
    const Layer *L = (const Layer *)layer.ctx;
    DMOE_REQUIRE(L != nullptr, "layer_dims: null layer");
    if (out_hidden) *out_hidden = L->D;
    if (out_ffn) *out_ffn = L->F;
    if (out_n_slots) *out_n_slots = L->E;
    if (out_top_k) *out_top_k = L->K;
    return DMOE_OK;
}

int dmoe_layer_destroy(dmoe_layer layer) {
    if (layer.ctx) free_layer((Layer *)layer.ctx);
    return DMOE_OK;
}

// `route` (optional): the gate's selection has not run yet and is to share a launch with the packing; it fills
// d_indices and d_scores (= route->out_idx, route->out_w) on the way.
static int forward_common(uint16_t *d_out, uint16_t *y_out, Layer *L, const uint16_t *d_x, const uint32_t *d_indices,
                          const float *d_scores, int T, bool apply_remap, bool with_shared, dmoe_workspace ws,
                          dmoe_stream s, const RouteArgs *route = nullptr) {
    DMOE_REQUIRE(T >= 0, "forward: T=%d", T);
    if (T == 0) return DMOE_OK;
    DMOE_REQUIRE(d_x && d_indices, "forward: null pointer");
    DMOE_REQUIRE(((uintptr_t)d_x % 16) == 0, "forward: x must be 16-byte aligned");
    DMOE_REQUIRE(y_out || (d_out && ((uintptr_t)d_out % 16) == 0), "forward: out must be 16-byte aligned and non-null");
    hipStream_t st = to_hip(s);
    FwdLayout f = forward_layout(L, T, with_shared && !y_out);
    Workspace *w = nullptr;
    DMOE_TRY(workspace_reserve(ws, f.total, &w));
    w->last_with_shared = with_shared && !y_out;
    DMOE_TRY(stage_begin(w, DMOE_STAGE_PACK, st));
    const bool remap = apply_remap && L->remap;
    // The shared expert does not depend on the routing: it runs on the workspace's side stream, forked
    // here and joined before the combine, so its two small dense GEMMs overlap pack and the routed GEMMs.
    // The routed launches are enqueued first: they are the critical path, and the host has all of their run
    // time to enqueue the side stream's work.
    const bool shared = with_shared && L->has_shared && !y_out;
    // else the shared expert is part of the routed launches, or (static scratch: no streams, no events) follows them
    const bool side_shared = shared && !f.fold && !w->fixed;
    if (side_shared) {
        DMOE_TRY(side_stream_ready(w));
        DMOE_HIP(hipEventRecord(w->fork, st));
    }
    DMOE_TRY(routed_forward(L, w, f, d_x, d_indices, remap, d_scores, T, y_out, st, route));
    if (side_shared) {
        DMOE_HIP(hipStreamWaitEvent(w->side, w->fork, 0));
        DMOE_TRY(stage_begin(w, DMOE_STAGE_SHARED, w->side));
        DMOE_TRY(shared_forward(L, w, f, d_x, T, w->side));
        DMOE_TRY(stage_end(w, DMOE_STAGE_SHARED, w->side));
        DMOE_HIP(hipEventRecord(w->join, w->side));
    }
    if (shared && !f.fold && w->fixed) DMOE_TRY(shared_forward(L, w, f, d_x, T, st));
    if (y_out) return DMOE_OK;
    if (side_shared) DMOE_HIP(hipStreamWaitEvent(st, w->join, 0));
    DMOE_TRY(stage_begin(w, DMOE_STAGE_COMBINE, st));
    size_t total = (size_t)T * (L->D / 8);
    hipLaunchKernelGGL(combine_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, d_out,
                       at<uint16_t>(w, f.y), L->score_before_down ? nullptr : d_scores,
                       !shared ? nullptr : f.fold ? at<uint16_t>(w, f.y) + (size_t)T * L->K * L->D : at<uint16_t>(w, f.sh_y), T,
                       L->K, L->D);
    DMOE_LAUNCH_CHECK();
    DMOE_TRY(stage_end(w, DMOE_STAGE_COMBINE, st));
    return DMOE_OK;
}

int dmoe_moe_forward(uint16_t *d_out, dmoe_layer layer, const uint16_t *d_x, const uint32_t *d_indices,
                     const float *d_scores, int T, dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(layer.ctx, "moe_forward: layer handle is null");
    DMOE_REQUIRE(d_scores || T == 0, "moe_forward: scores pointer is null");
    return forward_common(d_out, nullptr, (Layer *)layer.ctx, d_x, d_indices, d_scores, T, true, true, ws, s);
}

int dmoe_switch_glu_forward_no_scores(uint16_t *d_out, dmoe_layer layer, const uint16_t *d_x,
                                      const uint32_t *d_slot_indices, int T, dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(layer.ctx, "switch_glu_forward_no_scores: layer handle is null");
    DMOE_REQUIRE(d_out || T == 0, "switch_glu_forward_no_scores: out is null");
    DMOE_REQUIRE(((uintptr_t)d_out % 8) == 0, "switch_glu_forward_no_scores: out must be 8-byte aligned");
    return forward_common(nullptr, d_out, (Layer *)layer.ctx, d_x, d_slot_indices, nullptr, T, false, false, ws, s);
}

int dmoe_moe_layer_forward(uint16_t *d_out, uint32_t *d_out_indices, float *d_out_weights, dmoe_layer layer,
                           const uint16_t *d_x, const float *d_scores, const float *d_bias,
                           const uint8_t *d_resident_mask, int T, int E_total, int renorm, float route_scale,
                           dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(layer.ctx, "moe_layer_forward: layer handle is null");
    Layer *L = (Layer *)layer.ctx;
    DMOE_REQUIRE(T >= 0, "moe_layer_forward: T=%d", T);
    if (T == 0) return DMOE_OK;
    if (L->remap) DMOE_REQUIRE(E_total == L->n_total, "moe_layer_forward: E_total %d != remap length %d", E_total, L->n_total);
    else DMOE_REQUIRE(E_total == L->E, "moe_layer_forward: E_total %d != resident experts %d", E_total, L->E);
    // routing outputs live in caller memory when given, else in a private tail of the workspace
    FwdLayout f = forward_layout(L, T);
    size_t n = (size_t)T * L->K;
    Bump b;
    b.off = f.total;
    size_t o_idx = b.take(n * 4), o_w = b.take(n * 4);
    Workspace *w = nullptr;
    DMOE_TRY(workspace_reserve(ws, b.off, &w));
    uint32_t *idx = d_out_indices ? d_out_indices : at<uint32_t>(w, o_idx);
    float *wts = d_out_weights ? d_out_weights : at<float>(w, o_w);
    RouteArgs r;
    r.out_idx = idx, r.out_w = wts, r.scores = d_scores, r.bias = d_bias, r.resident = d_resident_mask;
    r.T = T, r.E = E_total, r.K = L->K, r.normalize = renorm, r.apply_scale = 1, r.route_scale = route_scale;
    DMOE_REQUIRE(d_scores != nullptr, "moe_layer_forward: scores is null");
    // one or two sequences: the selection shares a launch with the packing (and is timed as the packing stage)
    if (route_pack_tiny_supports(r)) return forward_common(d_out, nullptr, L, d_x, idx, wts, T, true, true, ws, s, &r);
    DMOE_TRY(stage_begin(w, DMOE_STAGE_ROUTE, to_hip(s)));
    DMOE_TRY(launch_route(r, to_hip(s)));
    DMOE_TRY(stage_end(w, DMOE_STAGE_ROUTE, to_hip(s)));
    return forward_common(d_out, nullptr, L, d_x, idx, wts, T, true, true, ws, s);
}

int dmoe_moe_layer_forward_static(uint16_t *d_out, uint32_t *d_out_indices, float *d_out_weights, dmoe_layer layer,
                                  const uint16_t *d_x, const float *d_scores, const float *d_bias,
                                  const uint8_t *d_resident_mask, int T, int E_total, int renorm, float route_scale,
                                  dmoe_stream s) {
    DMOE_REQUIRE(layer.ctx, "moe_layer_forward_static: layer handle is null");
    const Layer *L = (const Layer *)layer.ctx;
    DMOE_REQUIRE(T >= 0, "moe_layer_forward_static: T=%d", T);
    Workspace *w = nullptr;
    DMOE_TRY(static_workspace(&w));
    DMOE_REQUIRE(L->device == w->device, "moe_layer_forward_static: the layer lives on device %d, the current device is %d",
                 L->device, w->device);
    // same layout as dmoe_moe_layer_forward: the forward's buffers, then the routing outputs
    const size_t need = forward_layout(L, T).total + 2 * (((size_t)T * L->K * 4 + 255) & ~(size_t)255);
    DMOE_REQUIRE(need <= w->bytes,
                 "moe_layer_forward_static: T=%d tokens need %zu bytes of scratch memory, the static device scratch holds "
                 "%zu (use dmoe_moe_layer_forward with a workspace for larger batches)", T, need, w->bytes);
    dmoe_workspace ws;
    ws.ctx = w;
    return dmoe_moe_layer_forward(d_out, d_out_indices, d_out_weights, layer, d_x, d_scores, d_bias, d_resident_mask, T,
                                  E_total, renorm, route_scale, ws, s);
}

int dmoe_debug_last_activations(uint16_t *d_out, dmoe_layer layer, int T, dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(layer.ctx && ws.ctx && d_out, "debug_last_activations: null argument");
    Layer *L = (Layer *)layer.ctx;
    Workspace *w = (Workspace *)ws.ctx;
    FwdLayout f = forward_layout(L, T, w->last_with_shared);
    DMOE_REQUIRE(w->bytes >= f.total, "debug_last_activations: no forward of this size has run on the workspace");
    size_t n = (size_t)T * L->K, rv = (size_t)L->F / 8, total = n * rv;
    if (total == 0) return DMOE_OK;
    hipLaunchKernelGGL(scatter_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, to_hip(s),
                       (uint4 *)d_out, (const uint4 *)at<uint16_t>(w, f.h), at<uint32_t>(w, f.order), rv, total);
    DMOE_LAUNCH_CHECK();
    return DMOE_OK;
}

static int gather_qmm_view(uint16_t *d_out, const uint16_t *d_x, const QView &v, const uint32_t *d_lhs_indices,
                           const uint32_t *d_rhs_indices, int R, dmoe_workspace ws, dmoe_stream s) {
    DMOE_REQUIRE(R >= 0, "gather_qmm: R=%d", R);
    if (R == 0) return DMOE_OK;
    DMOE_REQUIRE(d_out && d_x && d_rhs_indices, "gather_qmm: null pointer");
    DMOE_REQUIRE(v.n_mats <= 1024, "gather_qmm: more than 1024 matrices in the stack");
    hipStream_t st = to_hip(s);
    const bool small = use_small_path((size_t)R, v.n_mats, v);
    DMOE_REQUIRE(small || qgemm_mfma_supports(v) || gemm_bf16_supports(v), "gather_qmm: unsupported weight shape rows=%d cols=%d", v.rows, v.cols);
    const int tile_m = small ? qgemm_skinny_tile_m(v) : qgemm_mfma_tile_m(v);
    const int max_tiles = pack_max_tiles((size_t)R, v.n_mats, tile_m);
    Bump b;
    size_t o_order = b.take((size_t)R * 4), o_arows = b.take((size_t)R * 4);
    size_t o_tiles = b.take((size_t)max_tiles * sizeof(Tile)), o_nt = b.take(4);
    size_t o_scr = b.take(pack_scratch_bytes((size_t)R, v.n_mats));
    Workspace *w = nullptr;
    DMOE_TRY(workspace_reserve(ws, b.off, &w));
    PackOut po;
    po.order = at<uint32_t>(w, o_order);
    po.tiles = at<Tile>(w, o_tiles);
    po.n_tiles = at<uint32_t>(w, o_nt);
    po.bad_ids = w->flags + 1;
    DMOE_TRY(launch_pack(po, d_rhs_indices, (size_t)R, 1, v.n_mats, tile_m, at<void>(w, o_scr), st));
    const uint32_t *a_rows = po.order;
    if (d_lhs_indices) {
        uint32_t *ar = at<uint32_t>(w, o_arows);
        hipLaunchKernelGGL(compose_rows_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0, st, ar,
                           d_lhs_indices, po.order, (size_t)R);
        DMOE_LAUNCH_CHECK();
        a_rows = ar;
    }
    GemmArgs g;
    g.b0 = v;
    g.a = d_x;
    g.a_rows = a_rows;
    g.out = d_out;
    g.ldo = v.rows;
    g.out_rows = po.order;
    g.tiles = po.tiles;
    g.n_tiles = po.n_tiles;
    g.max_tiles = max_tiles;
    g.tile_m = tile_m;
    return run_gemm(g, small, st, small ? 0 : prefill_small_rows(v, v), few_rows((size_t)R, v.n_mats));
}

int dmoe_gather_qmm(uint16_t *d_out, const uint16_t *d_x, const dmoe_qweight *qw, const uint32_t *d_lhs_indices,
                    const uint32_t *d_rhs_indices, int R, int sorted, dmoe_workspace ws, dmoe_stream s) {
    (void)sorted; // the counting sort is a no-op on already grouped rows
    QView v;
    DMOE_TRY(make_qview(&v, qw, "gather_qmm"));
    Workspace *w = (Workspace *)ws.ctx;
    if (w && w->cache_weights && can_pack(v)) {
        // the workspace keeps a re-ordered copy of this stack: the same kernels on the layout they stream
        const QView *cached = nullptr;
        DMOE_TRY(weight_cache_find_or_add(w, qw, &cached, to_hip(s)));
        return gather_qmm_view(d_out, d_x, *cached, d_lhs_indices, d_rhs_indices, R, ws, s);
    }
    return gather_qmm_view(d_out, d_x, v, d_lhs_indices, d_rhs_indices, R, ws, s);
}

int dmoe_resident_weight_create(dmoe_resident_weight *out, const dmoe_qweight *qw, int weight_source, dmoe_stream s) {
    DMOE_REQUIRE(out && qw, "resident_weight_create: null argument");
    out->ctx = nullptr;
    DMOE_REQUIRE(weight_source >= 0 && weight_source <= 2, "resident_weight_create: bad weight_source %d", weight_source);
    QOwned *q = new (std::nothrow) QOwned();
    DMOE_REQUIRE(q != nullptr, "resident_weight_create: out of host memory");
    int rc = adopt(q, qw, weight_source, "resident_weight", to_hip(s));
    if (rc == DMOE_OK && hipStreamSynchronize(to_hip(s)) != hipSuccess) rc = hip_fail(hipGetLastError(), "hipStreamSynchronize");
    if (rc != DMOE_OK) {
        free_owned(*q);
        delete q;
        return rc;
    }
    out->ctx = q;
    return DMOE_OK;
}

int dmoe_resident_weight_destroy(dmoe_resident_weight w) {
    QOwned *q = (QOwned *)w.ctx;
    if (!q) return DMOE_OK;
    free_owned(*q);
    delete q;
    return DMOE_OK;
}

int dmoe_gather_qmm_resident(uint16_t *d_out, const uint16_t *d_x, dmoe_resident_weight w, const uint32_t *d_lhs_indices,
                             const uint32_t *d_rhs_indices, int R, int sorted, dmoe_workspace ws, dmoe_stream s) {
    (void)sorted;
    const QOwned *q = (const QOwned *)w.ctx;
    DMOE_REQUIRE(q != nullptr, "gather_qmm_resident: null weight handle");
    return gather_qmm_view(d_out, d_x, q->view, d_lhs_indices, d_rhs_indices, R, ws, s);
}

} // extern "C"
