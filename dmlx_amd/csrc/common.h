// Shared host/device helpers of libdmoe (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "dmoe.h"

namespace dmoe {

// ---- errors (thread-local message, mlx-c style rc) ---------------------------------------------
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int hip_fail(hipError_t e, const char *what);

#define DMOE_HIP(call)                                                   \
    do {                                                                 \
        hipError_t e__ = (call);                                         \
        if (e__ != hipSuccess) return ::dmoe::hip_fail(e__, #call);      \
    } while (0)

#define DMOE_REQUIRE(cond, ...)                                          \
    do {                                                                 \
        if (!(cond)) {                                                   \
            ::dmoe::set_error(__VA_ARGS__);                              \
            return DMOE_ERR_INVALID;                                     \
        }                                                                \
    } while (0)

#define DMOE_TRY(expr)                                                   \
    do {                                                                 \
        int rc__ = (expr);                                               \
        if (rc__ != DMOE_OK) return rc__;                                \
    } while (0)

// checks the launch itself (bad configuration shows up here, not later)
#define DMOE_LAUNCH_CHECK() DMOE_HIP(hipGetLastError())

inline hipStream_t to_hip(dmoe_stream s) { return (hipStream_t)s.ctx; }

// ---- workspace: one grow-only device allocation, carved with a bump allocator ---------------------
// Per stage a ring of event pairs: the steps of a measurement run are enqueued back to back, and the host waits for
// events only when a ring is full or the totals are read.
constexpr int kStageRing = 64;
struct StageTimer {
    bool enabled = false;
    hipEvent_t start[DMOE_STAGE_COUNT][kStageRing] = {}, stop[DMOE_STAGE_COUNT][kStageRing] = {};
    int pending[DMOE_STAGE_COUNT] = {}; // event pairs recorded and not yet read, slots 0 .. pending - 1
    bool open[DMOE_STAGE_COUNT] = {};   // start recorded, stop not yet
    float total_ms[DMOE_STAGE_COUNT] = {};
    int samples[DMOE_STAGE_COUNT] = {};
};

struct Workspace {
    void *base = nullptr;
    size_t bytes = 0;
    int device = 0;
    StageTimer timer;
    // side stream (default priority) + fork/join events for work that overlaps the main stream
    hipStream_t side = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    hipEvent_t packed = nullptr, small_done = nullptr; // prefill: the small tiles' GEMMs run on the side stream
    bool last_with_shared = true; // layout of the last forward on this workspace (for dmoe_debug_last_activations)
    // Device words that outlive workspace growth, read and cleared by dmoe_workspace_check: [0] counts waits inside a
    // paired GEMM launch that gave up (see GemmArgs::wait_expired), [1] counts expert ids outside [0, E) met by the
    // pack kernels (see PackOut::bad_ids).
    uint32_t *flags = nullptr;
    uint32_t spin_limit = 1u << 16; // polls of ~0.25 us a waiting workgroup makes before it gives up (~16 ms)
    // Opt-in (dmoe_workspace_set_weight_cache): re-ordered resident copies of the borrowed MLX-layout stacks that
    // dmoe_gather_qmm has been called with on this workspace, keyed by the stack's pointers and shape. Owned by
    // layer.hip (weight_cache_find_or_add / weight_cache_clear).
    bool cache_weights = false;
    void *weight_cache = nullptr;
    size_t cache_limit_bytes = (size_t)32 << 30; // copies beyond this many bytes push out the least recently used ones
    // gate/up and down of a decode step share one launch (down workgroups wait per tile for gate/up). Switched off by
    // dmoe_workspace_set_paired_launch, and by dmoe_workspace_check once a wait gave up: the two GEMMs then run as two
    // launches in a row, which wait for nothing.
    bool paired = true;
    // a workspace over memory it does not own (the static device scratch of the allocation-free entry point):
    // reserve() never grows it, and nothing that would create a stream or an event runs on it
    bool fixed = false;
};
int side_stream_ready(Workspace *w);  // creates the side stream and its events on first use

// stage timing helpers (no-ops unless enabled on the workspace)
int stage_begin(Workspace *w, int stage, hipStream_t st);
int stage_end(Workspace *w, int stage, hipStream_t st);
int stage_flush(Workspace *w);

// makes sure at least `bytes` are reserved (may synchronize the device and reallocate)
int workspace_reserve(dmoe_workspace ws, size_t bytes, Workspace **out);
// drops every cached resident copy of the workspace (layer.hip)
void weight_cache_clear(Workspace *w);
int weight_cache_invalidate(Workspace *w, const dmoe_qweight *qw);  // one stack's copy, or every copy (qw == null)
int weight_cache_stats(Workspace *w, size_t *out_bytes, int *out_stacks);
// the current device's workspace over the static device scratch (layer.hip); resolves its address on first use
int static_workspace(Workspace **out);

struct Bump {
    size_t off = 0;
    size_t take(size_t bytes) {
        size_t o = off;
        off += (bytes + 255) & ~(size_t)255;
        return o;
    }
};

template <typename T>
inline T *at(Workspace *w, size_t off) {
    return (T *)((char *)w->base + off);
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Dynamic-LDS limit of a kernel above 64 KiB: hipFuncSetAttribute belongs to (function, device), so every kernel
// instantiation keeps one of these and raises its limit once per device. dmoe_init raises all of them for its device
// (prepare_kernels), so that no launch made later - possibly under stream capture, possibly from another thread - has
// host-side set-up left to do.
constexpr int kMaxDevices = 64;
struct LdsLimit {
    unsigned long long raised = 0; // bit d: done on device d (read and written under lds_limit_mutex)
};
int raise_lds_limit(LdsLimit &state, const void *kernel, int bytes);
// raise the limits of every kernel instantiation of the GEMM files on the current device
int qgemm_wide_prepare();
int qgemm_mfma_prepare();
int qgemm_skinny_prepare();

// ---- tile list produced by the pack kernels ----------------------------------------------------------
// one entry per (expert segment, row tile): rows [row0, row0 + nrows) of the sorted row order
struct Tile {
    uint32_t expert;
    uint32_t row0;
    uint32_t nrows;
    uint32_t flags; // kTileDense: rows of the always-on expert folded into a routed launch
};
constexpr uint32_t kTileDense = 1u;

struct PackOut {
    uint32_t *order = nullptr, *inv = nullptr, *token = nullptr, *sorted_e = nullptr;
    uint32_t *counts = nullptr, *offsets = nullptr, *live = nullptr, *n_live = nullptr;
    Tile *tiles = nullptr;       // capacity pack_max_tiles(n, E, tile_m) (+ the dense tiles below)
    uint32_t *n_tiles = nullptr; // device scalar
    // Optional always-on expert folded into the same tile list: `dense_rows` extra sorted rows n .. n+dense_rows-1
    // (row n+t = token t) of matrix `dense_expert`, cut into tiles of `tile_m` rows that come FIRST in the list,
    // flagged kTileDense. order / token / sorted_e then hold n + dense_rows entries.
    uint32_t dense_rows = 0, dense_expert = 0;
    // optional per-tile completion counters (n_done of them), zeroed by the pack kernels: see GemmArgs::tile_done
    uint32_t *tile_done = nullptr;
    uint32_t n_done = 0;
    // optional device counter: +1 for every expert id >= E met (such a row is packed under expert E - 1 so that every
    // access stays in bounds; the host learns about it from dmoe_workspace_check)
    uint32_t *bad_ids = nullptr;
    // optional map applied to every id before it is packed (global expert id -> resident slot; an id outside the
    // table maps to slot 0 like an expert that is not loaded)
    const int32_t *remap = nullptr;
    uint32_t n_remap = 0;
};

inline int pack_max_tiles(size_t n, int E, int tile_m) {
    size_t full = n / (size_t)tile_m;
    size_t part = n < (size_t)E ? n : (size_t)E;
    return (int)(full + part);
}
size_t pack_scratch_bytes(size_t n, int E);
// stable counting sort of n = T*K expert ids (< E) + tile list with `tile_m` rows per tile (0 = none)
int launch_pack(const PackOut &o, const uint32_t *d_idx, size_t n, int K, int E, int tile_m,
                void *d_scratch, hipStream_t st);
// The gate's selection (dmoe_gate_route) as one argument, for the launch that does selection and packing together
struct RouteArgs {
    uint32_t *out_idx = nullptr; // [T, K] router expert ids
    float *out_w = nullptr;      // [T, K]
    const float *scores = nullptr, *bias = nullptr;
    const uint8_t *resident = nullptr;
    int T = 0, E = 0, K = 0, normalize = 0, apply_scale = 1;
    float route_scale = 1.0f;
};
int launch_route(const RouteArgs &r, hipStream_t st);
// One or two sequences (T * K <= 16 rows, at most 256 router experts): selection and packing in ONE launch of T
// wavefronts, one token each; wavefront 0 then packs the rows by itself. Same results as launch_route + launch_pack;
// `E` = resident expert slots (what the ids are packed by, after o.remap).
bool route_pack_tiny_supports(const RouteArgs &r);
int launch_route_pack_tiny(const PackOut &o, const RouteArgs &r, int E, int tile_m, hipStream_t st);

// ---- grouped quantized GEMM ----------------------------------------------------------------------------
struct QView { // device view of one dmoe_qweight stack
    const uint8_t *w = nullptr, *scales = nullptr, *biases = nullptr;
    size_t w_mat = 0, s_mat = 0;   // bytes between consecutive matrices
    size_t w_row = 0, s_row = 0;   // bytes between consecutive rows
    int rows = 0, cols = 0, n_mats = 0;
    int mode = 0, bits = 4, group = 64;
    // packed (resident) layout, see qformat.h: w holds the re-ordered chunks, meta the interleaved
    // scale/bias words (affine) or exponents (mxfp4); scales still holds the per-row f32 scales of fp8row
    bool packed = false;
    const uint8_t *meta = nullptr;
    size_t m_mat = 0;
};
// bytes of the packed copies of a stack (rows must be a multiple of 32)
size_t packed_w_bytes(const QView &v);
size_t packed_meta_bytes(const QView &v);
bool can_pack(const QView &v);
// d_w / d_meta receive the packed layout of the MLX-layout stack `src` (all device memory)
int launch_repack(void *d_w, void *d_meta, const QView &src, hipStream_t st);
int make_qview(QView *out, const dmoe_qweight *q, const char *name);
size_t qweight_w_bytes(const dmoe_qweight *q);
size_t qweight_s_bytes(const dmoe_qweight *q);
size_t qweight_b_bytes(const dmoe_qweight *q);

struct GemmArgs {
    QView b0, b1;                 // b1 = up projection when gate_up
    bool gate_up = false;         // out[p, f] = swiglu(x.b0[f], x.b1[f]) instead of x.b0[n]
    const uint16_t *a = nullptr;  // bf16 [*, cols]
    const uint32_t *a_rows = nullptr;   // nullable: source row of sorted row p
    uint16_t *out = nullptr;      // bf16 [*, ldo]
    int ldo = 0;
    const uint32_t *out_rows = nullptr; // nullable: destination row of sorted row p
    const float *row_scale = nullptr;   // nullable: multiplier of sorted row p's output
    const uint32_t *row_scale_idx = nullptr; // nullable: row_scale index of sorted row p (else p)
    const Tile *tiles = nullptr;  // nullable: dense mode (one segment, expert 0, `dense_rows` rows)
    const uint32_t *n_tiles = nullptr;
    int max_tiles = 0;
    int tile_m = 0;               // rows per tile the tile list (or the dense split) was built with
    int dense_rows = 0;
    float swiglu_limit = 0.0f;
    // a launch serves the tiles with min_rows <= nrows <= max_rows of the list (prefill: the matrix-core kernels take the
    // large tiles, the weight-streaming kernel the small ones)
    int min_rows = 0, max_rows = 0x7fffffff;
    // weight-streaming kernel, launches of a handful of tiles: the reduction of a tile split over two groups of
    // wavefronts (see qgemm_skinny_ksplit_ok: packed layout, tiles of at most 8 rows)
    int ksplit = 0;
    // Paired launch (gate/up and down of a decode step in ONE launch): the workgroups of a gate/up tile add 1 to
    // tile_done[tile] after their stores, a down workgroup of that tile waits for tile_done_target before it reads h.
    uint32_t *tile_done = nullptr;
    uint32_t tile_done_target = 0;
    // a waiting workgroup polls at most spin_limit times; one that gives up adds 1 to *wait_expired (may be null)
    // and goes on with whatever the rows hold, so the launch always ends and the host can see that it went wrong
    uint32_t spin_limit = 1u << 16;
    uint32_t *wait_expired = nullptr;
    float swiglu_limit_dense = 0.0f;    // the limit for tiles flagged kTileDense
    uint32_t row_scale_rows = 0xffffffffu; // row_scale applies to sorted rows below this
};
// tile_m the kernels were built for
constexpr int kSkinnyTileM = 32;          // most rows a skinny tile can hold (see qgemm_skinny_tile_m)
constexpr int kSkinnyDenseTileM = 8;      // dense (one matrix) launches: small tiles, many workgroups per row block
constexpr int kMfmaTileM = 128;
constexpr int kMfmaWideTileM = 128;
int launch_qgemm_skinny(const GemmArgs &g, hipStream_t st);
// gate/up + down of one tile list in one launch (down waits per tile for gate/up); gu.tile_done must be zeroed
bool qgemm_skinny_pair_supports(const GemmArgs &gu, const GemmArgs &dn);
int launch_qgemm_skinny_pair(const GemmArgs &gu, const GemmArgs &dn, hipStream_t st);
int launch_qgemm_mfma(const GemmArgs &g, hipStream_t st); // picks the wide kernel when the format allows it
int launch_qgemm_wide(const GemmArgs &g, hipStream_t st);
bool qgemm_skinny_supports(const QView &b);
// unquantized bf16 weights (DMOE_QUANT_NONE): one kernel for every size
bool gemm_bf16_supports(const QView &b);
int launch_gemm_bf16(const GemmArgs &g, hipStream_t st);
bool qgemm_skinny_ksplit_ok(const QView &b); // the shape allows GemmArgs::ksplit
int qgemm_skinny_tile_m(const QView &b);  // rows per tile to build tile lists with for the skinny path
bool qgemm_mfma_supports(const QView &b);
bool qgemm_wide_supports(const QView &b);
bool qgemm_wide_bf16_supports(const QView &b); // unquantized weights in the packed resident layout (launch_qgemm_wide takes them too)
// tile size to build tile lists with for the MFMA path of this weight matrix
inline int qgemm_mfma_tile_m(const QView &b) { return qgemm_wide_supports(b) ? kMfmaWideTileM : kMfmaTileM; }

} // namespace dmoe

// ---- device helpers ------------------------------------------------------------------------------------
#if defined(__HIPCC__)
namespace dmoe {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// round to nearest even, one v_cvt_pk_bf16_f32 per pair
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    bf16x2_t v;
    v.x = (__bf16)lo;
    v.y = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    return (uint16_t)(pack_bf16x2(f, 0.0f) & 0xffffu);
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// limited SwiGLU on the bf16-rounded projections (deepseek_v4.zig:947-966); limit <= 0: plain SwiGLU
__device__ __forceinline__ float limited_swiglu(float g, float u, float limit) {
    // both roundings in one v_cvt_pk_bf16_f32, the halves widened again with a shift and a mask
    const uint32_t gu = pack_bf16x2(g, u);
    g = __uint_as_float(gu << 16);
    u = __uint_as_float(gu & 0xffff0000u);
    if (limit > 0.0f) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    float silu = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); // 1-ulp reciprocal; the result is rounded to bf16
    return silu * u;
}

} // namespace dmoe
#endif
