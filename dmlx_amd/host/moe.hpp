// Host-side layer over the C ABI (include/dmoe.h), mirroring the call surface of the reference's Zig
// modules for this path so that a caller of dmlx finds the same names, argument meaning and error
// behaviour:
//
//   src/moe_router.zig            MoERouterConfig, RouteResult, MoERouter{init, topkRoute, expandTokens,
//                                 reduceExperts}
//   src/models/deepseek_v4.zig    DSV4Gate.forward (from the scores on), DSV4SwitchGLU.{forward,
//                                 forwardNoScores}, DSV4MoE.forward
//   src/models/expert_provider.zig  ExpertProvider{forward, getCacheBias, deinit}
//   src/models/deepseek_v4_loader.zig  SmeltConfig.buildMask, expert_remap construction
//   src/batch_builder.zig         build (token concatenation and positions; the attention mask is not
//                                 part of this path)
//
// The reference is Zig over mlx-c; this header is the same layer in C++ because no Zig toolchain is
// available where this is built (dmlx_amd/zig/dmoe.zig is the @cImport binding a Zig caller would use).
// Arrays are device buffers owned by the caller-visible handle (as mlx arrays are refcounted handles in
// the reference); every failing C call throws dmoe::Error carrying dmoe_last_error(), the way the
// reference turns a non-zero mlx-c return code into error.MlxError.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "dmoe.h"

namespace dmoe {

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &m) : std::runtime_error(m), code(c) {}
};

inline void check(int rc) {
    if (rc != DMOE_OK) throw Error(rc, dmoe_last_error());
}

// Execution context: the stream every op is enqueued on plus the scratch workspace (EagerContext of the
// reference carries the mlx stream).
class Context {
  public:
    explicit Context(int device = 0) {
        check(dmoe_init(device));
        check(dmoe_stream_create(&stream_));
        check(dmoe_workspace_create(&ws_, 0));
    }
    ~Context() {
        dmoe_stream_synchronize(stream_);
        dmoe_workspace_destroy(ws_);
        dmoe_stream_destroy(stream_);
    }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    dmoe_stream stream() const { return stream_; }
    dmoe_workspace workspace() const { return ws_; }
    // Array.eval(): the host-visible sync point, where a failed step surfaces (a bounded wait inside a kernel that
    // gave up throws here, as a failed lazy graph throws at eval() in the reference)
    void synchronize() const { check(dmoe_workspace_check(ws_, stream_)); }
    void setWaitLimit(unsigned polls) const { check(dmoe_workspace_set_wait_limit(ws_, polls)); }
    // decode steps: gate/up and down in one launch (default) or as two launches that wait for nothing; a step that
    // reported a time-out at synchronize() has already switched the workspace to two launches
    // gatherQmm on borrowed MLX-layout arrays: keep re-ordered resident copies of the stacks seen (see dmoe.h)
    void setWeightCache(bool enabled) const { check(dmoe_workspace_set_weight_cache(ws_, enabled ? 1 : 0)); }
    // before a cached stack is freed or rewritten (null: every copy); the cap pushes out least recently used copies
    void invalidateWeightCache(const dmoe_qweight *qw = nullptr) const { check(dmoe_workspace_weight_cache_invalidate(ws_, qw)); }
    void setWeightCacheLimit(size_t max_bytes) const { check(dmoe_workspace_set_weight_cache_limit(ws_, max_bytes)); }
    void setPairedLaunch(bool enabled) const { check(dmoe_workspace_set_paired_launch(ws_, enabled ? 1 : 0)); }

  private:
    dmoe_stream stream_{};
    dmoe_workspace ws_{};
};

enum class DType { float32, bfloat16, uint32, int32, uint8 };
inline size_t dtype_size(DType t) {
    switch (t) {
    case DType::bfloat16: return 2;
    case DType::uint8: return 1;
    default: return 4;
    }
}

// A dense row-major device array (the path only needs 1-D..3-D). Copying shares the buffer, like the
// reference's refcounted mlx_array handles; deinit() is implicit.
class Array {
  public:
    Array() = default;
    Array(const Context &ctx, DType dtype, std::vector<int> shape) : ctx_(&ctx), dtype_(dtype), shape_(std::move(shape)) {
        void *p = nullptr;
        check(dmoe_malloc(&p, nbytes()));
        buf_ = std::shared_ptr<void>(p, [](void *q) { dmoe_free(q); });
    }
    // Array.fromData: copies host data to the device
    template <typename T>
    static Array fromData(const Context &ctx, const T *data, std::vector<int> shape, DType dtype) {
        Array a(ctx, dtype, std::move(shape));
        if (sizeof(T) != dtype_size(dtype)) throw Error(DMOE_ERR_INVALID, "fromData: element size does not match dtype");
        check(dmoe_copy_to_device(a.data(), data, a.nbytes(), ctx.stream()));
        return a;
    }
    // dataSlice: reads the array back (waits for the stream)
    template <typename T>
    std::vector<T> dataSlice() const {
        if (sizeof(T) != dtype_size(dtype_)) throw Error(DMOE_ERR_INVALID, "dataSlice: element size does not match dtype");
        std::vector<T> out(size());
        check(dmoe_copy_to_host(out.data(), data(), nbytes(), ctx_->stream()));
        return out;
    }
    size_t size() const {
        size_t n = 1;
        for (int d : shape_) n *= (size_t)d;
        return n;
    }
    size_t nbytes() const { return size() * dtype_size(dtype_); }
    const std::vector<int> &shape() const { return shape_; }
    DType dtype() const { return dtype_; }
    void *data() const { return buf_.get(); }
    bool valid() const { return (bool)buf_ || size() == 0; }
    Array reshaped(std::vector<int> shape) const {
        Array a = *this;
        a.shape_ = std::move(shape);
        if (a.size() != size()) throw Error(DMOE_ERR_INVALID, "reshape: element count differs");
        return a;
    }

  private:
    const Context *ctx_ = nullptr;
    DType dtype_ = DType::float32;
    std::vector<int> shape_;
    std::shared_ptr<void> buf_;
};

// ---- moe_router.zig ----------------------------------------------------------------------------------

struct RouteResult {      // moe_router.zig:21-33
    Array indices;        // [num_tokens, k] u32
    Array weights;        // [num_tokens, k] f32
    size_t k = 0;
};

struct MoERouterConfig {  // moe_router.zig:36-41
    size_t num_experts = 0;
    size_t top_k = 0;
    bool normalize_weights = true;
};

class MoERouter {         // moe_router.zig:44-165
  public:
    MoERouterConfig config;
    static MoERouter init(MoERouterConfig c) { return MoERouter{c}; }

    // scores [num_tokens, num_experts] f32 -> indices / weights [num_tokens, k] (columns in ascending score order)
    RouteResult topkRoute(const Context &ctx, const Array &scores) const {
        const int T = scores.shape().at(0), E = scores.shape().at(1), K = (int)config.top_k;
        if ((size_t)E != config.num_experts) throw Error(DMOE_ERR_INVALID, "topkRoute: scores do not have num_experts columns");
        RouteResult r{Array(ctx, DType::uint32, {T, K}), Array(ctx, DType::float32, {T, K}), config.top_k};
        check(dmoe_topk_route((uint32_t *)r.indices.data(), (float *)r.weights.data(), (const float *)scores.data(), T, E, K,
                              config.normalize_weights ? 1 : 0, ctx.stream()));
        return r;
    }
    // x [num_tokens, hidden] -> [num_tokens * k, hidden]
    static Array expandTokens(const Context &ctx, const Array &x, const RouteResult &route) {
        const int T = x.shape().at(0), D = x.shape().at(1), K = (int)route.k;
        Array out(ctx, x.dtype(), {T * K, D});
        check(dmoe_expand_tokens(out.data(), x.data(), T, D, K, (int)dtype_size(x.dtype()), ctx.stream()));
        return out;
    }
    // expert_outs [num_tokens * k, hidden] -> [num_tokens, hidden] f32, weighted by route.weights
    static Array reduceExperts(const Context &ctx, const Array &expert_outs, const RouteResult &route) {
        const int T = route.weights.shape().at(0), K = (int)route.k, D = expert_outs.shape().at(1);
        Array out(ctx, DType::float32, {T, D});
        check(dmoe_reduce_experts((float *)out.data(), expert_outs.data(), expert_outs.dtype() == DType::bfloat16 ? 1 : 0,
                                  (const float *)route.weights.data(), T, K, D, ctx.stream()));
        return out;
    }
};

// ---- deepseek_v4_loader.zig: SmeltConfig -------------------------------------------------------------------

struct SmeltConfig {      // deepseek_v4_loader.zig:250-294
    enum class Strategy { uniform = 0, first = 1 };
    bool enabled = false;
    float load_fraction = 1.0f;
    Strategy strategy = Strategy::uniform;

    std::vector<uint8_t> buildMask(size_t n_experts) const {
        std::vector<uint8_t> mask(n_experts);
        int n = 0;
        check(dmoe_smelt_build_mask(mask.data(), &n, (int)n_experts, load_fraction, (int)strategy, enabled ? 1 : 0));
        return mask;
    }
    // expert_remap of DSV4MoE (deepseek_v4_loader.zig:2151-2168)
    static std::vector<int32_t> buildRemap(const std::vector<uint8_t> &mask) {
        std::vector<int32_t> remap(mask.size());
        check(dmoe_build_remap(remap.data(), mask.data(), (int)mask.size()));
        return remap;
    }
};

// ---- deepseek_v4.zig: gate epilogue, SwitchGLU, MoE ----------------------------------------------------------

// deepseek_v4.zig:82-86, plus sqrtsoftplus_stable (DMOE_SCORE_SQRTSOFTPLUS_STABLE: no counterpart in the reference)
enum class ScoringFunc { softmax, sigmoid, sqrtsoftplus, sqrtsoftplus_stable };

// DSV4Gate (deepseek_v4.zig:521-681). `forward(ctx, scores)` takes the result of the scoring function (the
// gate epilogue, :589-678); once `load` has uploaded the router weight, `forwardHidden` serves the whole
// DSV4Gate.forward(hidden_states, null, stream): matmul, scoring function, selection.
struct DSV4Gate {
    size_t topk = 0, n_routed_experts = 0;
    float route_scale = 1.0f;
    ScoringFunc scoring_func = ScoringFunc::sqrtsoftplus;
    bool is_hash = false;
    Array bias;        // optional [n_routed_experts] f32 selection bias
    Array smelt_mask;  // optional [n_routed_experts] u8 residency mask

    DSV4Gate() = default;
    DSV4Gate(const DSV4Gate &) = delete;
    DSV4Gate &operator=(const DSV4Gate &) = delete;
    ~DSV4Gate() { deinit(); }
    void deinit() {
        if (handle_.ctx) dmoe_gate_destroy(handle_);
        handle_.ctx = nullptr;
    }

    // uploads `weight` (HOST bf16 [n_routed_experts, dim]) together with the bias / mask given as host vectors
    void load(const Context &ctx, const uint16_t *weight, int dim, const float *host_bias = nullptr,
              const uint8_t *host_mask = nullptr, const int32_t *host_tid2eid = nullptr, int vocab_size = 0) {
        deinit();
        dmoe_gate_desc d{};
        d.weight = weight;
        d.bias = host_bias;
        d.resident_mask = host_mask;
        d.n_experts = (int)n_routed_experts;
        d.dim = dim;
        d.top_k = (int)topk;
        d.scoring_func = (int)scoring_func;
        d.route_scale = route_scale;
        d.is_hash = is_hash ? 1 : 0;
        d.tid2eid = host_tid2eid; // [vocab_size, topk] for hash layers (deepseek_v4.zig:525)
        d.vocab_size = vocab_size;
        d.weight_source = DMOE_WEIGHTS_COPY_FROM_HOST;
        check(dmoe_gate_create(&handle_, &d, ctx.stream()));
    }

    // returns (weights [T, topk] f32, indices [T, topk] u32) like the reference's tuple
    std::pair<Array, Array> forward(const Context &ctx, const Array &scores) const {
        const int T = scores.shape().at(0), E = scores.shape().at(1), K = (int)topk;
        Array idx(ctx, DType::uint32, {T, K}), w(ctx, DType::float32, {T, K});
        check(dmoe_gate_route((uint32_t *)idx.data(), (float *)w.data(), (const float *)scores.data(),
                              bias.data() ? (const float *)bias.data() : nullptr,
                              smelt_mask.data() ? (const uint8_t *)smelt_mask.data() : nullptr, T, E, K,
                              scoring_func != ScoringFunc::softmax ? 1 : 0, route_scale, ctx.stream()));
        return {w, idx};
    }

    // hidden_states bf16 [T, dim] (or [B, S, dim]), optional input_ids u32 [T] (hash layers) -> (weights, indices);
    // needs load()
    std::pair<Array, Array> forwardHidden(const Context &ctx, const Array &hidden_states,
                                          const Array *input_ids = nullptr) const {
        if (!handle_.ctx) throw Error(DMOE_ERR_INVALID, "DSV4Gate.forwardHidden: no router weight loaded");
        const auto &sh = hidden_states.shape();
        int T = 1;
        for (size_t i = 0; i + 1 < sh.size(); ++i) T *= sh[i];
        const int K = (int)topk;
        Array idx(ctx, DType::uint32, {T, K}), w(ctx, DType::float32, {T, K});
        check(dmoe_gate_forward((uint32_t *)idx.data(), (float *)w.data(), nullptr, handle_,
                                (const uint16_t *)hidden_states.data(),
                                input_ids ? (const uint32_t *)input_ids->data() : nullptr, T, ctx.workspace(),
                                ctx.stream()));
        return {w, idx};
    }

  private:
    dmoe_gate handle_{};
};

// Quantized stack description on the host side (QuantizedWeight + QuantConfig of mlx-zig)
struct QuantizedWeight {
    const void *data = nullptr, *scales = nullptr, *biases = nullptr; // host or device memory, see weight_source
    int n_mats = 1, rows = 0, cols = 0;
    int group_size = 64, bits = 4;
    // "affine" | "mxfp4" | "fp8" | "none": unquantized bf16 [n_mats, rows, cols] (bits 16, no scales), the
    // is_quantized == false arm of DSV4SwitchGLU (deepseek_v4.zig:969-979, ops.gatherMm)
    std::string mode = "affine";
    static QuantizedWeight unquantized(const void *bf16_data, int n_mats, int rows, int cols) {
        QuantizedWeight q;
        q.data = bf16_data;
        q.n_mats = n_mats;
        q.rows = rows;
        q.cols = cols;
        q.group_size = 0;
        q.bits = 16;
        q.mode = "none";
        return q;
    }
    dmoe_qweight c() const {
        dmoe_qweight q{};
        q.w = data;
        q.scales = scales;
        q.biases = biases;
        q.n_mats = n_mats;
        q.rows = rows;
        q.cols = cols;
        q.mode = dmoe_quant_mode_from_string(mode.c_str());
        q.bits = bits;
        q.group_size = group_size;
        if (q.mode < 0) throw Error(DMOE_ERR_INVALID, "unknown quantization mode " + mode);
        return q;
    }
};

// One MoE layer's resident experts: DSV4SwitchGLU (routed, deepseek_v4.zig:687-980) + the shared
// DSV4Expert (:442-518) + expert_remap (:991-993). Owns a dmoe_layer.
class DSV4SwitchGLU {
  public:
    struct Options {
        float swiglu_limit = 0.0f;
        bool score_before_down = false; // true: DSV4SwitchGLU.forward (:796-806); false: provider paths
        const QuantizedWeight *shared_gate = nullptr, *shared_up = nullptr, *shared_down = nullptr;
        float shared_swiglu_limit = 0.0f;
        std::vector<int32_t> remap;     // router id -> slot; empty = identity
        dmoe_weight_source source = DMOE_WEIGHTS_COPY_FROM_HOST;
    };
    DSV4SwitchGLU(const Context &ctx, int hidden, int ffn, int top_k, const QuantizedWeight &gate, const QuantizedWeight &up,
                  const QuantizedWeight &down, const Options &opt)
        : hidden_(hidden), ffn_(ffn), top_k_(top_k) {
        dmoe_layer_desc d{};
        d.hidden = hidden;
        d.ffn = ffn;
        d.top_k = top_k;
        d.gate = gate.c();
        d.up = up.c();
        d.down = down.c();
        d.swiglu_limit = opt.swiglu_limit;
        d.score_before_down = opt.score_before_down ? 1 : 0;
        if (opt.shared_gate) {
            d.has_shared = 1;
            d.shared_gate = opt.shared_gate->c();
            d.shared_up = opt.shared_up->c();
            d.shared_down = opt.shared_down->c();
            d.shared_swiglu_limit = opt.shared_swiglu_limit;
        }
        if (!opt.remap.empty()) {
            d.remap = opt.remap.data();
            d.n_experts_total = (int)opt.remap.size();
        }
        d.weight_source = opt.source;
        check(dmoe_layer_create(&layer_, &d, ctx.stream()));
    }
    // Resident upload from MLX-format safetensors shards (replaces TensorIndex + LayerExpertMeta + the stream
    // provider set up in model_registry.zig:255-329). `smelt_mask` empty = every expert of the file.
    struct FileOptions {
        std::string mode = "mxfp4"; // the reference passes ("mxfp4", 32, 4) (:318-321)
        int group_size = 32, bits = 4;
        float swiglu_limit = 0.0f, shared_swiglu_limit = 0.0f;
        bool score_before_down = false, load_shared = true;
        std::vector<uint8_t> smelt_mask;
    };
    DSV4SwitchGLU(const Context &ctx, const std::vector<std::string> &paths, int layer_idx, int top_k,
                  const FileOptions &opt) {
        std::vector<const char *> p;
        for (const auto &s : paths) p.push_back(s.c_str());
        dmoe_safetensors_opts o{};
        o.top_k = top_k;
        o.mode = opt.mode.c_str();
        o.group_size = opt.group_size;
        o.bits = opt.bits;
        o.swiglu_limit = opt.swiglu_limit;
        o.score_before_down = opt.score_before_down ? 1 : 0;
        o.load_shared = opt.load_shared ? 1 : 0;
        o.shared_swiglu_limit = opt.shared_swiglu_limit;
        if (!opt.smelt_mask.empty()) {
            o.resident_mask = opt.smelt_mask.data();
            o.n_experts_total = (int)opt.smelt_mask.size();
        }
        check(dmoe_layer_create_from_safetensors(&layer_, p.data(), (int)p.size(), layer_idx, &o, ctx.stream()));
        check(dmoe_layer_dims(&hidden_, &ffn_, nullptr, &top_k_, layer_));
    }
    ~DSV4SwitchGLU() { dmoe_layer_destroy(layer_); } // deinit()
    DSV4SwitchGLU(const DSV4SwitchGLU &) = delete;
    DSV4SwitchGLU &operator=(const DSV4SwitchGLU &) = delete;

    // x [N, hidden] bf16, indices [N, topk] u32 (router ids), scores [N, topk] f32 -> [N, hidden] bf16
    // (routed experts, weighted sum over k, plus the shared expert when the layer has one)
    Array forward(const Context &ctx, const Array &x, const Array &indices, const Array &scores) const {
        const int T = x.shape().at(0);
        Array out(ctx, DType::bfloat16, {T, hidden_});
        check(dmoe_moe_forward((uint16_t *)out.data(), layer_, (const uint16_t *)x.data(), (const uint32_t *)indices.data(),
                               (const float *)scores.data(), T, ctx.workspace(), ctx.stream()));
        return out;
    }
    // expert outputs without scores, [N, topk, hidden] bf16 (deepseek_v4.zig:855-945); indices are slot ids
    Array forwardNoScores(const Context &ctx, const Array &x, const Array &slot_indices) const {
        const int T = x.shape().at(0);
        Array out(ctx, DType::bfloat16, {T, top_k_, hidden_});
        check(dmoe_switch_glu_forward_no_scores((uint16_t *)out.data(), layer_, (const uint16_t *)x.data(),
                                                (const uint32_t *)slot_indices.data(), T, ctx.workspace(), ctx.stream()));
        return out;
    }
    // DSV4MoE.forward from the gate's scores on (deepseek_v4.zig:1021-1052) in one call: selection (bias, Smelt mask,
    // renormalisation, route_scale as in DSV4Gate.forward :589-678), then forward(). scores f32 [N, n_experts_total];
    // bias f32 [n_experts_total] / resident_mask u8 [n_experts_total] or null.
    Array forwardFromScores(const Context &ctx, const Array &x, const Array &scores, const Array *bias, const Array *resident_mask,
                            bool renorm, float route_scale) const {
        const int T = x.shape().at(0), E = scores.shape().at(1);
        Array out(ctx, DType::bfloat16, {T, hidden_});
        check(dmoe_moe_layer_forward((uint16_t *)out.data(), nullptr, nullptr, layer_, (const uint16_t *)x.data(),
                                     (const float *)scores.data(), bias ? (const float *)bias->data() : nullptr,
                                     resident_mask ? (const uint8_t *)resident_mask->data() : nullptr, T, E, renorm ? 1 : 0,
                                     route_scale, ctx.workspace(), ctx.stream()));
        return out;
    }
    dmoe_layer handle() const { return layer_; }
    int hidden() const { return hidden_; }
    int top_k() const { return top_k_; }

  private:
    dmoe_layer layer_{};
    int hidden_, ffn_, top_k_;
};

// The sort block of DSV4SwitchGLU.forward (deepseek_v4.zig:749-784) on its own: rows (t * K + k) grouped by expert, ties
// in ascending flat index. order = argsort(flat indices) (:753), inv_order = argsort(order) (:758), token = order / K
// (:765-772), plus rows per expert and their exclusive scan (offsets has n_experts + 1 entries).
struct SortedRows {
    Array order, inv_order, token, counts, offsets;
};
inline SortedRows sortByExpert(const Context &ctx, const Array &indices, int n_experts) {
    const int T = indices.shape().at(0), K = indices.shape().at(1);
    SortedRows r{Array(ctx, DType::uint32, {T * K}), Array(ctx, DType::uint32, {T * K}), Array(ctx, DType::uint32, {T * K}),
                 Array(ctx, DType::uint32, {n_experts}), Array(ctx, DType::uint32, {n_experts + 1})};
    check(dmoe_pack((uint32_t *)r.order.data(), (uint32_t *)r.inv_order.data(), (uint32_t *)r.token.data(), nullptr,
                    (uint32_t *)r.counts.data(), (uint32_t *)r.offsets.data(), nullptr, nullptr, (const uint32_t *)indices.data(), T,
                    K, n_experts, ctx.workspace(), ctx.stream()));
    return r;
}
// mlx_take(expert_remap, indices).astype(u32) (deepseek_v4.zig:1035-1039, expert_preload.zig:200-206); remap i32 on the device
inline Array remapIndices(const Context &ctx, const Array &remap, const Array &indices) {
    Array out(ctx, DType::uint32, indices.shape());
    check(dmoe_remap_indices((uint32_t *)out.data(), (const int32_t *)remap.data(), (const uint32_t *)indices.data(), indices.size(),
                             (int)remap.size(), ctx.stream()));
    return out;
}

// ---- expert_provider.zig --------------------------------------------------------------------------------------

// ExpertProvider.VTable (expert_provider.zig:12-48) as an abstract class.
class ExpertProvider {
  public:
    virtual ~ExpertProvider() = default;                                   // deinit
    virtual Array forward(const Context &ctx, size_t layer_idx, const Array &flat_x, const Array &indices,
                          const Array &scores) = 0;
    virtual bool getCacheBias(size_t /*layer_idx*/, std::vector<float> * /*out*/) { return false; } // optional
};

// Experts resident in HBM: what replaces ExpertStreamProvider / ExpertPreloadProvider (no SSD, no cache).
class ResidentExpertProvider : public ExpertProvider {
  public:
    void addLayer(std::unique_ptr<DSV4SwitchGLU> layer, std::vector<float> cache_bias = {}) {
        layers_.push_back(std::move(layer));
        cache_bias_.push_back(std::move(cache_bias));
    }
    Array forward(const Context &ctx, size_t layer_idx, const Array &flat_x, const Array &indices, const Array &scores) override {
        if (layer_idx >= layers_.size()) throw Error(DMOE_ERR_INVALID, "PreloadProviderNotInitialized: no such layer");
        return layers_[layer_idx]->forward(ctx, flat_x, indices, scores);
    }
    bool getCacheBias(size_t layer_idx, std::vector<float> *out) override {
        if (layer_idx >= cache_bias_.size() || cache_bias_[layer_idx].empty()) return false;
        *out = cache_bias_[layer_idx];
        return true;
    }
    // expert_preload.zig:141-160: remap + cache bias (0 loaded, -1000 not loaded) for a list of loaded ids
    static std::pair<std::vector<int32_t>, std::vector<float>> preloadRemap(const std::vector<uint32_t> &ids, size_t n_total) {
        std::vector<int32_t> remap(n_total);
        std::vector<float> bias(n_total);
        check(dmoe_preload_remap(remap.data(), bias.data(), ids.data(), (int)ids.size(), (int)n_total));
        return {remap, bias};
    }

  private:
    std::vector<std::unique_ptr<DSV4SwitchGLU>> layers_;
    std::vector<std::vector<float>> cache_bias_;
};

// DSV4MoE.forward from the gate scores on (deepseek_v4.zig:1010-1056): hidden [B, S, D] -> [B, S, D].
struct DSV4MoE {
    DSV4Gate gate;
    ExpertProvider *stream_provider = nullptr; // owned by the model, as in the reference
    size_t layer_idx = 0;

    Array forward(const Context &ctx, const Array &hidden_states, const Array &scores) const {
        const auto &sh = hidden_states.shape();
        const int B = sh.at(0), S = sh.at(1), D = sh.at(2);
        Array flat = hidden_states.reshaped({B * S, D});
        auto routed = gate.forward(ctx, scores);
        if (!stream_provider) throw Error(DMOE_ERR_INVALID, "PreloadProviderNotInitialized");
        Array y = stream_provider->forward(ctx, layer_idx, flat, routed.second, routed.first);
        return y.reshaped({B, S, D});
    }
    // DSV4MoE.forward(hidden_states, input_ids, stream) as the reference declares it (deepseek_v4.zig:1010-1056): the
    // gate runs from the hidden states (router weight uploaded with gate.load), input_ids only matter on hash layers
    Array forward(const Context &ctx, const Array &hidden_states, const Array *input_ids = nullptr) const {
        const auto &sh = hidden_states.shape();
        const int B = sh.at(0), S = sh.at(1), D = sh.at(2);
        Array flat = hidden_states.reshaped({B * S, D});
        auto routed = gate.forwardHidden(ctx, flat, input_ids);
        if (!stream_provider) throw Error(DMOE_ERR_INVALID, "PreloadProviderNotInitialized");
        Array y = stream_provider->forward(ctx, layer_idx, flat, routed.second, routed.first);
        return y.reshaped({B, S, D});
    }
};

// ---- batch_builder.zig ----------------------------------------------------------------------------------------

struct Request {                     // the fields of scheduler.zig's Request that build() reads
    enum class State { waiting, prefilling, decoding, done } state = State::waiting;
    std::vector<uint32_t> prompt_tokens, generated_tokens;
    size_t prefill_offset = 0;
    size_t seqLen() const { return prompt_tokens.size() + generated_tokens.size(); }
};

struct BatchResult {                 // batch_builder.zig:24-43 without the [T,T] mask
    std::vector<uint32_t> batched_tokens;
    std::vector<int32_t> position_ids;
    std::vector<int32_t> request_offsets; // start of each request in the flat batch, plus the total
    size_t total_tokens = 0, num_requests = 0;
};

namespace batch_builder {
// getRequestTokens (batch_builder.zig:47-83)
inline std::vector<uint32_t> getRequestTokens(const Request &r) {
    switch (r.state) {
    case Request::State::prefilling:
    case Request::State::waiting:
        if (r.prefill_offset >= r.prompt_tokens.size()) {
            if (!r.prompt_tokens.empty()) return {r.prompt_tokens.back()};
            return {};
        }
        return std::vector<uint32_t>(r.prompt_tokens.begin() + (long)r.prefill_offset, r.prompt_tokens.end());
    case Request::State::decoding:
        if (!r.generated_tokens.empty()) return {r.generated_tokens.back()};
        if (!r.prompt_tokens.empty()) return {r.prompt_tokens.back()};
        return {};
    default: return {};
    }
}
// build (batch_builder.zig:90-214): prefill requests first, then decode requests
inline BatchResult build(const std::vector<const Request *> &prefill_requests, const std::vector<const Request *> &decode_requests) {
    BatchResult out;
    std::vector<const Request *> all(prefill_requests);
    all.insert(all.end(), decode_requests.begin(), decode_requests.end());
    out.num_requests = all.size();
    for (const Request *r : all) {
        std::vector<uint32_t> toks = getRequestTokens(*r);
        size_t base = 0;
        switch (r->state) {
        case Request::State::prefilling:
        case Request::State::waiting: base = r->prefill_offset; break;
        case Request::State::decoding: base = r->seqLen() > 0 ? r->seqLen() - toks.size() : 0; break;
        default: base = 0;
        }
        out.request_offsets.push_back((int32_t)out.batched_tokens.size());
        for (size_t j = 0; j < toks.size(); ++j) {
            out.batched_tokens.push_back(toks[j]);
            out.position_ids.push_back((int32_t)(base + j));
        }
    }
    out.total_tokens = out.batched_tokens.size();
    out.request_offsets.push_back((int32_t)out.total_tokens);
    return out;
}
// the same batch on the device: tokens, positions, [T,T] mask (optional) and the token -> request map
struct DeviceBatch {
    Array batched_tokens, position_ids, attention_mask, request_of_token;
    size_t total_tokens = 0, num_requests = 0;
};
inline DeviceBatch buildOnDevice(const Context &ctx, const std::vector<const Request *> &prefill_requests,
                                 const std::vector<const Request *> &decode_requests, bool want_mask) {
    const BatchResult host = build(prefill_requests, decode_requests);
    DeviceBatch out;
    out.total_tokens = host.total_tokens;
    out.num_requests = host.num_requests;
    const int T = (int)host.total_tokens, n = (int)host.num_requests;
    if (T == 0) return out; // emptyBatch
    std::vector<int32_t> lens((size_t)n), base((size_t)n);
    for (int i = 0; i < n; ++i) {
        lens[(size_t)i] = host.request_offsets[(size_t)i + 1] - host.request_offsets[(size_t)i];
        base[(size_t)i] = lens[(size_t)i] ? host.position_ids[(size_t)host.request_offsets[(size_t)i]] : 0;
    }
    out.batched_tokens = Array(ctx, DType::uint32, {T});
    out.position_ids = Array(ctx, DType::int32, {T});
    out.request_of_token = Array(ctx, DType::uint32, {T});
    if (want_mask) out.attention_mask = Array(ctx, DType::float32, {T, T});
    check(dmoe_batch_build((uint32_t *)out.batched_tokens.data(), (int32_t *)out.position_ids.data(),
                           want_mask ? (float *)out.attention_mask.data() : nullptr,
                           (uint32_t *)out.request_of_token.data(), host.batched_tokens.data(), lens.data(), base.data(), n, T,
                           ctx.workspace(), ctx.stream()));
    return out;
}
} // namespace batch_builder

// ---- quantize_mod / ops leaf calls (mlx-zig; call shapes at deepseek_v4.zig:976-978, expert_preload.zig:265) ------
namespace quantize_mod {
// gatherQmm(ctx, x, w, scales, biases, lhs_indices?, rhs_indices, transpose=true, config, sorted): row r of the
// result is x[lhs[r] or r] times the transposed matrix rhs[r] of the stack. `w` describes DEVICE memory here.
inline Array gatherQmm(const Context &ctx, const Array &x, const QuantizedWeight &w, const Array *lhs_indices,
                       const Array &rhs_indices, bool sorted) {
    if (x.dtype() != DType::bfloat16 || x.shape().size() != 2 || x.shape()[1] != w.cols)
        throw Error(DMOE_ERR_INVALID, "gatherQmm: x must be bfloat16 [rows, cols of the weights]");
    if (rhs_indices.dtype() != DType::uint32 || (lhs_indices && (lhs_indices->dtype() != DType::uint32 ||
                                                                 lhs_indices->size() != rhs_indices.size())))
        throw Error(DMOE_ERR_INVALID, "gatherQmm: indices must be uint32 and of equal length");
    const int R = (int)rhs_indices.size();
    Array out(ctx, DType::bfloat16, {R, w.rows});
    dmoe_qweight q = w.c();
    check(dmoe_gather_qmm((uint16_t *)out.data(), (const uint16_t *)x.data(), &q,
                          lhs_indices ? (const uint32_t *)lhs_indices->data() : nullptr,
                          (const uint32_t *)rhs_indices.data(), R, sorted ? 1 : 0, ctx.workspace(), ctx.stream()));
    return out;
}
// A QuantizedWeight made resident once in the layout the kernels stream (the long-lived weight Arrays of the
// reference's layer structs); gatherQmm on it gives the same bits as on the MLX layout, about 1.3 times faster at
// decode sizes.
class ResidentWeight {
  public:
    ResidentWeight(const Context &ctx, const QuantizedWeight &w, int weight_source) : rows_(w.rows), cols_(w.cols) {
        dmoe_qweight q = w.c();
        check(dmoe_resident_weight_create(&handle_, &q, weight_source, ctx.stream()));
    }
    ~ResidentWeight() { dmoe_resident_weight_destroy(handle_); }
    ResidentWeight(const ResidentWeight &) = delete;
    ResidentWeight &operator=(const ResidentWeight &) = delete;
    Array gatherQmm(const Context &ctx, const Array &x, const Array *lhs_indices, const Array &rhs_indices, bool sorted) const {
        if (x.dtype() != DType::bfloat16 || x.shape().size() != 2 || x.shape()[1] != cols_)
            throw Error(DMOE_ERR_INVALID, "gatherQmm: x must be bfloat16 [rows, cols of the weights]");
        if (rhs_indices.dtype() != DType::uint32 || (lhs_indices && (lhs_indices->dtype() != DType::uint32 ||
                                                                     lhs_indices->size() != rhs_indices.size())))
            throw Error(DMOE_ERR_INVALID, "gatherQmm: indices must be uint32 and of equal length");
        const int R = (int)rhs_indices.size();
        Array out(ctx, DType::bfloat16, {R, rows_});
        check(dmoe_gather_qmm_resident((uint16_t *)out.data(), (const uint16_t *)x.data(), handle_,
                                       lhs_indices ? (const uint32_t *)lhs_indices->data() : nullptr,
                                       (const uint32_t *)rhs_indices.data(), R, sorted ? 1 : 0, ctx.workspace(), ctx.stream()));
        return out;
    }

  private:
    dmoe_resident_weight handle_{};
    int rows_ = 0, cols_ = 0;
};
// mlx_dequantize of one matrix of the stack -> bf16 [rows, cols]
inline Array dequantize(const Context &ctx, const QuantizedWeight &w, int mat_index) {
    Array out(ctx, DType::bfloat16, {w.rows, w.cols});
    dmoe_qweight q = w.c();
    check(dmoe_dequantize((uint16_t *)out.data(), &q, mat_index, ctx.stream()));
    return out;
}
// dequantFp8(ctx, weight, scale, block_size) (deepseek_v4_loader.zig:922-990): weight uint8 [rows, cols] (E4M3FN), scale
// f32 or uint8 (E8M0) [ceil(rows / block), ceil(cols / block)] -> bf16 [rows, cols]
inline Array dequantFp8(const Context &ctx, const Array &weight, const Array &scale, int block_size) {
    if (weight.shape().size() != 2) throw Error(DMOE_ERR_INVALID, "dequantFp8: weight must be [rows, cols]");
    const int rows = weight.shape()[0], cols = weight.shape()[1];
    Array out(ctx, DType::bfloat16, {rows, cols});
    check(dmoe_dequant_fp8_block((uint16_t *)out.data(), (const uint8_t *)weight.data(), scale.data(),
                                 scale.dtype() == DType::uint8 ? 1 : 0, rows, cols, block_size, ctx.stream()));
    return out;
}
} // namespace quantize_mod
namespace ops {
// gatherMm(ctx, a, b, lhs?, rhs, sorted) with unquantized experts (deepseek_v4.zig:978). The reference hands over
// the transposed view [E, in, out] of its [E, out, in] weights; this takes the [E, out, in] array itself (bf16).
inline Array gatherMm(const Context &ctx, const Array &a, const Array &weight, const Array *lhs_indices,
                      const Array &rhs_indices, bool sorted) {
    if (weight.dtype() != DType::bfloat16 || weight.shape().size() != 3)
        throw Error(DMOE_ERR_INVALID, "gatherMm: weight must be bfloat16 [n_experts, out, in]");
    const QuantizedWeight q = QuantizedWeight::unquantized(weight.data(), weight.shape()[0], weight.shape()[1], weight.shape()[2]);
    return quantize_mod::gatherQmm(ctx, a, q, lhs_indices, rhs_indices, sorted);
}
} // namespace ops

// ---- the step after the layer (deepseek_v4.zig:2450-2499, 2652-2654, 2674) ---------------------------------
// mhcPost(x, residual, post_mix, comb_mix): x [T,H] bf16, residual [T,hc_mult,H] bf16, post_mix [T,hc_mult(,1)]
// f32, comb_mix [T,hc_mult,hc_mult] f32 -> [T,hc_mult,H] in x's dtype.
inline Array mhcPost(const Context &ctx, const Array &x, const Array &residual, const Array &post_mix,
                     const Array &comb_mix) {
    if (x.dtype() != DType::bfloat16 || residual.dtype() != DType::bfloat16)
        throw Error(DMOE_ERR_INVALID, "mhcPost: x and residual must be bfloat16");
    if (post_mix.dtype() != DType::float32 || comb_mix.dtype() != DType::float32)
        throw Error(DMOE_ERR_INVALID, "mhcPost: mixes must be float32");
    const std::vector<int> &xs = x.shape(), &rs = residual.shape();
    if (xs.size() != 2 || rs.size() != 3 || rs[0] != xs[0] || rs[2] != xs[1])
        throw Error(DMOE_ERR_INVALID, "mhcPost: x [T,H] and residual [T,hc_mult,H] do not match");
    const int T = xs[0], H = xs[1], m = rs[1];
    if (post_mix.size() != (size_t)T * m || comb_mix.size() != (size_t)T * m * m)
        throw Error(DMOE_ERR_INVALID, "mhcPost: post_mix must hold T*hc_mult values, comb_mix T*hc_mult*hc_mult");
    Array out(ctx, DType::bfloat16, {T, m, H});
    check(dmoe_block_post((uint16_t *)out.data(), (const uint16_t *)x.data(), (const uint16_t *)residual.data(),
                          (const float *)post_mix.data(), (const float *)comb_mix.data(), T, H, m, ctx.stream()));
    return out;
}
// the standard residual connection of the block (mHC disabled): after_attn + ffn_out
inline Array residualAdd(const Context &ctx, const Array &residual, const Array &ffn_out) {
    if (ffn_out.dtype() != DType::bfloat16 || residual.dtype() != DType::bfloat16)
        throw Error(DMOE_ERR_INVALID, "residualAdd: bfloat16 only");
    const std::vector<int> &xs = ffn_out.shape();
    if (xs.size() != 2 || residual.shape() != xs) throw Error(DMOE_ERR_INVALID, "residualAdd: shapes differ");
    Array out(ctx, DType::bfloat16, {xs[0], xs[1]});
    check(dmoe_block_post((uint16_t *)out.data(), (const uint16_t *)ffn_out.data(), (const uint16_t *)residual.data(), nullptr,
                          nullptr, xs[0], xs[1], 0, ctx.stream()));
    return out;
}

} // namespace dmoe
