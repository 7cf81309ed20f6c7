//! Zig binding of libdmoe (include/dmoe.h) with the call surface of dmlx's own modules, so that
//! `src/moe_router.zig` and the provider arm of `DSV4MoE.forward` can switch from mlx-c to this library
//! without touching their callers. It is imported the way dmlx imports mlx-c:
//!
//!     const c = @cImport({ @cInclude("dmoe.h"); });
//!
//! NOTE: written against Zig 0.16 (the version dmlx pins) but NOT compiled in this repository: the build
//! environment has no Zig toolchain. The C++ twin of this file (dmlx_amd/host/moe.hpp) is compiled and
//! tested; the two are kept line-for-line parallel. build.zig additions:
//!     exe.addIncludePath(.{ .cwd_relative = "<repo>/include" });
//!     exe.addLibraryPath(.{ .cwd_relative = "<repo>/dmlx_amd/lib" });
//!     exe.linkSystemLibrary("dmoe");
const std = @import("std");
pub const c = @cImport({
    @cInclude("dmoe.h");
});

pub const Error = error{DmoeError};

/// Same contract as mlx-zig's `c.check`: a non-zero return code becomes one Zig error after the
/// library's message has been logged.
pub fn check(rc: c_int) Error!void {
    if (rc != 0) {
        std.log.err("dmoe: {s}", .{std.mem.span(c.dmoe_last_error())});
        return Error.DmoeError;
    }
}

/// Stream + scratch workspace (what `EagerContext` carries in dmlx).
pub const Context = struct {
    stream: c.dmoe_stream,
    ws: c.dmoe_workspace,

    pub fn init(device: c_int) Error!Context {
        try check(c.dmoe_init(device));
        var s: c.dmoe_stream = undefined;
        try check(c.dmoe_stream_create(&s));
        var w: c.dmoe_workspace = undefined;
        try check(c.dmoe_workspace_create(&w, 0));
        return .{ .stream = s, .ws = w };
    }
    pub fn deinit(self: Context) void {
        _ = c.dmoe_stream_synchronize(self.stream);
        _ = c.dmoe_workspace_destroy(self.ws);
        _ = c.dmoe_stream_destroy(self.stream);
    }
    /// Array.eval(): the host-visible synchronisation point; a step whose kernels gave up a bounded wait fails here
    pub fn eval(self: Context) Error!void {
        try check(c.dmoe_workspace_check(self.ws, self.stream));
    }
    pub fn setWaitLimit(self: Context, polls: c_uint) Error!void {
        try check(c.dmoe_workspace_set_wait_limit(self.ws, polls));
    }
    /// gatherQmm on borrowed MLX-layout arrays: keep re-ordered resident copies of the stacks seen (see dmoe.h)
    pub fn setWeightCache(self: Context, enabled: bool) Error!void {
        try check(c.dmoe_workspace_set_weight_cache(self.ws, @intFromBool(enabled)));
    }
    /// before a cached stack is freed or rewritten while the cache is on (null: drop every copy)
    pub fn invalidateWeightCache(self: Context, qw: ?*const c.dmoe_qweight) Error!void {
        try check(c.dmoe_workspace_weight_cache_invalidate(self.ws, qw));
    }
    /// byte cap of the cached copies (0 = none); a new stack beyond it pushes out the least recently used ones
    pub fn setWeightCacheLimit(self: Context, max_bytes: usize) Error!void {
        try check(c.dmoe_workspace_set_weight_cache_limit(self.ws, max_bytes));
    }
    /// decode steps: gate/up and down in one launch (default) or as two launches that wait for nothing; after `eval`
    /// reported a time-out the workspace is already on two launches
    pub fn setPairedLaunch(self: Context, enabled: bool) Error!void {
        try check(c.dmoe_workspace_set_paired_launch(self.ws, @intFromBool(enabled)));
    }
};

/// Dense row-major device array; `deinit` frees it (handles are owned, as `Array.fromHandle` results are).
pub fn DeviceArray(comptime T: type) type {
    return struct {
        ptr: ?*anyopaque,
        len: usize,
        const Self = @This();
        pub fn alloc(len: usize) Error!Self {
            var p: ?*anyopaque = null;
            try check(c.dmoe_malloc(&p, len * @sizeOf(T)));
            return .{ .ptr = p, .len = len };
        }
        pub fn fromData(ctx: Context, data: []const T) Error!Self {
            const a = try alloc(data.len);
            try check(c.dmoe_copy_to_device(a.ptr, data.ptr, data.len * @sizeOf(T), ctx.stream));
            return a;
        }
        pub fn dataSlice(self: Self, ctx: Context, out: []T) Error!void {
            try check(c.dmoe_copy_to_host(out.ptr, self.ptr, self.len * @sizeOf(T), ctx.stream));
        }
        pub fn deinit(self: Self) void {
            _ = c.dmoe_free(self.ptr);
        }
    };
}

// ---- src/moe_router.zig ------------------------------------------------------------------------------

pub const RouteResult = struct {
    indices: DeviceArray(u32), // [num_tokens, k]
    weights: DeviceArray(f32), // [num_tokens, k]
    k: usize,
    num_tokens: usize,
    pub fn deinit(self: RouteResult) void {
        self.indices.deinit();
        self.weights.deinit();
    }
};

pub const MoERouterConfig = struct {
    num_experts: usize,
    top_k: usize,
    normalize_weights: bool = true,
};

pub const MoERouter = struct {
    config: MoERouterConfig,

    pub fn init(config: MoERouterConfig) MoERouter {
        return .{ .config = config };
    }

    /// scores: [num_tokens, num_experts] f32 on the device
    pub fn topkRoute(self: *const MoERouter, ctx: Context, scores: DeviceArray(f32), num_tokens: usize) Error!RouteResult {
        const k = self.config.top_k;
        const idx = try DeviceArray(u32).alloc(num_tokens * k);
        errdefer idx.deinit();
        const w = try DeviceArray(f32).alloc(num_tokens * k);
        errdefer w.deinit();
        try check(c.dmoe_topk_route(@ptrCast(@alignCast(idx.ptr)), @ptrCast(@alignCast(w.ptr)), @ptrCast(@alignCast(scores.ptr)), @intCast(num_tokens), @intCast(self.config.num_experts), @intCast(k), @intFromBool(self.config.normalize_weights), ctx.stream));
        return .{ .indices = idx, .weights = w, .k = k, .num_tokens = num_tokens };
    }

    /// x: [num_tokens, hidden] -> [num_tokens * k, hidden]
    pub fn expandTokens(ctx: Context, comptime T: type, x: DeviceArray(T), hidden: usize, route: RouteResult) Error!DeviceArray(T) {
        const out = try DeviceArray(T).alloc(route.num_tokens * route.k * hidden);
        errdefer out.deinit();
        try check(c.dmoe_expand_tokens(out.ptr, x.ptr, @intCast(route.num_tokens), @intCast(hidden), @intCast(route.k), @sizeOf(T), ctx.stream));
        return out;
    }

    /// expert_outs: [num_tokens * k, hidden] f32 -> [num_tokens, hidden] f32
    pub fn reduceExperts(ctx: Context, expert_outs: DeviceArray(f32), hidden: usize, route: RouteResult) Error!DeviceArray(f32) {
        const out = try DeviceArray(f32).alloc(route.num_tokens * hidden);
        errdefer out.deinit();
        try check(c.dmoe_reduce_experts(@ptrCast(@alignCast(out.ptr)), expert_outs.ptr, 0, @ptrCast(@alignCast(route.weights.ptr)), @intCast(route.num_tokens), @intCast(route.k), @intCast(hidden), ctx.stream));
        return out;
    }
};

// ---- src/models/deepseek_v4.zig: gate epilogue and the provider arm of DSV4MoE.forward ----------------------

/// DSV4Gate.forward from the scores on (deepseek_v4.zig:589-678)
pub fn gateRoute(ctx: Context, scores: DeviceArray(f32), bias: ?DeviceArray(f32), smelt_mask: ?DeviceArray(u8), num_tokens: usize, n_experts: usize, topk: usize, renorm: bool, route_scale: f32) Error!RouteResult {
    const idx = try DeviceArray(u32).alloc(num_tokens * topk);
    errdefer idx.deinit();
    const w = try DeviceArray(f32).alloc(num_tokens * topk);
    errdefer w.deinit();
    try check(c.dmoe_gate_route(@ptrCast(@alignCast(idx.ptr)), @ptrCast(@alignCast(w.ptr)), @ptrCast(@alignCast(scores.ptr)), if (bias) |b| @ptrCast(@alignCast(b.ptr)) else null, if (smelt_mask) |m| @ptrCast(@alignCast(m.ptr)) else null, @intCast(num_tokens), @intCast(n_experts), @intCast(topk), @intFromBool(renorm), route_scale, ctx.stream));
    return .{ .indices = idx, .weights = w, .k = topk, .num_tokens = num_tokens };
}

/// DSV4Gate (deepseek_v4.zig:521-681) with the router weight resident on the device: `forward` is the whole
/// DSV4Gate.forward(hidden_states, null, stream) -- matmul, scoring function, selection.
pub const ResidentGate = struct {
    handle: c.dmoe_gate,
    topk: usize,

    /// weight: host bf16 bits [n_experts * dim]; bias / mask: host slices or null
    pub fn init(ctx: Context, weight: []const u16, bias: ?[]const f32, smelt_mask: ?[]const u8, n_experts: usize, dim: usize, topk: usize, scoring_func: c_int, route_scale: f32) Error!ResidentGate {
        var d = std.mem.zeroes(c.dmoe_gate_desc);
        d.weight = weight.ptr;
        d.bias = if (bias) |b| b.ptr else null;
        d.resident_mask = if (smelt_mask) |m| m.ptr else null;
        d.n_experts = @intCast(n_experts);
        d.dim = @intCast(dim);
        d.top_k = @intCast(topk);
        d.scoring_func = scoring_func;
        d.route_scale = route_scale;
        d.weight_source = c.DMOE_WEIGHTS_COPY_FROM_HOST;
        var h: c.dmoe_gate = undefined;
        try check(c.dmoe_gate_create(&h, &d, ctx.stream));
        return .{ .handle = h, .topk = topk };
    }

    pub fn deinit(self: *ResidentGate) void {
        _ = c.dmoe_gate_destroy(self.handle);
    }

    pub fn forward(self: *ResidentGate, ctx: Context, hidden_states: DeviceArray(u16), input_ids: ?DeviceArray(u32), num_tokens: usize) Error!RouteResult {
        const idx = try DeviceArray(u32).alloc(num_tokens * self.topk);
        errdefer idx.deinit();
        const w = try DeviceArray(f32).alloc(num_tokens * self.topk);
        errdefer w.deinit();
        try check(c.dmoe_gate_forward(@ptrCast(@alignCast(idx.ptr)), @ptrCast(@alignCast(w.ptr)), null, self.handle, @ptrCast(@alignCast(hidden_states.ptr)), if (input_ids) |ids| @ptrCast(@alignCast(ids.ptr)) else null, @intCast(num_tokens), ctx.ws, ctx.stream));
        return .{ .indices = idx, .weights = w, .k = self.topk, .num_tokens = num_tokens };
    }
};

/// batch_builder.build with the per-token work on the device (src/batch_builder.zig:90-214): `tokens` are the
/// concatenated getRequestTokens results, prefill requests first.
pub fn batchBuild(ctx: Context, tokens: []const u32, seq_lens: []const i32, base_pos: []const i32, out_tokens: DeviceArray(u32), out_positions: DeviceArray(i32), out_mask: ?DeviceArray(f32)) Error!void {
    try check(c.dmoe_batch_build(@ptrCast(@alignCast(out_tokens.ptr)), @ptrCast(@alignCast(out_positions.ptr)), if (out_mask) |m| @ptrCast(@alignCast(m.ptr)) else null, null, tokens.ptr, seq_lens.ptr, base_pos.ptr, @intCast(seq_lens.len), @intCast(tokens.len), ctx.ws, ctx.stream));
}

/// quantize_mod.gatherQmm (call shape at src/models/deepseek_v4.zig:976): row r of the result is x[lhs[r] or r]
/// times the transposed matrix rhs[r] of the stack `q` (device memory). With `q.mode = c.DMOE_QUANT_NONE`, `q.bits = 16`
/// and no scales this is ops.gatherMm on the untransposed [E, out, in] bf16 weights (:978).
pub fn gatherQmm(ctx: Context, x: DeviceArray(u16), q: *const c.dmoe_qweight, lhs_indices: ?DeviceArray(u32), rhs_indices: DeviceArray(u32), sorted: bool) Error!DeviceArray(u16) {
    const out = try DeviceArray(u16).alloc(rhs_indices.len * @as(usize, @intCast(q.rows)));
    errdefer out.deinit();
    try check(c.dmoe_gather_qmm(@ptrCast(@alignCast(out.ptr)), @ptrCast(@alignCast(x.ptr)), q, if (lhs_indices) |l| @ptrCast(@alignCast(l.ptr)) else null, @ptrCast(@alignCast(rhs_indices.ptr)), @intCast(rhs_indices.len), @intFromBool(sorted), ctx.ws, ctx.stream));
    return out;
}

/// dequantFp8(ctx, weight, scale, block_size) (src/models/deepseek_v4_loader.zig:922-990): FP8 E4M3 bytes [rows, cols]
/// with one scale per block_size x block_size tile (f32, or E8M0 bytes with `scale_is_e8m0`) -> bf16 [rows, cols].
pub fn dequantFp8(ctx: Context, weight: DeviceArray(u8), scale_ptr: *const anyopaque, scale_is_e8m0: bool, rows: usize, cols: usize, block_size: usize) Error!DeviceArray(u16) {
    const out = try DeviceArray(u16).alloc(rows * cols);
    errdefer out.deinit();
    try check(c.dmoe_dequant_fp8_block(@ptrCast(@alignCast(out.ptr)), @ptrCast(weight.ptr), scale_ptr, @intFromBool(scale_is_e8m0), @intCast(rows), @intCast(cols), @intCast(block_size), ctx.stream));
    return out;
}

/// A weight stack made resident once in the layout the kernels stream (the long-lived weight Arrays of the
/// reference's layer structs); `gatherQmm` on it gives the same bits as on the MLX layout, faster.
pub const ResidentWeight = struct {
    handle: c.dmoe_resident_weight,
    rows: usize,

    pub fn init(ctx: Context, q: *const c.dmoe_qweight, weight_source: c_int) Error!ResidentWeight {
        var h: c.dmoe_resident_weight = undefined;
        try check(c.dmoe_resident_weight_create(&h, q, weight_source, ctx.stream));
        return .{ .handle = h, .rows = @intCast(q.rows) };
    }
    pub fn deinit(self: *ResidentWeight) void {
        _ = c.dmoe_resident_weight_destroy(self.handle);
    }
    pub fn gatherQmm(self: *const ResidentWeight, ctx: Context, x: DeviceArray(u16), lhs_indices: ?DeviceArray(u32), rhs_indices: DeviceArray(u32), sorted: bool) Error!DeviceArray(u16) {
        const out = try DeviceArray(u16).alloc(rhs_indices.len * self.rows);
        errdefer out.deinit();
        try check(c.dmoe_gather_qmm_resident(@ptrCast(@alignCast(out.ptr)), @ptrCast(@alignCast(x.ptr)), self.handle, if (lhs_indices) |l| @ptrCast(@alignCast(l.ptr)) else null, @ptrCast(@alignCast(rhs_indices.ptr)), @intCast(rhs_indices.len), @intFromBool(sorted), ctx.ws, ctx.stream));
        return out;
    }
};

/// DSV4HyperConn.post / mhcPost (src/models/deepseek_v4.zig:2450-2499) when `hc_mult` > 0, the plain residual add
/// of the block (:2674) when it is 0 (mixes null).
pub fn blockPost(ctx: Context, out: DeviceArray(u16), ffn_out: DeviceArray(u16), residual: DeviceArray(u16), post_mix: ?DeviceArray(f32), comb_mix: ?DeviceArray(f32), n_tokens: usize, dim: usize, hc_mult: usize) Error!void {
    try check(c.dmoe_block_post(@ptrCast(@alignCast(out.ptr)), @ptrCast(@alignCast(ffn_out.ptr)), @ptrCast(@alignCast(residual.ptr)), if (post_mix) |p| @ptrCast(@alignCast(p.ptr)) else null, if (comb_mix) |p| @ptrCast(@alignCast(p.ptr)) else null, @intCast(n_tokens), @intCast(dim), @intCast(hc_mult), ctx.stream));
}

/// One-time resident upload of a layer's experts from MLX-format safetensors shards (what
/// model_registry.zig:255-329 prepares for on-demand reads). `paths` are NUL-terminated.
pub fn layerFromSafetensors(ctx: Context, paths: []const [*:0]const u8, layer_idx: usize, top_k: usize, mode: [*:0]const u8, group_size: i32, bits: i32, swiglu_limit: f32, smelt_mask: ?[]const u8) Error!c.dmoe_layer {
    var o = std.mem.zeroes(c.dmoe_safetensors_opts);
    o.top_k = @intCast(top_k);
    o.mode = mode;
    o.group_size = group_size;
    o.bits = bits;
    o.swiglu_limit = swiglu_limit;
    o.load_shared = 1;
    if (smelt_mask) |m| {
        o.resident_mask = m.ptr;
        o.n_experts_total = @intCast(m.len);
    }
    var layer: c.dmoe_layer = undefined;
    try check(c.dmoe_layer_create_from_safetensors(&layer, @ptrCast(paths.ptr), @intCast(paths.len), @intCast(layer_idx), &o, ctx.stream));
    return layer;
}

/// ExpertProvider over HBM-resident experts: `forward(layer_idx, flat_x, indices, scores)` as in
/// src/models/expert_provider.zig:21; replaces ExpertStreamProvider.streamForward (expert_stream.zig:245-261).
pub const ResidentExpertProvider = struct {
    layers: []c.dmoe_layer,
    hidden: usize,

    pub fn forward(self: *ResidentExpertProvider, ctx: Context, layer_idx: usize, flat_x: DeviceArray(u16), indices: DeviceArray(u32), scores: DeviceArray(f32), num_tokens: usize) Error!DeviceArray(u16) {
        if (layer_idx >= self.layers.len) return Error.DmoeError; // error.PreloadProviderNotInitialized in dmlx
        const out = try DeviceArray(u16).alloc(num_tokens * self.hidden);
        errdefer out.deinit();
        try check(c.dmoe_moe_forward(@ptrCast(@alignCast(out.ptr)), self.layers[layer_idx], @ptrCast(@alignCast(flat_x.ptr)), @ptrCast(@alignCast(indices.ptr)), @ptrCast(@alignCast(scores.ptr)), @intCast(num_tokens), ctx.ws, ctx.stream));
        return out;
    }

    pub fn deinit(self: *ResidentExpertProvider) void {
        for (self.layers) |l| _ = c.dmoe_layer_destroy(l);
    }
};

/// SmeltConfig.buildMask (deepseek_v4_loader.zig:272-293)
pub fn smeltBuildMask(allocator: std.mem.Allocator, n_experts: usize, load_fraction: f32, first: bool, enabled: bool) ![]u8 {
    const mask = try allocator.alloc(u8, n_experts);
    errdefer allocator.free(mask);
    var n: c_int = 0;
    try check(c.dmoe_smelt_build_mask(mask.ptr, &n, @intCast(n_experts), load_fraction, @intFromBool(first), @intFromBool(enabled)));
    return mask;
}

/// expert_remap (deepseek_v4_loader.zig:2151-2168)
pub fn buildRemap(allocator: std.mem.Allocator, mask: []const u8) ![]i32 {
    const remap = try allocator.alloc(i32, mask.len);
    errdefer allocator.free(remap);
    try check(c.dmoe_build_remap(remap.ptr, mask.ptr, @intCast(mask.len)));
    return remap;
}
