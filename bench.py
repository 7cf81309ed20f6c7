#!/usr/bin/env python3
"""Benchmark of the quantized MoE expert-FFN path on one MI355X.

One "step" is one pass of the whole path over one batch of synthetic input already resident in HBM:
gate routing (top-k on biased scores, renormalised weights) -> token->expert packing -> grouped gate/up
GEMM + limited SwiGLU -> grouped down GEMM -> weighted combine + shared expert, all through the C ABI
(dmoe_moe_layer_forward). Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1] [--windows 9] [--settle-ms 1000]

--config selects the benchmark configuration (0..4, as listed in BASELINE.json); default 1: the 64-sequence decode
step the headline metric is quoted on. The metric's other half - the fraction of the bf16 MFMA peak at the 8k-token
ragged prefill, configuration 3 - is measured in the same run with the same procedure and reported under the key
`prefill_c3`, and so are configurations 2 (`decode_c2`) and 4 (`mixed_c4`) (switch all three off with --no-prefill).

Timing procedure, per configuration: a pre-run of at least --settle-ms of steps brings clocks and memory to their
loaded state (reported as `settle`, separate from `warmup`); then W untimed warm-up steps; then --windows windows of
EXACTLY K steps each, every window bracketed by device synchronisations. `ms_per_step` is the MEDIAN window, all
windows are listed in `window_ms_per_step`. Each window is followed by K more steps with the library's per-stage HIP
events (recorded on the launch stream) switched on; `roofline` describes the dominant kernel of the step with the
median of those per-window stage times. `cpu_baseline` is the CPU restatement of the dmlx/MLX op sequence (the oracle)
timed on this box's host cores on a bounded sample. `roofline.traffic` and `mfma_busy` are read from the rocprofv3
counter summaries under profiles/ (a counter cannot be read from inside the timed run).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

COPY_PROBE_BYTES = 256 << 20  # --copy-probe: bytes read (and written) by each calibration copy
COUNTERS_FILE = os.path.join(ROOT, "profiles", "counters.json")   # written by dmlx_amd/rocprof_summary.py from rocprofv3 --pmc output
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
SMALL_PATH_AVG_ROWS = 16     # at most this many rows per resident expert on average: weight-streaming kernel (kSkinnyAvgRows in csrc/layer.hip)
WIDE_TILE_ROWS = 128         # rows per tile of the library's matrix-core kernels (kMfmaWideTileM in csrc/common.h)


def recorded_counters():
    """Counter readings per (configuration, kernel) recorded under profiles/ ({} when the file is missing)."""
    try:
        with open(COUNTERS_FILE) as f:
            return json.load(f)
    except OSError:
        return {}


def cpu_baseline(wl, max_tokens, min_seconds=10.0, max_runs=5):
    """Time the oracle (route + MoE forward) on the first `max_tokens` tokens of the workload."""
    import numpy as np
    from oracle import oracle
    from oracle.oracle import bf16_bits, qmat

    n = min(wl.T, max_tokens)
    scores = wl.scores[:n].cpu().numpy()
    bias = None if wl.bias is None else wl.bias.cpu().numpy()
    mask = None if wl.resident_mask is None else wl.resident_mask.cpu().numpy()
    x = bf16_bits(wl.x[:n])
    gate, up, down = qmat(wl.gate), qmat(wl.up), qmat(wl.down)
    shared = None if wl.shared is None else tuple(qmat(q) for q in wl.shared)
    remap = None if wl.remap is None else np.array(wl.remap, np.int32)

    def step():
        idx, w = oracle.gate_route(scores, bias, mask, wl.K, wl.renorm, wl.route_scale)
        if remap is not None:
            idx = oracle.remap(remap, idx)
        return oracle.moe_forward(x, idx, w, gate, up, down, swiglu_limit=wl.swiglu_limit,
                                  score_before_down=wl.score_before_down, shared=shared,
                                  shared_swiglu_limit=wl.shared_swiglu_limit)

    times, t_all = [], time.perf_counter()
    while len(times) < max_runs and (not times or time.perf_counter() - t_all < min_seconds):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": n / med, "unit": "tokens/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{len(times)} run(s) of route+FFN+combine on the first {n} of {wl.T} tokens of the same "
                      f"workload, median {med:.3f} s (CPU restatement of the dmlx/MLX op sequence, OpenMP)"}


def measured_peaks(torch):
    """What simple library kernels reach on this GPU, reported next to the published peaks: a device-to-device copy
    (read + written bytes per second), a square bf16 GEMM through torch (hipBLASLt), a loop of matrix instructions
    alone and a kernel that only reads."""
    out = {}
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    a = torch.randn((8192, 8192), device="cuda", dtype=torch.bfloat16)
    b = torch.randn((8192, 8192), device="cuda", dtype=torch.bfloat16)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for name, fn, work in (("d2d_copy_GBs", lambda: dst.copy_(src), 2.0 * n / 1e9),
                           ("bf16_gemm_TFLOPs", lambda: torch.matmul(a, b), 2.0 * 8192 ** 3 / 1e12)):
        for _ in range(3):
            fn()
        e0.record()
        for _ in range(10):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out[name] = work / (e0.elapsed_time(e1) / 10 * 1e-3)
    # the matrix cores alone: the library's loop of bf16 matrix instructions on operands in registers (no loads, no
    # LDS, no decode), on all-zero and on random operands. The gap between the two is power: the prefill kernels'
    # ceiling on real data is the second figure, not the published peak the roofline fraction is quoted against.
    from dmlx_amd import capi
    iters = 20000
    g = torch.Generator(device="cuda").manual_seed(2)
    rnd = torch.randn((capi.MFMA_LOOP_OPERANDS,), generator=g, device="cuda")
    rnd[:capi.MFMA_LOOP_OPERANDS // 3] *= 0.02          # the weight fragments, scaled like the benchmark's weights
    sink = torch.empty((capi.MFMA_LOOP_OUT,), dtype=torch.float32, device="cuda")
    for name, ops in (("mfma_loop_zero_operands_TFLOPs", torch.zeros_like(rnd).to(torch.bfloat16)),
                      ("mfma_loop_random_operands_TFLOPs", rnd.to(torch.bfloat16))):
        for _ in range(3):
            capi.mfma_loop(ops, iters, sink)
        e0.record()
        for _ in range(5):
            capi.mfma_loop(ops, iters, sink)
        e1.record()
        torch.cuda.synchronize()
        out[name] = capi.MFMA_LOOP_FLOP_PER_ITER * iters / 1e12 / (e0.elapsed_time(e1) / 5 * 1e-3)
    # a kernel that only reads (2 GiB, far beyond the memory-side cache): what the decode launch's weight streaming
    # could reach at most. Few workgroups with long private streams do best; the best of three grid sizes is reported.
    del dst, a, b
    big = torch.empty(2 << 30, dtype=torch.uint8, device="cuda")
    big.fill_(1)
    best = 0.0
    for wgs in (256, 512, 8192):
        for _ in range(3):
            nbytes = capi.read_stream(big, wgs)
        e0.record()
        for _ in range(10):
            capi.read_stream(big, wgs)
        e1.record()
        torch.cuda.synchronize()
        rate = nbytes / 1e9 / (e0.elapsed_time(e1) / 10 * 1e-3)
        if rate > best:
            best, out["read_stream_workgroups"] = rate, wgs
    out["read_stream_GBs"] = best
    return out


FP32_VALU_PEAK_TFLOPS = 157.3    # MI355X fp32, published (vector and matrix alike)


def time_gate(torch, steps, windows):
    """DSV4Gate.forward (router matmul + sqrt-softplus scoring + biased top-6, deepseek_v4.zig:546-681) from the
    hidden states on, at the decode and the prefill batch size of the benchmark configurations. It runs in front
    of the timed step (which starts from the scores). The matmul's additions are kept in a fixed order so that the
    selected experts are reproducible bit for bit: fp32 FMAs on the vector ALU for small batches, the f32 matrix
    instruction (which accumulates in that same order) for large ones; both have the same published peak."""
    from dmlx_amd import capi

    g = torch.Generator(device="cuda").manual_seed(1)
    E, D, K = 256, 4096, 6
    wg = (torch.randn((E, D), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    bias = torch.randn((E,), generator=g, device="cuda") * 0.1
    gate = capi.Gate(wg, K, capi.SCORE_SQRTSOFTPLUS, 1.5, bias=bias)
    ws = capi.Workspace()
    out = []
    for T in (64, 8192):
        x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
        for _ in range(steps):
            gate.forward(x, ws)
        torch.cuda.synchronize()
        ms = []
        for _ in range(windows):
            t0 = time.perf_counter()
            for _ in range(steps):
                gate.forward(x, ws)
            torch.cuda.synchronize()
            ms.append((time.perf_counter() - t0) * 1e3 / steps)
        m = statistics.median(ms)
        tf = 2.0 * T * D * E / (m * 1e-3) / 1e12
        out.append({"tokens": T, "experts": E, "hidden": D, "ms": m, "fp32_TFLOPs": tf,
                    "frac_of_fp32_peak": tf / FP32_VALU_PEAK_TFLOPS})
    gate.close()
    ws.close()
    return out


def time_gather_qmm(torch, steps, windows):
    """The leaf operator on its own (quantize_mod.gatherQmm, call shape deepseek_v4.zig:976): the gate and the down
    projection of configuration 1 with that step's routing (384 rows over the live experts), three ways of holding the
    weights: the caller's MLX-layout arrays as they are (dmoe_gather_qmm), the same call with the workspace's opt-in
    cache of re-ordered copies, and a stack made resident once (dmoe_gather_qmm_resident). GB/s of the live experts'
    weight bytes over the whole call (packing launch included)."""
    from dmlx_amd import capi, workloads

    wl = workloads.make(1, device="cuda")
    ws = capi.Workspace()
    idx, _ = capi.gate_route(wl.scores, wl.bias, None, wl.K, wl.renorm, wl.route_scale)
    rhs = idx.reshape(-1).contiguous()
    live = int(torch.unique(rhs).numel())
    x_d = wl.x.repeat_interleave(wl.K, 0).contiguous()
    g = torch.Generator(device="cuda").manual_seed(2)
    x_f = torch.randn((x_d.shape[0], wl.F), generator=g, device="cuda").to(torch.bfloat16)
    out = []
    for name, q, x in (("gate_proj [E, F, D]", wl.gate, x_d), ("down_proj [E, D, F]", wl.down, x_f)):
        per = q.nbytes() // q.n_mats
        res = capi.ResidentWeight(q)
        calls = {"mlx_layout": lambda: capi.gather_qmm(x, q, rhs, ws),
                 "resident": lambda: res.gather_qmm(x, rhs, ws)}
        row = {"projection": name, "rows": int(rhs.numel()), "live_experts": live, "weight_bytes": live * per}
        for key in ("mlx_layout", "resident", "mlx_layout_cached"):
            if key == "mlx_layout_cached":
                ws.set_weight_cache(True)
                fn = calls["mlx_layout"]
            else:
                fn = calls[key]
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            ms = []
            for _ in range(windows):
                t0 = time.perf_counter()
                for _ in range(steps):
                    fn()
                torch.cuda.synchronize()
                ms.append((time.perf_counter() - t0) * 1e3 / steps)
            m = statistics.median(ms)
            row[key] = {"ms": m, "GBs": live * per / (m * 1e-3) / 1e9, "frac_of_hbm_peak": live * per / (m * 1e-3) / 1e9 / HBM_PEAK_GBS}
            if key == "mlx_layout_cached":
                ws.set_weight_cache(False)
        res.close()
        out.append(row)
    ws.check()
    ws.close()
    return out


def time_float_arm(torch, steps, windows):
    """The same step on UNQUANTIZED (bf16) experts, the `is_quantized == false` arm of dispatchGatherMm
    (deepseek_v4.zig:978, ops.gatherMm): configurations 1 and 3 with their seeded routing, the routed experts replaced
    by bf16 matrices drawn like the quantized ones (no shared expert). Decode: GB/s of the live experts' weights over
    the whole step; prefill: TFLOP/s of the three GEMMs over the whole step."""
    from dmlx_amd import capi, workloads

    out = []
    for config in (1, 3):
        wl = workloads.make(config, device="cuda")
        del wl.gate, wl.up, wl.down
        wl.shared = None
        torch.cuda.empty_cache()
        gate, up, down = workloads._experts(wl.E, wl.D, wl.F, "bf16", workloads._gen(90 + config, "cuda"), "cuda")
        layer = capi.Layer(wl.D, wl.F, wl.K, gate, up, down, swiglu_limit=wl.swiglu_limit,
                           score_before_down=wl.score_before_down, shared=None, remap=wl.remap)
        del gate, up, down      # the layer holds its own resident copy
        torch.cuda.empty_cache()
        ws = capi.Workspace(1 << 30)
        res = torch.empty((wl.T, wl.D), dtype=torch.bfloat16, device="cuda")
        step = lambda: layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws, out=res)
        _, idx, _ = layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws,
                                        want_routing=True)
        live = int(torch.unique(idx).numel())
        for _ in range(max(steps, 20)):
            step()
        torch.cuda.synchronize()
        ms = []
        for _ in range(windows):
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            ms.append((time.perf_counter() - t0) * 1e3 / steps)
        ws.check()
        m = statistics.median(ms)
        wbytes = live * 3 * wl.D * wl.F * 2
        flops = 2.0 * wl.T * wl.K * 3 * wl.D * wl.F
        row = {"workload": f"shapes and routing of configuration {config}, bf16 experts, no shared expert", "tokens": wl.T, "live_experts": live,
               "ms_per_step": m, "weight_bytes": wbytes, "flops": flops}
        if config == 1:
            row.update({"GBs": wbytes / (m * 1e-3) / 1e9, "frac_of_hbm_peak": wbytes / (m * 1e-3) / 1e9 / HBM_PEAK_GBS})
        else:
            row.update({"TFLOPs": flops / (m * 1e-3) / 1e12, "frac_of_mfma_peak": flops / (m * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS})
        out.append(row)
        layer.close()
        ws.close()
        del layer, ws, wl
        torch.cuda.empty_cache()
    return out


def run_config(torch, config, steps, warmup, windows, settle_ms, copy_probe=False, score_before_down=False):
    """Builds configuration `config`, times it as the module docstring says and returns (workload, timing, analysis
    inputs). The layer and its workspace are released before returning."""
    from dmlx_amd import capi, workloads

    wl = workloads.make(config, device="cuda")
    wl.score_before_down = bool(score_before_down)
    layer = capi.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap, borrow=True)
    ws = capi.Workspace()
    out = torch.empty((wl.T, wl.D), dtype=torch.bfloat16, device="cuda")

    def step():
        return layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws, out=out)

    if copy_probe:
        src = torch.ones(COPY_PROBE_BYTES // 4, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # clock-settling pre-run: steps in batches until the wall clock says enough
    step()
    torch.cuda.synchronize()
    settle_steps, t0 = 0, time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        settle_steps += steps
    settle = {"steps": settle_steps, "ms": (time.perf_counter() - t0) * 1e3}

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    window_ms, window_stages = [], []
    for _ in range(windows):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        window_ms.append((time.perf_counter() - t0) * 1e3 / steps)
        # the same K steps again with per-stage HIP events (recorded by the library on the launch stream)
        ws.set_stage_timing(True)
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        window_stages.append({k: (ms / n if n else 0.0) for k, (ms, n) in ws.stage_times().items()})
        ws.set_stage_timing(False)
    ws.check()   # no bounded wait gave up, no expert id out of range, in any step above
    assert torch.isfinite(out.float()).all()
    stages = {k: statistics.median(w[k] for w in window_stages) for k in window_stages[0]}

    # distinct live experts of this batch (each expert's weights are read once per step)
    idx, _ = capi.gate_route(wl.scores, wl.bias, wl.resident_mask, wl.K, wl.renorm, wl.route_scale)
    if wl.remap is not None:
        idx = capi.remap_indices(torch.tensor(wl.remap, dtype=torch.int32, device="cuda"), idx)
    packed = capi.pack(idx, wl.E, ws)
    n_live = int(packed["n_live"].item())
    counts = packed["counts"].cpu()
    layer.close()
    ws.close()
    timing = {"ms_per_step": statistics.median(window_ms), "window_ms_per_step": window_ms, "settle": settle,
              "stages": stages}
    return wl, timing, n_live, counts


def describe(torch, wl, config, timing, U, counts, steps, warmup, counters):
    """The JSON fields of one configuration: throughput, roofline of the dominant kernel, whole-step fractions."""
    stages, ms_per_step = timing["stages"], timing["ms_per_step"]
    rows = wl.T * wl.K
    gate_up_w = (wl.gate.nbytes() + wl.up.nbytes()) // wl.E
    down_w = wl.down.nbytes() // wl.E
    kern = "gate_up" if stages["gate_up"] >= stages["down"] else "down"
    decode = rows <= SMALL_PATH_AVG_ROWS * wl.E   # the library's own rule for the small-M path
    # At decode sizes a shared expert of the routed experts' format rides in the routed launches as one more expert
    # with T rows (the library's rule: small-M path, same shape / mode / bits / group): its weights and rows count.
    sh = wl.shared
    folded = decode and sh is not None and all(
        (a.rows, a.cols, a.mode, a.bits, a.group_size) == (b.rows, b.cols, b.mode, b.bits, b.group_size)
        for a, b in ((sh[0], wl.gate), (sh[1], wl.up), (sh[2], wl.down)))
    k_experts, k_rows = U + (1 if folded else 0), rows + (wl.T if folded else 0)
    # Prefill on packed 4-bit weights: each grouped GEMM is two launches on one tile list. The matrix-core kernel (the
    # dominant one, timed as the gate_up / down stage) takes the tiles above 8 rows; an expert's rows are cut into
    # tiles of `tile` rows, so only a remainder of at most 8 rows goes to the weight-streaming kernel (stages *_small).
    split = (not decode) and stages.get("gate_up_small", 0.0) > 0.0
    if split:
        tile = WIDE_TILE_ROWS
        c = counts.to(torch.int64)
        rem = c % tile
        wide = c - torch.where(rem <= 8, rem, torch.zeros_like(rem))
        k_experts, k_rows = int((wide > 0).sum()), int(wide.sum())
    gu_bytes = k_experts * gate_up_w + min(wl.T, k_rows) * wl.D * 2 + k_rows * wl.F * 2
    dn_bytes = k_experts * down_w + k_rows * wl.F * 2 + k_rows * wl.D * 2
    gu_flops, dn_flops = 2.0 * k_rows * 2 * wl.D * wl.F, 2.0 * k_rows * wl.D * wl.F
    # decode steps run both GEMMs as ONE launch (a down workgroup waits for its own tile's gate/up workgroups): the
    # library then reports the launch under the gate/up stage and nothing under down
    paired = decode and stages["down"] == 0.0
    if paired:
        # the intermediate h ([rows, F], written by one half of the launch and read by the other) is not algorithmic traffic
        kern, k_bytes, k_flops = "gate_up+down", gu_bytes + dn_bytes - 2 * k_rows * wl.F * 2, gu_flops + dn_flops
    elif kern == "gate_up":
        k_bytes, k_flops = gu_bytes, gu_flops
    else:
        k_bytes, k_flops = dn_bytes, dn_flops
    k_ms = stages["gate_up"] if paired else stages[kern]
    hbm = k_bytes / (k_ms * 1e-3) / 1e9
    mfma = k_flops / (k_ms * 1e-3) / 1e12
    by_bound = {"hbm": {"bound": "hbm", "achieved": hbm, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm / HBM_PEAK_GBS},
                "mfma": {"bound": "mfma", "achieved": mfma, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": mfma / MFMA_BF16_PEAK_TFLOPS}}
    # Which roofline bounds the launch follows from its arithmetic intensity against the machine balance (published
    # peaks: 2500 TFLOP/s / 8000 GB/s = 312.5 flop per byte), both taken from the ALGORITHMIC flops and bytes: decode
    # launches sit far below it (HBM), the 4-bit prefill far above (matrix core), the mixed batch of configuration 4
    # (8-bit weights, 2080 tokens) below it at 130 flop per byte. The fraction of the other peak is reported as well.
    intensity = k_flops / k_bytes
    ridge = MFMA_BF16_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    first = "hbm" if intensity < ridge else "mfma"
    roof = dict(by_bound[first])
    roof["other_bound"] = by_bound["mfma" if first == "hbm" else "hbm"]
    roof["flop_per_byte"] = intensity
    roof["fractions_use"] = "algorithmic bytes and flops of the launch (not the counted traffic)"
    rec = counters.get(f"c{config}", {}).get(kern, {})
    roof["traffic"] = rec.get("traffic_bytes")
    if "mfma_busy" in rec:
        roof["mfma_busy"] = rec["mfma_busy"]              # SQ_VALU_MFMA_BUSY_CYCLES / (SIMDs x kernel cycles)
        roof["valu_per_mfma"] = rec.get("valu_per_mfma")  # other vector instructions per MFMA
    if "wait_share" in rec:
        roof["wait_share"] = rec["wait_share"]            # SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES
    if rec:
        roof["counters_from"] = rec.get("source")
    launches = (["qgemm_skinny_kernel (gate/up and down tiles in one launch)"] if paired else ["qgemm_skinny_kernel"] if decode else
                ["qgemm_wide_kernel"])  # the benchmark's layers hold their weights in the packed resident layout
    if split:
        roof["rows_in_launch"] = k_rows
        roof["small_tile_launch_ms"] = stages[kern + "_small"]
    roof.update({"kernel": f"grouped {kern} GEMM ({'small-M' if decode else 'MFMA'} path)", "launches": launches, "kernel_ms": k_ms,
                 "algorithmic_bytes": k_bytes, "algorithmic_flops": k_flops, "live_experts": U,
                 "shared_expert_in_launch": bool(folded)})

    step_bytes = U * wl.expert_bytes() + wl.shared_bytes() + 2 * wl.T * wl.D * 2 + wl.T * wl.E_total * 4 + rows * 8
    step_flops = wl.routed_flops() + wl.shared_flops()
    return {
        "value": wl.T / (ms_per_step * 1e-3), "unit": "tokens/s", "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "window_ms_per_step": timing["window_ms_per_step"], "settle": timing["settle"],
        "config": {"workload": wl.name, "baseline_config": config, "tokens": wl.T, "hidden": wl.D,
                   "ffn": wl.F, "experts": wl.E_total, "resident_experts": wl.E, "top_k": wl.K,
                   "shared_expert": wl.shared is not None,
                   "routing_weight": "before the down projection (DSV4SwitchGLU.forward)" if wl.score_before_down
                   else "after the down projection (expert provider paths)",
                   "weights": {0: "affine", 1: "mxfp4", 2: "fp8row", 3: "unquantized"}[wl.gate.mode] + f"-{wl.gate.bits}bit",
                   "max_rows_per_expert": int(counts.max()),
                   "experts_by_rows": {"0": int((counts == 0).sum()), "1-9": int(((counts >= 1) & (counts < 10)).sum()),
                                       "10-99": int(((counts >= 10) & (counts < 100)).sum()),
                                       "100-499": int(((counts >= 100) & (counts < 500)).sum()),
                                       "500+": int((counts >= 500).sum())},
                   "request_lengths": wl.seg_lens},
        "roofline": roof,
        "step": {"algorithmic_bytes": step_bytes, "algorithmic_flops": step_flops,
                 "hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 "mfma_frac": step_flops / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                 "stage_ms": stages},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--windows", type=int, default=9, help="timed windows of --steps steps; the median is reported")
    ap.add_argument("--settle-ms", type=float, default=1000.0, help="clock-settling pre-run before the warm-up")
    ap.add_argument("--config", type=int, default=1, choices=[0, 1, 2, 3, 4])
    ap.add_argument("--score-before-down", type=int, default=0, choices=[0, 1],
                    help="1: routing weight applied to the activation before the down projection (DSV4SwitchGLU.forward); "
                         "0: to the expert outputs (expert provider paths)")
    ap.add_argument("--no-prefill", action="store_true", help="with --config 1: do not also time configurations 3, 2 and 4")
    ap.add_argument("--no-gate", action="store_true", help="do not also time the router (DSV4Gate.forward) in front of the step, the gatherQmm leaf operator and the step on unquantized experts")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-peaks", action="store_true", help="skip the library copy / GEMM reference measurements")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three plain 256 MiB device copies first: the known-size kernel that scales the "
                         "FETCH_SIZE / WRITE_SIZE counters when this command runs under rocprofv3 --pmc")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the one-GPU path only: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    assert args.steps >= 1 and args.windows >= 1 and args.warmup >= 0

    import torch
    from dmlx_amd import capi

    torch.cuda.set_device(0)
    capi.init(0)
    counters = recorded_counters()

    wl, timing, U, counts = run_config(torch, args.config, args.steps, args.warmup, args.windows, args.settle_ms,
                                       args.copy_probe, args.score_before_down)
    body = describe(torch, wl, args.config, timing, U, counts, args.steps, args.warmup, counters)
    result = {"metric": "MoE-FFN tokens/s; HBM GB/s at decode, MFMA % at prefill (4-bit top-6/256)",
              "value": body.pop("value"), "unit": body.pop("unit"), "n_gpus": 1, "steps": args.steps,
              "warmup": args.warmup, "ms_per_step": body.pop("ms_per_step"), "higher_is_better": True,
              "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}
    body.pop("steps"), body.pop("warmup")
    result.update(body)
    result["timing"] = (f"median of {args.windows} windows of {args.steps} steps after a {args.settle_ms:.0f} ms "
                        f"pre-run and {args.warmup} warm-up steps")
    if not args.no_peaks:
        result["roofline"]["measured_peaks"] = measured_peaks(torch)
    decode = wl.T * wl.K <= SMALL_PATH_AVG_ROWS * wl.E
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(wl, max_tokens=64 if decode else 256)
    else:
        result["cpu_baseline"] = None
    del wl
    torch.cuda.empty_cache()

    if args.config == 1 and not args.no_prefill:
        # the metric's prefill half (configuration 3) and the two remaining configurations (2: MXFP4 decode with 51
        # resident experts; 4: mixed batch, 8-bit routed + FP8 shared expert), each with the same procedure and its
        # own roofline block
        for key, cfg in (("prefill_c3", 3), ("decode_c2", 2), ("mixed_c4", 4)):
            wl_n, timing_n, U_n, counts_n = run_config(torch, cfg, args.steps, args.warmup, args.windows, args.settle_ms,
                                                       score_before_down=args.score_before_down)
            result[key] = describe(torch, wl_n, cfg, timing_n, U_n, counts_n, args.steps, args.warmup, counters)
            del wl_n
            torch.cuda.empty_cache()
    if not args.no_gate:
        result["gate"] = time_gate(torch, args.steps, args.windows)
        result["gather_qmm"] = time_gather_qmm(torch, args.steps, args.windows)
        result["float_arm"] = time_float_arm(torch, args.steps, args.windows)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
