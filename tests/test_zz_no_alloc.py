"""dmoe_moe_layer_forward_static (the entry point that allocates nothing) against dmoe_moe_layer_forward.

The static entry point keeps every intermediate buffer in a device array that is part of the library, shared by all
calls on a GPU and never cleared between them. Each case makes two calls in a row, the second on a smaller batch, and
compares outputs and routing bit for bit with the workspace entry point (integer results and bf16 outputs of the
same kernels: the bar is equality).
"""
import pytest
import torch

from dmlx_amd import workloads

pytestmark = pytest.mark.gpu


def _layer(dmoe, wl):
    return dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                      score_before_down=wl.score_before_down, shared=wl.shared,
                      shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap)


def _both(layer, wl, T, ws):
    x, scores = wl.x[:T].contiguous(), wl.scores[:T].contiguous()
    args = (x, scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale)
    want = layer.layer_forward(*args, ws, want_routing=True)
    got = layer.layer_forward(*args, None, want_routing=True)
    torch.cuda.synchronize()
    ws.check()
    return got, want


@pytest.mark.parametrize("config,scale,sizes", [
    (1, 0.5, (64, 24)),       # decode kernels, shared expert folded into the routed launches
    (2, 0.5, (64, 7)),        # MXFP4 + Smelt remap
    (4, 0.125, (292, 33)),    # matrix-core kernels, FP8 shared expert run behind the routed launches
    (1, 1.0, (64, 1)),        # the benchmark's decode step at full size
])
def test_static_entry_point_matches_the_workspace_one(dmoe, ws, config, scale, sizes):
    wl = workloads.make(config, device="cuda", scale=scale)
    layer = _layer(dmoe, wl)
    try:
        for T in sizes:   # the second call is smaller and finds the first call's data in the scratch array
            T = min(T, wl.T)
            (out, idx, w), (want_out, want_idx, want_w) = _both(layer, wl, T, ws)
            assert torch.equal(idx, want_idx), f"config {config} T={T}: routing indices differ"
            assert torch.equal(w.view(torch.int32), want_w.view(torch.int32)), f"config {config} T={T}: weights differ"
            assert torch.equal(out.view(torch.int16), want_out.view(torch.int16)), f"config {config} T={T}: outputs differ"
            assert torch.isfinite(out.float()).all()
    finally:
        layer.close()


def test_static_entry_point_allocates_nothing_and_rejects_large_batches(dmoe, ws):
    wl = workloads.make(1, device="cuda", scale=0.5)
    layer = _layer(dmoe, wl)
    try:
        out = torch.empty((wl.T, wl.D), dtype=torch.bfloat16, device="cuda")
        args = (wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale)
        layer.layer_forward(*args, None, out=out)   # first call: kernels loaded, scratch address resolved
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        for _ in range(5):
            layer.layer_forward(*args, None, out=out)
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        assert free1 == free0, f"device memory in use changed by {free0 - free1} bytes across allocation-free calls"
        # a batch whose buffers exceed the static array is refused with a message that names the size
        T_big = 8192
        big_x = torch.zeros((T_big, wl.D), dtype=torch.bfloat16, device="cuda")
        big_scores = torch.rand((T_big, wl.E_total), dtype=torch.float32, device="cuda")
        with pytest.raises(dmoe.DmoeError, match="static device scratch holds"):
            layer.layer_forward(big_x, big_scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, None)
        # and the array still serves the next call
        again = layer.layer_forward(*args, None)
        want = layer.layer_forward(*args, ws)
        torch.cuda.synchronize()
        assert torch.equal(again.view(torch.int16), want.view(torch.int16))
    finally:
        layer.close()


@pytest.mark.parametrize("config,scale,T", [(1, 0.5, 48), (4, 0.125, 200)])
def test_static_entry_point_under_graph_capture(dmoe, ws, config, scale, T):
    """The callers this entry point is for include code under HIP graph capture: one static forward is captured
    (after an eager call, so that nothing host-side is left to set up) and replayed on changing inputs, with eager
    work and synchronizations between the replays; every replay must give the bits of the workspace entry point."""
    wl = workloads.make(config, device="cuda", scale=scale)
    T = min(T, wl.T)
    layer = _layer(dmoe, wl)
    try:
        scores = wl.scores[:T].contiguous()
        x_a = wl.x[:T].contiguous()
        x_b = torch.roll(x_a, 1, dims=0).contiguous()
        route = (wl.bias, wl.resident_mask, wl.renorm, wl.route_scale)
        want_a = layer.layer_forward(x_a, scores, *route, ws).clone()
        want_b = layer.layer_forward(x_b, scores, *route, ws).clone()
        x_in = x_a.clone()
        out = torch.empty((T, wl.D), dtype=torch.bfloat16, device="cuda")
        layer.layer_forward(x_in, scores, *route, None, out=out)     # eager static call first
        torch.cuda.synchronize()
        assert torch.equal(out, want_a)
        free0, _ = torch.cuda.mem_get_info()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            layer.layer_forward(x_in, scores, *route, None, out=out)
        torch.cuda.synchronize()
        for i, (x, want) in enumerate([(x_a, want_a), (x_b, want_b), (x_b, want_b), (x_a, want_a)]):
            x_in.copy_(x)
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want), f"config {config}: replay {i} of the captured static forward differs"
            eager = layer.layer_forward(x, scores, *route, ws)        # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(eager, want)
        ws.check()
        del graph
        torch.cuda.synchronize()
    finally:
        layer.close()
