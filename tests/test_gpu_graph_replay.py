"""A whole layer step (route -> pack -> both GEMMs on their streams -> shared expert -> combine) recorded into a
HIP graph replays to the same bits as the eager call: every replay is checked, with eager steps and
synchronizations between the replays, for the decode configurations (three streams, two tile classes) and a
prefill-sized one."""
import pytest
import torch

from dmlx_amd import workloads

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("config,scale", [(1, 0.5), (2, 0.5), (4, 0.125)])
def test_layer_step_replays_bit_identically(dmoe, ws, config, scale):
    wl = workloads.make(config, scale=scale)
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap)

    def step(x):
        return layer.layer_forward(x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws)

    x_a = wl.x
    x_b = torch.roll(wl.x, 1, dims=0).contiguous()
    want_a, want_b = step(x_a).clone(), step(x_b).clone()   # also sizes the workspace before the capture
    torch.cuda.synchronize()

    x_in = x_a.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = step(x_in)
    torch.cuda.synchronize()

    for i, (x, want) in enumerate([(x_a, want_a), (x_b, want_b), (x_a, want_a), (x_b, want_b)]):
        x_in.copy_(x)
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i} differs from the eager result"
        eager = step(x)                                      # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(eager, want)
