"""A whole layer step (route -> pack -> both GEMMs on their streams -> shared expert -> combine) recorded into a
HIP graph replays to the same bits as the eager call: every replay is checked, with eager steps and
synchronizations between the replays, for the decode configurations (three streams, two tile classes) and a
prefill-sized one."""
import pytest
import torch

from dmlx_amd import workloads

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("config,scale,tokens", [(1, 0.5, None), (2, 0.5, None), (4, 0.125, None), (1, 1.0, 1), (2, 1.0, 1)])
def test_layer_step_replays_bit_identically(dmoe, ws, config, scale, tokens):
    """tokens = 1: a single sequence at full size, whose launch splits every tile's reduction over two groups of
    wavefronts (twice the workgroups per tile, the halves meeting in LDS)."""
    wl = workloads.make(config, scale=scale)
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap, borrow=tokens is not None)
    scores = wl.scores if tokens is None else wl.scores[:tokens].contiguous()

    def step(x):
        return layer.layer_forward(x, scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws)

    x_a = wl.x if tokens is None else wl.x[:tokens].contiguous()
    x_b = torch.roll(wl.x, 1, dims=0).contiguous() if tokens is None else wl.x[tokens:2 * tokens].contiguous()
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


@pytest.mark.parametrize("config", [1, 2])
def test_decode_step_is_reproducible_call_after_call(dmoe, ws, config):
    """The decode step runs gate/up and down tiles in one launch, the down tiles waiting on per-tile counters for the
    gate/up tiles. 200 calls in a row, with other work queued between them, give the same bits every time."""
    wl = workloads.make(config)
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap, borrow=True)
    want = layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws).clone()
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    bad = 0
    for i in range(200):
        if i % 3 == 0:
            scratch.fill_(i & 0xff)          # other traffic through the caches between the steps
        out = layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws)
        bad += int(not torch.equal(out, want))
    torch.cuda.synchronize()
    assert bad == 0, f"{bad} of 200 calls differ from the first"


def test_decode_step_reports_a_wait_that_gave_up(dmoe, ws):
    """Failure handling of the decode launch: its down-projection workgroups wait a bounded number of polls for
    their tile's gate/up workgroups. With the bound forced to zero from the host they give up at once (every kernel
    still runs to its end), and the workspace check at the next sync point must say so, once. From then on the
    workspace runs the two projections as two launches, which wait for nothing: the next steps are correct and
    clean even with the zero bound still in place. Switching the paired launch back on restores it."""
    from dmlx_amd.capi import DmoeError
    wl = workloads.make(1, scale=0.25)
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap, borrow=True)
    step = lambda: layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws)
    want = step().clone()
    ws.check()                                   # a normal step leaves nothing behind
    ws.set_wait_limit(0)
    try:
        for _ in range(3):
            step()
        with pytest.raises(DmoeError, match="gave up"):
            ws.check()
        ws.check()                               # reported once, then cleared
        for _ in range(3):                       # fallen back to two launches: no wait, so no time-out, right bits
            out = step()
            ws.check()
            assert torch.equal(out, want)
    finally:
        ws.set_wait_limit(1 << 16)
    ws.set_paired_launch(True)
    out = step()
    ws.check()
    assert torch.equal(out, want)
    ws.set_paired_launch(False)                  # the API switch gives the same bits
    out = step()
    ws.check()
    assert torch.equal(out, want)
    layer.close()


def test_pack_reports_expert_ids_out_of_range(dmoe, ws):
    """An expert id >= E is packed under the last expert (every access stays in bounds) and the workspace check
    reports it once, for the one-launch and the three-launch packing kernels."""
    from dmlx_amd.capi import DmoeError
    E, K = 16, 2
    for T in (64, 2000):
        idx = torch.randint(0, E, (T, K), dtype=torch.int32, device="cuda")
        dmoe.pack(idx, E, ws)
        ws.check()
        idx[T // 2, 1] = E + 3
        p = dmoe.pack(idx, E, ws)
        with pytest.raises(DmoeError, match="outside the layer's expert range"):
            ws.check()
        ws.check()
        assert int(p["counts"].sum()) == T * K and int(p["offsets"][E]) == T * K
