"""GPU parity of DSV4Gate.forward from the hidden states on (router matmul -> scoring -> selection), through
the C ABI, against the oracle. The library and the oracle fix the same accumulation order and the same
polynomial exp / log, so scores, routing weights and indices must match bit for bit."""
import numpy as np
import pytest
import torch

from tests.helpers import bf16_bits, to_np_u32

pytestmark = pytest.mark.gpu


def _case(seed, T, D, E, with_bias, with_mask, spread):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = (torch.randn((T, D), generator=g, device="cuda") * spread).to(torch.bfloat16)
    wg = (torch.randn((E, D), generator=g, device="cuda") * (1.0 / D ** 0.5)).to(torch.bfloat16)
    bias = torch.randn(E, generator=g, device="cuda") * 0.1 if with_bias else None
    mask = None
    if with_mask:
        mask = (torch.rand(E, generator=g, device="cuda") < 0.4).to(torch.uint8)
        mask[:8] = 1  # at least K resident experts
    return x, wg, bias, mask


@pytest.mark.parametrize("func", [0, 1, 2, 3])
@pytest.mark.parametrize("T,D,E,K,with_bias,with_mask", [
    (64, 4096, 256, 6, True, False),     # decode shape of configuration 1: one reduction segment per wavefront
    (5, 200, 72, 3, True, True),         # short last segment, experts not a multiple of 64, Smelt mask
    (1, 128, 8, 2, False, False),
    (700, 1024, 64, 4, True, False),     # several segments per wavefront, sums through scratch
    (4200, 256, 128, 6, True, False),    # many tokens: a wavefront walks all segments itself
    (1100, 4096, 256, 6, True, False),   # the prefill shape of configurations 3 / 4
    (900, 520, 300, 5, False, True),     # more than 256 experts, short last segment
    (6200, 520, 300, 5, False, True),    # enough tiles for the f32 matrix-core kernel: ragged tokens and experts, short last segment
    (12345, 256, 128, 6, True, False),   # the same kernel, whole segments, a partial last token tile
    (9000, 392, 300, 6, True, True),     # more than 2048 tiles: two expert blocks per wavefront, the last block partly past E
])
def test_gate_forward_bit_exact(dmoe, orc, ws, func, T, D, E, K, with_bias, with_mask):
    x, wg, bias, mask = _case(7 + func, T, D, E, with_bias, with_mask, spread=2.0)
    gate = dmoe.Gate(wg, K, func, route_scale=1.5, bias=bias, resident_mask=mask)
    idx, w, scores = gate.forward(x, ws, want_scores=True)
    logits = orc.gate_logits(bf16_bits(x), bf16_bits(wg))
    want_scores = orc.gate_scores_det(logits, func)
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    want_idx, want_w = orc.gate_route(want_scores, None if bias is None else bias.cpu().numpy(),
                                      None if mask is None else mask.cpu().numpy(), K, func != 0, 1.5)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    # without the inspection output the routing is the same
    idx2, w2 = gate.forward(x, ws)
    assert torch.equal(idx2, idx) and torch.equal(w2, w)
    gate.close()


def test_gate_prefill_full_size_bit_exact(dmoe, orc, ws):
    """The router of the 8192-token prefill (f32 matrix-core kernel, one 32 x 32 tile per wavefront) at full size: logits
    after scoring, selected experts and weights bit for bit against the CPU restatement, whose sums are fmaf chains."""
    T, D, E, K = 8192, 4096, 256, 6
    x, wg, bias, _ = _case(31, T, D, E, True, False, spread=2.0)
    gate = dmoe.Gate(wg, K, 2, route_scale=1.5, bias=bias)
    idx, w, scores = gate.forward(x, ws, want_scores=True)
    want_scores = orc.gate_scores_det(orc.gate_logits(bf16_bits(x), bf16_bits(wg)), 2)
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    want_idx, want_w = orc.gate_route(want_scores, bias.cpu().numpy(), None, K, True, 1.5)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    gate.close()


def test_gate_extreme_logits(dmoe, orc, ws):
    """Saturating inputs: sigmoid -> 0 / 1, softplus overflow of the reference's literal form (exp -> inf), and the
    overflow-free variant on the same logits."""
    T, D, E = 4, 64, 64
    x = torch.full((T, D), 8.0, device="cuda").to(torch.bfloat16)
    wg = torch.zeros((E, D), device="cuda")
    wg[0] = 0.25      # logit 128: exp overflows, log(inf) = inf
    wg[1] = -0.25     # logit -128
    wg[2] = 0.0
    wg = wg.to(torch.bfloat16)
    for func in (1, 2, 3):
        gate = dmoe.Gate(wg, 2, func)
        _, _, scores = gate.forward(x, ws, want_scores=True)
        want = orc.gate_scores_det(orc.gate_logits(bf16_bits(x), bf16_bits(wg)), func)
        np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want.view(np.uint32))
        if func == 2:
            assert bool(torch.isinf(scores[:, 0]).all())
        if func == 3:   # the overflow-free softplus: sqrt(128) where the literal form gives infinity
            assert bool((scores[:, 0] == 128.0 ** 0.5).all()) and bool(torch.isfinite(scores).all())
        gate.close()


@pytest.mark.parametrize("func", [0, 2])
def test_hash_gate_takes_experts_from_the_table(dmoe, orc, ws, func):
    """Hash layers (deepseek_v4.zig:619-636): indices = tid2eid[input_ids]; weights from the unbiased scores."""
    T, D, E, K, vocab = 37, 256, 64, 6, 500
    x, wg, bias, _ = _case(21, T, D, E, True, False, spread=2.0)
    g = torch.Generator(device="cuda").manual_seed(5)
    tid2eid = torch.stack([torch.randperm(E, generator=g, device="cuda")[:K] for _ in range(vocab)]).to(torch.int32)
    ids = torch.randint(0, vocab, (T,), generator=g, device="cuda", dtype=torch.int32)
    gate = dmoe.Gate(wg, K, func, route_scale=2.5, bias=bias, tid2eid=tid2eid)
    idx, w, scores = gate.forward(x, ws, want_scores=True, input_ids=ids)
    want_scores = orc.gate_scores_det(orc.gate_logits(bf16_bits(x), bf16_bits(wg)), func)
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    want_idx, want_w = orc.gate_hash_route(want_scores, tid2eid.cpu().numpy(), to_np_u32(ids), func != 0, 2.5)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    # the table decides, not the scores: the indices are exactly the rows of the table
    np.testing.assert_array_equal(to_np_u32(idx), tid2eid.cpu().numpy()[to_np_u32(ids).astype(np.int64)].astype(np.uint32))
    # the same call without a scores output (the scores then live in the workspace only)
    idx3, w3 = gate.forward(x, ws, input_ids=ids)
    assert torch.equal(idx3, idx) and torch.equal(w3, w)
    # without token ids a hash gate falls back to score-based top-k, like the reference
    idx2, w2 = gate.forward(x, ws)
    ref_idx, ref_w = orc.gate_route(want_scores, bias.cpu().numpy(), None, K, func != 0, 2.5)
    np.testing.assert_array_equal(to_np_u32(idx2), ref_idx)
    np.testing.assert_array_equal(w2.cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
    gate.close()


def test_gate_rejects_bad_arguments(dmoe):
    wg = torch.zeros((8, 64), device="cuda", dtype=torch.bfloat16)
    with pytest.raises(dmoe.DmoeError):
        dmoe.Gate(wg, 9, 1)            # top_k > experts
    with pytest.raises(dmoe.DmoeError):
        dmoe.Gate(wg[:, :60].contiguous(), 2, 1)   # dim not a multiple of 8
    with pytest.raises(dmoe.DmoeError):
        dmoe.Gate(wg, 2, 7)            # unknown scoring function


@pytest.mark.parametrize("T", [40, 6200])
def test_gate_logits_tiny_and_huge_magnitudes(dmoe, orc, ws, T):
    """Both matmul kernels (vector ALU for 40 tokens, f32 matrix core for 6200) on operands whose sums overflow to
    infinity (both signs) next to operands whose products are f32 denormals: the scores must still be the oracle's
    bits. (Logits that small all score like 0, so this checks that tiny operands produce nothing else - no NaN, no
    stray value - not how the hardware rounds denormals; the overflowing sums do tell saturation from infinity.)"""
    D, E = 256, 300
    g = torch.Generator(device="cuda").manual_seed(17)
    sign = lambda *s: torch.where(torch.rand(s, generator=g, device="cuda") < 0.5, -1.0, 1.0)
    x = torch.full((T, D), 2.0 ** -90, device="cuda") * sign(T, D) * (1 + torch.rand((T, D), generator=g, device="cuda"))
    wg = torch.full((E, D), 2.0 ** -50, device="cuda") * sign(E, D) * (1 + torch.rand((E, D), generator=g, device="cuda"))
    x[1::2] = x[1::2] * 2.0 ** 150          # every second token: products near 2^10, still ordinary numbers
    x[3::8] = 2.0 ** 100                    # some tokens against ...
    wg[5::16] = 2.0 ** 27                   # ... some experts: 256 products of 2^127 overflow the sum
    x, wg = x.to(torch.bfloat16), wg.to(torch.bfloat16)
    logits = orc.gate_logits(bf16_bits(x), bf16_bits(wg))
    assert np.isinf(logits).any() and (np.abs(logits[np.isfinite(logits)]) < 2.0 ** -126).any(), "the case must reach both ends"
    for func in (1, 2, 3):
        gate = dmoe.Gate(wg, 4, func)
        _, _, scores = gate.forward(x, ws, want_scores=True)
        want = orc.gate_scores_det(logits, func)
        np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want.view(np.uint32))
        gate.close()
