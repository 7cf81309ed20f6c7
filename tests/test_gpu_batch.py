"""GPU parity of the device-side batch builder against the oracle's restatement of batch_builder.build:
tokens, positions and the block-diagonal causal mask bit for bit."""
import numpy as np
import pytest
import torch

from tests.helpers import to_np_u32

pytestmark = pytest.mark.gpu


def _requests(seed, lens):
    rng = np.random.default_rng(seed)
    toks = [rng.integers(0, 50000, n).astype(np.uint32) for n in lens]
    base = [int(rng.integers(0, 4000)) if n == 1 else int(rng.integers(0, 100)) for n in lens]
    return toks, base


def test_batch_build_reference_cases(dmoe, ws, golden):
    """The literal cases of the reference's batch builder tests (src/tests/batch_builder_tests.zig:61-316)."""
    for case in golden["batch_builder"]["cases"]:
        lens = [len(r["tokens"]) for r in case["requests"]]
        flat = [t for r in case["requests"] for t in r["tokens"]]
        d_tok, d_pos, d_mask, d_req = dmoe.batch_build(flat, lens, [r["base"] for r in case["requests"]], ws)
        assert d_tok.numel() == case.get("total_tokens", sum(lens)) and int(d_req.max()) + 1 == case["num_requests"]
        if case["tokens"] is not None:
            np.testing.assert_array_equal(to_np_u32(d_tok), case["tokens"], err_msg=case["name"])
        if case["positions"] is not None:
            np.testing.assert_array_equal(d_pos.cpu().numpy(), case["positions"], err_msg=case["name"])
        m = d_mask.cpu().numpy()
        assert m.shape == (len(flat), len(flat))
        for r, c, att in case["attending"]:
            assert (m[r, c] == 0.0) == bool(att), (case["name"], r, c)


@pytest.mark.parametrize("lens", [[5, 3, 1, 1], [512, 512, 1, 1, 1, 7], [1], [3, 0, 4], [129, 2]])
def test_batch_build_matches_oracle(dmoe, orc, ws, lens):
    toks, base = _requests(3, lens)
    want_tok, want_pos, offs = orc.batch_concat(toks, base)
    want_mask = orc.batch_mask(lens)
    flat = np.concatenate(toks) if sum(lens) else np.zeros(0, np.uint32)
    d_tok, d_pos, d_mask, d_req = dmoe.batch_build(flat.tolist(), lens, base, ws)
    np.testing.assert_array_equal(to_np_u32(d_tok), want_tok)
    np.testing.assert_array_equal(d_pos.cpu().numpy(), want_pos)
    np.testing.assert_array_equal(d_mask.cpu().numpy().view(np.uint32), want_mask.view(np.uint32))
    want_req = np.repeat(np.arange(len(lens)), lens)
    np.testing.assert_array_equal(d_req.cpu().numpy(), want_req)
    # mask properties of the reference's tests: 0 on and below the diagonal inside a request, -inf elsewhere
    m = d_mask.cpu().numpy()
    assert np.isneginf(m[np.triu_indices(m.shape[0], 1)]).all() and (np.diag(m) == 0).all()


def test_batch_build_baseline_config_4_shape(dmoe, orc, ws):
    """4 x 512 prefill rows then 32 decode rows (the mixed batch of configuration 4), without the mask too."""
    lens = [512] * 4 + [1] * 32
    toks, base = _requests(4, lens)
    flat = np.concatenate(toks)
    _, d_pos, d_mask, d_req = dmoe.batch_build(flat.tolist(), lens, base, ws, want_mask=False)
    assert d_mask is None
    _, want_pos, _ = orc.batch_concat(toks, base)
    np.testing.assert_array_equal(d_pos.cpu().numpy(), want_pos)
    assert int(d_req[-1]) == len(lens) - 1


def test_batch_build_rejects_inconsistent_requests(dmoe, ws):
    with pytest.raises(dmoe.DmoeError, match="sum"):
        dmoe.batch_build([1, 2, 3], [2, 2], [0, 0], ws)
    with pytest.raises(dmoe.DmoeError, match="negative"):
        dmoe.batch_build([1, 2, 3], [4, -1], [0, 0], ws)
