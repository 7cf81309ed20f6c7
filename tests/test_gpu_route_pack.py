"""GPU parity: router top-k, remap, expand/reduce and packing, through the C ABI, against the oracle.
Integer results (indices, permutations, offsets) and routing weights must match bit for bit."""
import numpy as np
import pytest
import torch

from tests.helpers import to_np_u32

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _f32_bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ---- reference vectors through the GPU path -------------------------------------------------------------

@pytest.mark.parametrize("case", ["topk_no_normalize", "topk_normalize", "topk_8_experts_top3"])
def test_topk_reference_vectors(dmoe, golden, case):
    g = golden[case]
    scores = np.array(g["scores"], np.float32)
    idx, w = dmoe.topk_route(_dev(scores), g["k"], case == "topk_normalize")
    idx, w = to_np_u32(idx), w.cpu().numpy()
    for t, want in enumerate(g["selected_sets"]):
        assert sorted(idx[t].tolist()) == want
    if "weight_sums" in g:
        np.testing.assert_allclose(w.sum(1), g["weight_sums"], atol=g["tol"])
    if "weight_of_expert" in g:
        for j, e in enumerate(idx[0]):
            assert abs(w[0, j] - g["weight_of_expert"][str(int(e))]) < g["tol"]


def test_expand_reduce_reference_vectors(dmoe, golden):
    g = golden["expand"]
    out = dmoe.expand_tokens(_dev(np.array(g["x"], np.float32)), g["k"])
    np.testing.assert_array_equal(out.cpu().numpy(), np.array(g["expected"], np.float32))
    g = golden["reduce"]
    out = dmoe.reduce_experts(_dev(np.array(g["expert_outs"], np.float32)), _dev(np.array(g["weights"], np.float32)))
    np.testing.assert_allclose(out.cpu().numpy(), g["expected"], atol=g["tol"])
    g = golden["route_expand_reduce_identity"]
    x = _dev(np.array(g["x"], np.float32))
    idx, w = dmoe.topk_route(_dev(np.array(g["scores"], np.float32)), g["k"], True)
    out = dmoe.reduce_experts(dmoe.expand_tokens(x, g["k"]), w)
    np.testing.assert_allclose(out.cpu().numpy(), x.cpu().numpy(), atol=g["tol"])


def test_remap_reference_vectors(dmoe, golden):
    g = golden["remap_take"]
    table = np.zeros(g["n_experts"], np.int32)
    for k, v in g["remap_nonzero"].items():
        table[int(k)] = v
    for shape in ((6,), (1, 6)):
        idx = np.array(g["indices"], np.int32).reshape(shape)
        out = dmoe.remap_indices(_dev(table), _dev(idx))
        assert out.shape == shape and out.cpu().numpy().reshape(-1).tolist() == g["expected"]


# ---- bit-exact parity with the oracle ----------------------------------------------------------------------

@pytest.mark.parametrize("T,E,K,normalize", [(1, 4, 1, True), (16, 8, 2, True), (64, 256, 6, True), (33, 100, 7, False),
                                             (257, 64, 64, True), (5, 1024, 8, True), (8192, 256, 6, True), (0, 8, 2, True)])
def test_topk_route_bit_exact(dmoe, orc, T, E, K, normalize):
    rng = np.random.default_rng(T + E + K)
    scores = rng.random((T, E), dtype=np.float32)
    if T > 1:
        scores[1, :] = 0.25                               # a row of ties
        scores[0, : E // 2] = scores[0, E // 2: E // 2 * 2]  # pairwise ties
    idx, w = dmoe.topk_route(_dev(scores), K, normalize)
    want_idx, want_w = orc.topk_route(scores, K, normalize)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(_f32_bits(w.cpu().numpy()), _f32_bits(want_w))


@pytest.mark.parametrize("T,E,K", [(50, 24, 5), (7, 256, 6), (300, 100, 64), (3, 1024, 8)])
def test_topk_route_special_values_bit_exact(dmoe, orc, T, E, K):
    """Negative scores, both zeros, denormals, both infinities and NaNs of both signs: the selection follows the same
    total order as the oracle (ascending, -0 equal to +0, NaN last, ties to the higher index); the weights are the
    selected scores' bits (no normalisation, so that NaN and infinity stay where they are)."""
    from tests.test_oracle_golden import _special_scores
    scores = _special_scores(T, E, T + E)
    idx, w = dmoe.topk_route(_dev(scores), K, False)
    want_idx, want_w = orc.topk_route(scores, K, False)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(_f32_bits(w.cpu().numpy()), _f32_bits(want_w))
    # the gate's selection on the same values (bias zero, no mask, no renormalisation, scale 1)
    idx2, w2 = dmoe.gate_route(_dev(scores), None, None, K, False, 1.0)
    g_idx, g_w = orc.gate_route(scores, None, None, K, False, 1.0)
    np.testing.assert_array_equal(to_np_u32(idx2), g_idx)
    np.testing.assert_array_equal(_f32_bits(w2.cpu().numpy()), _f32_bits(g_w))


def test_property_18_on_gpu(dmoe):
    """moe_router.zig:455-628 through the GPU path."""
    rng = np.random.default_rng(18)
    for _ in range(100):
        T = int(rng.choice([1, 2, 3, 4, 5, 8]))
        E = int(rng.choice([4, 6, 8, 12, 16]))
        K = min(int(rng.choice([1, 2, 3, 4])), E)
        normalize = bool(rng.integers(0, 2))
        scores = (rng.integers(0, 10001, (T, E)) / 10000.0).astype(np.float32)
        idx, w = dmoe.topk_route(_dev(scores), K, normalize)
        idx, w = to_np_u32(idx), w.cpu().numpy()
        for t in range(T):
            kth = np.sort(scores[t])[::-1][K - 1]
            sel = scores[t, idx[t]]
            assert len(set(idx[t].tolist())) == K and (sel >= kth - 1e-5).all()
            unsel = np.delete(scores[t], idx[t])
            assert unsel.size == 0 or unsel.max() <= sel.min() + 1e-5
            if normalize:
                assert abs(w[t].sum() - 1.0) < 1e-4
            else:
                np.testing.assert_allclose(w[t], sel, atol=1e-5)


@pytest.mark.parametrize("T,E,K,masked", [(64, 256, 6, False), (64, 256, 6, True), (2080, 256, 6, False), (7, 16, 3, True)])
def test_gate_route_bit_exact(dmoe, orc, T, E, K, masked):
    rng = np.random.default_rng(E + K + masked)
    scores = (1 / (1 + np.exp(-rng.standard_normal((T, E))))).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.1).astype(np.float32)
    resident = None
    if masked:
        resident = np.zeros(E, np.uint8)
        resident[rng.choice(E, max(K, E // 5), replace=False)] = 1
    for renorm, scale in ((True, 1.5), (False, 1.0)):
        idx, w = dmoe.gate_route(_dev(scores), _dev(bias), None if resident is None else _dev(resident), K, renorm, scale)
        want_idx, want_w = orc.gate_route(scores, bias, resident, K, renorm, scale)
        np.testing.assert_array_equal(to_np_u32(idx), want_idx)
        np.testing.assert_array_equal(_f32_bits(w.cpu().numpy()), _f32_bits(want_w))
        if masked:
            assert resident[want_idx].all()
    # -inf in place of the reference's -1e9 selects the same experts
    if masked:
        ninf = np.where(resident, 0, -np.inf).astype(np.float32)
        idx2, _ = dmoe.gate_route(_dev(scores), _dev(bias + ninf), None, K, True, 1.5)
        np.testing.assert_array_equal(np.sort(to_np_u32(idx2), 1), np.sort(want_idx, 1))


@pytest.mark.parametrize("T,K,E", [(0, 6, 8), (1, 1, 4), (16, 2, 8), (64, 6, 256), (64, 6, 51), (170, 6, 256),
                                   # up to 16 rows: the single-wavefront kernel (one sequence, 16 rows exactly, 1024
                                   # experts, nearly every row on the same few experts); and sizes just above it
                                   (1, 6, 256), (2, 8, 1024), (16, 1, 16), (5, 3, 3), (3, 5, 40), (2, 6, 256),
                                   (10, 6, 256), (64, 1, 16), (8, 8, 1024), (9, 7, 3), (17, 1, 40),
                                   (171, 6, 256), (2080, 6, 256), (8192, 6, 256), (5000, 3, 1000), (300, 1, 1)])
def test_pack_bit_exact(dmoe, orc, ws, T, K, E):
    rng = np.random.default_rng(T * 7 + K + E)
    if T >= 2000:  # skewed: a few heavy experts, many empty ones
        p = 1.0 / np.arange(1, E + 1) ** 1.1
        idx = rng.choice(E, (T, K), p=p / p.sum()).astype(np.int32)
    else:
        idx = rng.integers(0, E, (T, K)).astype(np.int32)
    got = dmoe.pack(_dev(idx), E, ws)
    want = orc.pack(idx.view(np.uint32), E)
    for name in ("order", "inv", "token", "sorted_e", "counts", "offsets"):
        np.testing.assert_array_equal(to_np_u32(got[name]), want[name], err_msg=name)
    uniq, _ = orc.dedup(idx.view(np.uint32), E)
    n_live = int(got["n_live"].item())
    assert n_live == len(uniq)
    np.testing.assert_array_equal(to_np_u32(got["live"])[:n_live], uniq)


@pytest.mark.parametrize("T,K,D", [(37, 6, 200),      # rows of whole 16-byte pieces: the vector kernels
                                   (5, 3, 37),        # ragged rows: one element per thread
                                   (300, 8, 4100)])   # f32 rows in pieces, bf16 rows ragged (4100 = 4 * 1025)
def test_expand_reduce_match_oracle(dmoe, orc, T, K, D):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((T, D)).astype(np.float32)
    w = rng.random((T, K)).astype(np.float32)
    ex = dmoe.expand_tokens(_dev(x), K)
    np.testing.assert_array_equal(ex.cpu().numpy(), orc.expand_tokens(x, K))
    xb = _dev(x).to(torch.bfloat16)
    exb = dmoe.expand_tokens(xb, K)
    assert torch.equal(exb, xb.repeat_interleave(K, 0))
    eo = rng.standard_normal((T * K, D)).astype(np.float32)
    red = dmoe.reduce_experts(_dev(eo), _dev(w))
    np.testing.assert_array_equal(red.cpu().numpy(), orc.reduce_experts(eo, w))
    eob = _dev(eo).to(torch.bfloat16)
    redb = dmoe.reduce_experts(eob, _dev(w))
    np.testing.assert_array_equal(redb.cpu().numpy(), orc.reduce_experts(eob.float().cpu().numpy(), w))
