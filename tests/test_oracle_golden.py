"""Pins the CPU oracle: against the vectors the reference's own tests hold (tests/golden/), against the
properties its property test asserts, and — where the reference holds nothing — against closed forms,
library routines (numpy stable argsort, torch fp8/bf16 casts, float64 matmul) and brute force.
CPU only."""
import numpy as np
import pytest
import torch

from dmlx_amd import quantize as Q
from dmlx_amd.capi import QUANT_AFFINE, QUANT_FP8_ROW, QUANT_MXFP4, QUANT_NONE, QWeight
from tests.helpers import bf16_bits, max_abs_rel, qmat


# ---------------------------------------------------------------- router (moe_router.zig tests) ----

@pytest.mark.parametrize("case", ["topk_no_normalize", "topk_normalize", "topk_8_experts_top3"])
def test_topk_reference_vectors(orc, golden, case):
    g = golden[case]
    scores = np.array(g["scores"], np.float32)
    normalize = case == "topk_normalize"
    idx, w = orc.topk_route(scores, g["k"], normalize)
    for t, want in enumerate(g["selected_sets"]):
        assert sorted(idx[t].tolist()) == want
    if "weight_sums" in g:
        np.testing.assert_allclose(w.sum(1), g["weight_sums"], atol=g["tol"])
    if "weight_of_expert" in g:
        for j, e in enumerate(idx[0]):
            assert abs(w[0, j] - g["weight_of_expert"][str(int(e))]) < g["tol"]
    if not normalize:  # weights are the scores at the selected experts (moe_router.zig:433-438)
        np.testing.assert_allclose(w, np.take_along_axis(scores, idx.astype(np.int64), 1), atol=g["tol"])


def test_expand_reduce_reference_vectors(orc, golden):
    g = golden["expand"]
    np.testing.assert_array_equal(orc.expand_tokens(np.array(g["x"], np.float32), g["k"]),
                                  np.array(g["expected"], np.float32))
    g = golden["reduce"]
    out = orc.reduce_experts(np.array(g["expert_outs"], np.float32), np.array(g["weights"], np.float32))
    np.testing.assert_allclose(out, g["expected"], atol=g["tol"])


def test_route_expand_reduce_identity(orc, golden):
    g = golden["route_expand_reduce_identity"]
    x = np.array(g["x"], np.float32)
    idx, w = orc.topk_route(np.array(g["scores"], np.float32), g["k"], True)
    out = orc.reduce_experts(orc.expand_tokens(x, g["k"]), w)
    np.testing.assert_allclose(out, x, atol=g["tol"])


def test_property_18_topk_selection(orc):
    """moe_router.zig:455-628: shapes, selected >= k-th score, no unselected above the minimum selected,
    weights are the scores or sum to one; same draw ranges, 100 iterations."""
    rng = np.random.default_rng(18)
    for _ in range(100):
        T = int(rng.choice([1, 2, 3, 4, 5, 8]))
        E = int(rng.choice([4, 6, 8, 12, 16]))
        K = min(int(rng.choice([1, 2, 3, 4])), E)
        normalize = bool(rng.integers(0, 2))
        scores = (rng.integers(0, 10001, (T, E)) / 10000.0).astype(np.float32)
        idx, w = orc.topk_route(scores, K, normalize)
        assert idx.shape == (T, K) and w.shape == (T, K)
        for t in range(T):
            kth = np.sort(scores[t])[::-1][K - 1]
            sel = scores[t, idx[t]]
            assert len(set(idx[t].tolist())) == K and (idx[t] < E).all()
            assert (sel >= kth - 1e-5).all()
            unsel = np.delete(scores[t], idx[t])
            assert unsel.size == 0 or unsel.max() <= sel.min() + 1e-5
            if normalize:
                assert abs(w[t].sum() - 1.0) < 1e-4
            else:
                np.testing.assert_allclose(w[t], sel, atol=1e-5)


def test_topk_matches_stable_argsort_and_tie_rule(orc):
    """The oracle's own sort against numpy's stable argsort (a library routine), ties included:
    columns are the last K of the ascending order, so equal scores resolve to the higher index."""
    rng = np.random.default_rng(0)
    scores = rng.integers(0, 6, (64, 32)).astype(np.float32)  # many ties
    idx, w = orc.topk_route(scores, 5, False)
    want = np.argsort(scores, axis=1, kind="stable")[:, -5:]
    np.testing.assert_array_equal(idx, want.astype(np.uint32))
    idx, _ = orc.topk_route(np.array([[1.0, 1.0, 1.0, 0.5]], np.float32), 2, False)
    assert idx.tolist() == [[1, 2]]
    # weights in ascending order, largest last
    assert (np.diff(w, axis=1) >= 0).all()


def _special_scores(T, E, seed):
    """Scores with negative values, both zeros, denormals, both infinities and NaNs, several of each per row."""
    rng = np.random.default_rng(seed)
    s = rng.standard_normal((T, E)).astype(np.float32)
    special = np.array([0.0, -0.0, 1e-40, -1e-40, np.inf, -np.inf, np.nan, -np.nan, 3e38, -3e38], np.float32)
    pick = rng.random((T, E)) < 0.4
    s[pick] = special[rng.integers(0, len(special), int(pick.sum()))]
    return s


def test_topk_order_of_special_values_matches_numpy(orc):
    """The order the oracle sorts by (ascending, -0 equal to +0, NaN of either sign after +inf, ties by index) is the one
    numpy's stable argsort uses; selection on rows full of such values against that library routine."""
    scores = _special_scores(50, 24, 11)
    for K in (1, 5, 24):
        idx, w = orc.topk_route(scores, K, False)
        want = np.argsort(scores, axis=1, kind="stable")[:, -K:]
        np.testing.assert_array_equal(idx, want.astype(np.uint32))
        np.testing.assert_array_equal(w.view(np.uint32), np.take_along_axis(scores, want, 1).view(np.uint32))


def test_gate_route_bias_mask_renorm_scale(orc):
    """deepseek_v4.zig:589-678 by brute force: selection on biased+masked scores, weights from the raw
    scores, renormalised and scaled; -1e9, -1000 and -inf masks select the same experts."""
    rng = np.random.default_rng(1)
    T, E, K = 32, 64, 6
    scores = (1 / (1 + np.exp(-rng.standard_normal((T, E))))).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.1).astype(np.float32)
    resident = (rng.random(E) < 0.3).astype(np.uint8)
    resident[:K] = 1
    idx, w = orc.gate_route(scores, bias, resident, K, True, 1.5)
    choice = scores + bias + np.where(resident, np.float32(0), np.float32(-1e9))
    want = np.argsort(choice, axis=1, kind="stable")[:, -K:]
    np.testing.assert_array_equal(idx, want.astype(np.uint32))
    assert resident[idx].all()
    raw = np.take_along_axis(scores, want, 1).astype(np.float64)
    np.testing.assert_allclose(w, raw / raw.sum(1, keepdims=True) * 1.5, rtol=1e-5)
    for neg in (-1000.0, -np.inf):
        alt = np.argsort(scores + bias + np.where(resident, 0, neg).astype(np.float32), axis=1, kind="stable")[:, -K:]
        np.testing.assert_array_equal(np.sort(alt, 1), np.sort(want, 1))
    # softmax scoring: no renormalisation (deepseek_v4.zig:663)
    _, w2 = orc.gate_route(scores, None, None, K, False, 2.0)
    np.testing.assert_allclose(w2, np.sort(scores, 1)[:, -K:] * 2.0, rtol=1e-6)


def test_gate_scores_closed_forms(orc):
    x = np.linspace(-8, 8, 4 * 16, dtype=np.float32).reshape(4, 16)
    xd = x.astype(np.float64)
    sm = np.exp(xd - xd.max(1, keepdims=True))
    np.testing.assert_allclose(orc.gate_scores(x, orc.SCORE_SOFTMAX), sm / sm.sum(1, keepdims=True), rtol=1e-5)
    np.testing.assert_allclose(orc.gate_scores(x, orc.SCORE_SIGMOID), 1 / (1 + np.exp(-xd)), rtol=1e-5)
    np.testing.assert_allclose(orc.gate_scores(x, orc.SCORE_SQRTSOFTPLUS), np.sqrt(np.log1p(np.exp(xd))), rtol=1e-4)
    np.testing.assert_allclose(orc.gate_scores(x, orc.SCORE_SQRTSOFTPLUS_STABLE), np.sqrt(np.logaddexp(xd, 0.0)), rtol=1e-6)


# ---------------------------------------------------------------- remap / dedup / smelt ----------------

def test_remap_reference_vectors(orc, golden):
    g = golden["remap_take"]
    table = np.zeros(g["n_experts"], np.int32)
    for k, v in g["remap_nonzero"].items():
        table[int(k)] = v
    idx = np.array(g["indices"], np.uint32)
    assert orc.remap(table, idx).tolist() == g["expected"]                      # 1-D
    assert orc.remap(table, idx.reshape(1, 6)).reshape(-1).tolist() == g["expected"]  # [1, 6]
    g = golden["remap_construction"]
    remap, _ = orc.preload_remap(g["unique_ids"], g["n_experts"])
    for i, e in enumerate(g["unique_ids"]):
        assert remap[e] == i
    for e in g["non_selected"]:
        assert remap[e] == 0


def test_dedup_reference_vectors(orc, golden):
    g = golden["dedup_prefill"]
    idx = np.array(g["indices"], np.uint32)
    uniq, remap = orc.dedup(idx, g["n_experts"])
    assert g["unique_count_min"] <= len(uniq) <= g["unique_count_max"] and len(uniq) < idx.size
    assert uniq.tolist() == sorted(set(idx.reshape(-1).tolist()))
    assert all(remap[e] == i for i, e in enumerate(uniq))                         # remap[e] = slot
    mapped = orc.remap(remap, idx)
    assert (mapped < len(uniq)).all() and len(set(remap[uniq].tolist())) == len(uniq)  # in bounds, bijective
    g = golden["dedup_shared_experts"]
    uniq, remap = orc.dedup(np.array(g["indices"], np.uint32), g["n_experts"])
    assert uniq.tolist() == g["unique_ids"]
    g = golden["dedup_disjoint"]
    uniq, _ = orc.dedup(np.array(g["indices"], np.uint32), g["n_experts"])
    assert len(uniq) == g["unique_count"]


def test_smelt_mask_and_remap_closed_form(orc):
    """deepseek_v4_loader.zig:272-293 / :2151-2168, re-evaluated with numpy float32 arithmetic."""
    mask, n = orc.smelt_mask(256, 0.2, orc.SMELT_UNIFORM)
    assert n == 51 and mask[0] == 1 and mask[255] == 1
    step = np.float32(255) / np.float32(50)
    want = sorted({min(255, int(np.floor(np.float32(step * np.float32(i)) + np.float32(0.5)))) for i in range(51)})
    assert np.flatnonzero(mask).tolist() == want
    mask_f, n_f = orc.smelt_mask(256, 0.2, orc.SMELT_FIRST)
    assert n_f == 51 and mask_f[:51].all() and not mask_f[51:].any()
    full, n_full = orc.smelt_mask(16, 1.0, orc.SMELT_UNIFORM)
    assert n_full == 16 and full.all()
    off, n_off = orc.smelt_mask(16, 0.1, orc.SMELT_UNIFORM, enabled=False)
    assert n_off == 16
    tiny, n_tiny = orc.smelt_mask(8, 0.01, orc.SMELT_FIRST)       # max(1, round(0.08)) = 1
    assert n_tiny == 1 and tiny[0] == 1
    remap = orc.build_remap(mask)
    assert remap[np.flatnonzero(mask)].tolist() == list(range(51))   # running slot index
    assert (remap[mask == 0] == 0).all()                             # unloaded -> row 0
    r2, cb = orc.preload_remap([4, 9, 1], 12)
    assert r2.tolist() == [0, 2, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0]
    assert cb.tolist() == [-1000.0 if e not in (4, 9, 1) else 0.0 for e in range(12)]


# ---------------------------------------------------------------- packing ---------------------------------

@pytest.mark.parametrize("T,K,E", [(1, 1, 4), (16, 2, 8), (64, 6, 256), (300, 6, 64), (0, 6, 8)])
def test_pack_invariants_and_library_sort(orc, T, K, E):
    rng = np.random.default_rng(T * 31 + K)
    idx = rng.integers(0, E, (T, K)).astype(np.uint32)
    p = orc.pack(idx, E)
    flat = idx.reshape(-1)
    n = T * K
    np.testing.assert_array_equal(p["order"], np.argsort(flat, kind="stable").astype(np.uint32))
    assert sorted(p["order"].tolist()) == list(range(n))                          # a permutation
    assert (np.diff(flat[p["order"]].astype(np.int64)) >= 0).all()                 # grouped by expert
    same = flat[p["order"]][1:] == flat[p["order"]][:-1]
    assert (np.diff(p["order"].astype(np.int64))[same] > 0).all()                  # stable inside a segment
    np.testing.assert_array_equal(p["inv"][p["order"]], np.arange(n, dtype=np.uint32))
    np.testing.assert_array_equal(p["token"], p["order"] // K)
    np.testing.assert_array_equal(p["sorted_e"], flat[p["order"]])
    np.testing.assert_array_equal(p["counts"], np.bincount(flat, minlength=E).astype(np.uint32))
    np.testing.assert_array_equal(p["offsets"], np.concatenate([[0], np.cumsum(p["counts"])]).astype(np.uint32))
    assert p["offsets"][E] == n


# ---------------------------------------------------------------- number formats ------------------------

def test_bf16_rounding_matches_torch(orc):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-6, 6, 20000).astype(np.float32)
    ties = np.array([1.00390625, 1.01171875, -1.00390625, 3.0e38, 1e-40, 0.0, -0.0, np.inf], np.float32)
    x = np.concatenate([x, ties])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(orc.f32_to_bf16(x), want)
    got_scalar = np.array([orc.lib().orc_f32_to_bf16(float(v)) for v in ties], np.uint16)
    np.testing.assert_array_equal(got_scalar, want[-len(ties):])


def test_fp8_e4m3_all_codes_match_torch(orc):
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    qm = orc.QMat(codes.numpy().reshape(1, 1, 256), np.ones((1, 1), np.float32), None, 1, 256, orc.FP8_ROW, 8, 0)
    got = np.array([orc.dequant_value(qm, 0, 0, c) for c in range(256)], np.float32)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9
    # row scale multiplies in f32, then one rounding to bf16
    qm2 = orc.QMat(codes.numpy().reshape(1, 1, 256), np.array([[0.37]], np.float32), None, 1, 256, orc.FP8_ROW, 8, 0)
    deq = orc.bf16_to_f32(orc.dequantize(qm2))[0]
    ref = (torch.from_numpy(want) * torch.tensor(0.37)).to(torch.bfloat16).float().numpy()
    ok = ~np.isnan(ref)
    np.testing.assert_array_equal(deq[ok], ref[ok])


@pytest.mark.parametrize("rows,cols,block", [(256, 384, 128), (200, 330, 128), (7, 50, 16), (33, 64, 1)])
def test_fp8_block_dequant_matches_the_reference_op_sequence_in_torch(orc, rows, cols, block):
    """dequantFp8 (deepseek_v4_loader.zig:922-990) evaluated with torch on the CPU exactly as the reference writes it -
    fromFp8 to bf16, zero-pad to whole blocks, view as [m/bs, bs, n/bs, bs], times scale[:, None, :, None] in f32, back,
    truncate, astype(bf16) - against the oracle's per-element restatement. Shapes that need the padding, a block of one,
    f32 scales and E8M0 scales (the reference's exp((s - 127) ln 2) taken as the exact power of two)."""
    g = torch.Generator().manual_seed(rows * 1000 + cols)
    w = torch.randint(0, 256, (rows, cols), generator=g, dtype=torch.uint8)
    w[0, :min(cols, 256)] = torch.arange(min(cols, 256), dtype=torch.uint8)
    sr, sc = -(-rows // block), -(-cols // block)
    for e8m0 in (False, True):
        if e8m0:
            scale = torch.randint(100, 140, (sr, sc), generator=g, dtype=torch.uint8)
            scale_f32 = torch.exp2(scale.float() - 127.0)
        else:
            scale = (torch.rand((sr, sc), generator=g) * 0.01 + 1e-4).float()
            scale_f32 = scale
        w_bf16 = w.view(torch.float8_e4m3fn).to(torch.bfloat16)
        pm, pn = sr * block, sc * block
        padded = torch.zeros((pm, pn), dtype=torch.bfloat16)
        padded[:rows, :cols] = w_bf16
        scaled = padded.reshape(sr, block, sc, block).float() * scale_f32[:, None, :, None]
        want = scaled.reshape(pm, pn)[:rows, :cols].to(torch.bfloat16)
        got = orc.dequant_fp8_block(w.numpy(), scale.numpy(), block)
        want_bits = want.view(torch.int16).numpy().view(np.uint16)
        nan = np.isnan(want.float().numpy())
        assert nan.any() == bool(((w & 0x7F) == 0x7F).any())
        np.testing.assert_array_equal(got[~nan], want_bits[~nan])
        assert ((got[nan] & 0x7FFF) > 0x7F80).all()


def test_mxfp4_codes_and_scales(orc, golden):
    """E2M1 table of deepseek_v4_loader.zig:861-863 times 2^(s-127), low nibble first; exact in bf16."""
    table = np.array(golden["e2m1_table"]["values"], np.float64)
    codes = np.arange(32, dtype=np.uint32) % 16
    words = np.zeros(4, np.uint32)
    for i, c in enumerate(codes):
        words[i // 8] |= np.uint32(c) << np.uint32(4 * (i % 8))
    for s in (0, 1, 100, 126, 127, 128, 140, 252):
        qm = orc.QMat(words.reshape(1, 1, 4), np.array([[[s]]], np.uint8), None, 1, 32, orc.MXFP4, 4, 32)
        got = orc.bf16_to_f32(orc.dequantize(qm))[0].astype(np.float64)
        np.testing.assert_array_equal(got, table[codes] * 2.0 ** (s - 127))
    # quantize -> dequantize round trip: error below half the largest E2M1 gap at the block's scale
    w = torch.randn(4, 64, generator=torch.Generator().manual_seed(5)) * 0.02
    pw, ps = Q.quantize_mxfp4(w)
    qm = qmat(QWeight(pw, ps, None, 4, 64, QUANT_MXFP4, 4, 32))
    deq = orc.bf16_to_f32(orc.dequantize(qm))
    scale = 2.0 ** (ps.numpy().astype(np.float64) - 127).repeat(32, axis=-1)
    assert (np.abs(deq - w.numpy()) <= scale * 1.0 + 1e-12).all()


@pytest.mark.parametrize("bits,group", [(4, 64), (4, 32), (4, 128), (8, 64)])
def test_affine_dequant_layout_and_rounding(orc, bits, group):
    """Layout: a single non-zero code at element i must come back at column i (catches a wrong nibble or
    word order). Value: q*scale + bias in float64, rounded once to bf16 by torch. Round trip: quantize
    then dequantize stays within one step of the input."""
    cols, per = 256, 32 // bits
    s_bits = orc.f32_to_bf16(np.full((1, 1, cols // group), 0.0123, np.float32))
    b_bits = orc.f32_to_bf16(np.full((1, 1, cols // group), -0.0771, np.float32))
    s, b = float(orc.bf16_to_f32(s_bits)[0, 0, 0]), float(orc.bf16_to_f32(b_bits)[0, 0, 0])
    for i in (0, 1, per - 1, per, cols // 2 + 3, cols - 1):
        q = (1 << bits) - 2
        words = np.zeros((1, 1, cols // per), np.uint32)
        words[0, 0, i // per] = np.uint32(q) << np.uint32(bits * (i % per))
        qm = orc.QMat(words, s_bits, b_bits, 1, cols, orc.AFFINE, bits, group)
        got = orc.bf16_to_f32(orc.dequantize(qm))[0]
        want = np.full(cols, b)
        want[i] = q * s + b
        ref = torch.from_numpy(want).float().to(torch.bfloat16).float().numpy()
        np.testing.assert_array_equal(got, ref)
    w = torch.randn(3, 8, cols, generator=torch.Generator().manual_seed(7)) * 0.02
    pw, ps, pb = Q.quantize_affine(w, group, bits)
    qm = qmat(QWeight(pw, ps, pb, 8, cols, QUANT_AFFINE, bits, group))
    step = np.abs(ps.float().numpy()).repeat(group, axis=-1)
    for m in range(3):
        deq = orc.bf16_to_f32(orc.dequantize(qm, m))
        # one quantization step, the final rounding to bf16 (8 significant bits), and the bf16 rounding of the
        # scale accumulated over the code range
        bound = step[m] * (1.01 + (2 ** bits - 1) * 2.0 ** -9) + np.abs(w[m].numpy()) * 2.0 ** -8 + 1e-6
        assert (np.abs(deq - w[m].numpy()) <= bound).all()


# ---------------------------------------------------------------- gather_qmm / layer --------------------

def _small_layer(fmt, E=4, D=256, F=128, seed=11):
    g = torch.Generator().manual_seed(seed)
    mk = {"affine4": lambda w: Q.quantize_affine(w, 64, 4), "affine8": lambda w: Q.quantize_affine(w, 64, 8),
          "mxfp4": lambda w: Q.quantize_mxfp4(w) + (None,), "fp8row": lambda w: Q.quantize_fp8_row(w) + (None,),
          "bf16": lambda w: (w.to(torch.bfloat16), None, None)}[fmt]
    mode, bits, group = {"affine4": (QUANT_AFFINE, 4, 64), "affine8": (QUANT_AFFINE, 8, 64),
                         "mxfp4": (QUANT_MXFP4, 4, 32), "fp8row": (QUANT_FP8_ROW, 8, 0),
                         "bf16": (QUANT_NONE, 16, 0)}[fmt]
    out = []
    for rows, cols in ((F, D), (F, D), (D, F)):
        w = torch.randn(E, rows, cols, generator=g) * 0.02
        a, s, b = mk(w)
        out.append(QWeight(a, s, b, rows, cols, mode, bits, group))
    return out


@pytest.mark.parametrize("fmt", ["affine4", "affine8", "mxfp4", "fp8row", "bf16"])
def test_gather_qmm_reduces_to_dense_matmul(orc, fmt):
    gate, _, _ = _small_layer(fmt)
    qm = qmat(gate)
    if fmt == "bf16":   # unquantized: the "dequantized" matrix is the matrix itself
        np.testing.assert_array_equal(orc.dequantize(qm, 2), bf16_bits(gate.w[2]))
    rng = np.random.default_rng(2)
    R = 10
    x = rng.standard_normal((R, 256)).astype(np.float32)
    xb = orc.f32_to_bf16(x)
    rhs = rng.integers(0, 4, R).astype(np.uint32)
    lhs = rng.integers(0, R, R).astype(np.uint32)
    deq = [orc.dequantize_f32(qm, m).astype(np.float64) for m in range(4)]
    assert deq[1][5, 77] == np.float32(orc.dequant_value(qm, 1, 5, 77))
    xf = orc.bf16_to_f32(xb).astype(np.float64)
    for use_lhs in (False, True):
        want = np.stack([xf[lhs[r] if use_lhs else r] @ deq[rhs[r]].T for r in range(R)])
        got_f32 = orc.gather_qmm(orc.bf16_to_f32(xb), qm, rhs, lhs if use_lhs else None)
        np.testing.assert_allclose(got_f32, want, rtol=2e-5, atol=2e-6)
        got_bf = orc.gather_qmm(xb, qm, rhs, lhs if use_lhs else None)      # bf16 in -> bf16-rounded out
        ref_bf = torch.from_numpy(want).float().to(torch.bfloat16).float().numpy()
        assert max_abs_rel(got_bf, ref_bf) < 8e-3 and np.mean(got_bf == ref_bf) > 0.95


def _dense_reference(orc, x_bits, idx, w, gate, up, down, limit, shared=None):
    """float64 evaluation of sum_k w * down(silu(min(g,L)) * clip(u)) + shared, no intermediate rounding"""
    def deq_all(qm, n):
        return [orc.dequantize_f32(qm, m).astype(np.float64) for m in range(n)]
    x = orc.bf16_to_f32(x_bits).astype(np.float64)

    def ffn(xr, g_, u_, d_, L):
        g, u = g_ @ xr, u_ @ xr
        if L > 0:
            g, u = np.minimum(g, L), np.clip(u, -L, L)
        return d_ @ (g / (1 + np.exp(-g)) * u)
    G, U, Dn = deq_all(gate, gate.n), deq_all(up, up.n), deq_all(down, down.n)
    out = np.zeros((x.shape[0], down.rows))
    for t in range(x.shape[0]):
        for k in range(idx.shape[1]):
            e = idx[t, k]
            out[t] += w[t, k] * ffn(x[t], G[e], U[e], Dn[e], limit)
        if shared is not None:
            sg, su, sd = (deq_all(q, 1)[0] for q in shared)
            out[t] += ffn(x[t], sg, su, sd, 0.0)
    return out


@pytest.mark.parametrize("fmt,before", [("affine4", False), ("affine4", True), ("mxfp4", False), ("affine8", False)])
def test_moe_forward_against_dense_float64(orc, fmt, before):
    gate, up, down = (qmat(q) for q in _small_layer(fmt))
    sh = tuple(qmat(q) for q in _small_layer(fmt, E=1, seed=12))
    rng = np.random.default_rng(4)
    T, K = 6, 2
    x_bits = orc.f32_to_bf16(rng.standard_normal((T, 256)).astype(np.float32) * 3)
    idx = np.stack([rng.choice(4, K, replace=False) for _ in range(T)]).astype(np.uint32)
    w = rng.random((T, K)).astype(np.float32)
    out, h = orc.moe_forward(x_bits, idx, w, gate, up, down, swiglu_limit=1.0, score_before_down=before,
                             shared=sh, want_h=True)
    want = _dense_reference(orc, x_bits, idx, w, gate, up, down, 1.0, sh)
    assert max_abs_rel(out, want) < 1e-2
    assert h.shape == (T * K, 128) and np.abs(h).max() <= 1.0 * 1.0 + 1e-6    # silu(min(g,1)) * clip(u) bounded by L*L
    # the score position only moves roundings
    other = orc.moe_forward(x_bits, idx, w, gate, up, down, swiglu_limit=1.0, score_before_down=not before, shared=sh)
    assert max_abs_rel(other, out) < 1e-2
    # zero routing weights leave the shared expert alone; doubling them doubles the routed part (score-after path)
    only_shared = orc.moe_forward(x_bits, idx, np.zeros_like(w), gate, up, down, swiglu_limit=1.0, shared=sh)
    np.testing.assert_allclose(only_shared, _dense_reference(orc, x_bits, idx, 0 * w, gate, up, down, 1.0, sh),
                               atol=2e-2 * np.abs(want).max())
    routed1 = orc.moe_forward(x_bits, idx, w, gate, up, down, swiglu_limit=1.0)
    routed2 = orc.moe_forward(x_bits, idx, 2 * w, gate, up, down, swiglu_limit=1.0)
    np.testing.assert_allclose(routed2, 2 * routed1, rtol=1e-6, atol=1e-9)
    # permuting the k columns (with their weights) changes at most the summation order
    perm = orc.moe_forward(x_bits, idx[:, ::-1].copy(), w[:, ::-1].copy(), gate, up, down, swiglu_limit=1.0)
    np.testing.assert_allclose(perm, routed1, rtol=1e-5, atol=1e-6)


def test_grouped_float64_reference_equals_the_row_by_row_one(orc):
    """tests/helpers.dense_reference_f64 (rows grouped by expert, used by the GPU accuracy-margin tests at full size)
    against the row-by-row float64 evaluation above, with separate limits for routed and shared experts."""
    from tests.helpers import dense_reference_f64
    gate, up, down = (qmat(q) for q in _small_layer("affine4"))
    sh = tuple(qmat(q) for q in _small_layer("affine4", E=1, seed=12))
    rng = np.random.default_rng(9)
    T, K = 7, 3
    x_bits = orc.f32_to_bf16(rng.standard_normal((T, 256)).astype(np.float32) * 2)
    idx = np.stack([rng.choice(4, K, replace=False) for _ in range(T)]).astype(np.uint32)
    w = rng.random((T, K)).astype(np.float32)
    want = _dense_reference(orc, x_bits, idx, w, gate, up, down, 0.7, sh)
    got = dense_reference_f64(x_bits, idx, w, gate, up, down, 0.7, sh, 0.0)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-14)
    clamped = dense_reference_f64(x_bits, idx, w, gate, up, down, 0.7, sh, 0.01)
    assert np.abs(clamped - want).max() > 1e-6      # the shared expert's own limit is applied
    # the torch twin that the GPU tests use on whole prefill batches (run here on the CPU)
    import torch
    from tests.helpers import dense_reference_f64_device
    x_t = torch.from_numpy(orc.bf16_to_f32(x_bits)).to(torch.bfloat16)
    twin = dense_reference_f64_device(x_t, idx, w, gate, up, down, 0.7, sh, 0.0, device="cpu").numpy()
    np.testing.assert_allclose(twin, want, rtol=1e-10, atol=1e-13)
    twin_clamped = dense_reference_f64_device(x_t, idx, w, gate, up, down, 0.7, sh, 0.01, device="cpu").numpy()
    np.testing.assert_allclose(twin_clamped, clamped, rtol=1e-10, atol=1e-13)


# ---------------------------------------------------------------- batch builder --------------------------------

def test_batch_builder_reference_cases(orc, golden):
    """The literal expectations of src/tests/batch_builder_tests.zig: token order (prefill requests first), positions,
    request count and the isAttending assertions (mask value 0 = attends, batch_builder.zig:253-256)."""
    for case in golden["batch_builder"]["cases"]:
        toks = [np.array(r["tokens"], np.uint32) for r in case["requests"]]
        base = np.array([r["base"] for r in case["requests"]], np.int32)
        flat, pos, offs = orc.batch_concat(toks, base)
        lens = [len(t) for t in toks]
        assert len(offs) - 1 == case["num_requests"], case["name"]
        assert flat.size == case.get("total_tokens", sum(lens))
        if case["tokens"] is not None:
            np.testing.assert_array_equal(flat, case["tokens"], err_msg=case["name"])
        if case["positions"] is not None:
            np.testing.assert_array_equal(pos, case["positions"], err_msg=case["name"])
        m = orc.batch_mask(lens)
        assert m.shape == (flat.size, flat.size)
        for r, c, att in case["attending"]:
            assert (m[r, c] == 0.0) == bool(att), (case["name"], r, c)


def test_batch_concat_and_mask_properties(orc):
    """batch_builder.zig:90-214 and Property 11 of src/tests/batch_builder_tests.zig: total_tokens is the
    sum of the request lengths, positions restart per request, requests never attend to each other."""
    rng = np.random.default_rng(11)
    for _ in range(20):
        n = int(rng.integers(1, 6))
        lens = rng.integers(1, 9, n)
        toks = [rng.integers(0, 1000, l).astype(np.uint32) for l in lens]
        base = rng.integers(0, 50, n).astype(np.int32)
        flat, pos, offs = orc.batch_concat(toks, base)
        assert flat.size == lens.sum() and offs[-1] == lens.sum()
        np.testing.assert_array_equal(flat, np.concatenate(toks))
        for i in range(n):
            np.testing.assert_array_equal(pos[offs[i]:offs[i + 1]], base[i] + np.arange(lens[i]))
        m = orc.batch_mask(lens)
        T = int(lens.sum())
        owner = np.repeat(np.arange(n), lens)
        for r in range(T):
            for c in range(T):
                allowed = owner[r] == owner[c] and c <= r
                assert m[r, c] == (0.0 if allowed else -np.inf)


# ---- router matmul and scoring with fixed arithmetic (assumption u7) ----------------------------------------

def test_det_exp_log_within_one_ulp_of_the_exact_value(orc):
    """Pins the polynomial exp / log against the mathematical functions (float64 numpy), not against themselves."""
    x = np.linspace(-87.0, 88.0, 4001).astype(np.float32)
    got = orc.det_expf(x).astype(np.float64)
    ref = np.exp(x.astype(np.float64))
    assert (np.abs(got - ref) / np.spacing(ref.astype(np.float32)).astype(np.float64)).max() < 1.0
    y = np.exp(np.linspace(np.log(1e-30), np.log(3e38), 4001)).astype(np.float32)
    got = orc.det_logf(y).astype(np.float64)
    ref = np.log(y.astype(np.float64))
    assert (np.abs(got - ref) / np.spacing(np.abs(ref).astype(np.float32)).astype(np.float64)).max() < 1.0
    # special values
    assert orc.det_expf([0.0])[0] == 1.0 and orc.det_expf([-100.0])[0] == 0.0 and np.isinf(orc.det_expf([100.0])[0])
    assert orc.det_logf([1.0])[0] == 0.0 and np.isinf(orc.det_logf([np.inf])[0]) and np.isnan(orc.det_logf([-1.0])[0])
    assert np.isnan(orc.det_expf([np.nan])[0])


def test_det_softplus_against_the_exact_function(orc):
    """The overflow-free softplus behind DMOE_SCORE_SQRTSOFTPLUS_STABLE, against float64 logaddexp(x, 0): within
    two units in the last place from -85 to 200 (a dropped log1p correction, a wrong sign of |x| or a missing max(x, 0)
    each miss that by orders of magnitude somewhere on the range), equal to x where exp(-x) no longer registers, and
    finite where the reference's literal log(1 + exp(x)) overflows. Where the literal form is accurate the two agree to
    rounding; below x = -15 the literal form has lost the value (1 + exp(x) rounds to 1) and the stable one has not."""
    x = np.concatenate([np.linspace(-85.0, 200.0, 5701), [0.0, -0.0, 1e-6, -1e-6, 16.6, 17.4, 88.7, 88.8]]).astype(np.float32)
    got = orc.det_softplusf(x).astype(np.float64)
    ref = np.logaddexp(x.astype(np.float64), 0.0)
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    assert (np.abs(got - ref) / ulp).max() < 2.0, (np.abs(got - ref) / ulp).max()
    big = np.array([30.0, 88.8, 128.0, 3e38], np.float32)
    np.testing.assert_array_equal(orc.det_softplusf(big), big)
    assert orc.det_softplusf([0.0])[0] == np.float32(np.log(2.0)) and orc.det_softplusf([-100.0])[0] == 0.0
    assert np.isnan(orc.det_softplusf([np.nan])[0]) and np.isinf(orc.det_softplusf([np.inf])[0])
    # the scoring function built on it, next to the literal one
    xs = np.linspace(-20.0, 100.0, 9 * 40).astype(np.float32).reshape(9, 40)
    stable, literal = orc.gate_scores_det(xs, orc.SCORE_SQRTSOFTPLUS_STABLE), orc.gate_scores_det(xs, orc.SCORE_SQRTSOFTPLUS)
    np.testing.assert_allclose(stable, np.sqrt(np.logaddexp(xs.astype(np.float64), 0.0)), rtol=3e-7)
    ok = np.isfinite(literal) & (xs > -6.0)
    assert not ok.all() and np.isinf(literal[xs > 88.8]).all() and np.isfinite(stable).all()
    np.testing.assert_allclose(stable[ok], literal[ok], rtol=2e-5)   # 1 + exp(x) rounded: up to 2^-24 / exp(-6) on the log
    assert (literal[xs < -17.0] == 0.0).all() and (stable[xs < -17.0] > 0.0).all()


def test_gate_logits_match_a_float64_matmul(orc):
    rng = np.random.default_rng(5)
    T, D, E = 7, 392, 24      # a short last segment (392 = 3 * 128 + 8)
    x = orc.f32_to_bf16(rng.standard_normal((T, D)).astype(np.float32))
    w = orc.f32_to_bf16((rng.standard_normal((E, D)) / 16).astype(np.float32))
    got = orc.gate_logits(x, w)
    exact = orc.bf16_to_f32(x).astype(np.float64) @ orc.bf16_to_f32(w).astype(np.float64).T
    # every logit is a bf16 number within one bf16 rounding step of the exact dot product
    assert np.array_equal(orc.bf16_to_f32(orc.f32_to_bf16(got)), got)
    assert (np.abs(got - exact) <= np.abs(exact) * 2.0 ** -8 + 1e-6).all()
    # a single product: exact
    one = orc.gate_logits(orc.f32_to_bf16(np.array([[1.5] + [0.0] * 7], np.float32)),
                          orc.f32_to_bf16(np.array([[-2.25] + [0.0] * 7], np.float32)))
    assert one[0, 0] == -3.375


def test_gate_scores_det_agree_with_libm(orc):
    rng = np.random.default_rng(6)
    logits = orc.bf16_to_f32(orc.f32_to_bf16((rng.standard_normal((9, 70)) * 4).astype(np.float32)))
    for func in (0, 1, 2, 3):
        a, b = orc.gate_scores_det(logits, func), orc.gate_scores(logits, func)
        np.testing.assert_allclose(a, b, rtol=2e-6, atol=1e-12)
    sm = orc.gate_scores_det(logits, 0)
    np.testing.assert_allclose(sm.sum(1), 1.0, rtol=1e-6)


def test_hash_route_is_a_table_lookup_with_renormalised_scores(orc):
    rng = np.random.default_rng(8)
    T, E, K, vocab = 11, 16, 3, 40
    scores = rng.random((T, E)).astype(np.float32)
    t2e = np.stack([rng.permutation(E)[:K] for _ in range(vocab)]).astype(np.int32)
    ids = rng.integers(0, vocab, T).astype(np.uint32)
    idx, w = orc.gate_hash_route(scores, t2e, ids, True, 1.5)
    np.testing.assert_array_equal(idx, t2e[ids].astype(np.uint32))
    picked = np.take_along_axis(scores, t2e[ids].astype(np.int64), 1).astype(np.float64)
    np.testing.assert_allclose(w, 1.5 * picked / picked.sum(1, keepdims=True), rtol=1e-6)
    np.testing.assert_allclose(w.sum(1), 1.5, rtol=1e-6)
    _, w_raw = orc.gate_hash_route(scores, t2e, ids, False, 1.0)
    np.testing.assert_array_equal(w_raw, np.take_along_axis(scores, t2e[ids].astype(np.int64), 1))


def _bf16(a):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16)


def test_block_post_matches_float64_einsum_and_hand_values(orc):
    """mhcPost (deepseek_v4.zig:2450-2499): comb is used TRANSPOSED and post_mix multiplies the layer output, not
    the residual. Hand values that a swapped index or operand would miss, then a float64 einsum on random data."""
    from tests.helpers import bf16_bits
    # T=1, D=8, two streams; comb = [[1, 2], [4, 8]]: out_0 = 1*r0 + 4*r1, out_1 = 2*r0 + 8*r1 (plus x * post)
    x = _bf16(np.full((1, 8), 2.0))
    res = _bf16(np.stack([np.full(8, 1.0), np.full(8, 3.0)])[None])
    post = np.array([[0.5, 4.0]], np.float32)
    comb = np.array([[[1.0, 2.0], [4.0, 8.0]]], np.float32)
    out = orc.block_post(bf16_bits(x), bf16_bits(res), post, comb)
    got = torch.from_numpy(out.view(np.int16)).view(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(got[0, 0], np.full(8, 2.0 * 0.5 + 1.0 + 12.0))
    np.testing.assert_array_equal(got[0, 1], np.full(8, 2.0 * 4.0 + 2.0 + 24.0))
    # random data against float64
    rng = np.random.default_rng(11)
    T, D, m = 9, 64, 4
    x = _bf16(rng.standard_normal((T, D)))
    res = _bf16(rng.standard_normal((T, m, D)) * 3)
    post = rng.random((T, m)).astype(np.float32) * 2
    comb = rng.random((T, m, m)).astype(np.float32)
    out = orc.block_post(bf16_bits(x), bf16_bits(res), post, comb)
    got = torch.from_numpy(out.view(np.int16)).view(torch.bfloat16).float().numpy()
    x64, r64 = x.double().numpy(), res.double().numpy()
    want = x64[:, None, :] * post.astype(np.float64)[:, :, None] + np.einsum("tji,tjd->tid", comb.astype(np.float64), r64)
    assert np.max(np.abs(got - want) / (np.abs(want) + 1.0)) < 2 ** -8   # one bf16 rounding
    # residual add: exactly the correctly rounded sum
    a, b = _bf16(rng.standard_normal((5, 16))), _bf16(rng.standard_normal((5, 16)))
    out = orc.block_post(bf16_bits(a), bf16_bits(b))
    want = (a.float() + b.float()).to(torch.bfloat16)
    np.testing.assert_array_equal(out, bf16_bits(want))
