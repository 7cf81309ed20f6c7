"""GPU parity: dequantize (bit-exact), gather_qmm and the MoE layer forward (bf16 outputs within
max-abs-rel 1e-2 of the fp32-accumulating oracle), through the C ABI, for every weight format and for both
GEMM paths (small-M decode kernel, MFMA prefill kernel)."""
import numpy as np
import pytest
import torch

from dmlx_amd import quantize as Q
from dmlx_amd import workloads
from dmlx_amd.capi import QUANT_AFFINE, QUANT_FP8_ROW, QUANT_MXFP4, QUANT_NONE, QWeight
from tests.helpers import bf16_bits, max_abs_rel, max_abs_rel_rows, oracle_forward, qmat, to_np_u32

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-2   # max |gpu - oracle| / max |oracle| on bf16 outputs
ROW_TOL = 2e-2   # the same ratio taken per output row


def _stack(fmt, n, rows, cols, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    w = torch.randn((n, rows, cols), generator=g, device="cuda") * 0.02
    if fmt == "affine4":
        a, s, b = Q.quantize_affine(w, 64, 4)
        return QWeight(a, s, b, rows, cols, QUANT_AFFINE, 4, 64)
    if fmt == "affine4g32":
        a, s, b = Q.quantize_affine(w, 32, 4)
        return QWeight(a, s, b, rows, cols, QUANT_AFFINE, 4, 32)
    if fmt == "affine4g128":
        a, s, b = Q.quantize_affine(w, 128, 4)
        return QWeight(a, s, b, rows, cols, QUANT_AFFINE, 4, 128)
    if fmt == "affine8":
        a, s, b = Q.quantize_affine(w, 64, 8)
        return QWeight(a, s, b, rows, cols, QUANT_AFFINE, 8, 64)
    if fmt == "affine8g32":
        a, s, b = Q.quantize_affine(w, 32, 8)
        return QWeight(a, s, b, rows, cols, QUANT_AFFINE, 8, 32)
    if fmt == "mxfp4":
        a, s = Q.quantize_mxfp4(w)
        return QWeight(a, s, None, rows, cols, QUANT_MXFP4, 4, 32)
    if fmt == "bf16":     # unquantized experts (the float arm of dispatchGatherMm)
        return QWeight(w.to(torch.bfloat16), None, None, rows, cols, QUANT_NONE, 16, 0)
    a, s = Q.quantize_fp8_row(w)
    return QWeight(a, s, None, rows, cols, QUANT_FP8_ROW, 8, 0)


FORMATS = ["affine4", "affine4g32", "affine4g128", "affine8", "mxfp4", "fp8row", "bf16"]


@pytest.mark.parametrize("fmt", FORMATS)
def test_dequantize_bit_exact(dmoe, orc, fmt):
    qw = _stack(fmt, 3, 96, 512, 1)
    if fmt == "mxfp4":   # exercise extreme shared exponents and every code
        qw.scales[0, 0, :4] = torch.tensor([0, 1, 254, 200], dtype=torch.uint8, device="cuda")
        qw.w[0, 0, :4] = torch.tensor([0x76543210, -19088744, 0x0F0F0F0F, 0x7F7F7F7F], dtype=torch.int32, device="cuda")
    if fmt == "fp8row":  # every byte value, NaN codes included
        qw.w[0, 0, :256] = torch.arange(256, dtype=torch.uint8, device="cuda")
    qm = qmat(qw)
    for m in range(3):
        want = orc.dequantize(qm, m)
        nan = (want & 0x7FFF) > 0x7F80
        for fused in (False, True) if fmt != "bf16" else (False,):   # fused: the prefill kernels' in-register decoder
            got = bf16_bits(dmoe.dequantize(qw, m, fused=fused))
            np.testing.assert_array_equal(got[~nan], want[~nan], err_msg=f"{fmt} fused={fused}")
            assert ((got[nan] & 0x7FFF) > 0x7F80).all()


@pytest.mark.parametrize("rows,cols,block", [(512, 768, 128), (200, 336, 128), (37, 50, 16), (64, 48, 24), (33, 64, 1),
                                             (4096, 2048, 128)])
def test_dequant_fp8_block_bit_exact(dmoe, orc, rows, cols, block):
    """dmoe_dequant_fp8_block (dequantFp8, deepseek_v4_loader.zig:922-990) against the oracle: every E4M3 byte, shapes
    that are not whole blocks, block sizes that send the call to the one-value-per-thread kernel (columns or blocks not
    multiples of 16), f32 and E8M0 scales with the extreme exponents, and one weight matrix of a real expert's size."""
    g = torch.Generator(device="cuda").manual_seed(rows + cols)
    w = torch.randint(0, 256, (rows, cols), generator=g, device="cuda", dtype=torch.uint8)
    w[0, :min(cols, 256)] = torch.arange(min(cols, 256), dtype=torch.uint8, device="cuda")
    sr, sc = -(-rows // block), -(-cols // block)
    scale_f = (torch.rand((sr, sc), generator=g, device="cuda") * 0.01 + 1e-4).float()
    scale_e = torch.randint(90, 150, (sr, sc), generator=g, device="cuda", dtype=torch.uint8)
    scale_e.view(-1)[:3] = torch.tensor([0, 254, 255], dtype=torch.uint8, device="cuda")[:scale_e.numel()][:3]
    for scale in (scale_f, scale_e):
        got = bf16_bits(dmoe.dequant_fp8_block(w, scale, block))
        want = orc.dequant_fp8_block(w.cpu().numpy(), scale.cpu().numpy(), block)
        nan = (want & 0x7FFF) > 0x7F80
        np.testing.assert_array_equal(got[~nan], want[~nan])
        assert ((got[nan] & 0x7FFF) > 0x7F80).all()
    with pytest.raises(dmoe.DmoeError):
        dmoe.check(dmoe.lib().dmoe_dequant_fp8_block(None, None, None, 0, 4, 4, 2, None))


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("R,n_mats,rows,cols", [(24, 8, 256, 1024),     # small-M path (<= 4 rows per expert on average)
                                                (700, 4, 256, 512),     # MFMA path, ragged segments
                                                (130, 1, 128, 2048),    # single expert, MFMA, partial tile
                                                (700, 4, 256, 384),     # reduction not a multiple of the pipeline depth
                                                (1200, 2, 192, 640),    # 256-row tiles, idle wavefronts in the last strip
                                                (900, 12, 256, 2048),   # MFMA path for the large tiles + weight-streaming kernel for the small ones
                                                (60, 8, 256, 2048),     # small-M path, some experts above 8 rows (restaged tiles)
                                                (30, 4, 192, 2048)])    # same, weight rows not a multiple of the workgroup's
def test_gather_qmm_matches_oracle(dmoe, orc, ws, fmt, R, n_mats, rows, cols):
    qw = _stack(fmt, n_mats, rows, cols, 2)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn((R + 5, cols), generator=g, device="cuda").to(torch.bfloat16)
    rhs = torch.randint(0, n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
    lhs = torch.randint(0, R + 5, (R,), generator=g, device="cuda", dtype=torch.int32)
    qm = qmat(qw)
    for use_lhs in (False, True):
        got = dmoe.gather_qmm(x, qw, rhs, ws, lhs if use_lhs else None).float().cpu().numpy()
        want = orc.gather_qmm(bf16_bits(x), qm, to_np_u32(rhs), to_np_u32(lhs) if use_lhs else None)
        assert max_abs_rel(got, want) < OUT_TOL, (fmt, use_lhs, max_abs_rel(got, want))
    # sorted indices (the reference's sorted=true call) give the same rows
    srt = torch.sort(rhs).values.to(torch.int32)
    got_s = dmoe.gather_qmm(x, qw, srt, ws, None, sorted_indices=True).float().cpu().numpy()
    want_s = orc.gather_qmm(bf16_bits(x), qm, to_np_u32(srt), None)
    assert max_abs_rel(got_s, want_s) < OUT_TOL


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("R,n_mats,rows,cols", [(40, 16, 256, 2048), (900, 6, 256, 1024), (12, 3, 96, 512), (50, 4, 40, 256)])
def test_gather_qmm_on_a_resident_stack(dmoe, orc, ws, fmt, R, n_mats, rows, cols):
    """dmoe_gather_qmm_resident: the stack copied once into the kernels' layout. At decode sizes the same bits as the
    call on the MLX layout (the same kernel with other addressing); at prefill sizes the packed 4-bit formats take
    another kernel, so the two agree to rounding. Always within the output bar of the oracle. The last shape cannot
    be re-ordered (rows not a multiple of 32) and stays in the MLX layout inside the handle."""
    qw = _stack(fmt, n_mats, rows, cols, 7)
    g = torch.Generator(device="cuda").manual_seed(R)
    x = torch.randn((R + 3, cols), generator=g, device="cuda").to(torch.bfloat16)
    rhs = torch.randint(0, n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
    lhs = torch.randint(0, R + 3, (R,), generator=g, device="cuda", dtype=torch.int32)
    res = dmoe.ResidentWeight(qw)
    for use_lhs in (False, True):
        got = res.gather_qmm(x, rhs, ws, lhs if use_lhs else None)
        plain = dmoe.gather_qmm(x, qw, rhs, ws, lhs if use_lhs else None)
        if R <= 16 * n_mats:   # both calls on the weight-streaming kernel
            assert torch.equal(got, plain), (fmt, use_lhs)
        else:
            # one bf16 step of the largest output at most (2^-7 of its value)
            assert max_abs_rel(got.float().cpu().numpy(), plain.float().cpu().numpy()) < 8e-3, (fmt, use_lhs)
        want = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), to_np_u32(lhs) if use_lhs else None)
        assert max_abs_rel(got.float().cpu().numpy(), want) < OUT_TOL
    res.close()
    host = dmoe.ResidentWeight(qw.to("cpu"))          # the same stack handed over from host memory
    assert torch.equal(host.gather_qmm(x, rhs, ws), got if False else dmoe.ResidentWeight(qw).gather_qmm(x, rhs, ws))
    host.close()


@pytest.mark.parametrize("fmt", ["affine4", "mxfp4", "affine8g32"])
@pytest.mark.parametrize("rows,cols", [(96, 512), (200, 1536), (256, 4096), (64, 1024)])
def test_gather_qmm_mlx_layout_line_loads(dmoe, orc, ws, fmt, rows, cols):
    """Decode-sized calls on the MLX layout whose scale rows are whole 16-byte blocks: the weight-streaming kernel then
    loads whole 128-byte lines and turns them in LDS, and takes scales / biases eight steps at a time. Reductions of one
    half round (8 steps), of rounds plus a half, of several rounds; weight rows that end inside a wavefront's block.
    Same bits as the re-ordered copy of the stack, and the oracle's values within the output bar."""
    n_mats = 5
    qw = _stack(fmt, n_mats, rows, cols, 11)
    g = torch.Generator(device="cuda").manual_seed(rows + cols)
    for R in (1, 7, 33):
        x = torch.randn((R + 2, cols), generator=g, device="cuda").to(torch.bfloat16)
        rhs = torch.randint(0, n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
        lhs = torch.randint(0, R + 2, (R,), generator=g, device="cuda", dtype=torch.int32)
        got = dmoe.gather_qmm(x, qw, rhs, ws, lhs)
        want = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), to_np_u32(lhs))
        assert max_abs_rel(got.float().cpu().numpy(), want) < OUT_TOL, (fmt, R)
        if rows % 32 == 0:
            res = dmoe.ResidentWeight(qw)
            assert torch.equal(got, res.gather_qmm(x, rhs, ws, lhs)), (fmt, R)
            res.close()
    ws.check()


def test_gather_qmm_weight_cache_gives_the_resident_results(dmoe, orc, ws):
    """dmoe_workspace_set_weight_cache: the unchanged gatherQmm call (borrowed MLX-layout arrays) is served from a
    re-ordered copy the workspace makes on first sight. Same bits as the explicit resident handle, the oracle's values
    within the output tolerance, one copy per stack however often it is called, and dropped when switched off."""
    g = torch.Generator(device="cuda").manual_seed(77)
    stacks = [_stack("affine4", 6, 256, 512, 301), _stack("mxfp4", 5, 128, 256, 302), _stack("affine8", 4, 128, 256, 303)]
    R = 24
    ws.set_weight_cache(True)
    try:
        for rep in range(3):
            for qw in stacks:
                x = torch.randn((R, qw.cols), generator=g, device="cuda").to(torch.bfloat16)
                rhs = torch.randint(0, qw.n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
                got = dmoe.gather_qmm(x, qw, rhs, ws)
                res = dmoe.ResidentWeight(qw)
                assert torch.equal(got, res.gather_qmm(x, rhs, ws))
                res.close()
                want = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), None)
                assert max_abs_rel(got.float().cpu().numpy(), want) < OUT_TOL
        ws.check()
    finally:
        ws.set_weight_cache(False)
    qw = stacks[0]
    x = torch.randn((R, qw.cols), generator=g, device="cuda").to(torch.bfloat16)
    rhs = torch.randint(0, qw.n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
    plain = dmoe.gather_qmm(x, qw, rhs, ws)       # cache off again: the MLX-layout path, same values
    want = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), None)
    assert max_abs_rel(plain.float().cpu().numpy(), want) < OUT_TOL


def test_gather_qmm_weight_cache_invalidate_and_cap(dmoe, orc, ws):
    """A stack rewritten in place keeps its pointers, so the cache cannot tell: it serves the old copy until the
    caller invalidates that stack, after which the call sees the new bytes. The byte cap pushes out the least recently
    used copies; results stay right throughout."""
    g = torch.Generator(device="cuda").manual_seed(5)
    qw = _stack("affine4", 4, 128, 512, 401)
    other = _stack("mxfp4", 3, 128, 512, 402)
    R = 16
    x = torch.randn((R, qw.cols), generator=g, device="cuda").to(torch.bfloat16)
    rhs = torch.randint(0, 3, (R,), generator=g, device="cuda", dtype=torch.int32)
    ws.set_weight_cache(True)
    try:
        old = dmoe.gather_qmm(x, qw, rhs, ws)
        dmoe.gather_qmm(x, other, rhs, ws)
        assert ws.weight_cache_stats()[1] == 2
        fresh = _stack("affine4", 4, 128, 512, 403)
        qw.w.copy_(fresh.w), qw.scales.copy_(fresh.scales), qw.biases.copy_(fresh.biases)   # same addresses, new values
        want_new = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), None)
        stale = dmoe.gather_qmm(x, qw, rhs, ws)
        assert torch.equal(stale, old)                           # what the documentation warns about
        ws.invalidate_weight_cache(qw)
        assert ws.weight_cache_stats()[1] == 1                   # only that stack's copy went
        got = dmoe.gather_qmm(x, qw, rhs, ws)
        assert max_abs_rel(got.float().cpu().numpy(), want_new) < OUT_TOL
        assert not torch.equal(got, old)
        held, n = ws.weight_cache_stats()
        assert n == 2 and held > 0
        # cap below two copies: adding a third stack leaves only the most recent ones that fit
        ws.set_weight_cache_limit(held)
        third = _stack("affine8", 2, 128, 512, 404)
        got3 = dmoe.gather_qmm(x, third, rhs % 2, ws)
        want3 = orc.gather_qmm(bf16_bits(x), qmat(third), to_np_u32(rhs % 2), None)
        assert max_abs_rel(got3.float().cpu().numpy(), want3) < OUT_TOL
        held3, n3 = ws.weight_cache_stats()
        assert held3 <= held and 1 <= n3 <= 2
        again = dmoe.gather_qmm(x, qw, rhs, ws)                  # possibly re-made: same bits either way
        assert torch.equal(again, got)
        ws.invalidate_weight_cache()
        assert ws.weight_cache_stats() == (0, 0)
        ws.check()
    finally:
        ws.set_weight_cache_limit(32 << 30)
        ws.set_weight_cache(False)


@pytest.mark.parametrize("fmt", FORMATS)
def test_gather_qmm_seeded_random_shapes(dmoe, orc, ws, fmt):
    """Twelve seeded shapes per format across both paths and both layouts: odd expert counts, weight rows that are
    not a multiple of the 32-row blocks, reductions from one to 24 granules, row counts on either side of the
    decode / prefill threshold, with and without a row gather."""
    rng = np.random.default_rng(sum(map(ord, fmt)))
    for case in range(12):
        n_mats = int(rng.integers(1, 13))
        rows = 4 * int(rng.integers(2, 81)) if case % 3 else 32 * int(rng.integers(1, 9))
        cols = 128 * int(rng.integers(1, 13)) if fmt == "affine4g128" else 64 * int(rng.integers(1, 25))
        R = int(rng.integers(1, 40)) if case % 2 else int(rng.integers(16 * n_mats + 1, 16 * n_mats + 600))
        qw = _stack(fmt, n_mats, rows, cols, 100 + case)
        g = torch.Generator(device="cuda").manual_seed(case)
        x = torch.randn((R + 2, cols), generator=g, device="cuda").to(torch.bfloat16)
        rhs = torch.randint(0, n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
        lhs = torch.randint(0, R + 2, (R,), generator=g, device="cuda", dtype=torch.int32) if case % 4 == 0 else None
        want = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), None if lhs is None else to_np_u32(lhs))
        got = dmoe.gather_qmm(x, qw, rhs, ws, lhs).float().cpu().numpy()
        assert max_abs_rel(got, want) < OUT_TOL, (fmt, "MLX layout", n_mats, rows, cols, R, max_abs_rel(got, want))
        res = dmoe.ResidentWeight(qw)
        got_r = res.gather_qmm(x, rhs, ws, lhs).float().cpu().numpy()
        res.close()
        assert max_abs_rel(got_r, want) < OUT_TOL, (fmt, "resident", n_mats, rows, cols, R, max_abs_rel(got_r, want))


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("R", [9, 16, 17, 29, 32])
def test_gather_qmm_one_expert_takes_every_row(dmoe, orc, ws, fmt, R):
    """Small-M path with a single tile of 9..32 rows (activations restaged span by span) beside empty experts."""
    n_mats, rows, cols = 4, 160, 2048
    qw = _stack(fmt, n_mats, rows, cols, 5)
    g = torch.Generator(device="cuda").manual_seed(R)
    x = torch.randn((R, cols), generator=g, device="cuda").to(torch.bfloat16)
    rhs = torch.full((R,), 2, device="cuda", dtype=torch.int32)
    got = dmoe.gather_qmm(x, qw, rhs, ws, None).float().cpu().numpy()
    want = orc.gather_qmm(bf16_bits(x), qmat(qw), to_np_u32(rhs), None)
    assert max_abs_rel(got, want) < OUT_TOL, (fmt, R, max_abs_rel(got, want))


def _adversarial_affine(bits, n_mats, rows, cols, seed):
    """Random codes with HAND-SET bf16 scales and biases: every group takes one of seven relations between the bias b
    and the scale s that a min/max quantizer never produces together: b = 0, |b| = s / 256, b = +3 s, |b| = 100 s,
    b = -7.5 s (the usual case, for contrast), b = -s, and a negative scale with a positive bias. Scales are
    (1 + m / 128) 2^e with all eight significant bits in use."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    n_groups = cols // 64
    codes = torch.randint(0, 2 ** bits, (n_mats, rows, cols), generator=g, device="cuda")
    mant = torch.randint(0, 128, (n_mats, rows, n_groups), generator=g, device="cuda").float()
    expo = torch.randint(-9, -5, (n_mats, rows, n_groups), generator=g, device="cuda").float()
    s = ((1.0 + mant / 128.0) * torch.exp2(expo)).to(torch.bfloat16)
    kind = (torch.arange(n_groups, device="cuda")[None, None, :] + torch.arange(rows, device="cuda")[None, :, None]) % 7
    sf = s.float()
    b = torch.zeros_like(sf)
    b = torch.where(kind == 1, -sf / 256.0, b)
    b = torch.where(kind == 2, 3.0 * sf, b)
    b = torch.where(kind == 3, -100.0 * sf, b)
    b = torch.where(kind == 4, -7.5 * sf, b)
    b = torch.where(kind == 5, -sf, b)
    s = torch.where(kind == 6, -sf, sf).to(torch.bfloat16)
    b = torch.where(kind == 6, 11.0 * sf, b).to(torch.bfloat16)
    return QWeight(Q._pack_codes(codes, bits), s, b, rows, cols, QUANT_AFFINE, bits, 64)


@pytest.mark.parametrize("bits", [4, 8])
def test_affine_decode_on_adversarial_scales_and_biases(dmoe, orc, ws, bits):
    """The in-kernel affine decode (prefill kernels: (1024 + c) s + (b - 1024 s) through an f16 magic number; decode
    kernel: scales factored out of the matrix product) on scale / bias pairs for which b - 1024 s is NOT exactly
    representable in f32, on zero and positive biases and on biases far above the scale. dmoe_dequantize must give
    the oracle's bits; every GEMM path must stay within the output bar of the oracle; and the prefill and the decode
    kernels, fed the same rows, must agree to two bf16 steps of the value (plus accumulation-order noise). Two, not
    one: the prefill kernels multiply bf16-rounded weights (the values of dmoe_dequantize), the 4-bit decode kernel
    factors the scale out of the matrix product and never rounds a weight, and where |b| = 100 |s| that rounding is a
    fifth of a code step per weight."""
    n_mats, rows, cols = 3, 128, 1024
    qw = _adversarial_affine(bits, n_mats, rows, cols, 40 + bits)
    qm = qmat(qw)
    for m in range(n_mats):
        want_bits = orc.dequantize(qm, m)
        np.testing.assert_array_equal(bf16_bits(dmoe.dequantize(qw, m)), want_bits)
        # the decoder fused into the prefill kernels: the same bits, also where b - 1024 s would not be representable
        np.testing.assert_array_equal(bf16_bits(dmoe.dequantize(qw, m, fused=True)), want_bits)
    g = torch.Generator(device="cuda").manual_seed(bits)
    R = 16 * n_mats + 400                                 # prefill-sized: the matrix-core kernels
    x = torch.randn((R, cols), generator=g, device="cuda").to(torch.bfloat16)
    rhs = torch.randint(0, n_mats, (R,), generator=g, device="cuda", dtype=torch.int32)
    want = orc.gather_qmm(bf16_bits(x), qm, to_np_u32(rhs), None)
    res = dmoe.ResidentWeight(qw)
    big = {"resident": res.gather_qmm(x, rhs, ws), "mlx": dmoe.gather_qmm(x, qw, rhs, ws)}
    for name, got in big.items():
        err = max_abs_rel(got.float().cpu().numpy(), want)
        assert err < OUT_TOL, (bits, "prefill kernels", name, err)
    # the same rows in decode-sized calls (8 rows per matrix at most): the weight-streaming kernel
    step = 8 * n_mats
    small = {"resident": [], "mlx": []}
    for r0 in range(0, 3 * step, step):
        small["resident"].append(res.gather_qmm(x[r0:r0 + step].contiguous(), rhs[r0:r0 + step].contiguous(), ws))
        small["mlx"].append(dmoe.gather_qmm(x[r0:r0 + step].contiguous(), qw, rhs[r0:r0 + step].contiguous(), ws))
    top = float(np.abs(want).max())
    for name in small:
        got = torch.cat(small[name]).float().cpu().numpy()
        err = max_abs_rel(got, want[:3 * step])
        assert err < OUT_TOL, (bits, "decode kernel", name, err)
        ref = big[name][:3 * step].float().cpu().numpy()
        gap = np.abs(got - ref)
        allowed = np.maximum(np.abs(got), np.abs(ref)) * 2.0 ** -6 + 1e-3 * top
        assert (gap <= allowed).all(), (bits, name, "prefill and decode kernels differ by more than two bf16 steps",
                                        float((gap - allowed).max()))
    res.close()
    ws.check()


def _route(dmoe, orc, wl):
    idx, w = dmoe.gate_route(wl.scores, wl.bias, wl.resident_mask, wl.K, wl.renorm, wl.route_scale)
    want_idx, want_w = orc.gate_route(wl.scores.cpu().numpy(), None if wl.bias is None else wl.bias.cpu().numpy(),
                                      None if wl.resident_mask is None else wl.resident_mask.cpu().numpy(),
                                      wl.K, wl.renorm, wl.route_scale)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    return idx, w, want_idx, want_w


def _check_layer(dmoe, orc, ws, wl, check_h=True):
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap)
    idx, w, want_idx, want_w = _route(dmoe, orc, wl)
    out = layer.forward(wl.x, idx, w, ws)
    slots = want_idx if wl.remap is None else orc.remap(np.array(wl.remap, np.int32), want_idx)
    want, want_h = oracle_forward(wl, slots, want_w, want_h=True)
    err = max_abs_rel(out.float().cpu().numpy(), want)
    assert err < OUT_TOL, (wl.name, err)
    # the same measure row by row (each token against its own largest output), so that no row hides behind the
    # largest row of the tensor; two bf16 roundings of the row maximum on either side leave room for 2e-2
    err_rows = max_abs_rel_rows(out.float().cpu().numpy(), want)
    assert err_rows < ROW_TOL, (wl.name, "per-row", err_rows)
    if check_h:
        h = layer.last_activations(wl.T, ws).float().cpu().numpy()
        scale = want_w.reshape(-1, 1) if wl.score_before_down else 1.0
        # an intermediate, not an output: the oracle rounds sigmoid, silu and the product to bf16 one by
        # one, the kernel rounds once, so the bar here is two bf16 roundings wider than OUT_TOL
        err_h = max_abs_rel(h, want_h * scale)
        assert err_h < 2e-2, (wl.name, "activations", err_h)
    print(f"[parity] {wl.name}: T={wl.T} out max-abs-rel {err:.3e} per-row {err_rows:.3e}")
    # one call from the gate scores on gives the same bytes as route + forward
    out2, idx2, w2 = layer.layer_forward(wl.x, wl.scores, wl.bias, wl.resident_mask, wl.renorm, wl.route_scale, ws,
                                         want_routing=True)
    assert torch.equal(out2, out) and torch.equal(idx2, idx) and torch.equal(w2, w)
    layer.close()
    return err


def test_c0_small_layer_full_size(dmoe, orc, ws):
    """Benchmark configuration 0 at its real size: 16 tokens, D=1024, E=8, top-2, F=2048, affine-4 g64, softmax scores
    renormalised over the top-k (MoERouter.topkRoute)."""
    wl = workloads.make(0)
    idx, w = dmoe.topk_route(wl.scores, wl.K, True)
    want_idx, want_w = orc.topk_route(wl.scores.cpu().numpy(), wl.K, True)
    np.testing.assert_array_equal(to_np_u32(idx), want_idx)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down)
    out = layer.forward(wl.x, idx, w, ws)
    want = oracle_forward(wl, want_idx, want_w)
    assert max_abs_rel(out.float().cpu().numpy(), want) < OUT_TOL
    # MoERouter surface: expand -> (expert fn) -> reduce reproduces the same layer output
    y = layer.forward_no_scores(wl.x, idx, ws)                       # [T, K, D]
    red = dmoe.reduce_experts(y.reshape(wl.T * wl.K, wl.D), w)
    assert max_abs_rel(red.cpu().numpy(), want) < OUT_TOL
    layer.close()


@pytest.mark.parametrize("config,scale", [(1, 0.0625), (1, 0.125), (1, 0.5), (2, 0.0625), (2, 0.125), (2, 0.5), (3, 0.125),
                                          (4, 0.125)])
def test_configs_reduced_size(dmoe, orc, ws, config, scale):
    """Configurations 1-4 with E, D, F shrunk (same formats, routing rules and raggedness). Scales 0.5 and 0.125 keep
    the decode configurations on the small-M kernel (at most 16 rows per expert on average), 0.0625 (16 experts) puts
    them on the MFMA kernel."""
    wl = workloads.make(config, scale=scale)
    _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("before", [False, True])
def test_score_position_variants(dmoe, orc, ws, before):
    wl = workloads.make(1, scale=0.125)
    wl.score_before_down = before
    _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("config", [1, 2])
@pytest.mark.parametrize("limit,shared_limit,before", [(0.05, 0.0, False), (0.05, 0.02, True), (0.0, 0.05, True)])
def test_shared_expert_inside_the_routed_launches(dmoe, orc, ws, config, limit, shared_limit, before):
    """Decode sizes with a shared expert of the routed experts' format: its rows ride in the routed GEMM launches as
    an always-on expert. Limits small enough to clamp, different for routed and shared rows; with the routing weight
    before the down projection the shared rows must stay unscaled."""
    wl = workloads.make(config, scale=0.25)
    wl.swiglu_limit, wl.shared_swiglu_limit, wl.score_before_down = limit, shared_limit, before
    _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("config,T", [(1, 300), (2, 700)])
def test_prefill_sized_batch_with_4bit_shared_expert(dmoe, orc, ws, config, T):
    """A prefill-sized batch on the decode configurations: routed experts AND the dense shared expert (4-bit) on the
    256-row matrix-core kernel, the latter in its dense mode (no tile list); 300 and 700 rows leave a partial tile."""
    wl = workloads.make(config, scale=0.125)
    g = torch.Generator(device="cuda").manual_seed(11)
    wl.T = T
    wl.x = torch.randn((T, wl.D), generator=g, device="cuda").to(torch.bfloat16)
    wl.scores = torch.sigmoid(torch.randn((T, wl.E_total), generator=g, device="cuda"))
    _check_layer(dmoe, orc, ws, wl)


def test_c1_decode_full_size(dmoe, orc, ws):
    """Benchmark configuration 1 at full size (64 x 1 tokens, D=4096, 256 experts top-6 + shared, F=2048, affine-4)."""
    wl = workloads.make(1)
    _check_layer(dmoe, orc, ws, wl, check_h=True)


def test_c2_decode_mxfp4_smelt_full_size(dmoe, orc, ws):
    wl = workloads.make(2)
    assert wl.E == 51 and int(wl.resident_mask.sum()) == 51
    _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("config", [3, 4])
def test_prefill_configs_full_size(dmoe, orc, ws, config):
    """Benchmark configurations 3 (8192-token ragged prefill, Zipf routing, affine-4) and 4 (2080-token mixed batch, affine-8
    routed + FP8 shared expert) at full size. Routing and packing are compared bit for bit with the oracle on the
    whole batch. The oracle's FFN would take minutes on 49 152 rows, so the outputs are pinned two ways that do not
    depend on the batch size: a sample of 64 tokens (the rows of the most and of the least loaded experts, the
    first and last tokens, random ones) against the oracle at full D, F and E, and the same 64 tokens run alone,
    which takes the decode kernels instead of the prefill ones and must give the same rows."""
    import copy
    wl = workloads.make(config)
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit,
                       score_before_down=wl.score_before_down, shared=wl.shared,
                       shared_swiglu_limit=wl.shared_swiglu_limit, remap=wl.remap)
    idx, w, want_idx, want_w = _route(dmoe, orc, wl)
    got = dmoe.pack(idx, wl.E, ws)
    want = orc.pack(want_idx, wl.E)
    for name in ("order", "inv", "token", "sorted_e", "counts", "offsets"):
        np.testing.assert_array_equal(to_np_u32(got[name]), want[name], err_msg=name)
    counts = want["counts"].astype(np.int64)
    assert counts.sum() == wl.T * wl.K
    out = layer.forward(wl.x, idx, w, ws)
    assert out.shape == (wl.T, wl.D) and bool(torch.isfinite(out.float()).all())

    rng = np.random.default_rng(config)
    live = np.nonzero(counts)[0]
    heavy, light = live[np.argmax(counts[live])], live[np.argmin(counts[live])]
    tok_of = lambda e: np.nonzero((want_idx == e).any(axis=1))[0]
    pick = np.concatenate([tok_of(heavy)[:16], tok_of(light)[:8], [0, 1, wl.T - 2, wl.T - 1],
                           rng.integers(0, wl.T, 64)])
    sample = np.unique(pick)[:64]
    sel = torch.from_numpy(sample).to("cuda")
    sub = copy.copy(wl)
    sub.x, sub.T = wl.x[sel].contiguous(), len(sample)
    want_out = oracle_forward(sub, want_idx[sample], want_w[sample])
    got_out = out[sel].float().cpu().numpy()
    err = max_abs_rel(got_out, want_out)
    assert err < OUT_TOL, (wl.name, "sample against the oracle", err)
    alone = layer.forward(sub.x, idx[sel].contiguous(), w[sel].contiguous(), ws).float().cpu().numpy()
    err_alone = max_abs_rel(alone, want_out)
    assert err_alone < OUT_TOL, (wl.name, "sample run alone against the oracle", err_alone)
    err_paths = max_abs_rel(alone, got_out)
    assert err_paths < OUT_TOL, (wl.name, "prefill kernels against decode kernels", err_paths)
    print(f"[parity] {wl.name}: T={wl.T} rows/expert max {counts.max()} min {counts[live].min()} "
          f"sample err {err:.3e}, alone {err_alone:.3e}, prefill vs decode {err_paths:.3e}")
    layer.close()


@pytest.mark.parametrize("config,scale", [(1, 0.25), (3, 0.125), (4, 0.25)])
def test_unquantized_experts_layer(dmoe, orc, ws, config, scale):
    """A layer whose experts (and shared expert) are plain bf16 matrices: the float arm of dispatchGatherMm
    (deepseek_v4.zig:978, ops.gatherMm) and of DSV4Expert.expertMatmul, at a decode and at two prefill sizes."""
    wl = workloads.make(config, scale=scale)
    wl.gate, wl.up = _stack("bf16", wl.E, wl.F, wl.D, 21), _stack("bf16", wl.E, wl.F, wl.D, 22)
    wl.down = _stack("bf16", wl.E, wl.D, wl.F, 23)
    if wl.shared is not None:
        wl.shared = (_stack("bf16", 1, wl.F, wl.D, 24), _stack("bf16", 1, wl.F, wl.D, 25), _stack("bf16", 1, wl.D, wl.F, 26))
    _check_layer(dmoe, orc, ws, wl)


def test_unquantized_tiny_model_shape(dmoe, orc, ws):
    """The shape of the reference's own DSV4 smoke tests (src/tests/deepseek_v4_tests.zig:398-610): 2 experts, top-2,
    D=16, F=8, float weights. All-zero weights must give zeros (finite); random ones must match the oracle. F=8 makes
    the down projection's reduction half an MFMA step, D=16 keeps the weights in their row-major layout."""
    E, K, D, F, T = 2, 2, 16, 8, 5
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
    idx = torch.tensor([[0, 1], [1, 0], [0, 1], [1, 0], [0, 1]], dtype=torch.int32, device="cuda")
    w = torch.full((T, K), 0.5, dtype=torch.float32, device="cuda")
    zeros = lambda r, c: QWeight(torch.zeros((E, r, c), dtype=torch.bfloat16, device="cuda"), None, None, r, c, QUANT_NONE, 16, 0)
    layer = dmoe.Layer(D, F, K, zeros(F, D), zeros(F, D), zeros(D, F))
    out = layer.forward(x, idx, w, ws)
    assert out.shape == (T, D) and bool((out == 0).all())
    layer.close()
    gate, up, down = _stack("bf16", E, F, D, 31), _stack("bf16", E, F, D, 32), _stack("bf16", E, D, F, 33)
    for q in (gate, up, down):
        q.w *= 40.0  # N(0, 0.8): outputs well above the bf16 rounding of a 16-term sum
    layer = dmoe.Layer(D, F, K, gate, up, down)
    out = layer.forward(x, idx, w, ws).float().cpu().numpy()
    want = orc.moe_forward(bf16_bits(x), to_np_u32(idx), w.cpu().numpy(), qmat(gate), qmat(up), qmat(down))
    assert max_abs_rel(out, want) < OUT_TOL, max_abs_rel(out, want)
    layer.close()


@pytest.mark.parametrize("fmt", ["affine4", "mxfp4", "affine8", "bf16"])
def test_layer_seeded_random_shapes(dmoe, orc, ws, fmt):
    """Eight seeded layers per routed format: hidden / FFN sizes in steps of 64, 2..40 experts, top-1..8, 1..600
    tokens (both GEMM paths), no shared expert or one in the routed format, FP8 or 4-bit affine, either position of
    the routing weight, with and without the SwiGLU limits and a selection bias."""
    rng = np.random.default_rng(sum(map(ord, fmt)) + 1)
    for case in range(8):
        D, F = 64 * int(rng.integers(2, 17)), 64 * int(rng.integers(2, 13))
        E = int(rng.integers(2, 41))
        K = int(rng.integers(1, min(E, 8) + 1))
        T = int(rng.integers(1, 33)) if case % 2 else int(rng.integers(33, 601))
        g = torch.Generator(device="cuda").manual_seed(1000 + case)
        x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
        scores = torch.sigmoid(torch.randn((T, E), generator=g, device="cuda"))
        bias = torch.randn((E,), generator=g, device="cuda") * 0.1 if case % 3 == 0 else None
        sfmt = [None, fmt, "fp8row", "affine4"][case % 4]
        shared = None if sfmt is None else (_stack(sfmt, 1, F, D, 70 + case), _stack(sfmt, 1, F, D, 80 + case),
                                            _stack(sfmt, 1, D, F, 90 + case))
        wl = workloads.Workload(f"random {fmt} #{case}", T, D, F, E, E, K, x, scores, bias, None, None, True, 1.5,
                                _stack(fmt, E, F, D, 40 + case), _stack(fmt, E, F, D, 50 + case),
                                _stack(fmt, E, D, F, 60 + case), shared,
                                swiglu_limit=7.0 if case % 2 else 0.0, shared_swiglu_limit=3.0 if case % 4 == 1 else 0.0,
                                score_before_down=bool(case & 4))
        _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("fmt,T", [("affine4", 24), ("affine4", 330), ("mxfp4", 330)])
def test_layer_with_a_hidden_size_that_is_not_a_power_of_two(dmoe, orc, ws, fmt, T):
    """D = 7168 (112 reduction steps of 64: not a multiple of the kernels' ring rounds, unroll trips or span counts), F =
    2048, 16 experts top-4 with a shared expert: the decode kernel at 24 tokens (6 rows per expert, partial last round),
    the matrix-core kernels at 330 (82 rows per expert, 28 whole trips of the activation ring)."""
    D, F, E, K = 7168, 2048, 16, 4
    g = torch.Generator(device="cuda").manual_seed(7000 + T)
    x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
    scores = torch.sigmoid(torch.randn((T, E), generator=g, device="cuda"))
    shared = (_stack(fmt, 1, F, D, 711), _stack(fmt, 1, F, D, 712), _stack(fmt, 1, D, F, 713))
    wl = workloads.Workload(f"D=7168 {fmt} T={T}", T, D, F, E, E, K, x, scores, None, None, None, True, 2.5,
                            _stack(fmt, E, F, D, 701), _stack(fmt, E, F, D, 702), _stack(fmt, E, D, F, 703), shared,
                            swiglu_limit=7.0)
    _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("fmt", ["affine4", "affine4g32", "affine4g128", "affine8", "mxfp4", "fp8row", "bf16"])
def test_single_sequence_decode_step(dmoe, orc, ws, fmt):
    """Steps of at most 8 sorted rows (one or two sequences): the weight-streaming kernel splits every tile's
    reduction over two groups of wavefronts that meet in LDS. D = 2048 and F = 1024 are whole ring rounds per half
    for every format, so the split kernel runs; D = 1536 is not (its steps do not halve into whole rounds for the
    4-bit formats) and takes the unsplit kernel on the same rows. With a shared expert of the routed format (it rides
    in the routed launch as one more row per token), of another format (a launch of its own), and none; both
    positions of the routing weight; SwiGLU limits that clamp a fifth of the values (gate and up values have a
    standard deviation of 0.9 here; limits far below that would shrink the activations, against which their error is
    measured, a hundredfold while the 8-bit and the unfactored 4-bit decoders' bf16 weight rounding stays what it is)."""
    E = 12
    case = 0
    for D, F in ((2048, 1024), (1536, 1024)):
        routed = (_stack(fmt, E, F, D, 9001), _stack(fmt, E, F, D, 9002), _stack(fmt, E, D, F, 9003))
        for T, K in ((1, 6), (1, 8), (2, 3), (2, 4), (3, 2)):
            for sfmt in (fmt, None, "fp8row" if fmt != "fp8row" else "affine8"):
                case += 1
                if T * K + (T if sfmt == fmt else 0) > 8 and D != 2048:
                    continue
                g = torch.Generator(device="cuda").manual_seed(9100 + case)
                x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
                scores = torch.sigmoid(torch.randn((T, E), generator=g, device="cuda"))
                shared = None if sfmt is None else (_stack(sfmt, 1, F, D, 9200 + case), _stack(sfmt, 1, F, D, 9300 + case),
                                                    _stack(sfmt, 1, D, F, 9400 + case))
                wl = workloads.Workload(f"single sequence {fmt} D={D} T={T} K={K} shared={sfmt}", T, D, F, E, E, K, x,
                                        scores, None, None, None, True, 1.5, *routed, shared,
                                        swiglu_limit=1.0 if case % 2 else 0.0, shared_swiglu_limit=0.5 if case % 3 == 0 else 0.0,
                                        score_before_down=bool(case % 4 < 2))
                _check_layer(dmoe, orc, ws, wl)


@pytest.mark.parametrize("fmt,D,F,E,K,T", [("bf16", 512, 512, 4, 2, 64),      # 32-row tiles over an 8 KiB activation window
                                           ("bf16", 256, 256, 4, 2, 1),       # one sequence: split reduction, 4 KiB window
                                           ("affine4", 128, 256, 8, 2, 8),    # a 2 KiB window
                                           ("affine4", 192, 128, 8, 2, 3),
                                           ("affine8", 64, 64, 4, 2, 5),      # 1 KiB
                                           ("mxfp4", 1024, 64, 4, 2, 40)])    # down projection: a reduction of one step
def test_short_reduction_dimensions(dmoe, orc, ws, fmt, D, F, E, K, T):
    """Hidden / FFN sizes so small that the activations of a tile take less LDS than the sums the wavefronts exchange
    once the reduction is done (up to 16 KiB for a 32-row gate/up tile): the exchange must still have its room. With
    and without a shared expert riding in the routed launch."""
    g = torch.Generator(device="cuda").manual_seed(D + F + T)
    x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
    scores = torch.sigmoid(torch.randn((T, E), generator=g, device="cuda"))
    for with_shared in (False, True):
        shared = (_stack(fmt, 1, F, D, 61), _stack(fmt, 1, F, D, 62), _stack(fmt, 1, D, F, 63)) if with_shared else None
        wl = workloads.Workload(f"short reduction {fmt} D={D} F={F} T={T} shared={with_shared}", T, D, F, E, E, K, x, scores,
                                None, None, None, True, 1.5, _stack(fmt, E, F, D, 51), _stack(fmt, E, F, D, 52),
                                _stack(fmt, E, D, F, 53), shared)
        for q in (wl.gate, wl.up, wl.down):
            if fmt == "bf16":
                q.w *= 4.0   # outputs well above the bf16 rounding of the short sums
        _check_layer(dmoe, orc, ws, wl)


def test_forward_edge_cases(dmoe, orc, ws):
    wl = workloads.make(1, scale=0.125)
    layer = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit, shared=wl.shared)
    # empty batch: nothing enqueued, no error
    empty = layer.forward(wl.x[:0], torch.empty((0, wl.K), dtype=torch.int32, device="cuda"),
                          torch.empty((0, wl.K), dtype=torch.float32, device="cuda"), ws)
    assert empty.shape == (0, wl.D)
    # every token on the same K experts (maximally unbalanced segments)
    T = 40
    idx = torch.arange(wl.K, dtype=torch.int32, device="cuda").repeat(T, 1)
    w = torch.full((T, wl.K), 1.0 / wl.K, device="cuda")
    x = wl.x[:T].contiguous()
    out = layer.forward(x, idx, w, ws)
    wl.x, wl.T = x, T
    want = oracle_forward(wl, to_np_u32(idx), w.cpu().numpy())
    assert max_abs_rel(out.float().cpu().numpy(), want) < OUT_TOL
    # a single token
    out1 = layer.forward(x[:1].contiguous(), idx[:1].contiguous(), w[:1].contiguous(), ws)
    assert max_abs_rel(out1.float().cpu().numpy(), want[:1]) < OUT_TOL
    # bad arguments are rejected with a message, nothing is launched
    with pytest.raises(dmoe.DmoeError):
        dmoe.topk_route(wl.scores, 2000, True)
    with pytest.raises(dmoe.DmoeError):
        dmoe.Layer(wl.D, wl.F + 8, wl.K, wl.gate, wl.up, wl.down)
    layer.close()


def test_mfma_calibration_loop_counts_what_it_claims(dmoe):
    """The benchmark's matrix-core calibration (dmoe_debug_mfma_loop) reports flops as iterations x a constant: with
    every operand 1.0 each of a lane's 128 accumulators grows by 16 per instruction and 64 per iteration, so the lane
    checksum must be 128 x 64 x iters exactly, i.e. the loop really issues 32 instructions of k = 16 per iteration."""
    ones = torch.ones((dmoe.MFMA_LOOP_OPERANDS,), dtype=torch.bfloat16, device="cuda")
    for iters in (1, 3):
        out = dmoe.mfma_loop(ones, iters)
        torch.cuda.synchronize()
        assert out.shape == (dmoe.MFMA_LOOP_OUT,)
        assert torch.equal(out, torch.full_like(out, 128.0 * 64.0 * iters))
    assert dmoe.MFMA_LOOP_FLOP_PER_ITER == 512 * 4 * 32 * 2.0 * 32 * 32 * 16
    with pytest.raises(dmoe.DmoeError, match="iters"):
        dmoe.mfma_loop(ones, 0)


def test_read_stream_calibration_reads_what_it_reports(dmoe):
    """dmoe_debug_read_stream reports the bytes one launch reads: whole 8 KiB chunks per wavefront, never past the
    buffer, and each wavefront's checksum is the XOR of exactly its own part."""
    wgs, chunk = 3, 8192
    n = 4 * wgs * 2 * chunk + 5000                       # two chunks per wavefront and a ragged rest that is not read
    src = torch.randint(0, 2 ** 31 - 1, (n // 4,), dtype=torch.int32, device="cuda")
    sink = torch.zeros((4 * wgs,), dtype=torch.int32, device="cuda")
    got = dmoe.read_stream(src, wgs, sink)
    torch.cuda.synchronize()
    assert got == 4 * wgs * 2 * chunk
    per_wave = src[: got // 4].view(4 * wgs, -1).cpu().numpy()
    import numpy as np
    want = np.bitwise_xor.reduce(per_wave, axis=1)
    assert np.array_equal(sink.cpu().numpy(), want)
    with pytest.raises(dmoe.DmoeError, match="less than one"):
        dmoe.read_stream(src[:1024], wgs, sink)
