"""Shared helpers of the test-suite (conversions between the product's tensors and the oracle's arrays)."""
import numpy as np
import torch

from dmlx_amd import capi
from oracle import oracle


def to_np_u32(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def bf16_bits(t):
    """torch bf16 tensor -> numpy uint16 bit patterns"""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_to_f32(t):
    return t.detach().cpu().float().numpy()


def qmat(qw):
    """capi.QWeight (torch, any device) -> oracle.QMat (numpy)"""
    w = qw.w.detach().cpu().contiguous()
    if qw.mode == capi.QUANT_NONE:
        return oracle.QMat(bf16_bits(w), None, None, qw.rows, qw.cols, oracle.NONE, 16, 0)
    s = qw.scales.detach().cpu().contiguous()
    b = None if qw.biases is None else qw.biases.detach().cpu().contiguous()
    if qw.mode == capi.QUANT_FP8_ROW:
        return oracle.QMat(w.numpy(), s.numpy(), None, qw.rows, qw.cols, oracle.FP8_ROW, 8, 0)
    if qw.mode == capi.QUANT_MXFP4:
        return oracle.QMat(w.numpy().view(np.uint32), s.numpy(), None, qw.rows, qw.cols, oracle.MXFP4, 4, 32)
    return oracle.QMat(w.numpy().view(np.uint32), bf16_bits(s), None if b is None else bf16_bits(b),
                       qw.rows, qw.cols, oracle.AFFINE, qw.bits, qw.group_size)


def max_abs_rel(got, ref):
    """max |got - ref| / max |ref|: the error measure of the 1e-2 output bar."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    denom = np.abs(ref).max()
    return float(np.abs(got - ref).max() / (denom if denom > 0 else 1.0))


def oracle_forward(wl, idx_slots, weights, want_h=False):
    """Run the oracle's MoE forward on a Workload with given slot indices / weights (numpy)."""
    shared = None if wl.shared is None else tuple(qmat(q) for q in wl.shared)
    return oracle.moe_forward(bf16_bits(wl.x), idx_slots, weights, qmat(wl.gate), qmat(wl.up), qmat(wl.down),
                              swiglu_limit=wl.swiglu_limit, score_before_down=wl.score_before_down,
                              shared=shared, shared_swiglu_limit=wl.shared_swiglu_limit, want_h=want_h)


def max_abs_rel_rows(got, ref):
    """Largest per-row error: max over rows of (max |got - ref| over the row) / (max |ref| over the row)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    denom = np.abs(ref).max(axis=-1)
    denom[denom == 0] = 1.0
    return float((np.abs(got - ref).max(axis=-1) / denom).max())


def dense_reference_f64(x_bits, idx, w, gate, up, down, limit=0.0, shared=None, shared_limit=0.0):
    """The layer in float64 with no intermediate rounding: sum_k w[t,k] * down_e(silu(min(g, L)) * clip(u, -L, L)) +
    shared(x), from the dequantized weights (oracle.QMat stacks; idx = slot ids). Rows are grouped by expert so that
    each expert is dequantized once; this is the exact value both the kernels and the oracle approximate."""
    x = oracle.bf16_to_f32(x_bits).astype(np.float64)
    T, K = idx.shape

    def ffn(xr, g_, u_, d_, L):          # xr [n, D]
        g, u = xr @ g_.T, xr @ u_.T
        if L > 0:
            g, u = np.minimum(g, L), np.clip(u, -L, L)
        return (g / (1.0 + np.exp(-g)) * u) @ d_.T

    deq = lambda qm, m: oracle.dequantize_f32(qm, m).astype(np.float64)
    out = np.zeros((T, down.rows))
    flat = idx.reshape(-1).astype(np.int64)
    for e in np.unique(flat):
        pos = np.nonzero(flat == e)[0]
        tok = pos // K
        y = ffn(x[tok], deq(gate, int(e)), deq(up, int(e)), deq(down, int(e)), limit)
        np.add.at(out, tok, y * w.reshape(-1)[pos].astype(np.float64)[:, None])
    if shared is not None:
        out += ffn(x, deq(shared[0], 0), deq(shared[1], 0), deq(shared[2], 0), shared_limit)
    return out
