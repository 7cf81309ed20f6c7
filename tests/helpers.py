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
