"""ctypes front end of the CPU oracle (oracle/dmoe_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg. The product never imports this module.

All arrays are numpy, C-contiguous. bf16 travels as uint16.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libdmoe_oracle.so")

AFFINE, MXFP4, FP8_ROW, NONE = 0, 1, 2, 3
SCORE_SOFTMAX, SCORE_SIGMOID, SCORE_SQRTSOFTPLUS, SCORE_SQRTSOFTPLUS_STABLE = 0, 1, 2, 3
SMELT_UNIFORM, SMELT_FIRST = 0, 1


def build():
    """Compile the oracle with its Makefile (gcc)."""
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


class _QMat(C.Structure):
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
                ("rows", C.c_int), ("cols", C.c_int),
                ("mode", C.c_int), ("bits", C.c_int), ("group", C.c_int)]


class _Layer(C.Structure):
    _fields_ = [("T", C.c_int), ("D", C.c_int), ("F", C.c_int), ("K", C.c_int), ("E", C.c_int),
                ("gate", _QMat), ("up", _QMat), ("down", _QMat),
                ("swiglu_limit", C.c_float), ("score_before_down", C.c_int),
                ("has_shared", C.c_int),
                ("sh_gate", _QMat), ("sh_up", _QMat), ("sh_down", _QMat),
                ("shared_swiglu_limit", C.c_float)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        srcs = [os.path.join(os.path.dirname(os.path.abspath(__file__)), f) for f in ("dmoe_oracle.c", "dmoe_oracle.h")]
        if not os.path.exists(_LIB_PATH) or any(os.path.getmtime(f) > os.path.getmtime(_LIB_PATH) for f in srcs):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_dequant_value.restype = C.c_float
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
        _lib.orc_bf16_to_f32.restype = C.c_float
        _lib.orc_bf16_to_f32.argtypes = [C.c_uint16]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads():
    return int(lib().orc_num_threads())


def f32_to_bf16(x):
    """Round-to-nearest-even f32 -> bf16 bits (uint16), vectorised twin of orc_f32_to_bf16."""
    u = _c(x, np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_to_f32(h):
    return (_c(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


class QMat:
    """A stack [n, rows, cols] of quantized matrices in MLX layout (numpy-held)."""

    def __init__(self, w, scales, biases, rows, cols, mode, bits, group):
        self.mode, self.bits, self.group, self.rows, self.cols = mode, bits, group, rows, cols
        if mode == NONE:
            self.w = _c(w, np.uint16)
            self.scales = None
            self.biases = None
        elif mode == FP8_ROW:
            self.w = _c(w, np.uint8)
            self.scales = _c(scales, np.float32)
            self.biases = None
        elif mode == MXFP4:
            self.w = _c(w, np.uint32)
            self.scales = _c(scales, np.uint8)
            self.biases = None
        else:
            self.w = _c(w, np.uint32)
            self.scales = _c(scales, np.uint16)
            self.biases = None if biases is None else _c(biases, np.uint16)
        self.n = self.w.shape[0] if self.w.ndim == 3 else 1

    def c(self):
        return _QMat(_p(self.w), _p(self.scales), _p(self.biases), self.rows, self.cols,
                     self.mode, self.bits, self.group)


def bf16_bits(t):
    """A torch bf16 tensor (any device) -> numpy uint16 bit patterns."""
    import torch
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def qmat(qw):
    """A weight stack as the harness holds it (torch tensors `w`, `scales`, `biases` in MLX layout plus `rows`, `cols`,
    `mode`, `bits`, `group_size`; the mode numbers are those of include/dmoe.h) -> QMat over numpy copies."""
    w = qw.w.detach().cpu().contiguous()
    if qw.mode == NONE:
        return QMat(bf16_bits(w), None, None, qw.rows, qw.cols, NONE, 16, 0)
    s = qw.scales.detach().cpu().contiguous()
    b = None if qw.biases is None else qw.biases.detach().cpu().contiguous()
    if qw.mode == FP8_ROW:
        return QMat(w.numpy(), s.numpy(), None, qw.rows, qw.cols, FP8_ROW, 8, 0)
    if qw.mode == MXFP4:
        return QMat(w.numpy().view(np.uint32), s.numpy(), None, qw.rows, qw.cols, MXFP4, 4, 32)
    return QMat(w.numpy().view(np.uint32), bf16_bits(s), None if b is None else bf16_bits(b),
                qw.rows, qw.cols, AFFINE, qw.bits, qw.group_size)


def topk_route(scores, K, normalize=True):
    s = _c(scores, np.float32)
    T, E = s.shape
    idx = np.empty((T, K), np.uint32)
    w = np.empty((T, K), np.float32)
    lib().orc_topk_route(_p(s), T, E, K, int(normalize), _p(idx), _p(w))
    return idx, w


def gate_scores(logits, func):
    x = _c(logits, np.float32)
    T, E = x.shape
    out = np.empty_like(x)
    lib().orc_gate_scores(_p(x), T, E, func, _p(out))
    return out


def gate_logits(x_bf16, wg_bf16):
    """x, wg: uint16 arrays of bf16 bits, [T,D] and [E,D] -> f32 [T,E] (bf16-valued)"""
    x = _c(x_bf16, np.uint16)
    w = _c(wg_bf16, np.uint16)
    T, D = x.shape
    E = w.shape[0]
    out = np.empty((T, E), np.float32)
    lib().orc_gate_logits(_p(x), _p(w), T, D, E, _p(out))
    return out


def gate_scores_det(logits, func):
    x = _c(logits, np.float32)
    T, E = x.shape
    out = np.empty_like(x)
    lib().orc_gate_scores_det(_p(x), T, E, func, _p(out))
    return out


def det_expf(x):
    f = lib().orc_det_expf
    f.restype = C.c_float
    return np.array([f(C.c_float(float(v))) for v in np.asarray(x, np.float32).ravel()], np.float32)


def det_logf(x):
    f = lib().orc_det_logf
    f.restype = C.c_float
    return np.array([f(C.c_float(float(v))) for v in np.asarray(x, np.float32).ravel()], np.float32)


def det_softplusf(x):
    f = lib().orc_det_softplusf
    f.restype = C.c_float
    return np.array([f(C.c_float(float(v))) for v in np.asarray(x, np.float32).ravel()], np.float32)


def gate_route(scores, bias, resident, K, renorm, route_scale):
    s = _c(scores, np.float32)
    T, E = s.shape
    b = None if bias is None else _c(bias, np.float32)
    m = None if resident is None else _c(resident, np.uint8)
    idx = np.empty((T, K), np.uint32)
    w = np.empty((T, K), np.float32)
    lib().orc_gate_route(_p(s), _p(b), _p(m), T, E, K, int(renorm), C.c_float(route_scale),
                         _p(idx), _p(w))
    return idx, w


def gate_hash_route(scores, tid2eid, ids, renorm, route_scale):
    s = _c(scores, np.float32)
    t2e = _c(tid2eid, np.int32)
    i = _c(ids, np.uint32)
    T, E = s.shape
    K = t2e.shape[1]
    idx = np.empty((T, K), np.uint32)
    w = np.empty((T, K), np.float32)
    lib().orc_gate_hash_route(_p(s), _p(t2e), _p(i), T, E, K, int(renorm), C.c_float(route_scale), _p(idx), _p(w))
    return idx, w


def block_post(x_bits, residual_bits, post_mix=None, comb_mix=None):
    """residual add (no mixes) or mhcPost; bf16 bit patterns in and out"""
    x = _c(x_bits, np.uint16)
    r = _c(residual_bits, np.uint16)
    T, D = x.shape
    m = 0 if post_mix is None else r.shape[1]
    out = np.empty_like(r)
    pm = None if post_mix is None else _c(post_mix, np.float32).reshape(T, m)
    cm = None if comb_mix is None else _c(comb_mix, np.float32).reshape(T, m, m)
    lib().orc_block_post(_p(x), _p(r), _p(pm), _p(cm), T, D, m, _p(out))
    return out


def remap(remap_table, idx):
    r = _c(remap_table, np.int32)
    i = _c(idx, np.uint32)
    out = np.empty_like(i)
    lib().orc_remap(_p(r), _p(i), C.c_size_t(i.size), _p(out))
    return out


def smelt_mask(n_experts, load_fraction, strategy=SMELT_UNIFORM, enabled=True):
    m = np.zeros(n_experts, np.uint8)
    n = lib().orc_smelt_mask(n_experts, C.c_float(load_fraction), strategy, int(enabled), _p(m))
    return m, int(n)


def build_remap(mask):
    m = _c(mask, np.uint8)
    out = np.empty(m.size, np.int32)
    lib().orc_build_remap(_p(m), m.size, _p(out))
    return out


def preload_remap(expert_ids, n_total):
    ids = _c(expert_ids, np.uint32)
    r = np.empty(n_total, np.int32)
    cb = np.empty(n_total, np.float32)
    lib().orc_preload_remap(_p(ids), ids.size, n_total, _p(r), _p(cb))
    return r, cb


def dedup(idx, n_experts):
    i = _c(idx, np.uint32)
    uniq = np.empty(n_experts, np.uint32)
    r = np.empty(n_experts, np.int32)
    n = lib().orc_dedup(_p(i), C.c_size_t(i.size), n_experts, _p(uniq), _p(r))
    return uniq[:n].copy(), r


def pack(idx, E):
    i = _c(idx, np.uint32)
    T, K = i.shape
    n = T * K
    order = np.empty(n, np.uint32)
    inv = np.empty(n, np.uint32)
    token = np.empty(n, np.uint32)
    se = np.empty(n, np.uint32)
    counts = np.empty(E, np.uint32)
    offsets = np.empty(E + 1, np.uint32)
    lib().orc_pack(_p(i), T, K, E, _p(order), _p(inv), _p(token), _p(se), _p(counts), _p(offsets))
    return dict(order=order, inv=inv, token=token, sorted_e=se, counts=counts, offsets=offsets)


def expand_tokens(x, K):
    x = _c(x, np.float32)
    T, D = x.shape
    out = np.empty((T * K, D), np.float32)
    lib().orc_expand_tokens(_p(x), T, D, K, _p(out))
    return out


def reduce_experts(expert_outs, w):
    eo = _c(expert_outs, np.float32)
    w = _c(w, np.float32)
    T, K = w.shape
    D = eo.shape[1]
    out = np.empty((T, D), np.float32)
    lib().orc_reduce_experts(_p(eo), _p(w), T, K, D, _p(out))
    return out


def dequantize(qm, mat_index=0):
    out = np.empty((qm.rows, qm.cols), np.uint16)
    c = qm.c()
    lib().orc_dequantize(C.byref(c), mat_index, _p(out))
    return out


def dequant_fp8_block(w, scale, block):
    """w uint8 [rows, cols]; scale float32 or uint8 (E8M0) [ceil(rows/block), ceil(cols/block)] -> uint16 (bf16) [rows, cols]"""
    w = _c(w, np.uint8)
    e8m0 = scale.dtype == np.uint8
    scale = _c(scale, np.uint8 if e8m0 else np.float32)
    rows, cols = w.shape
    assert scale.shape == (-(-rows // block), -(-cols // block)), scale.shape
    out = np.empty((rows, cols), np.uint16)
    lib().orc_dequant_fp8_block(_p(w), _p(scale), int(e8m0), rows, cols, block, _p(out))
    return out


def dequantize_f32(qm, mat_index=0):
    out = np.empty((qm.rows, qm.cols), np.float32)
    c = qm.c()
    lib().orc_dequantize_f32(C.byref(c), mat_index, _p(out))
    return out


def dequant_value(qm, mat_index, row, col):
    c = qm.c()
    return float(lib().orc_dequant_value(C.byref(c), mat_index, row, col))


def gather_qmm(x, qm, rhs, lhs=None):
    """x: uint16 (bf16) or float32 [Rx, cols]; returns f32 [R, rows]."""
    x_is_f32 = x.dtype == np.float32
    x = _c(x, np.float32 if x_is_f32 else np.uint16)
    rhs = _c(rhs, np.uint32).reshape(-1)
    lhs_a = None if lhs is None else _c(lhs, np.uint32).reshape(-1)
    R = rhs.size
    out = np.empty((R, qm.rows), np.float32)
    c = qm.c()
    lib().orc_gather_qmm(_p(x), int(x_is_f32), C.byref(c), _p(lhs_a), _p(rhs), R, _p(out))
    return out


def moe_forward(x, idx, w, gate, up, down, swiglu_limit=0.0, score_before_down=False,
                shared=None, shared_swiglu_limit=0.0, want_h=False):
    """x uint16 [T,D]; idx uint32 [T,K] (slot ids); w f32 [T,K]; gate/up/down QMat stacks;
    shared = (gate, up, down) QMat singles or None. Returns f32 [T,D] (and h f32 [T*K,F])."""
    x = _c(x, np.uint16)
    idx = _c(idx, np.uint32)
    w = _c(w, np.float32)
    T, D = x.shape
    K = idx.shape[1]
    F = gate.rows
    L = _Layer()
    L.T, L.D, L.F, L.K, L.E = T, D, F, K, gate.n
    L.gate, L.up, L.down = gate.c(), up.c(), down.c()
    L.swiglu_limit = swiglu_limit
    L.score_before_down = int(score_before_down)
    L.has_shared = int(shared is not None)
    if shared is not None:
        L.sh_gate, L.sh_up, L.sh_down = shared[0].c(), shared[1].c(), shared[2].c()
    L.shared_swiglu_limit = shared_swiglu_limit
    out = np.empty((T, D), np.float32)
    h = np.empty((T * K, F), np.float32) if want_h else None
    lib().orc_moe_forward(C.byref(L), _p(x), _p(idx), _p(w), _p(out), _p(h))
    return (out, h) if want_h else out


def batch_concat(req_tokens, base_pos):
    n = len(req_tokens)
    arrs = [_c(t, np.uint32) for t in req_tokens]
    lens = np.array([a.size for a in arrs], np.int32)
    total = int(lens.sum())
    ptrs = (C.c_void_p * max(n, 1))(*[a.ctypes.data for a in arrs])
    bp = _c(base_pos, np.int32)
    toks = np.empty(total, np.uint32)
    pos = np.empty(total, np.int32)
    offs = np.empty(n + 1, np.int32)
    lib().orc_batch_concat(ptrs, _p(lens), _p(bp), n, _p(toks), _p(pos), _p(offs))
    return toks, pos, offs


def batch_mask(lens):
    lens = _c(lens, np.int32)
    T = int(lens.sum())
    m = np.empty((T, T), np.float32)
    lib().orc_batch_mask(_p(lens), lens.size, _p(m))
    return m
