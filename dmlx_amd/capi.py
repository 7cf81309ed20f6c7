"""ctypes binding of libdmoe.so (include/dmoe.h) for Python callers.

PyTorch is used only as the owner of device memory and streams: every call passes
raw device pointers (tensor.data_ptr()) and the current HIP stream to the C ABI.
There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdmoe.so")

QUANT_AFFINE, QUANT_MXFP4, QUANT_FP8_ROW, QUANT_NONE = 0, 1, 2, 3
WEIGHTS_COPY_FROM_HOST, WEIGHTS_COPY_FROM_DEVICE, WEIGHTS_BORROW_DEVICE = 0, 1, 2


class DmoeError(RuntimeError):
    pass


class _Handle(C.Structure):
    _fields_ = [("ctx", C.c_void_p)]


class QWeightC(C.Structure):
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
                ("n_mats", C.c_int), ("rows", C.c_int), ("cols", C.c_int),
                ("mode", C.c_int), ("bits", C.c_int), ("group_size", C.c_int)]


class LayerDescC(C.Structure):
    _fields_ = [("hidden", C.c_int), ("ffn", C.c_int), ("top_k", C.c_int),
                ("gate", QWeightC), ("up", QWeightC), ("down", QWeightC),
                ("swiglu_limit", C.c_float), ("score_before_down", C.c_int),
                ("has_shared", C.c_int),
                ("shared_gate", QWeightC), ("shared_up", QWeightC), ("shared_down", QWeightC),
                ("shared_swiglu_limit", C.c_float),
                ("remap", C.c_void_p), ("n_experts_total", C.c_int),
                ("weight_source", C.c_int)]


class GateDescC(C.Structure):
    _fields_ = [("weight", C.c_void_p), ("bias", C.c_void_p), ("resident_mask", C.c_void_p),
                ("n_experts", C.c_int), ("dim", C.c_int), ("top_k", C.c_int),
                ("scoring_func", C.c_int), ("route_scale", C.c_float), ("is_hash", C.c_int),
                ("tid2eid", C.c_void_p), ("vocab_size", C.c_int), ("weight_source", C.c_int)]


class SafetensorsOptsC(C.Structure):
    _fields_ = [("top_k", C.c_int), ("mode", C.c_char_p), ("group_size", C.c_int), ("bits", C.c_int),
                ("swiglu_limit", C.c_float), ("score_before_down", C.c_int), ("load_shared", C.c_int),
                ("shared_mode", C.c_char_p), ("shared_group_size", C.c_int), ("shared_bits", C.c_int),
                ("shared_swiglu_limit", C.c_float), ("resident_mask", C.c_void_p), ("n_experts_total", C.c_int)]


SCORE_SOFTMAX, SCORE_SIGMOID, SCORE_SQRTSOFTPLUS, SCORE_SQRTSOFTPLUS_STABLE = 0, 1, 2, 3

# every symbol include/dmoe.h declares
EXPORTS = [
    "dmoe_quant_mode_from_string", "dmoe_version", "dmoe_dequant_fp8_block", "dmoe_last_error", "dmoe_init",
    "dmoe_stream_create", "dmoe_stream_destroy", "dmoe_stream_synchronize",
    "dmoe_malloc", "dmoe_free", "dmoe_copy_to_device", "dmoe_copy_to_host",
    "dmoe_workspace_create", "dmoe_workspace_destroy", "dmoe_workspace_reserved",
    "dmoe_workspace_check", "dmoe_workspace_set_wait_limit", "dmoe_workspace_set_paired_launch", "dmoe_workspace_set_weight_cache",
    "dmoe_workspace_weight_cache_invalidate", "dmoe_workspace_set_weight_cache_limit", "dmoe_workspace_weight_cache_stats",
    "dmoe_workspace_set_stage_timing", "dmoe_workspace_read_stage_times",
    "dmoe_topk_route", "dmoe_gate_route", "dmoe_remap_indices", "dmoe_expand_tokens",
    "dmoe_reduce_experts", "dmoe_smelt_build_mask", "dmoe_build_remap", "dmoe_preload_remap",
    "dmoe_pack", "dmoe_dequantize", "dmoe_gather_qmm",
    "dmoe_resident_weight_create", "dmoe_resident_weight_destroy", "dmoe_gather_qmm_resident",
    "dmoe_layer_create", "dmoe_layer_destroy", "dmoe_moe_forward",
    "dmoe_switch_glu_forward_no_scores", "dmoe_moe_layer_forward", "dmoe_moe_layer_forward_static",
    "dmoe_debug_last_activations", "dmoe_debug_dequantize_fused", "dmoe_debug_mfma_loop", "dmoe_debug_read_stream",
    "dmoe_gate_create", "dmoe_gate_destroy", "dmoe_gate_forward",
    "dmoe_layer_create_from_safetensors", "dmoe_layer_dims", "dmoe_batch_build", "dmoe_block_post",
]

_lib = None


def lib():
    """Load libdmoe.so (built by dmlx_amd/csrc/Makefile). Raises if it is not there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise DmoeError(f"{LIB_PATH} not found: build it with `make -C dmlx_amd/csrc` "
                            "(or __graft_entry__.build()); there is no fallback path")
        _lib = C.CDLL(LIB_PATH)
        _lib.dmoe_last_error.restype = C.c_char_p
    return _lib


def check(rc):
    if rc != 0:
        raise DmoeError(f"dmoe error {rc}: {lib().dmoe_last_error().decode()}")


def _ptr(t):
    if t is None:
        return None
    assert t.is_contiguous(), "dmoe takes dense row-major tensors"
    return C.c_void_p(t.data_ptr())


def _stream():
    return _Handle(C.c_void_p(torch.cuda.current_stream().cuda_stream))


def init(device=0):
    check(lib().dmoe_init(device))


class Workspace:
    def __init__(self, initial_bytes=0):
        self.h = _Handle()
        check(lib().dmoe_workspace_create(C.byref(self.h), C.c_size_t(initial_bytes)))

    def reserved(self):
        n = C.c_size_t()
        check(lib().dmoe_workspace_reserved(C.byref(n), self.h))
        return n.value

    def check(self):
        """Wait for the current stream; raises if a kernel launched with this workspace gave up a bounded wait."""
        check(lib().dmoe_workspace_check(self.h, _stream()))

    def set_wait_limit(self, polls):
        check(lib().dmoe_workspace_set_wait_limit(self.h, C.c_uint(polls)))

    def set_weight_cache(self, enabled):
        """gather_qmm keeps re-ordered resident copies of the stacks it sees (dmoe_workspace_set_weight_cache)"""
        check(lib().dmoe_workspace_set_weight_cache(self.h, int(enabled)))

    def invalidate_weight_cache(self, qw=None):
        """drop the cached copy of one stack (a QWeight), or every copy"""
        if qw is None:
            check(lib().dmoe_workspace_weight_cache_invalidate(self.h, None))
        else:
            c = qw.c()
            check(lib().dmoe_workspace_weight_cache_invalidate(self.h, C.byref(c)))

    def set_weight_cache_limit(self, max_bytes):
        check(lib().dmoe_workspace_set_weight_cache_limit(self.h, C.c_size_t(max_bytes)))

    def weight_cache_stats(self):
        b, n = C.c_size_t(0), C.c_int(0)
        check(lib().dmoe_workspace_weight_cache_stats(C.byref(b), C.byref(n), self.h))
        return b.value, n.value

    def set_paired_launch(self, enabled):
        check(lib().dmoe_workspace_set_paired_launch(self.h, int(enabled)))

    STAGES = ("route", "pack", "gate_up", "down", "shared", "combine", "gate_up_small", "down_small")

    def set_stage_timing(self, enabled):
        check(lib().dmoe_workspace_set_stage_timing(self.h, int(enabled)))

    def stage_times(self):
        """{stage: (total_ms, samples)} of the forward calls made since timing was enabled"""
        ms = (C.c_float * len(self.STAGES))()
        n = (C.c_int * len(self.STAGES))()
        check(lib().dmoe_workspace_read_stage_times(ms, n, self.h))
        return {s: (ms[i], n[i]) for i, s in enumerate(self.STAGES)}

    def close(self):
        if self.h.ctx:
            check(lib().dmoe_workspace_destroy(self.h))
            self.h = _Handle()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class QWeight:
    """A stack [n, rows, cols] of quantized matrices held as torch tensors (any device)."""

    def __init__(self, w, scales, biases, rows, cols, mode, bits, group_size):
        self.w, self.scales, self.biases = w.contiguous(), None if scales is None else scales.contiguous(), biases
        if self.biases is not None:
            self.biases = self.biases.contiguous()
        self.rows, self.cols, self.mode, self.bits, self.group_size = rows, cols, mode, bits, group_size
        self.n_mats = w.shape[0] if w.dim() == 3 else 1

    def to(self, device):
        return QWeight(self.w.to(device), None if self.scales is None else self.scales.to(device),
                       None if self.biases is None else self.biases.to(device),
                       self.rows, self.cols, self.mode, self.bits, self.group_size)

    def c(self):
        return QWeightC(_ptr(self.w), _ptr(self.scales), _ptr(self.biases), self.n_mats, self.rows,
                        self.cols, self.mode, self.bits, self.group_size)

    def nbytes(self):
        n = self.w.numel() * self.w.element_size()
        if self.scales is not None:
            n += self.scales.numel() * self.scales.element_size()
        if self.biases is not None:
            n += self.biases.numel() * self.biases.element_size()
        return n


def topk_route(scores, K, normalize=True):
    T, E = scores.shape
    idx = torch.empty((T, K), dtype=torch.int32, device=scores.device)
    w = torch.empty((T, K), dtype=torch.float32, device=scores.device)
    check(lib().dmoe_topk_route(_ptr(idx), _ptr(w), _ptr(scores), T, E, K, int(normalize), _stream()))
    return idx, w


def gate_route(scores, bias, resident_mask, K, renorm, route_scale):
    T, E = scores.shape
    idx = torch.empty((T, K), dtype=torch.int32, device=scores.device)
    w = torch.empty((T, K), dtype=torch.float32, device=scores.device)
    check(lib().dmoe_gate_route(_ptr(idx), _ptr(w), _ptr(scores), _ptr(bias), _ptr(resident_mask),
                                T, E, K, int(renorm), C.c_float(route_scale), _stream()))
    return idx, w


def remap_indices(remap, idx):
    out = torch.empty_like(idx)
    check(lib().dmoe_remap_indices(_ptr(out), _ptr(remap), _ptr(idx), C.c_size_t(idx.numel()),
                                   remap.numel(), _stream()))
    return out


def expand_tokens(x, K):
    T, D = x.shape
    out = torch.empty((T * K, D), dtype=x.dtype, device=x.device)
    check(lib().dmoe_expand_tokens(_ptr(out), _ptr(x), T, D, K, x.element_size(), _stream()))
    return out


def reduce_experts(expert_outs, weights):
    T, K = weights.shape
    D = expert_outs.shape[1]
    out = torch.empty((T, D), dtype=torch.float32, device=weights.device)
    check(lib().dmoe_reduce_experts(_ptr(out), _ptr(expert_outs), int(expert_outs.dtype == torch.bfloat16),
                                    _ptr(weights), T, K, D, _stream()))
    return out


def smelt_build_mask(n_experts, load_fraction, strategy=0, enabled=True):
    mask = (C.c_uint8 * n_experts)()
    n = C.c_int()
    check(lib().dmoe_smelt_build_mask(mask, C.byref(n), n_experts, C.c_float(load_fraction), strategy,
                                      int(enabled)))
    return list(mask), n.value


def build_remap(mask):
    n = len(mask)
    m = (C.c_uint8 * n)(*mask)
    out = (C.c_int32 * n)()
    check(lib().dmoe_build_remap(out, m, n))
    return list(out)


def preload_remap(expert_ids, n_total):
    ids = (C.c_uint32 * max(len(expert_ids), 1))(*expert_ids)
    out = (C.c_int32 * n_total)()
    cb = (C.c_float * n_total)()
    check(lib().dmoe_preload_remap(out, cb, ids, len(expert_ids), n_total))
    return list(out), list(cb)


def pack(idx, E, ws):
    T, K = idx.shape
    n = T * K
    dev = idx.device
    i32 = dict(dtype=torch.int32, device=dev)
    out = dict(order=torch.empty(n, **i32), inv=torch.empty(n, **i32), token=torch.empty(n, **i32),
               sorted_e=torch.empty(n, **i32), counts=torch.empty(E, **i32),
               offsets=torch.empty(E + 1, **i32), live=torch.full((E,), -1, **i32),
               n_live=torch.empty(1, **i32))
    check(lib().dmoe_pack(_ptr(out["order"]), _ptr(out["inv"]), _ptr(out["token"]), _ptr(out["sorted_e"]),
                          _ptr(out["counts"]), _ptr(out["offsets"]), _ptr(out["live"]), _ptr(out["n_live"]),
                          _ptr(idx), T, K, E, ws.h, _stream()))
    return out


def dequantize(qw, mat_index=0, fused=False):
    """dmoe_dequantize; fused=True: the same matrix through the prefill kernels' in-register decoder."""
    out = torch.empty((qw.rows, qw.cols), dtype=torch.bfloat16, device=qw.w.device)
    c = qw.c()
    fn = lib().dmoe_debug_dequantize_fused if fused else lib().dmoe_dequantize
    check(fn(_ptr(out), C.byref(c), mat_index, _stream()))
    return out


def dequant_fp8_block(w, scale, block_size):
    """dmoe_dequant_fp8_block: w uint8 [rows, cols] (E4M3FN), scale float32 or uint8 (E8M0)
    [ceil(rows / block), ceil(cols / block)] -> bf16 [rows, cols]."""
    rows, cols = w.shape
    assert w.dtype == torch.uint8 and w.is_contiguous() and scale.is_contiguous()
    assert scale.dtype in (torch.float32, torch.uint8) and tuple(scale.shape) == (-(-rows // block_size), -(-cols // block_size))
    out = torch.empty((rows, cols), dtype=torch.bfloat16, device=w.device)
    check(lib().dmoe_dequant_fp8_block(_ptr(out), _ptr(w), _ptr(scale), int(scale.dtype == torch.uint8), rows, cols,
                                       block_size, _stream()))
    return out


MFMA_LOOP_OPERANDS = 49152            # DMOE_MFMA_LOOP_OPERANDS
MFMA_LOOP_OUT = 131072                # DMOE_MFMA_LOOP_OUT
MFMA_LOOP_FLOP_PER_ITER = 2147483648.0


def mfma_loop(operands, iters, out=None):
    """dmoe_debug_mfma_loop: one launch of the matrix-instruction loop on `operands` (bf16 [MFMA_LOOP_OPERANDS])."""
    assert operands.dtype == torch.bfloat16 and operands.numel() == MFMA_LOOP_OPERANDS and operands.is_contiguous()
    if out is None:
        out = torch.empty((MFMA_LOOP_OUT,), dtype=torch.float32, device=operands.device)
    check(lib().dmoe_debug_mfma_loop(_ptr(out), _ptr(operands), int(iters), _stream()))
    return out


def read_stream(src, workgroups, sink=None):
    """dmoe_debug_read_stream: one launch that reads `src` (any contiguous tensor); returns the bytes it reads."""
    assert src.is_contiguous()
    if sink is None:
        sink = torch.empty((4 * workgroups,), dtype=torch.int32, device=src.device)
    n = C.c_size_t(0)
    check(lib().dmoe_debug_read_stream(C.byref(n), _ptr(sink), _ptr(src), C.c_size_t(src.numel() * src.element_size()),
                                       int(workgroups), _stream()))
    return n.value


class ResidentWeight:
    """A weight stack made resident once in the kernels' layout (dmoe_resident_weight)."""

    def __init__(self, qw):
        self.h = _Handle()
        self.rows, self.cols, self.n_mats = qw.rows, qw.cols, qw.n_mats
        c = qw.c()
        source = 1 if qw.w.is_cuda else 0   # DMOE_WEIGHTS_COPY_FROM_DEVICE / _FROM_HOST
        check(lib().dmoe_resident_weight_create(C.byref(self.h), C.byref(c), source, _stream()))

    def gather_qmm(self, x, rhs_indices, ws, lhs_indices=None, sorted_indices=False):
        R = rhs_indices.numel()
        out = torch.empty((R, self.rows), dtype=torch.bfloat16, device=x.device)
        check(lib().dmoe_gather_qmm_resident(_ptr(out), _ptr(x), self.h, _ptr(lhs_indices), _ptr(rhs_indices), R,
                                             int(sorted_indices), ws.h, _stream()))
        return out

    def close(self):
        if self.h.ctx:
            check(lib().dmoe_resident_weight_destroy(self.h))
            self.h = _Handle()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gather_qmm(x, qw, rhs_indices, ws, lhs_indices=None, sorted_indices=False):
    R = rhs_indices.numel()
    out = torch.empty((R, qw.rows), dtype=torch.bfloat16, device=x.device)
    c = qw.c()
    check(lib().dmoe_gather_qmm(_ptr(out), _ptr(x), C.byref(c), _ptr(lhs_indices), _ptr(rhs_indices), R,
                                int(sorted_indices), ws.h, _stream()))
    return out


def batch_build(tokens, seq_lens, base_pos, ws, want_mask=True):
    """dmoe_batch_build: host lists in, (tokens u32 [T], positions i32 [T], mask f32 [T,T] | None, request_of_token)"""
    T, n = len(tokens), len(seq_lens)
    dev = "cuda"
    d_tok = torch.empty(T, dtype=torch.int32, device=dev)
    d_pos = torch.empty(T, dtype=torch.int32, device=dev)
    d_req = torch.empty(T, dtype=torch.int32, device=dev)
    d_mask = torch.empty((T, T), dtype=torch.float32, device=dev) if want_mask else None
    h_tok = (C.c_uint32 * max(T, 1))(*[int(v) for v in tokens])
    h_len = (C.c_int32 * max(n, 1))(*[int(v) for v in seq_lens])
    h_base = (C.c_int32 * max(n, 1))(*[int(v) for v in base_pos])
    check(lib().dmoe_batch_build(_ptr(d_tok), _ptr(d_pos), _ptr(d_mask), _ptr(d_req), h_tok, h_len, h_base, n, T,
                                 ws.h, _stream()))
    return d_tok, d_pos, d_mask, d_req


def block_post(ffn_out, residual, post_mix=None, comb_mix=None):
    """dmoe_block_post: residual add (no mixes; residual [T,D]) or mhcPost (residual [T,m,D], post_mix [T,m] or
    [T,m,1], comb_mix [T,m,m])"""
    T, D = ffn_out.shape
    m = 0 if post_mix is None else residual.shape[1]
    out = torch.empty_like(residual)
    pm = None if post_mix is None else post_mix.reshape(T, m).contiguous()
    cm = None if comb_mix is None else comb_mix.reshape(T, m, m).contiguous()
    check(lib().dmoe_block_post(_ptr(out), _ptr(ffn_out), _ptr(residual), _ptr(pm), _ptr(cm), T, D, m, _stream()))
    return out


class Gate:
    """Resident router (dmoe_gate): DSV4Gate.forward from the hidden states on."""

    def __init__(self, weight, top_k, scoring_func, route_scale=1.0, bias=None, resident_mask=None, tid2eid=None):
        assert weight.dtype == torch.bfloat16 and weight.dim() == 2
        d = GateDescC()
        d.weight, d.bias, d.resident_mask = _ptr(weight), _ptr(bias), _ptr(resident_mask)
        d.n_experts, d.dim, d.top_k = weight.shape[0], weight.shape[1], top_k
        d.scoring_func, d.route_scale, d.is_hash = scoring_func, route_scale, int(tid2eid is not None)
        if tid2eid is not None:
            assert tid2eid.dtype == torch.int32 and tid2eid.shape[1] == top_k
            d.tid2eid, d.vocab_size = _ptr(tid2eid), tid2eid.shape[0]
        d.weight_source = WEIGHTS_COPY_FROM_DEVICE if weight.is_cuda else WEIGHTS_COPY_FROM_HOST
        for t in (bias, resident_mask, tid2eid):
            assert t is None or t.is_cuda == weight.is_cuda, "gate tensors must live on the same side"
        self.n_experts, self.top_k = weight.shape[0], top_k
        self.h = _Handle()
        check(lib().dmoe_gate_create(C.byref(self.h), C.byref(d), _stream()))

    def forward(self, x, ws, want_scores=False, input_ids=None):
        T = x.shape[0]
        idx = torch.empty((T, self.top_k), dtype=torch.int32, device=x.device)
        w = torch.empty((T, self.top_k), dtype=torch.float32, device=x.device)
        scores = torch.empty((T, self.n_experts), dtype=torch.float32, device=x.device) if want_scores else None
        check(lib().dmoe_gate_forward(_ptr(idx), _ptr(w), _ptr(scores), self.h, _ptr(x), _ptr(input_ids), T, ws.h,
                                      _stream()))
        return (idx, w, scores) if want_scores else (idx, w)

    def close(self):
        if self.h.ctx:
            check(lib().dmoe_gate_destroy(self.h))
            self.h = _Handle()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Layer:
    """Resident MoE layer (dmoe_layer). Weights are copied to (or borrowed from) device memory."""

    def __init__(self, hidden, ffn, top_k, gate, up, down, swiglu_limit=0.0, score_before_down=False,
                 shared=None, shared_swiglu_limit=0.0, remap=None, borrow=False):
        d = LayerDescC()
        d.hidden, d.ffn, d.top_k = hidden, ffn, top_k
        d.gate, d.up, d.down = gate.c(), up.c(), down.c()
        d.swiglu_limit = swiglu_limit
        d.score_before_down = int(score_before_down)
        d.has_shared = int(shared is not None)
        if shared is not None:
            d.shared_gate, d.shared_up, d.shared_down = shared[0].c(), shared[1].c(), shared[2].c()
        d.shared_swiglu_limit = shared_swiglu_limit
        self._remap_host = None
        if remap is not None:
            self._remap_host = (C.c_int32 * len(remap))(*[int(v) for v in remap])
            d.remap = C.cast(self._remap_host, C.c_void_p)
            d.n_experts_total = len(remap)
        on_device = gate.w.is_cuda
        d.weight_source = (WEIGHTS_BORROW_DEVICE if borrow else WEIGHTS_COPY_FROM_DEVICE) if on_device \
            else WEIGHTS_COPY_FROM_HOST
        self._keep = (gate, up, down, shared) if borrow else None
        self.hidden, self.ffn, self.top_k = hidden, ffn, top_k
        self.h = _Handle()
        check(lib().dmoe_layer_create(C.byref(self.h), C.byref(d), _stream()))

    @classmethod
    def from_safetensors(cls, paths, layer_idx, top_k, mode, group_size, bits, swiglu_limit=0.0,
                         score_before_down=False, load_shared=True, shared_swiglu_limit=0.0, resident_mask=None):
        """dmoe_layer_create_from_safetensors; `resident_mask` is a host sequence of 0/1 per expert in the file."""
        o = SafetensorsOptsC()
        o.top_k, o.mode, o.group_size, o.bits = top_k, mode.encode(), group_size, bits
        o.swiglu_limit, o.score_before_down, o.load_shared = swiglu_limit, int(score_before_down), int(load_shared)
        o.shared_mode, o.shared_group_size, o.shared_bits, o.shared_swiglu_limit = None, 0, 0, shared_swiglu_limit
        keep = None
        if resident_mask is not None:
            keep = (C.c_uint8 * len(resident_mask))(*[int(v) for v in resident_mask])
            o.resident_mask, o.n_experts_total = C.cast(keep, C.c_void_p), len(resident_mask)
        arr = (C.c_char_p * len(paths))(*[p.encode() for p in paths])
        self = cls.__new__(cls)
        self._remap_host, self._keep = None, None
        self.h = _Handle()
        check(lib().dmoe_layer_create_from_safetensors(C.byref(self.h), arr, len(paths), layer_idx, C.byref(o),
                                                       _stream()))
        d, f, n, k = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        check(lib().dmoe_layer_dims(C.byref(d), C.byref(f), C.byref(n), C.byref(k), self.h))
        self.hidden, self.ffn, self.n_slots, self.top_k = d.value, f.value, n.value, k.value
        return self

    def forward(self, x, indices, scores, ws):
        T = x.shape[0]
        out = torch.empty((T, self.hidden), dtype=torch.bfloat16, device=x.device)
        check(lib().dmoe_moe_forward(_ptr(out), self.h, _ptr(x), _ptr(indices), _ptr(scores), T, ws.h,
                                     _stream()))
        return out

    def forward_no_scores(self, x, slot_indices, ws):
        T = x.shape[0]
        out = torch.empty((T, self.top_k, self.hidden), dtype=torch.bfloat16, device=x.device)
        check(lib().dmoe_switch_glu_forward_no_scores(_ptr(out), self.h, _ptr(x), _ptr(slot_indices), T,
                                                      ws.h, _stream()))
        return out

    def layer_forward(self, x, scores, bias, resident_mask, renorm, route_scale, ws, want_routing=False, out=None):
        """dmoe_moe_layer_forward; ws=None calls dmoe_moe_layer_forward_static (the library's static device scratch,
        no allocation: pass `out` to keep torch from allocating too)."""
        T, E_total = scores.shape
        if out is None:
            out = torch.empty((T, self.hidden), dtype=torch.bfloat16, device=x.device)
        idx = w = None
        if want_routing:
            idx = torch.empty((T, self.top_k), dtype=torch.int32, device=x.device)
            w = torch.empty((T, self.top_k), dtype=torch.float32, device=x.device)
        if ws is None:
            check(lib().dmoe_moe_layer_forward_static(_ptr(out), _ptr(idx), _ptr(w), self.h, _ptr(x), _ptr(scores),
                                                      _ptr(bias), _ptr(resident_mask), T, E_total, int(renorm),
                                                      C.c_float(route_scale), _stream()))
        else:
            check(lib().dmoe_moe_layer_forward(_ptr(out), _ptr(idx), _ptr(w), self.h, _ptr(x), _ptr(scores),
                                               _ptr(bias), _ptr(resident_mask), T, E_total, int(renorm),
                                               C.c_float(route_scale), ws.h, _stream()))
        return (out, idx, w) if want_routing else out

    def last_activations(self, T, ws):
        out = torch.empty((T * self.top_k, self.ffn), dtype=torch.bfloat16, device="cuda")
        check(lib().dmoe_debug_last_activations(_ptr(out), self.h, T, ws.h, _stream()))
        return out

    def close(self):
        if self.h.ctx:
            check(lib().dmoe_layer_destroy(self.h))
            self.h = _Handle()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
