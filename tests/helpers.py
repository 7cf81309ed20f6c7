"""Shared helpers of the test-suite (conversions between the product's tensors and the oracle's arrays)."""
import numpy as np
import torch

from oracle import oracle
from oracle.oracle import bf16_bits, qmat  # noqa: F401  (re-exported: the tests import them from here)


def to_np_u32(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def bf16_to_f32(t):
    return t.detach().cpu().float().numpy()


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


def dense_reference_f64_device(x, idx, w, gate, up, down, limit=0.0, shared=None, shared_limit=0.0, device="cuda"):
    """dense_reference_f64 for whole prefill batches: the same float64 evaluation (no intermediate rounding), with the
    matrix products done by torch on `device`. The weights are the ORACLE's dequantized values (oracle.dequantize_f32
    on the CPU, one expert at a time, then copied over); nothing of the library under test takes part.
    x: torch bf16 [T, D]; idx: numpy [T, K] slot ids; w: numpy f32 [T, K]. Returns a float64 tensor [T, D] on `device`."""
    T, K = idx.shape
    xd = x.to(device).to(torch.float64)

    def deq(qm, m):
        return torch.from_numpy(oracle.dequantize_f32(qm, m)).to(device).to(torch.float64)

    def ffn(xr, g_, u_, d_, L):
        g, u = xr @ g_.T, xr @ u_.T
        if L > 0:
            g, u = torch.clamp(g, max=L), torch.clamp(u, -L, L)
        return (g / (1.0 + torch.exp(-g)) * u) @ d_.T

    out = torch.zeros((T, down.rows), dtype=torch.float64, device=device)
    flat = torch.from_numpy(idx.reshape(-1).astype(np.int64)).to(device)
    wf = torch.from_numpy(w.reshape(-1).astype(np.float64)).to(device)
    for e in np.unique(idx.reshape(-1)):
        pos = torch.nonzero(flat == int(e)).reshape(-1)
        tok = pos // K
        y = ffn(xd[tok], deq(gate, int(e)), deq(up, int(e)), deq(down, int(e)), limit)
        out.index_add_(0, tok, y * wf[pos][:, None])   # a token holds an expert at most once: no duplicate indices
    if shared is not None:
        out += ffn(xd, deq(shared[0], 0), deq(shared[1], 0), deq(shared[2], 0), shared_limit)
    return out
