"""Synthetic workloads for the MoE expert-FFN path (the five benchmark configurations).

Everything is seeded and generated with torch on the requested device; weights are drawn in f32 from
N(0, 0.02), quantized with dmlx_amd.quantize, activations are bf16 N(0,1), router logits f32 N(0,1).
A workload is plain data (tensors + scalars); it knows nothing about the kernels.
"""
from dataclasses import dataclass, field
from typing import Optional

import torch

from . import quantize as Q
from .capi import QUANT_AFFINE, QUANT_FP8_ROW, QUANT_MXFP4, QUANT_NONE, QWeight


@dataclass
class Workload:
    name: str
    T: int
    D: int
    F: int
    E_total: int                 # experts the router sees
    E: int                       # resident expert slots
    K: int
    x: torch.Tensor              # bf16 [T, D]
    scores: torch.Tensor         # f32 [T, E_total] (after the scoring function)
    bias: Optional[torch.Tensor]         # f32 [E_total] selection bias or None
    resident_mask: Optional[torch.Tensor]  # u8 [E_total] or None
    remap: Optional[list]        # router id -> slot, or None
    renorm: bool
    route_scale: float
    gate: QWeight = None
    up: QWeight = None
    down: QWeight = None
    shared: Optional[tuple] = None       # (gate, up, down) QWeight singles
    swiglu_limit: float = 0.0
    shared_swiglu_limit: float = 0.0
    score_before_down: bool = False
    scoring: str = "sigmoid"
    seg_lens: list = field(default_factory=list)   # request lengths for ragged batches

    def expert_bytes(self):
        """packed bytes of ONE routed expert (gate + up + down, scales and biases included)"""
        return (self.gate.nbytes() + self.up.nbytes() + self.down.nbytes()) // self.E

    def shared_bytes(self):
        return 0 if self.shared is None else sum(q.nbytes() for q in self.shared)

    def routed_flops(self):
        return 2 * self.T * self.K * 3 * self.D * self.F

    def shared_flops(self):
        return 0 if self.shared is None else 2 * self.T * 3 * self.D * self.shared[0].rows


def _quant_stack(n, rows, cols, fmt, gen, device, chunk=16):
    """n matrices [rows, cols] drawn N(0, 0.02) and quantized; generated in chunks to bound memory."""
    ws, ss, bs = [], [], []
    for i in range(0, n, chunk):
        m = min(chunk, n - i)
        w = torch.randn((m, rows, cols), generator=gen, device=device, dtype=torch.float32) * 0.02
        if fmt == "affine4":
            a, s, b = Q.quantize_affine(w, 64, 4)
        elif fmt == "affine8":
            a, s, b = Q.quantize_affine(w, 64, 8)
        elif fmt == "mxfp4":
            a, s = Q.quantize_mxfp4(w)
            b = None
        elif fmt == "fp8row":
            a, s = Q.quantize_fp8_row(w)
            b = None
        elif fmt == "bf16":   # unquantized experts
            a, s, b = w.to(torch.bfloat16), None, None
        else:
            raise ValueError(fmt)
        ws.append(a)
        ss.append(s)
        bs.append(b)
        del w
    w = torch.cat(ws)
    s = None if ss[0] is None else torch.cat(ss)
    b = None if bs[0] is None else torch.cat(bs)
    mode, bits, group = {"affine4": (QUANT_AFFINE, 4, 64), "affine8": (QUANT_AFFINE, 8, 64),
                         "mxfp4": (QUANT_MXFP4, 4, 32), "fp8row": (QUANT_FP8_ROW, 8, 0),
                         "bf16": (QUANT_NONE, 16, 0)}[fmt]
    return QWeight(w, s, b, rows, cols, mode, bits, group)


def _experts(E, D, F, fmt, gen, device):
    return (_quant_stack(E, F, D, fmt, gen, device), _quant_stack(E, F, D, fmt, gen, device),
            _quant_stack(E, D, F, fmt, gen, device))


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def ragged_lengths(n_req, lo, hi, total, gen):
    """n_req lengths uniform in [lo, hi], rescaled so they sum to `total` (each kept in [lo, hi])."""
    lens = torch.randint(lo, hi + 1, (n_req,), generator=gen, device=gen.device).cpu().tolist()
    for _ in range(64):
        diff = total - sum(lens)
        if diff == 0:
            break
        step = (diff // n_req) or (1 if diff > 0 else -1)
        for i in range(n_req):
            if sum(lens) == total:
                break
            lens[i] = min(hi, max(lo, lens[i] + step))
    return lens


def make(config, device="cuda", seed=None, scale=1.0):
    """Build benchmark configuration `config` (0..4). `scale` < 1 shrinks E, D, F for quick tests."""
    seed = config if seed is None else seed
    g = _gen(seed, device)
    rn = lambda *shape: torch.randn(shape, generator=g, device=device, dtype=torch.float32)

    def dims(D, F, E):
        if scale == 1.0:
            return D, F, E
        r = lambda v, q: max(q, int(v * scale) // q * q)
        return r(D, 256), r(F, 256), max(8, int(E * scale))

    if config == 0:
        # 16 tokens, D=1024, E=8, top-2, F=2048, affine-4 g64; softmax scores renormalised over the top-k
        T, (D, F, E), K = 16, dims(1024, 2048, 8), 2
        gate, up, down = _experts(E, D, F, "affine4", g, device)
        scores = torch.softmax(rn(T, E), dim=-1)
        return Workload("C0 small layer", T, D, F, E, E, K, rn(T, D).to(torch.bfloat16), scores, None, None, None,
                        True, 1.0, gate, up, down, scoring="softmax")
    if config in (1, 2):
        T, (D, F, E), K = 64, dims(4096, 2048, 256), 6
        K = min(K, E)
        fmt = "affine4" if config == 1 else "mxfp4"
        logits, bias = rn(T, E), rn(E) * 0.1
        scores = torch.sigmoid(logits)
        x = rn(T, D).to(torch.bfloat16)
        if config == 1:
            gate, up, down = _experts(E, D, F, fmt, g, device)
            shared = tuple(_quant_stack(1, r, c, fmt, g, device) for r, c in ((F, D), (F, D), (D, F)))
            return Workload("C1 decode 64x1 affine4", T, D, F, E, E, K, x, scores, bias, None, None, True, 1.5,
                            gate, up, down, shared, swiglu_limit=10.0)
        n_live = max(K, round(E * 51 / 256))
        perm = torch.randperm(E, generator=g, device=device)[:n_live].sort().values.cpu()
        mask = torch.zeros(E, dtype=torch.uint8)
        mask[perm] = 1
        remap, slot = [], 0
        for e in range(E):
            remap.append(slot if mask[e] else 0)
            slot += int(mask[e])
        gate, up, down = _experts(n_live, D, F, fmt, g, device)
        shared = tuple(_quant_stack(1, r, c, fmt, g, device) for r, c in ((F, D), (F, D), (D, F)))
        return Workload("C2 decode 64x1 mxfp4 smelt", T, D, F, E, n_live, K, x, scores, bias, mask.to(device),
                        remap, True, 1.5, gate, up, down, shared, swiglu_limit=10.0)
    if config == 3:
        (D, F, E), K = dims(4096, 2048, 256), 6
        K = min(K, E)
        total = 8192 if scale == 1.0 else max(256, int(8192 * scale))
        lo, hi = (64, 2048) if scale == 1.0 else (max(8, int(64 * scale)), max(16, int(2048 * scale)))
        lens = ragged_lengths(8, lo, hi, total, g)
        T = sum(lens)
        # Zipf(1.1) popularity over a seeded permutation of the experts, added as log p to the logits
        rank = torch.randperm(E, generator=g, device=device).float() + 1.0
        logp = -1.1 * torch.log(rank)
        logp = logp - torch.logsumexp(logp, 0)
        scores = torch.sigmoid(rn(T, E) + logp)
        gate, up, down = _experts(E, D, F, "affine4", g, device)
        return Workload("C3 ragged prefill zipf", T, D, F, E, E, K, rn(T, D).to(torch.bfloat16), scores, None,
                        None, None, True, 1.5, gate, up, down, swiglu_limit=10.0, seg_lens=lens)
    if config == 4:
        (D, F, E), K = dims(4096, 2048, 256), 6
        K = min(K, E)
        pre = 512 if scale == 1.0 else max(16, int(512 * scale))
        lens = [pre] * 4 + [1] * 32   # prefill requests first, then decode ones (batch_builder.zig:104-111)
        T = sum(lens)
        logits, bias = rn(T, E), rn(E) * 0.1
        gate, up, down = _experts(E, D, F, "affine8", g, device)
        shared = tuple(_quant_stack(1, r, c, "fp8row", g, device) for r, c in ((F, D), (F, D), (D, F)))
        return Workload("C4 mixed batch affine8 + fp8 shared", T, D, F, E, E, K, rn(T, D).to(torch.bfloat16),
                        torch.sigmoid(logits), bias, None, None, True, 1.5, gate, up, down, shared,
                        swiglu_limit=10.0, seg_lens=lens)
    raise ValueError(f"unknown config {config}")
