"""Weight quantizers used to prepare synthetic (and real) expert weights.

These produce the MLX on-disk/in-memory formats the MoE path consumes
(packed u32 words + per-group scales/biases). They are data preparation, not part
of the per-step hot path, and run as plain torch ops on whatever device holds the
weights. The rule for choosing scales is this repository's own (modelled on MLX's
published affine rule); parity of the hot path never depends on it because the
GPU kernels and their checker both consume the bytes produced here.

Formats
  affine  : q in [0, 2^bits), value = q*scale + bias; `32/bits` codes per u32,
            code i of a row at bits [bits*(i % per), +bits) of word i // per;
            scales/biases bf16 [..., rows, cols/group]
  mxfp4   : E2M1 codes (sign bit 3), 8 per u32 low nibble first; one E8M0
            exponent (u8, value 2^(s-127)) per 32 values
  fp8row  : E4M3FN bytes [..., rows, cols] with one f32 scale per output row
            (scale = amax_row / 448)
"""
import torch

E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def _pack_codes(q, bits):
    """q: integer codes [..., cols] -> int32 words [..., cols*bits/32] (u32 bit pattern)."""
    per = 32 // bits
    shp = q.shape
    q = q.reshape(*shp[:-1], shp[-1] // per, per).to(torch.int64)
    shifts = (torch.arange(per, device=q.device, dtype=torch.int64) * bits)
    words = (q << shifts).sum(-1)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32)


def quantize_affine(w, group=64, bits=4):
    """w: f32 [..., rows, cols] -> (words int32, scales bf16, biases bf16)."""
    n_bins = float(2 ** bits - 1)
    shp = w.shape
    wg = w.float().reshape(*shp[:-1], shp[-1] // group, group)
    w_max = wg.amax(-1)
    w_min = wg.amin(-1)
    use_min = w_min.abs() > w_max.abs()
    scale = torch.clamp((w_max - w_min) / n_bins, min=1e-7)
    scale = torch.where(use_min, scale, -scale)
    edge = torch.where(use_min, w_min, w_max)
    q0 = torch.round(edge / scale)
    scale = torch.where(q0 != 0, edge / q0, scale)
    bias = torch.where(q0 == 0, torch.zeros_like(edge), edge)
    scale_bf = scale.to(torch.bfloat16)
    bias_bf = bias.to(torch.bfloat16)
    s = scale_bf.float().unsqueeze(-1)
    b = bias_bf.float().unsqueeze(-1)
    q = torch.round((wg - b) / s).clamp_(0, n_bins).to(torch.uint8)
    words = _pack_codes(q.reshape(shp), bits)
    return words, scale_bf, bias_bf


def quantize_mxfp4(w):
    """w: f32 [..., rows, cols] -> (words int32 [..., cols/8], scales uint8 [..., cols/32])."""
    shp = w.shape
    wg = w.float().reshape(*shp[:-1], shp[-1] // 32, 32)
    amax = wg.abs().amax(-1)
    e = torch.ceil(torch.log2(torch.clamp(amax, min=1e-38) / 6.0))
    e = torch.where(amax > 0, e, torch.full_like(e, -127.0)).clamp_(-127, 127)
    scaled = wg / torch.exp2(e).unsqueeze(-1)
    mids = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], device=w.device)
    code = torch.bucketize(scaled.abs(), mids).to(torch.uint8)
    code = code | ((scaled < 0).to(torch.uint8) << 3)
    words = _pack_codes(code.reshape(shp), 4)
    return words, (e + 127).to(torch.uint8)


def quantize_fp8_row(w):
    """w: f32 [..., rows, cols] -> (bytes uint8 [..., rows, cols], scales f32 [..., rows])."""
    wf = w.float()
    amax = wf.abs().amax(-1)
    scale = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    q = (wf / scale.unsqueeze(-1)).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.view(torch.uint8), scale
