"""Resident upload of a layer's experts from MLX-format safetensors files (dmoe_layer_create_from_safetensors):
the layer built from the file must behave bit for bit like the layer built from the same tensors in memory,
including the Smelt subset with its remap; malformed files are rejected with a message."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from dmlx_amd import workloads
from tests.helpers import to_np_u32

pytestmark = pytest.mark.gpu

_DT = {torch.int32: "U32", torch.uint8: "U8", torch.bfloat16: "BF16", torch.float32: "F32"}


def write_safetensors(path, tensors, metadata=None):
    """8-byte little-endian header length + JSON header + raw tensor bytes (the layout the reference's own test
    writes, src/tests/numerical_equivalence_test.zig:29-88)."""
    header, blobs, off = {}, [], 0
    if metadata:
        header["__metadata__"] = metadata
    for name, t in tensors.items():
        t = t.contiguous().cpu()
        raw = t.view(torch.uint8).numpy().tobytes() if t.dtype != torch.uint8 else t.numpy().tobytes()
        header[name] = {"dtype": _DT[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


def _layer_tensors(wl, layer_idx, with_shared):
    base = f"model.layers.{layer_idx}.ffn."
    out = {}
    for proj, q in (("gate_proj", wl.gate), ("up_proj", wl.up), ("down_proj", wl.down)):
        out[base + f"switch_mlp.{proj}.weight"] = q.w
        if q.scales is not None:
            out[base + f"switch_mlp.{proj}.scales"] = q.scales
        if q.biases is not None:
            out[base + f"switch_mlp.{proj}.biases"] = q.biases
    if with_shared:
        for proj, q in zip(("gate_proj", "up_proj", "down_proj"), wl.shared):
            out[base + f"shared_experts.{proj}.weight"] = q.w[0]
            if q.scales is not None:
                out[base + f"shared_experts.{proj}.scales"] = q.scales[0]
            if q.biases is not None:
                out[base + f"shared_experts.{proj}.biases"] = q.biases[0]
    return out


@pytest.mark.parametrize("config,mode,group", [(1, "affine", 64), (2, "mxfp4", 32)])
def test_layer_from_safetensors_matches_layer_from_memory(dmoe, ws, tmp_path, config, mode, group):
    wl = workloads.make(config, scale=0.125)
    tensors = _layer_tensors(wl, 3, with_shared=True)
    keys = sorted(tensors)
    # two shards, as a sharded checkpoint would have them, plus an unrelated tensor and metadata
    p1, p2 = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    write_safetensors(p1, {k: tensors[k] for k in keys[::2]}, metadata={"format": "mlx"})
    write_safetensors(p2, {**{k: tensors[k] for k in keys[1::2]}, "model.norm.weight": torch.ones(8)})
    mem = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit, shared=wl.shared,
                     remap=wl.remap)
    # the file holds the resident experts only (the workload quantizes just those), so no mask here
    disk = dmoe.Layer.from_safetensors([p1, p2], 3, wl.K, mode, group, 4, swiglu_limit=wl.swiglu_limit)
    assert (disk.hidden, disk.ffn, disk.n_slots, disk.top_k) == (wl.D, wl.F, wl.E, wl.K)
    idx, w = dmoe.gate_route(wl.scores, wl.bias, wl.resident_mask, wl.K, wl.renorm, wl.route_scale)
    if wl.remap is not None:
        idx = dmoe.remap_indices(torch.tensor(wl.remap, dtype=torch.int32, device="cuda"), idx)
        mem.close()
        mem = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit, shared=wl.shared)
    a = mem.forward(wl.x, idx, w, ws)
    b = disk.forward(wl.x, idx, w, ws)
    assert torch.equal(a, b)
    mem.close()
    disk.close()


def test_smelt_subset_from_safetensors(dmoe, ws, tmp_path):
    """Only the masked experts are uploaded; router ids go through the remap built from the mask."""
    wl = workloads.make(1, scale=0.125)
    path = str(tmp_path / "l0.safetensors")
    write_safetensors(path, _layer_tensors(wl, 0, with_shared=False))
    mask = np.zeros(wl.E, np.uint8)
    mask[::3] = 1
    keep = torch.from_numpy(np.nonzero(mask)[0]).cuda()
    sub = lambda q: dmoe.QWeight(q.w[keep].contiguous(), q.scales[keep].contiguous(),
                                 None if q.biases is None else q.biases[keep].contiguous(), q.rows, q.cols, q.mode,
                                 q.bits, q.group_size)
    remap = dmoe.build_remap(mask)
    mem = dmoe.Layer(wl.D, wl.F, wl.K, sub(wl.gate), sub(wl.up), sub(wl.down), swiglu_limit=wl.swiglu_limit,
                     remap=list(remap))
    disk = dmoe.Layer.from_safetensors([path], 0, wl.K, "affine", 64, 4, swiglu_limit=wl.swiglu_limit,
                                       load_shared=False, resident_mask=mask.tolist())
    assert disk.n_slots == int(mask.sum())
    idx, w = dmoe.gate_route(wl.scores, wl.bias, torch.from_numpy(mask).cuda(), wl.K, wl.renorm, wl.route_scale)
    assert mask[to_np_u32(idx)].all()
    assert torch.equal(mem.forward(wl.x, idx, w, ws), disk.forward(wl.x, idx, w, ws))
    mem.close()
    disk.close()


def test_unquantized_experts_from_safetensors(dmoe, ws, tmp_path):
    """A float checkpoint: `switch_mlp.*.weight` are bf16 [E, rows, cols] and there are no scales (mode "none").
    Whole layer with its shared expert, then a Smelt subset of the same file."""
    wl = workloads.make(1, scale=0.125)
    g = torch.Generator(device="cuda").manual_seed(8)
    bf = lambda n, r, c: dmoe.QWeight((torch.randn((n, r, c), generator=g, device="cuda") * 0.02).to(torch.bfloat16),
                                      None, None, r, c, dmoe.QUANT_NONE, 16, 0)
    wl.gate, wl.up, wl.down = bf(wl.E, wl.F, wl.D), bf(wl.E, wl.F, wl.D), bf(wl.E, wl.D, wl.F)
    wl.shared = (bf(1, wl.F, wl.D), bf(1, wl.F, wl.D), bf(1, wl.D, wl.F))
    path = str(tmp_path / "float.safetensors")
    write_safetensors(path, _layer_tensors(wl, 2, with_shared=True))
    idx, w = dmoe.gate_route(wl.scores, wl.bias, None, wl.K, wl.renorm, wl.route_scale)
    mem = dmoe.Layer(wl.D, wl.F, wl.K, wl.gate, wl.up, wl.down, swiglu_limit=wl.swiglu_limit, shared=wl.shared)
    disk = dmoe.Layer.from_safetensors([path], 2, wl.K, "none", 0, 16, swiglu_limit=wl.swiglu_limit)
    assert (disk.hidden, disk.ffn, disk.n_slots) == (wl.D, wl.F, wl.E)
    assert torch.equal(mem.forward(wl.x, idx, w, ws), disk.forward(wl.x, idx, w, ws))
    mem.close()
    disk.close()
    with pytest.raises(dmoe.DmoeError, match="scales not found"):
        dmoe.Layer.from_safetensors([path], 2, wl.K, "affine", 64, 4)   # a float file is not an affine one
    mask = np.zeros(wl.E, np.uint8)
    mask[1::2] = 1
    keep = torch.from_numpy(np.nonzero(mask)[0]).cuda()
    sub = lambda q: dmoe.QWeight(q.w[keep].contiguous(), None, None, q.rows, q.cols, q.mode, q.bits, q.group_size)
    mem = dmoe.Layer(wl.D, wl.F, wl.K, sub(wl.gate), sub(wl.up), sub(wl.down), swiglu_limit=wl.swiglu_limit,
                     remap=list(dmoe.build_remap(mask)))
    disk = dmoe.Layer.from_safetensors([path], 2, wl.K, "none", 0, 16, swiglu_limit=wl.swiglu_limit,
                                       load_shared=False, resident_mask=mask.tolist())
    assert disk.n_slots == int(mask.sum())
    idx, w = dmoe.gate_route(wl.scores, wl.bias, torch.from_numpy(mask).cuda(), wl.K, wl.renorm, wl.route_scale)
    assert torch.equal(mem.forward(wl.x, idx, w, ws), disk.forward(wl.x, idx, w, ws))
    mem.close()
    disk.close()


def test_malformed_safetensors_are_rejected(dmoe, tmp_path):
    wl = workloads.make(1, scale=0.125)
    tensors = _layer_tensors(wl, 0, with_shared=False)
    good = str(tmp_path / "good.safetensors")
    write_safetensors(good, tensors)
    load = lambda paths, layer=0, **kw: dmoe.Layer.from_safetensors(paths, layer, wl.K, kw.get("mode", "affine"),
                                                                    kw.get("group", 64), 4, load_shared=False)
    with pytest.raises(dmoe.DmoeError, match="not found"):
        load([good], layer=1)                                  # no such layer in the file
    with pytest.raises(dmoe.DmoeError, match="cannot open"):
        load([str(tmp_path / "missing.safetensors")])
    with pytest.raises(dmoe.DmoeError, match="group size"):
        load([good], group=32)                                 # scales shape contradicts the group size
    with pytest.raises(dmoe.DmoeError, match="dtype"):
        load([good], mode="mxfp4", group=32)                   # bf16 scales are not E8M0 bytes
    bad = str(tmp_path / "bad.safetensors")
    with open(good, "rb") as f:
        blob = f.read()
    with open(bad, "wb") as f:
        f.write(blob[: len(blob) // 2])                        # truncated: offsets point outside the file
    with pytest.raises(dmoe.DmoeError, match="outside the file"):
        load([bad])
    with open(bad, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(dmoe.DmoeError, match="header length"):
        load([bad])
    with open(bad, "wb") as f:
        f.write(struct.pack("<Q", 9) + b'{"a": [1,')
    with pytest.raises(dmoe.DmoeError, match="malformed|JSON"):
        load([bad])
