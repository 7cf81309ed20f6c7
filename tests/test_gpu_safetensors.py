"""Resident upload of a layer's experts from MLX-format safetensors files (dmoe_layer_create_from_safetensors):
the layer built from the file must give the oracle's outputs when the oracle is fed the bytes an independent numpy
reader takes from the same file (the reference's own check is "partial read == load + take, bitwise",
src/tests/numerical_equivalence_test.zig:97-213), including the Smelt subset with its remap; it must also behave bit
for bit like the layer built from the same tensors in memory; malformed files are rejected with a message."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from dmlx_amd import workloads
from oracle import oracle
from tests.helpers import bf16_bits, max_abs_rel, to_np_u32

OUT_TOL = 1e-2   # bf16 outputs against the oracle, as everywhere else

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


_NP = {"U32": np.uint32, "U8": np.uint8, "BF16": np.uint16, "F32": np.float32}


def read_safetensors_numpy(path):
    """An independent reader for the test: 8-byte little-endian header length, JSON header, then the data section the
    offsets are relative to. bf16 comes back as uint16 bit patterns."""
    with open(path, "rb") as f:
        blob = f.read()
    (n,) = struct.unpack("<Q", blob[:8])
    header = json.loads(blob[8:8 + n].decode())
    data = blob[8 + n:]
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        out[name] = np.frombuffer(data[a:b], dtype=_NP[meta["dtype"]]).reshape(meta["shape"]).copy()
    return out


def _oracle_stack(tensors, layer_idx, group, proj, mode, bits, group_size):
    """oracle.QMat of `model.layers.{i}.ffn.{group}.{proj}` from the arrays read back from the file"""
    base = f"model.layers.{layer_idx}.ffn.{group}.{proj}."
    w = tensors[base + "weight"]
    if w.ndim == 2:
        w = w[None]
    per_word = 32 // bits
    rows, cols = w.shape[1], w.shape[2] * per_word
    scales = tensors[base + "scales"]
    biases = tensors.get(base + "biases")
    return oracle.QMat(np.ascontiguousarray(w), np.ascontiguousarray(scales),
                       None if biases is None else np.ascontiguousarray(biases), rows, cols, mode, bits, group_size)


@pytest.mark.parametrize("config,mode,group", [(1, "affine", 64), (2, "mxfp4", 32)])
def test_layer_from_safetensors_against_the_oracle(dmoe, orc, ws, tmp_path, config, mode, group):
    """File -> HBM -> kernels against file -> numpy -> oracle: routed experts and the shared expert, two shards."""
    wl = workloads.make(config, scale=0.125)
    tensors = _layer_tensors(wl, 5, with_shared=True)
    keys = sorted(tensors)
    p1, p2 = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    write_safetensors(p1, {k: tensors[k] for k in keys[::2]}, metadata={"format": "mlx"})
    write_safetensors(p2, {k: tensors[k] for k in keys[1::2]})
    disk = dmoe.Layer.from_safetensors([p1, p2], 5, wl.K, mode, group, 4, swiglu_limit=wl.swiglu_limit)
    back = {**read_safetensors_numpy(p1), **read_safetensors_numpy(p2)}
    omode = oracle.AFFINE if mode == "affine" else oracle.MXFP4
    stack = lambda grp, proj: _oracle_stack(back, 5, grp, proj, omode, 4, group)
    routed = [stack("switch_mlp", p) for p in ("gate_proj", "up_proj", "down_proj")]
    shared = tuple(stack("shared_experts", p) for p in ("gate_proj", "up_proj", "down_proj"))
    assert routed[0].n == wl.E and (routed[0].rows, routed[0].cols) == (wl.F, wl.D)
    idx, w = dmoe.gate_route(wl.scores, wl.bias, wl.resident_mask, wl.K, wl.renorm, wl.route_scale)
    if wl.remap is not None:   # the file holds the resident experts only: ids go through the workload's remap
        idx = dmoe.remap_indices(torch.tensor(wl.remap, dtype=torch.int32, device="cuda"), idx)
    got = disk.forward(wl.x, idx, w, ws).float().cpu().numpy()
    ws.check()
    want = orc.moe_forward(bf16_bits(wl.x), to_np_u32(idx), w.cpu().numpy(), *routed, swiglu_limit=wl.swiglu_limit,
                           shared=shared)
    err = max_abs_rel(got, want)
    assert err < OUT_TOL, err
    disk.close()


def test_smelt_subset_from_safetensors_against_the_oracle(dmoe, orc, ws, tmp_path):
    """Partial read == load + take: the layer uploads only the masked experts and remaps router ids to slots; the
    oracle takes ALL experts from the same file and the router ids as they are."""
    wl = workloads.make(1, scale=0.125)
    path = str(tmp_path / "l0.safetensors")
    write_safetensors(path, _layer_tensors(wl, 0, with_shared=False))
    mask = np.zeros(wl.E, np.uint8)
    mask[1::3] = 1
    disk = dmoe.Layer.from_safetensors([path], 0, wl.K, "affine", 64, 4, swiglu_limit=wl.swiglu_limit,
                                       load_shared=False, resident_mask=mask.tolist())
    assert disk.n_slots == int(mask.sum())
    back = read_safetensors_numpy(path)
    routed = [_oracle_stack(back, 0, "switch_mlp", p, oracle.AFFINE, 4, 64) for p in ("gate_proj", "up_proj", "down_proj")]
    idx, w = dmoe.gate_route(wl.scores, wl.bias, torch.from_numpy(mask).cuda(), wl.K, wl.renorm, wl.route_scale)
    assert mask[to_np_u32(idx)].all()
    got = disk.forward(wl.x, idx, w, ws).float().cpu().numpy()   # router ids in, the layer's own remap applied
    ws.check()
    want = orc.moe_forward(bf16_bits(wl.x), to_np_u32(idx), w.cpu().numpy(), *routed, swiglu_limit=wl.swiglu_limit)
    err = max_abs_rel(got, want)
    assert err < OUT_TOL, err
    disk.close()


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
    with pytest.raises(dmoe.DmoeError, match="group size must be"):
        load([good], group=0)                                  # would divide by zero
    with pytest.raises(dmoe.DmoeError, match="bits must be"):
        dmoe.Layer.from_safetensors([good], 0, wl.K, "affine", 64, 0, load_shared=False)
    uneven = dict(tensors)                                     # up_proj with one expert less than gate_proj
    for kind in ("weight", "scales", "biases"):
        k = f"model.layers.0.ffn.switch_mlp.up_proj.{kind}"
        uneven[k] = tensors[k][:-1]
    bad_n = str(tmp_path / "uneven.safetensors")
    write_safetensors(bad_n, uneven)
    mask = [1] * wl.E
    with pytest.raises(dmoe.DmoeError, match="experts"):
        dmoe.Layer.from_safetensors([bad_n], 0, wl.K, "affine", 64, 4, load_shared=False, resident_mask=mask)
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
