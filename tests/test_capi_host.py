"""CPU-side checks of the C ABI: the library loads, exports every symbol include/dmoe.h declares, and its
host-only entry points (Smelt mask, remap builders, mode names) agree with the oracle and the reference's
vectors. No GPU work is enqueued here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from dmlx_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    with open(os.path.join(ROOT, "include", "dmoe.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(dmoe_[a-z0-9_]+)\s*\(", header))
    assert declared == set(capi.EXPORTS), declared ^ set(capi.EXPORTS)
    for name in sorted(declared):
        assert hasattr(lib, name), f"libdmoe.so does not export {name}"
    assert lib.dmoe_version() == 100


def test_mode_names_and_error_reporting():
    lib = capi.lib()
    assert lib.dmoe_quant_mode_from_string(b"affine") == capi.QUANT_AFFINE
    assert lib.dmoe_quant_mode_from_string(b"mxfp4") == capi.QUANT_MXFP4
    assert lib.dmoe_quant_mode_from_string(b"fp8") == capi.QUANT_FP8_ROW
    assert lib.dmoe_quant_mode_from_string(b"nope") == -1
    # a rejected call returns non-zero and leaves a message, mlx-c style
    rc = lib.dmoe_smelt_build_mask(None, None, 0, C.c_float(0.5), 0, 1)
    assert rc == 1 and b"smelt" in lib.dmoe_last_error()
    with pytest.raises(capi.DmoeError):
        capi.smelt_build_mask(8, 0.5, strategy=7)
    with pytest.raises(capi.DmoeError):
        capi.preload_remap([1, 99], 8)


@pytest.mark.parametrize("n,frac,strategy", [(256, 0.2, 0), (256, 0.2, 1), (64, 0.5, 0), (8, 0.01, 0), (8, 0.01, 1),
                                             (16, 1.0, 0), (100, 0.33, 0), (7, 0.9, 0)])
def test_smelt_mask_and_remap_match_oracle(orc, n, frac, strategy):
    mask, cnt = capi.smelt_build_mask(n, frac, strategy)
    want, want_cnt = orc.smelt_mask(n, frac, strategy)
    assert mask == want.tolist() and cnt == want_cnt
    assert capi.build_remap(mask) == orc.build_remap(want).tolist()
    off, cnt_off = capi.smelt_build_mask(n, frac, strategy, enabled=False)
    assert cnt_off == n and all(off)


def test_remap_builders_reference_vectors(orc, golden):
    g = golden["remap_construction"]
    remap, cache_bias = capi.preload_remap(g["unique_ids"], g["n_experts"])
    want, want_cb = orc.preload_remap(g["unique_ids"], g["n_experts"])
    assert remap == want.tolist() and cache_bias == want_cb.tolist()
    for i, e in enumerate(g["unique_ids"]):
        assert remap[e] == i and cache_bias[e] == 0.0
    for e in g["non_selected"]:
        assert remap[e] == 0 and cache_bias[e] == -1000.0
    # 256 experts at 20 %: 51 resident, the C2 configuration
    mask, cnt = capi.smelt_build_mask(256, 0.2)
    assert cnt == 51
    remap = capi.build_remap(mask)
    assert [remap[e] for e in np.flatnonzero(mask)] == list(range(51))
