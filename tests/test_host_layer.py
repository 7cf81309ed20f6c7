"""The host layers above the C ABI: the header is valid C99 and C++17 (what @cImport / cgo-style bindings
parse), the C++ mirror of the reference's Zig call surface builds against it, and — on the GPU — the
reference's own router / remap / batch-builder vectors pass through that C++ layer."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dmoe.h")
HOST_HPP = os.path.join(ROOT, "dmlx_amd", "host", "moe.hpp")
HOST_BIN = os.path.join(ROOT, "tests", "host", "test_host_api")


def test_header_is_valid_c99_and_cxx17():
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c", HEADER], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c++", HEADER], check=True)


def test_host_layer_compiles_against_the_c_abi(tmp_path):
    src = tmp_path / "use.cpp"
    src.write_text('#include "dmlx_amd/host/moe.hpp"\nint main() { return sizeof(dmoe::MoERouter) ? 0 : 1; }\n')
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", f"-I{ROOT}/include", f"-I{ROOT}",
                    str(src)], check=True)


def test_zig_binding_names_the_same_entry_points():
    """dmlx_amd/zig/dmoe.zig cannot be compiled here (no Zig toolchain); at least every C symbol it calls
    must be one the header declares."""
    import re
    with open(os.path.join(ROOT, "dmlx_amd", "zig", "dmoe.zig")) as f:
        zig = f.read()
    with open(HEADER) as f:
        declared = set(re.findall(r"\b(dmoe_[a-z0-9_]+)\s*\(", f.read()))
    used = set(re.findall(r"\bc\.(dmoe_[a-z0-9_]+)\s*\(", zig))
    assert used and used <= declared, used - declared


@pytest.mark.gpu
def test_reference_vectors_through_the_cxx_host_layer():
    assert os.path.exists(HOST_BIN), "build it with make -C dmlx_amd/csrc (or __graft_entry__.build())"
    r = subprocess.run([HOST_BIN], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "ALL HOST TESTS PASSED" in r.stdout, r.stdout + r.stderr
