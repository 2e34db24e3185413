"""The C-ABI library builds into the tree, loads without a GPU, and exports exactly the symbols the header declares.
No compute is called here."""

import ctypes
import os
import re

import pytest
import torch

from halo_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "halo_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hmoe_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        from halo_amd.build import build

        build(verbose=False)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/halo_moe.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "the ctypes table and the header disagree"


def test_status_strings_and_version():
    lib = _lib.load()
    assert lib.hmoe_abi_version() == 1
    assert lib.hmoe_status_string(0) == b"ok"
    assert b"unsupported" in lib.hmoe_status_string(-2)


def test_header_is_plain_c():
    """The header compiles as C: plain pointers and sizes, no C++ or torch types."""
    import subprocess
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "t.c")
        with open(src, "w") as f:
            f.write('#include "halo_moe.h"\nint main(void) { return hmoe_abi_version() == 0; }\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", f"-I{ROOT}/include", src], check=True)


def test_cpu_tensors_are_refused_not_routed_to_a_fallback():
    from halo_amd.kernels.fused_glu import GluCombine
    from halo_amd.kernels.grouped_mm import grouped_mm
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert

    with pytest.raises(RuntimeError, match="device tensors only"):
        sort_routing_by_expert(torch.zeros(2, 2, dtype=torch.long), torch.rand(2, 2), 4, None)
    with pytest.raises(RuntimeError, match="device tensors only"):
        GluCombine.silu()(torch.randn(2, 8), torch.randn(2, 8))
    with pytest.raises(RuntimeError, match="device tensors only"):
        grouped_mm(torch.randn(4, 8), torch.randn(1, 8, 8), offs=torch.tensor([4], dtype=torch.int32))
    with pytest.raises(ValueError, match="2 receive counts for 4 local experts"):
        sort_routing_by_expert(torch.zeros(2, 2, dtype=torch.long), torch.rand(2, 2), 4, (3, 1))


def test_product_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "halo_amd")):
        for name in files:
            if name.endswith(".py"):
                text = open(os.path.join(dirpath, name)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f"{name} imports the oracle"
