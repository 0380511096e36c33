"""CPU-side checks of the boundary: the library loads, exports every symbol the header
declares, and the Python binding table covers exactly those symbols."""
import os
import re

from amct_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "amct_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(amct_[a-z0-9_]+)\s*\(", text))


def test_header_symbols_exported_and_bound():
    names = header_functions()
    assert "amct_gemm_w8a8" in names and len(names) >= 17
    lib = _lib.load()
    for n in names:
        assert hasattr(lib, n), n
    assert names == set(_lib.SIGNATURES), names ^ set(_lib.SIGNATURES)


def test_version_and_errors_without_gpu():
    lib = _lib.load()
    assert lib.amct_hip_version() >= 100
    assert b"bad argument" in lib.amct_hip_strerror(-1)
    # argument validation happens before any HIP call, so it works without a GPU
    assert lib.amct_minmax(None, None, None, 1, 1, 0, 0, None) == -1
    assert lib.amct_mx_quant(None, None, None, 1, 32, 0, 0, 2, None) == -1
    assert lib.amct_gemm_w8a8(None, None, None, None, None, 0, None, None, 1, 1, 1, 2, None) == -1


def test_cpu_tensors_are_rejected_loudly():
    import pytest
    import torch
    from amct_amd import ops
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.minmax(torch.zeros(4, 32))
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.fakequant_int(torch.zeros(4, 32), 8, True)
