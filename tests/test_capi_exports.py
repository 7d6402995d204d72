"""CPU: the C-ABI library loads and exports every symbol include/otter_hip_int8.h declares (no compute)."""
import os
import re

import pytest

from tensor_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "otter_hip_int8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(otter_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail("%s missing: run __graft_entry__.build()" % capi.LIB_PATH)
    lib = capi.load_cdll()
    names = declared_symbols()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), "library does not export " + name
    assert set(capi.EXPORTS) <= set(names)


def test_no_cpu_fallback_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError):
        capi.Library()
