"""The C-ABI library loads and exports every symbol include/joshua_hip.h
declares (no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

import pytest

from joshua_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "joshua_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:jq|joshua_npu)_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert declared_symbols() == sorted(capi.EXPORTS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail(f"{capi.LIB_PATH} not built: run `python -m joshua_amd.build`")
    L = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name


def test_block_geometry_needs_no_gpu():
    # reference: src/gguf_ext.rs:483-512
    assert capi.block_geometry(capi.Q4_K) == (256, 144)
    assert capi.block_geometry(capi.Q8_0) == (32, 34)
    assert capi.block_geometry(capi.Q2_K) == (256, 84)
    assert capi.block_geometry(capi.Q6_K) == (256, 210)
    assert capi.block_geometry(capi.IQ2_XXS) == (256, 66)
    assert capi.block_geometry(capi.MXFP4) == (32, 17)
    assert [capi.block_geometry(t) for t in capi.GENERIC_TYPES] == [(32, 18), (32, 20), (32, 22), (32, 24), (256, 110),
                                                                     (256, 176)]
    for unknown in (0, 1, 4, 5, 9, 15, 30, 40):      # no decode kernel: floats, removed ids, Q8_1, Q8_K
        with pytest.raises(capi.JoshuaHipError):
            capi.block_geometry(unknown)
