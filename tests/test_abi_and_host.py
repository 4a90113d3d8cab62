"""CPU-only checks of the boundary: the shared library loads, exports every symbol the header
declares (and nothing is declared twice), and the host-side format helpers keep the
reference's rejections.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

import helpers
import karume_amd
from karume_amd import _ffi

HEADER = os.path.join(helpers.ROOT, "include", "karume_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(krm_[a-z0-9_]+)\s*\(", text)


def test_header_symbols_are_exported_and_bound():
    names = declared_symbols()
    assert len(names) == len(set(names)) and len(names) >= 20
    lib = ctypes.CDLL(_ffi.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in karume_hip.h but not exported"
    assert set(names) == set(_ffi.PROTOTYPES), "ctypes prototypes and header disagree"
    loaded = _ffi.load()
    assert loaded.krm_version().decode().startswith("karume-hip")


def test_last_error_without_context_is_a_string():
    lib = _ffi.load()
    assert isinstance(lib.krm_last_error(None), bytes)
    # Context-less size queries need no device.
    nbytes = ctypes.c_size_t()
    assert lib.krm_attention_state_workspace(1, 32, 8, 1, 128, 0, 4095, 1,
                                             ctypes.byref(nbytes)) == 0
    assert nbytes.value >= 32 * 32 * 130 * 4
    assert lib.krm_attention_varlen_workspace(16, 32, 8, 128, 40000, ctypes.byref(nbytes)) == 0
    assert nbytes.value > 0


def test_pack_int4_matches_reference_vectors():
    # packages/runtime/tests/format_i4_test.ts:10-15, tools/exporter/tests/test_emit.py:588-600
    assert karume_amd.pack_int4(np.array([1, 2])).tolist() == [0xA9]
    assert karume_amd.pack_int4(np.array([-7, 7, 0, -7])).tolist() == [0xF1, 0x18]
    q = np.arange(-8, 8)
    assert np.array_equal(karume_amd.pack_int4(q), helpers.oracle.pack_i4(q))
    with pytest.raises(karume_amd.I4Error):
        karume_amd.pack_int4(np.array([1, 2, 3]))
    with pytest.raises(karume_amd.I4Error):
        karume_amd.pack_int4(np.array([8, 0]))


def test_check_int4_rejections():
    # packages/runtime/tests/format_i4_test.ts:108-141
    assert karume_amd.group_scale_shape([2, 4, 4], 8) == [2, 2]
    karume_amd.check_int4(8, [2, 8], [2, 2], 4)
    with pytest.raises(karume_amd.I4Error):
        karume_amd.check_int4(7, [2, 8], [2, 1], 8)
    with pytest.raises(karume_amd.I4Error):
        karume_amd.check_int4(8, [2, 8], [2, 1], 4)
    with pytest.raises(karume_amd.I4Error):
        karume_amd.check_int4(8, [2, 8], [2, 1], 3)
    with pytest.raises(karume_amd.I4Error):
        karume_amd.check_int4(0, [], [], 16)


def test_product_package_does_not_touch_the_oracle():
    """The oracle is test infrastructure: nothing under karume_amd/ may import or load it."""
    pkg = os.path.join(helpers.ROOT, "karume_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        for name in files:
            if name.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, name)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, name)
