"""The C ABI library loads and exports every symbol include/mxconv.h declares
(no device work: runs without a GPU)."""
import ctypes
import os
import re

import poplibs_amd as pa
from poplibs_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mxconv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mxconv_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = _declared_symbols()
    assert len(names) >= 25
    raw = ctypes.CDLL(pa.library_path())
    for name in names:
        assert hasattr(raw, name), name


def test_stamped_twin_exports_the_same_abi_and_its_two_switches():
    """libmxconv_stamps.so (the library with cycle and wall-clock stamps
    compiled into the two benchmark kernels, for tests/tools/kernel_stamps.py)
    is the same C ABI plus one switch per stamped kernel; the product library
    carries neither switch."""
    twin = os.path.join(os.path.dirname(pa.library_path()),
                        "libmxconv_stamps.so")
    assert os.path.exists(twin), "make -C poplibs_amd stamps"
    raw = ctypes.CDLL(twin)
    for name in _declared_symbols():
        assert hasattr(raw, name), name
    product = ctypes.CDLL(pa.library_path())
    for switch in ("mxk_patch_stamp_sink", "mxk_rows_stamp_sink"):
        assert hasattr(raw, switch)
        assert not hasattr(product, switch)


def test_python_binding_declares_every_symbol():
    assert set(_declared_symbols()) == set(pa.lib()._declared)


def test_struct_layout_matches_header():
    # 3 x int32 + pad, 1 + 4 + 4 + 3 u64, 2 x (5*4 u32 + 4 u8), 5*4 u32
    assert ctypes.sizeof(capi.CParams) == 16 + 8 * 12 + 2 * 84 + 80


def test_null_arguments_are_reported_not_crashed():
    L = pa.lib()
    assert L.mxconv_params_validate(None) == capi.Status.NULL_ARGUMENT
    assert b"null" in L.mxconv_last_error()
    assert L.mxconv_status_string(capi.Status.INVALID_OPTION) == \
        b"invalid option"
