"""The C-ABI library without a GPU: it loads, exports every symbol the header
declares, answers the geometry queries and refuses compute before init."""
import re

import pytest

from conftest import ROOT
from gufo_npu_amd import capi, synth


def declared_symbols():
    text = (ROOT / "include" / "gufo_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gufo_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load_library()
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(capi.SIGNATURES) == names


def test_block_geometry_without_device():
    assert [capi.block_bytes(t) for t in (12, 13, 14)] == [144, 176, 210]
    assert capi.block_bytes(synth.Q8_0) == 34 and capi.block_bytes(synth.F32) == 4
    assert capi.block_bytes(1) == 0 and capi.block_bytes(30) == 0   # F16, BF16: not taken
    assert capi.row_bytes(synth.Q8_0, 2048) == 2176
    assert capi.row_bytes(synth.F32, 512) == 2048
    assert capi.row_bytes(synth.Q8_0, 2016) == 0   # rows are multiples of 256 values here
    assert capi.row_bytes(synth.Q4_K, 2048) == 1152
    assert capi.row_bytes(synth.Q5_K, 512) == 352
    assert capi.row_bytes(synth.Q6_K, 6144) == 5040
    assert capi.row_bytes(synth.Q6_K, 100) == 0


def test_compute_before_init_is_refused():
    import ctypes as C
    lib = capi.load_library()
    handle = C.c_void_p()
    code = lib.gufo_hip_malloc(C.byref(handle), 64)
    if code == capi.OK:  # a GPU test initialised the library earlier in this process
        lib.gufo_hip_free(handle)
        pytest.skip("library already initialised")
    assert code == capi.ERR_NOT_INITIALIZED
    assert b"gufo_hip_init" in lib.gufo_hip_last_error()


def test_init_without_gpu_reports_no_device():
    import os
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    with pytest.raises(capi.NoDeviceError):
        capi.init(0)
