"""CPU-side checks of the C-ABI library: it loads, exports every symbol include/zyx_hip.h
declares, and reports a missing GPU through the reference's error statuses."""
import ctypes
import os
import re

import pytest

import zyx_amd
from zyx_amd import backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "zyx_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(zhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = backend.load_library()
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/zyx_hip.h but not exported"
    assert sorted(backend._EXPORTS) == names


def test_struct_layouts_match_header():
    assert ctypes.sizeof(backend.KernelDesc) == 4 * 4 + 8 * 8 + 8 * 4 + 24 * 4
    assert ctypes.sizeof(backend._Config) == 16


def test_error_status_values_follow_reference_order():
    # zyx/src/error.rs:125-153
    names = ["DyLibNotFound", "Initialization", "Deinitialization", "DeviceEnumeration", "DeviceQuery",
             "MemoryAllocation", "MemoryDeallocation", "MemoryCopyH2P", "MemoryCopyP2H", "IncorrectKernelArg",
             "KernelCompilation", "KernelLaunch", "KernelSync"]
    assert [s.name for s in zyx_amd.ErrorStatus] == names
    assert [int(s) for s in zyx_amd.ErrorStatus] == list(range(1, 14))


def test_disabled_backend_raises_like_reference():
    # device_ids: Some([]) disables the backend (zyx/src/backend/hip.rs:128-135)
    with pytest.raises(zyx_amd.BackendError) as ei:
        zyx_amd.initialize_device(zyx_amd.HIPConfig(device_ids=[]))
    assert ei.value.status == zyx_amd.ErrorStatus.Initialization


def test_no_gpu_is_an_error_not_a_fallback():
    try:
        n = backend.device_count()
    except zyx_amd.BackendError as e:
        assert e.status == zyx_amd.ErrorStatus.DeviceEnumeration
        return
    if n == 0:
        with pytest.raises(zyx_amd.BackendError):
            zyx_amd.initialize_device()
