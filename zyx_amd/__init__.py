"""MI355X (gfx950) HIP device backend for zyx: host-side mirror of the backend plugin
interface (`MemoryPool::HIP` / `Device::HIP`, zyx/src/backend/mod.rs, zyx/src/backend/hip.rs)
over the C ABI in ``include/zyx_hip.h``. All compute happens in ``libzyx_hip.so``; there is
no CPU fallback -- a missing library or GPU raises ``BackendError``.
"""
from .backend import (  # noqa: F401
    BackendError,
    DType,
    DeviceInfo,
    ErrorStatus,
    Event,
    HIPConfig,
    HIPDevice,
    HIPMemoryPool,
    KernelDesc,
    initialize_device,
    library_path,
)
from . import kernels  # noqa: F401
from . import safetensors_io  # noqa: F401
from . import ir  # noqa: F401
from . import graph  # noqa: F401

__all__ = ["BackendError", "DType", "DeviceInfo", "ErrorStatus", "Event", "HIPConfig", "HIPDevice", "HIPMemoryPool",
           "KernelDesc", "initialize_device", "library_path", "kernels"]
