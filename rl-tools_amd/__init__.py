"""MI355X (gfx950) backend for the dense-network training hot path of rl-tools: HIP kernels behind a C ABI
(include/rlt_rocm.h), the `devices::ROCM` host headers that bind the reference's overload set to it, and this
ctypes binding used by the tests and the benchmark."""
from . import capi  # noqa: F401
from .capi import Device, DeviceArray, load_library  # noqa: F401
