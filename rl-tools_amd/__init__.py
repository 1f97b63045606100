"""MI355X (gfx950) backend for the dense-network training hot path of rl-tools: HIP kernels (csrc/) behind a C ABI
(include/rlt_rocm.h, librlt_rocm.so next to this file) and this ctypes binding used by the tests and the benchmark (capi.py), with builders of networks and agents over it (builders.py). The C++ header layer
that binds the reference's own API to the C ABI (a `devices::ROCM` tag and its overloads) is under include/rl_tools/."""
from . import capi  # noqa: F401
from . import builders  # noqa: F401
from .capi import Device, DeviceArray, load_library  # noqa: F401
