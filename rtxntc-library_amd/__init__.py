"""MI355X-native decoder for LibNTC texture sets: Python plumbing over csrc/libntc_hip.so.

The product is the shared library (HIP kernels + C ABI, include/ntc_hip.h) and the C++
host layer in host/.  This package only assembles descriptors, generates seeded synthetic
inputs and calls the C ABI through ctypes for the tests and the benchmark.
"""
from . import abi, presets, synth, device  # noqa: F401
from .abi import NtcHipError, load_library  # noqa: F401
from .device import Device, DeviceBuffer, make_texture_set  # noqa: F401
