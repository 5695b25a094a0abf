"""rustorch_amd: MI355X (gfx950) backend for RusTorch's GGUF quantized-inference hot path.

The product is `librustorch_hip` (hand-written HIP kernels behind a C ABI, see
`include/rustorch_hip.h`).  This package is the host-side harness that mirrors
the reference's executor interface on top of that ABI through ctypes; the only
arithmetic it holds is the CLI's host-side token sampling (`sampling.py`), and it
raises if the native library is missing.
"""
from .errors import (  # noqa: F401
    RusTorchHipError, InvalidParameters, ShapeMismatch, DeviceNotAvailable, OutOfMemory, GpuError,
    UnsupportedOperation,
)
from .gguf import GGMLType  # noqa: F401

__all__ = [
    "RusTorchHipError", "InvalidParameters", "ShapeMismatch", "DeviceNotAvailable", "OutOfMemory", "GpuError",
    "UnsupportedOperation", "GGMLType",
]
