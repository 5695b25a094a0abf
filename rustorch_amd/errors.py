"""Status codes of the C ABI mapped onto the reference's error vocabulary.

The class names follow the `RusTorchError` variants the Rust shim would raise
(src/error.rs:15-300 in the reference): a GPU failure is an error, never a
silent CPU fallback (src/gpu/matrix_ops.rs:408-425).
"""


class RusTorchHipError(RuntimeError):
    code = -1


class InvalidParameters(RusTorchHipError):
    code = 1


class ShapeMismatch(RusTorchHipError):
    code = 2


class DeviceNotAvailable(RusTorchHipError):
    code = 3


class OutOfMemory(RusTorchHipError):
    code = 4


class GpuError(RusTorchHipError):
    code = 5


class UnsupportedOperation(RusTorchHipError):
    code = 6


BY_CODE = {c.code: c for c in (InvalidParameters, ShapeMismatch, DeviceNotAvailable, OutOfMemory, GpuError,
                               UnsupportedOperation)}
