"""Per-tensor affine quantized tensors: the host mirror of `QuantizedTensor<i8>`
(src/quantization/types.rs:206-276) with the one operation of it that reaches the device,
`qmatmul` (src/quantization/operations.rs:195-260, dispatched by
`OptimizedOps::qmatmul`, src/quantization/hardware/mod.rs:25-46).

The GGUF block formats do not use this type; it is here because Q8_0 with one shared `d`
is its degenerate case (zero point 0) and the reference routes every int8 matmul through it."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .errors import InvalidParameters, ShapeMismatch


@dataclass
class QuantizedTensor:
    data: np.ndarray          # int8, any shape
    scale: float
    zero_point: int = 0

    def __post_init__(self):
        self.data = np.ascontiguousarray(self.data)
        if self.data.dtype != np.int8:
            raise InvalidParameters("QuantizedTensor: data must be int8")
        self.scale = float(np.float32(self.scale))
        self.zero_point = int(self.zero_point)

    @property
    def shape(self):
        return self.data.shape

    def numel(self) -> int:
        return int(self.data.size)

    def ndim(self) -> int:
        return int(self.data.ndim)

    def dequantize(self) -> np.ndarray:
        """(q - zero_point) * scale in f32 (types.rs:270-276)."""
        return (self.data.astype(np.float32) - np.float32(self.zero_point)) * np.float32(self.scale)

    def qmatmul(self, other: "QuantizedTensor", executor) -> "QuantizedTensor":
        """self @ other on the device: exact integer sum, output scale = product of the scales, zero point 0."""
        if self.ndim() < 2 or other.ndim() < 2:
            raise InvalidParameters("Matrix multiplication requires at least 2D tensors")
        if self.shape[-1] != other.shape[-2]:
            raise ShapeMismatch("expected %d, got %d" % (self.shape[-1], other.shape[-2]))
        if self.ndim() != 2 or other.ndim() != 2:
            raise InvalidParameters("Only 2D matrix multiplication currently supported")
        out, scale, zp = executor.qmatmul_i8(self.data, self.scale, self.zero_point, other.data, other.scale, other.zero_point)
        return QuantizedTensor(out, scale, zp)
