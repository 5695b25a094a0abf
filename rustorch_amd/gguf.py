"""GGML tensor types as the reference's GGUF loader names them.

Mirrors `GGMLType` / `from_u32` / `type_size` of
example-cli/src/model/formats/gguf.rs:78-144 (same ids, same bytes per block).
"""
from __future__ import annotations

import enum


class GGMLType(enum.IntEnum):
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q8_1 = 9
    Q2_K = 10
    Q3_K = 11
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14
    Q8_K = 15
    I8 = 16
    I16 = 17
    I32 = 18

    @classmethod
    def from_u32(cls, value: int) -> "GGMLType":
        try:
            return cls(value)
        except ValueError:
            raise ValueError("Unknown GGML type: %d" % value) from None

    def type_size(self) -> int:
        """Bytes per block (per element for the plain types)."""
        return _TYPE_SIZE[self]

    def block_elems(self) -> int:
        """Elements per block."""
        if self in (GGMLType.Q2_K, GGMLType.Q3_K, GGMLType.Q4_K, GGMLType.Q5_K, GGMLType.Q6_K, GGMLType.Q8_K):
            return 256
        if self in (GGMLType.Q4_0, GGMLType.Q4_1, GGMLType.Q5_0, GGMLType.Q5_1, GGMLType.Q8_0, GGMLType.Q8_1):
            return 32
        return 1

    def row_bytes(self, n_cols: int) -> int:
        be = self.block_elems()
        if n_cols % be:
            raise ValueError("n_cols=%d is not a multiple of the block size %d" % (n_cols, be))
        return n_cols // be * self.type_size()


_TYPE_SIZE = {
    GGMLType.F32: 4, GGMLType.I32: 4, GGMLType.F16: 2, GGMLType.I16: 2, GGMLType.I8: 1,
    GGMLType.Q4_0: 18, GGMLType.Q4_1: 20, GGMLType.Q5_0: 22, GGMLType.Q5_1: 24, GGMLType.Q8_0: 34,
    GGMLType.Q8_1: 36, GGMLType.Q2_K: 82, GGMLType.Q3_K: 110, GGMLType.Q4_K: 144, GGMLType.Q5_K: 176,
    GGMLType.Q6_K: 210, GGMLType.Q8_K: 292,
}
