"""Writes tests/golden/blocks_golden.npz: raw blocks of every format and their
decoded float32 values from the scalar NumPy decoder in tests/np_blocks.py
(independent of the C oracle and of the HIP kernels).

Inputs are deterministic: numpy's PCG64 with a fixed seed for the payload bytes,
plus hand-placed edge blocks (zero scale, largest finite fp16 scale, fp16
subnormal scale, all-0x00 and all-0xFF payloads).  Run from the repo root:
    python tests/golden/make_golden.py
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import np_blocks as nb  # noqa: E402

OUT = Path(__file__).resolve().parent / "blocks_golden.npz"


def scale_bytes(v: float) -> np.ndarray:
    return np.frombuffer(np.float16(v).tobytes(), dtype=np.uint8)


def main() -> None:
    rng = np.random.Generator(np.random.PCG64(20250127))
    out = {}
    for t, (bb, be, fn) in nb.DECODERS.items():
        n = 12
        raw = rng.integers(0, 256, size=(n, bb), dtype=np.uint8)
        d_off = [208] if t == 14 else [108] if t == 11 else [80, 82] if t == 10 else ([0, 2] if t in (12, 13, 3, 7) else [0])     # d (and dmin / m) fields
        scales = rng.uniform(1e-3, 1e-2, size=(n, len(d_off)))
        for i in range(n):
            for k, off in enumerate(d_off):
                raw[i, off:off + 2] = scale_bytes(scales[i, k])
        # edge blocks
        raw[0, d_off[0]:d_off[0] + 2] = scale_bytes(0.0)
        raw[1, d_off[0]:d_off[0] + 2] = scale_bytes(65504.0)
        raw[2, d_off[0]:d_off[0] + 2] = np.array([0x01, 0x00], dtype=np.uint8)  # smallest fp16 subnormal
        raw[3, d_off[0]:d_off[0] + 2] = scale_bytes(-0.0123)
        payload = [i for i in range(bb) if all(not (o <= i < o + 2) for o in d_off)]
        raw[4, payload] = 0x00
        raw[5, payload] = 0xFF
        if t in (8, 9):
            raw[5, payload] = 0x81  # -127: keep away from the unused -128 only in this block
        vals = np.stack([fn(b) for b in raw])
        out["raw_%d" % t] = raw
        out["val_%d" % t] = vals.astype(np.float32)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
