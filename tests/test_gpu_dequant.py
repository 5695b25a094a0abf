"""Block decode on the GPU is bit-exact against the oracle and the committed golden vectors."""
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden" / "blocks_golden.npz"


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("t", [8, 9, 2, 3, 6, 7, 10, 11, 12, 13, 14])
def test_golden_vectors_bit_exact(ex, t):
    g = np.load(GOLDEN)
    raw, val = g["raw_%d" % t], g["val_%d" % t]
    print("dequant golden type", t, flush=True)
    w = ex.upload_qweight(t, raw.shape[0], val.shape[1], raw)
    got = ex.dequant(w)
    assert np.array_equal(bits(got), bits(val))   # includes zero, max-finite and subnormal fp16 scales


@pytest.mark.parametrize("t,rows,cols", [(8, 64, 4096), (2, 33, 11008), (12, 48, 4096), (12, 17, 11008), (14, 40, 4096), (14, 9, 11008), (13, 48, 4096), (13, 5, 11008),
                                         (9, 33, 4096), (9, 7, 11008), (3, 33, 4096), (6, 33, 11008), (7, 20, 4096), (1, 9, 4096), (0, 5, 1024), (11, 40, 4096), (11, 7, 11008), (10, 40, 4096), (10, 7, 11008)])
def test_synthetic_tensors_bit_exact(ex, orc, t, rows, cols):
    from rustorch_amd import synth
    print("dequant synthetic", t, rows, cols, flush=True)
    raw = synth.blocks(t, 2024, 11, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    assert w.nbytes == raw.nbytes
    assert np.array_equal(bits(ex.dequant(w)), bits(orc.dequant(t, raw, rows, cols)))


def test_upload_validates_payload(ex):
    from rustorch_amd import ShapeMismatch, UnsupportedOperation
    raw = np.zeros(144 * 4, dtype=np.uint8)
    with pytest.raises(ShapeMismatch):
        ex.upload_qweight(12, 4, 250, raw)         # not a multiple of the block
    with pytest.raises(ShapeMismatch):
        ex.upload_qweight(12, 5, 256, raw)         # byte count does not match
    with pytest.raises(ShapeMismatch):
        ex.upload_qweight(12, 0, 256, raw[:0])     # empty tensor
    with pytest.raises(UnsupportedOperation):
        ex.upload_qweight(15, 4, 256, raw)         # Q8_K: listed by the enum, an activation format with no kernel here
