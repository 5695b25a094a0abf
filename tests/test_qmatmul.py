"""Per-tensor affine int8 matmul (src/quantization/operations.rs:195-260): oracle against the reference's own
test vectors and a brute-force restatement; the GPU kernel against the oracle, bit for bit."""
import numpy as np
import pytest

from oracle import oracle as orc_mod


def brute(a, sa, za, b, sb, zb):
    """int64 sum, then the float round trip the reference writes, in numpy scalars."""
    s = (a.astype(np.int64) - za) @ (b.astype(np.int64) - zb)
    scale = np.float32(sa) * np.float32(sb)
    with np.errstate(all="ignore"):
        fp = s.astype(np.float32) * scale
        q = fp / scale
    q = np.where(np.isnan(q), np.float32(0), q)
    r = np.sign(q) * np.floor(np.abs(q) + np.float32(0.5))          # halves away from zero, as f32::round
    return np.clip(r, -128, 127).astype(np.int8), float(scale)


def test_reference_vector_and_scale():
    # test_quantized_matmul (operations.rs:569-585), test_qmatmul_i8_optimized (hardware/cpu.rs:428-442)
    a = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.int8)
    b = np.array([[7, 8], [9, 10], [11, 12]], dtype=np.int8)
    out, scale, zp = orc_mod.qmatmul_i8(a, 0.1, 0, b, 0.1, 0)
    assert out.shape == (2, 2) and zp == 0
    assert np.float32(scale) == np.float32(0.1) * np.float32(0.1)
    assert out.tolist() == [[58, 64], [127, 127]]                     # 139 and 154 saturate


def test_oracle_against_brute_force():
    rng = np.random.default_rng(5)
    for m, n, k, za, zb, sa, sb in ((3, 5, 7, 0, 0, 0.1, 0.1), (17, 9, 130, 3, -4, 0.02, 0.5), (8, 8, 64, -128, 127, 1.0, 1.0),
                                    (4, 4, 4, 0, 0, 0.0, 1.0), (5, 6, 33, 1024, -1024, 3e-3, 7e-3)):
        a = rng.integers(-128, 128, (m, k)).astype(np.int8); b = rng.integers(-128, 128, (k, n)).astype(np.int8)
        if k <= 8:                                              # keep some sums inside the int8 range
            a = (a // 32).astype(np.int8); b = (b // 32).astype(np.int8)
        got, scale, _ = orc_mod.qmatmul_i8(a, sa, za, b, sb, zb)
        exp, escale = brute(a, sa, za, b, sb, zb)
        assert np.float32(scale) == np.float32(escale)
        assert np.array_equal(got, exp), (m, n, k)


def test_host_mirror_dequantize_and_errors():
    from rustorch_amd.quantized import QuantizedTensor
    from rustorch_amd.errors import InvalidParameters, ShapeMismatch
    q = QuantizedTensor(np.array([[10, 20], [30, 40]], dtype=np.int8), 0.1, 0)       # types.rs:431-443
    assert np.allclose(q.dequantize().ravel(), [1.0, 2.0, 3.0, 4.0], atol=1e-6)
    assert q.numel() == 4 and q.ndim() == 2 and q.shape == (2, 2)
    z = QuantizedTensor(np.array([[1, 2, 3]], dtype=np.int8), 0.5, 1)
    assert np.array_equal(z.dequantize(), np.array([[0.0, 0.5, 1.0]], dtype=np.float32))
    with pytest.raises(ShapeMismatch):
        q.qmatmul(z, executor=None)
    with pytest.raises(InvalidParameters):
        QuantizedTensor(np.zeros((2, 2), dtype=np.int8), 1.0).qmatmul(QuantizedTensor(np.zeros((2, 2, 2), dtype=np.int8), 1.0), executor=None)
    with pytest.raises(InvalidParameters):
        QuantizedTensor(np.zeros(3, dtype=np.float32), 1.0)


@pytest.mark.gpu
def test_gpu_qmatmul_i8_matches_oracle(ex):
    from rustorch_amd.quantized import QuantizedTensor
    from rustorch_amd.errors import InvalidParameters
    rng = np.random.default_rng(6)
    cases = [(2, 2, 3, 0, 0, 0.1, 0.1), (64, 64, 64, 0, 0, 0.05, 0.05), (65, 130, 200, 5, -7, 0.01, 0.2), (1, 1, 1, 0, 0, 1.0, 1.0),
             (300, 17, 1000, -128, 127, 1e-3, 1e-3), (33, 70, 4096, 1024, -1024, 2e-3, 4e-3), (7, 9, 5, 0, 0, 0.0, 1.0)]
    for m, n, k, za, zb, sa, sb in cases:
        print("qmatmul_i8", m, n, k, za, zb, flush=True)
        a = rng.integers(-128, 128, (m, k)).astype(np.int8); b = rng.integers(-128, 128, (k, n)).astype(np.int8)
        if k <= 8:
            a = (a // 32).astype(np.int8); b = (b // 32).astype(np.int8)
        exp, escale, _ = orc_mod.qmatmul_i8(a, sa, za, b, sb, zb)
        got, scale, zp = ex.qmatmul_i8(a, sa, za, b, sb, zb)
        assert zp == 0 and np.float32(scale) == np.float32(escale)
        assert np.array_equal(got, exp), (m, n, k)
    # sparse operands keep the sums small, so the whole int8 range is exercised, not only the saturated ends
    a = np.zeros((40, 256), dtype=np.int8); b = np.zeros((256, 50), dtype=np.int8)
    a[np.arange(40), rng.integers(0, 256, 40)] = rng.integers(-11, 12, 40)
    b[rng.integers(0, 256, 200), rng.integers(0, 50, 200)] = rng.integers(-11, 12, 200)
    exp, _, _ = orc_mod.qmatmul_i8(a, 0.1, 0, b, 0.1, 0)
    got, _, _ = ex.qmatmul_i8(a, 0.1, 0, b, 0.1, 0)
    assert np.array_equal(got, exp)
    # the reference's own vector through the tensor mirror
    r = QuantizedTensor(np.array([[1, 2, 3], [4, 5, 6]], dtype=np.int8), 0.1).qmatmul(
        QuantizedTensor(np.array([[7, 8], [9, 10], [11, 12]], dtype=np.int8), 0.1), ex)
    assert r.data.tolist() == [[58, 64], [127, 127]] and r.zero_point == 0 and np.float32(r.scale) == np.float32(0.1) * np.float32(0.1)
    with pytest.raises(InvalidParameters):
        ex.qmatmul_i8(a, 0.1, 5000, b, 0.1, 0)
