"""Dequant-fused GEMV against the oracle at the benchmark shapes.

Tolerance (stated by the benchmark): max |delta| <= 1e-3 * ||w_row||_2 * ||x||_2 per element.
The kernels are held to a 50x tighter bound against the f64 yardstick."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3          # the benchmark's bound
TIGHT = 2e-5            # what the kernels are actually held to (vs f64 accumulation)

SHAPES = {
    "C1_q8_0": (8, 4096, 4096),
    "C2_q4_0_up": (2, 11008, 4096),
    "C2_q4_0_down": (2, 4096, 11008),
    "C3_q": (12, 4096, 4096),
    "C3_gate": (12, 11008, 4096),
    "C3_v": (14, 4096, 4096),
    "C3_down": (14, 4096, 11008),
    "q5_k_gate": (13, 11008, 4096),          # not a benchmark configuration: the Q5_K_M files' format, same shapes
    "q5_k_down": (13, 4096, 11008),
    "q2_k_gate": (10, 11008, 4096),
    "q2_k_down": (10, 4096, 11008),
    "q3_k_gate": (11, 11008, 4096),
    "q3_k_down": (11, 4096, 11008),
    "q4_1_up": (3, 11008, 4096),             # the older 32-element formats with an offset and / or a fifth bit
    "q5_0_down": (6, 4096, 11008),
    "q5_1_q": (7, 4096, 4096),
    "f16_q": (1, 4096, 4096),                # unquantized matrices: the formats the reference decodes itself
    "f16_down": (1, 4096, 11008),
    "f32_up": (0, 11008, 4096),
}


def check(y, y64, wn, x, what):
    xn = np.linalg.norm(np.atleast_2d(x).astype(np.float64), axis=1)[:, None]
    ratio = np.abs(np.atleast_2d(y) - np.atleast_2d(y64)) / (wn[None, :] * xn)
    worst = ratio.max()
    print("%s: max |delta| / (||w|| ||x||) = %.3e (bound %.0e, held to %.0e)" % (what, worst, REL_TOL, TIGHT), flush=True)
    assert np.isfinite(y).all()
    assert worst <= TIGHT


@pytest.mark.parametrize("name", list(SHAPES))
def test_gemv_config_shapes_batch1_and_8(ex, orc, name):
    from rustorch_amd import synth
    t, rows, cols = SHAPES[name]
    print("gemv", name, t, rows, cols, flush=True)
    raw = synth.blocks(t, 2025, 21, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    x = synth.normal(2025, 22, 8 * cols).reshape(8, cols)
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, x)
    y1 = ex.qgemv(w, x[0])
    check(y1, y64[0], wn, x[0], name + " batch 1")
    y8 = ex.qgemv(w, x)
    check(y8, y64, wn, x, name + " batch 8")
    if t in (12, 14):
        # Q4_K / Q6_K batches stream the weights once on the matrix cores: another summation order than the one-row kernel
        assert np.all(np.abs(y8[0] - y1) <= 2 * TIGHT * wn * np.linalg.norm(x[0].astype(np.float64)))
    else:
        assert np.array_equal(y8[0], y1)                   # a batch row is the single-vector result
    # faithful f32 sequential-sum oracle sits inside the same bound
    yo = orc.qgemv(t, raw, rows, cols, x[:2])
    check(yo, y64[:2], wn, x[:2], name + " oracle f32 vs f64")


@pytest.mark.parametrize("t", [8, 9, 2, 3, 6, 7, 10, 11, 12, 13, 14, 1, 0])
def test_gemv_edge_inputs(ex, orc, t):
    from rustorch_amd import synth
    be = 256 if t in (10, 11, 12, 13, 14) else 32                  # unquantized rows: any multiple of 32 columns
    rows, cols = 5, 3 * be                                  # ragged: fewer rows than a tile, odd block count
    print("gemv edge", t, rows, cols, flush=True)
    raw = synth.blocks(t, 7, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    W = orc.dequant(t, raw, rows, cols).astype(np.float64)
    assert np.array_equal(ex.qgemv(w, np.zeros(cols, np.float32)), np.zeros(rows, np.float32))
    for k in (0, be - 1, cols - 1):
        e = np.zeros(cols, np.float32); e[k] = 1.0
        assert np.allclose(ex.qgemv(w, e), W[:, k], rtol=1e-6, atol=1e-7 * np.abs(W).max())   # one-hot picks a column
    x = synth.normal(7, 2, cols)
    y = ex.qgemv(w, x)
    # two results that are each within the held bound of the exact one (formats with a minimum term cancel heavily,
    # so the yardstick is |w| |x|, not the result itself)
    both = 2 * TIGHT * np.linalg.norm(W, axis=1) * np.linalg.norm(x.astype(np.float64))
    assert np.all(np.abs(ex.qgemv(w, 3 * x) - 3 * y) <= 3 * both)          # linearity
    big = (x * 1e20).astype(np.float32); tiny = (x * 1e-20).astype(np.float32)
    assert np.all(np.abs(ex.qgemv(w, big) / 1e20 - y) <= both)
    assert np.all(np.abs(ex.qgemv(w, tiny) * 1e20 - y) <= both)
    x2 = x.copy(); x2[::2] = 0                                               # blocks with sparse content
    y64 = W @ x2.astype(np.float64)
    assert np.all(np.abs(ex.qgemv(w, x2) - y64) <= TIGHT * np.linalg.norm(W, axis=1) * np.linalg.norm(x2))


@pytest.mark.parametrize("t", [12, 14])
@pytest.mark.parametrize("rows,cols", [(37, 256), (256, 256), (16, 768), (1, 4096), (4099, 2048), (300, 11008), (40000, 512), (48, 28672)])
def test_batches_of_two_to_eight_on_the_matrix_cores(ex, orc, t, rows, cols):
    """Every batch size the one-pass kernel takes, with row counts that do not fill its groups of 16 and k slices that
    leave some of a workgroup's waves without work; rows past the batch must not be written."""
    from rustorch_amd import synth
    print("gemv small batch", t, rows, cols, flush=True)
    raw = synth.blocks(t, 31, 5, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    x = synth.normal(31, 6, 8 * cols).reshape(8, cols)
    x[3, : cols // 2] = 0                                    # a token with empty blocks
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, x)
    for b in range(2, 9):
        check(ex.qgemv(w, x[:b]), y64[:b], wn, x[:b], "type %d %dx%d batch %d" % (t, rows, cols, b))
    assert np.array_equal(ex.qgemv(w, np.zeros((5, cols), np.float32)), np.zeros((5, rows), np.float32))


@pytest.mark.parametrize("t", [12, 14, 8])
def test_rows_longer_than_the_default_lds(ex, orc, t):
    """K = 28 672 (the feed-forward width of a 70B-class model): the staged x is 68 KB, beyond the 64 KB a kernel gets
    without asking."""
    from rustorch_amd import synth
    rows, cols = 768, 28672
    print("gemv long rows", t, rows, cols, flush=True)
    raw = synth.blocks(t, 77, 3, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    x = synth.normal(77, 4, 2 * cols).reshape(2, cols)
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, x)
    check(ex.qgemv(w, x), y64, wn, x, "type %d K=%d" % (t, cols))


def test_grouped_launch_equals_single_launches(ex, orc):
    from rustorch_amd import synth
    specs = [(12, 4096, 4096), (12, 512, 4096), (14, 4096, 4096), (14, 256, 11008), (8, 100, 4096)]
    print("gemv grouped", specs, flush=True)
    ws, xs, ys, want = [], [], [], []
    for i, (t, r, c) in enumerate(specs):
        raw = synth.blocks(t, 99, i, r, c)
        w = ex.upload_qweight(t, r, c, raw)
        x = synth.normal(99, 50 + i, c)
        ws.append(w); xs.append(ex.to_device(x)); ys.append(ex.buffer(r * 4)); want.append(ex.qgemv(w, x))
    ex.qgemv_grouped_dev(ws, xs, ys)
    for y, wv in zip(ys, want):
        assert np.array_equal(y.download(np.float32), wv)


@pytest.mark.parametrize("batch", [1, 2, 5, 8])
def test_several_weights_against_one_batch(ex, orc, batch):
    """q / k / v of an attention block and gate / up of a feed-forward block meet the same rows: one quantizing launch,
    the Q4_K matrices in one launch and the Q6_K ones in another; a format the matrix-core kernel does not take (Q8_0) and
    batches below three run per weight."""
    from rustorch_amd import synth, ShapeMismatch
    cols = 2048
    specs = [(12, 1024), (12, 1024), (14, 512), (12, 37), (8, 256), (12, 2048), (14, 96)]
    print("gemv shared x", specs, "batch", batch, flush=True)
    x = synth.normal(98, 1, 8 * cols).reshape(8, cols)[:batch]
    dx = ex.to_device(x)
    ws, ys, raws = [], [], []
    for i, (t, r) in enumerate(specs):
        raw = synth.blocks(t, 98, 10 + i, r, cols)
        raws.append(raw); ws.append(ex.upload_qweight(t, r, cols, raw)); ys.append(ex.buffer(8 * r * 4))
    ex.qgemv_shared_x_dev(ws, dx, ys, batch)
    for (t, r), raw, w, y in zip(specs, raws, ws, ys):
        y64, wn = orc.qgemv_f64(t, raw, r, cols, x)
        got = y.download(np.float32, batch * r).reshape(batch, r)
        check(got, y64, wn, x, "type %d rows %d batch %d" % (t, r, batch))
        single = np.atleast_2d(ex.qgemv(w, x))
        assert np.all(np.abs(got - single) <= 2 * TIGHT * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None])
    other = ex.upload_qweight(12, 64, 1024, synth.blocks(12, 98, 30, 64, 1024))
    with pytest.raises(ShapeMismatch):
        ex.qgemv_shared_x_dev([ws[0], other], dx, ys[:2], batch)          # another number of columns


def test_device_pointer_form_and_errors(ex, orc):
    from rustorch_amd import synth, InvalidParameters, ShapeMismatch
    raw = synth.blocks(12, 3, 3, 64, 512)
    w = ex.upload_qweight(12, 64, 512, raw)
    x = synth.normal(3, 4, 2 * 512).reshape(2, 512)
    dx, dy = ex.to_device(x), ex.buffer(2 * 64 * 4)
    ex.qgemv_dev(w, dx, dy, 2)
    assert np.array_equal(dy.download(np.float32).reshape(2, 64), ex.qgemv(w, x))
    with pytest.raises(InvalidParameters):
        ex.qgemv_dev(w, dx, dy, 9)
    with pytest.raises(ShapeMismatch):
        ex.qgemv(w, np.zeros(100, np.float32))


def test_dense_matmul_f32_kat(ex):
    # src/tensor/ops/matrix.rs:328-336 through the executor signature of src/gpu/cuda_kernels.rs:231-239
    a = np.array([1, 2, 3, 4], dtype=np.float32); b = np.array([5, 6, 7, 8], dtype=np.float32)
    c = np.zeros(4, dtype=np.float32)
    ex.matmul_f32(a, b, c, 2, 2, 2)
    assert np.array_equal(c, np.array([19, 22, 43, 50], dtype=np.float32))
    rng = np.random.default_rng(0)
    A = rng.standard_normal((70, 45)).astype(np.float32); B = rng.standard_normal((45, 33)).astype(np.float32)
    Cm = np.zeros((70, 33), dtype=np.float32)
    ex.matmul_f32(A, B, Cm, 70, 33, 45)
    assert np.allclose(Cm, A.astype(np.float64) @ B.astype(np.float64), rtol=1e-5, atol=1e-5)
    # A . I == A, the check GpuValidator::validate_matrix_multiplication runs (src/gpu/validation.rs:116-166)
    I = np.eye(45, dtype=np.float32); out = np.zeros((70, 45), dtype=np.float32)
    ex.matmul_f32(A, I, out, 70, 45, 45)
    assert np.array_equal(out, A)


def test_dense_matmul_on_resident_buffers_and_batches(ex):
    """The dense product on device buffers that stay resident between calls (GpuBuffer, src/gpu/memory_ops/buffer.rs:22-48):
    the reference's known answer (src/tensor/ops/matrix.rs:328-336), a batch of products in one launch against NumPy f64
    (gpu_batch_matmul, src/gpu/matrix_ops.rs:562-595), the matrix-vector form (gpu_matvec: n = 1), and the same bits as the
    host-slice entry point."""
    from rustorch_amd import ShapeMismatch
    a = ex.to_device(np.array([1, 2, 3, 4], dtype=np.float32)); b = ex.to_device(np.array([5, 6, 7, 8], dtype=np.float32))
    c = ex.buffer(16)
    ex.matmul_f32_dev(a, b, c, 2, 2, 2)
    assert np.array_equal(c.download(np.float32), np.array([19, 22, 43, 50], dtype=np.float32))
    rng = np.random.default_rng(1)
    batch, m, n, k = 5, 70, 33, 45
    A = rng.standard_normal((batch, m, k)).astype(np.float32); B = rng.standard_normal((batch, k, n)).astype(np.float32)
    dA, dB, dC = ex.to_device(A), ex.to_device(B), ex.buffer(4 * batch * m * n)
    ex.matmul_f32_dev(dA, dB, dC, m, n, k, batch)
    got = dC.download(np.float32).reshape(batch, m, n)
    assert np.allclose(got, A.astype(np.float64) @ B.astype(np.float64), rtol=1e-5, atol=1e-5)
    one = np.zeros((m, n), dtype=np.float32)
    ex.matmul_f32(A[3], B[3], one, m, n, k)
    assert np.array_equal(got[3], one)
    ex.matmul_f32_dev(dA, dB, dC, m, n, k, batch)               # the operands are still there: no upload between the calls
    assert np.array_equal(dC.download(np.float32).reshape(batch, m, n), got)
    v = ex.to_device(B[0][:, 0].copy()); y = ex.buffer(4 * m)
    ex.matmul_f32_dev(dA, v, y, m, 1, k)
    assert np.allclose(y.download(np.float32), A[0].astype(np.float64) @ B[0][:, 0].astype(np.float64), rtol=1e-5, atol=1e-5)
    with pytest.raises(ShapeMismatch):
        ex.matmul_f32_dev(dA, dB, c, m, n, k, batch)
    for buf in (a, b, c, dA, dB, dC, v, y):
        buf.free()
