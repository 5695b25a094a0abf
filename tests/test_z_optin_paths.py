"""Code paths that are switched on by request (rt_hip_set_option), each against the same checks as the default path it
stands in for.  The file sorts after the other GPU tests on purpose: under `pytest -x` a failure here cannot hide them.

  * the lean decode GEMV (Q4_K / Q6_K / Q8_0 / Q4_0, rt_gemv_lean.h): the benchmark's matrices, edge inputs, grouped
    launches, in-place residuals through the model's decode step, and its bits against the general kernel's;
  * the dense f32 product on the matrix cores (v_mfma_f32_32x32x2f32)."""
import numpy as np
import pytest

import test_gpu_gemv as base

pytestmark = pytest.mark.gpu

LEAN_TYPES = (8, 2, 12, 14)


@pytest.fixture(params=[1, 2], ids=["lean", "lean-five-waves"])
def lean(ex, request):
    """1: the lean kernel at four waves per SIMD; 2: launches without a gate / up pair run its 640-thread, five-wave form."""
    ex.set_option(ex.OPT_GEMV_LEAN, request.param)
    assert ex.get_option(ex.OPT_GEMV_LEAN) == request.param
    yield request.param
    ex.set_option(ex.OPT_GEMV_LEAN, 0)


@pytest.fixture
def dense_mfma(ex):
    ex.set_option(ex.OPT_DENSE_MFMA, 1)
    yield
    ex.set_option(ex.OPT_DENSE_MFMA, 0)


def test_options_are_refused_when_unknown(ex):
    from rustorch_amd import InvalidParameters
    assert ex.get_option(ex.OPT_GEMV_LEAN) in (0, 1)
    with pytest.raises(InvalidParameters):
        ex.set_option(99, 1)
    with pytest.raises(InvalidParameters):
        ex.set_option(ex.OPT_GEMV_LEAN, 3)
    with pytest.raises(InvalidParameters):
        ex.set_option(ex.OPT_DENSE_MFMA, 2)
    with pytest.raises(InvalidParameters):
        ex.get_option(0)


@pytest.mark.parametrize("t", LEAN_TYPES)
def test_lean_gemv_edge_inputs(ex, orc, lean, t):
    """Rows shorter than one pass, fewer rows than waves, one-hot and scaled inputs."""
    base.test_gemv_edge_inputs(ex, orc, t)


@pytest.mark.parametrize("name", ["C1_q8_0", "C2_q4_0_up", "C2_q4_0_down", "C3_q", "C3_gate", "C3_v", "C3_down"])
def test_lean_gemv_config_shapes(ex, orc, lean, name):
    base.test_gemv_config_shapes_batch1_and_8(ex, orc, name)


@pytest.mark.parametrize("t,rows,cols", [(12, 4096, 4096), (14, 4096, 4096), (8, 4096, 2048), (2, 5504, 2048), (12, 77, 1024), (14, 5, 768), (8, 5, 96)])
@pytest.mark.parametrize("value", [1, 2])
def test_lean_rows_of_one_pass_have_the_general_kernels_bits(ex, t, rows, cols, value):
    """Same x layout and the same arithmetic per unit: a row of one pass (64 units: 4096 elements of Q4_K / Q6_K, 2048 of
    Q8_0 / Q4_0) must come out bit for bit as from the general kernel."""
    from rustorch_amd import synth
    raw = synth.blocks(t, 41, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    x = synth.normal(41, 2, 2 * cols).reshape(2, cols)
    ex.set_option(ex.OPT_GEMV_LEAN, 0)
    y_general = ex.qgemv(w, x)
    ex.set_option(ex.OPT_GEMV_LEAN, value)
    try:
        print("launch:", ex.qgemv_describe([w]), flush=True)
        y_lean = ex.qgemv(w, x)
    finally:
        ex.set_option(ex.OPT_GEMV_LEAN, 0)
    print("lean (%d) vs general, type %d %d x %d: %d of %d elements differ" % (value, t, rows, cols, int((y_lean != y_general).sum()), y_lean.size), flush=True)
    assert np.array_equal(y_lean, y_general)


def test_lean_grouped_launch_equals_single_launches(ex, orc, lean):
    base.test_grouped_launch_equals_single_launches(ex, orc)


def test_lean_long_rows_stay_within_the_held_bound_of_the_general_kernel(ex, orc):
    """Rows of several passes (K = 11008) add their passes' wave sums in another order than the general kernel: both within
    the held bound of the f64 products, and the lean result the same whether the row stands alone or in a grouped launch."""
    from rustorch_amd import synth
    t, rows, cols = 14, 4096, 11008
    raw = synth.blocks(t, 43, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    x = synth.normal(43, 2, cols)
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, x)
    y_general = ex.qgemv(w, x)
    ex.set_option(ex.OPT_GEMV_LEAN, 1)
    try:
        y_lean = ex.qgemv(w, x)
        ex.set_option(ex.OPT_GEMV_LEAN, 2)
        assert np.array_equal(ex.qgemv(w, x), y_lean)        # the cut of a launch (here: ten waves per workgroup) never changes a result
        other = ex.upload_qweight(12, 512, 4096, synth.blocks(12, 43, 3, 512, 4096))
        dx, dx2 = ex.to_device(x), ex.to_device(synth.normal(43, 4, 4096))
        dy, dy2 = ex.buffer(rows * 4), ex.buffer(512 * 4)
        ex.qgemv_grouped_dev([w, other], [dx, dx2], [dy, dy2])
        y_grouped = dy.download(np.float32)
    finally:
        ex.set_option(ex.OPT_GEMV_LEAN, 0)
    base.check(y_general, y64, wn, x, "general, rows of three passes")
    base.check(y_lean, y64, wn, x, "lean, rows of three passes")
    assert np.array_equal(y_lean, y_grouped)


def test_lean_decode_steps_match_the_general_path_and_the_oracle(ex, orc):
    """A small model's decode steps (RMSNorm-staged q/k/v and gate/up with the SwiGLU pair form, in-place residual adds) with
    the lean GEMV against the same steps with the general one and against the oracle."""
    from rustorch_amd import llama
    cfg = dict(n_layers=2, hidden=512, n_heads=4, ffn=1536, vocab=320, max_pos=16)
    om = orc.OracleLlama(**cfg)
    toks = [3, 77, 100, 5, 319]
    logits = {}
    for which in (0, 1, 2):
        ex.set_option(ex.OPT_GEMV_LEAN, which)
        try:
            gm = llama.HipLlama(ex, **cfg)
            llama.load_synthetic(gm, 11, om.set_tensor if which == 0 else None)
            out = []
            for p, t in enumerate(toks):
                gm.step(t, p)
                out.append(gm.logits().copy())
            gm.close()
        finally:
            ex.set_option(ex.OPT_GEMV_LEAN, 0)
        logits[which] = np.stack(out)
    want = om.forward(toks, 0)
    scale = np.abs(want).max(axis=1)[:, None]
    for which in (0, 1, 2):
        err = np.abs(logits[which] - want).max()
        print("decode steps, lean %d: max |delta logit| %.3e (logit scale %.3e)" % (which, err, scale.max()), flush=True)
        assert np.all(np.abs(logits[which] - want) <= 1e-3 * scale + 1e-3)
    assert np.all(np.abs(logits[1] - logits[0]) <= 2e-4 * scale + 1e-4) and np.all(np.abs(logits[2] - logits[0]) <= 2e-4 * scale + 1e-4)


@pytest.mark.parametrize("batch,m,n,k", [(1, 128, 128, 16), (3, 200, 136, 72), (1, 130, 132, 20), (2, 64, 64, 260), (1, 257, 384, 128), (1, 96, 64, 64)])
def test_dense_matmul_on_the_matrix_cores(ex, dense_mfma, batch, m, n, k):
    """Products whose rows are whole 16-byte pieces and that fill tiles take the f32 matrix-core kernel (whole tiles, ragged
    edges in m, n and k, batches): against NumPy f64, held to 4 * sqrt(k) roundings of the row and column norms; a
    product with the identity returns its operand bit for bit (GpuValidator::validate_matrix_multiplication,
    src/gpu/validation.rs:116-166)."""
    print("dense matmul on the matrix cores: batch %d, %d x %d x %d" % (batch, m, n, k), flush=True)
    rng = np.random.default_rng(m + n + k)
    A = rng.standard_normal((batch, m, k)).astype(np.float32); B = rng.standard_normal((batch, k, n)).astype(np.float32)
    dA, dB, dC = ex.to_device(A), ex.to_device(B), ex.buffer(4 * batch * m * n)
    ex.matmul_f32_dev(dA, dB, dC, m, n, k, batch)
    got = dC.download(np.float32).reshape(batch, m, n)
    want = A.astype(np.float64) @ B.astype(np.float64)
    bound = 4 * np.sqrt(k) * 2.0 ** -24 * np.linalg.norm(A.astype(np.float64), axis=2)[:, :, None] * np.linalg.norm(B.astype(np.float64), axis=1)[:, None, :]
    assert np.isfinite(got).all() and np.all(np.abs(got - want) <= bound)
    if k == n:
        eye = np.broadcast_to(np.eye(k, dtype=np.float32), (batch, k, k)).copy()
        dI = ex.to_device(eye)
        ex.matmul_f32_dev(dA, dI, dC, m, n, k, batch)
        assert np.array_equal(dC.download(np.float32).reshape(batch, m, n), A)
        dI.free()
    one = np.zeros((m, n), dtype=np.float32)
    ex.matmul_f32(A[0], B[0], one, m, n, k)                    # the host-slice entry point runs the same kernel
    assert np.array_equal(one, got[0])
    for buf in (dA, dB, dC):
        buf.free()
