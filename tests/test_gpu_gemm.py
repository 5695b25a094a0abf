"""Prefill contraction (MFMA path) against the oracle.

Bound stated by the benchmark: max |delta| <= 1e-3 * ||w_row||_2 * ||x_row||_2 per element.  The fp16 operands
of the matrix cores keep the kernel about 20x inside it; the test holds it to 1e-4 at K = 4096 (scaled by sqrt(4096/K))."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
HELD = 1e-4


def check(Y, rows, toks, raw, t, n_rows, n_cols, X, orc, what):
    """Compare Y[toks][:, rows] with the f64 yardstick on the sampled weight rows / tokens."""
    rb = len(raw) // n_rows
    worst = 0.0
    for r0, r1 in rows:
        sub = raw[r0 * rb:r1 * rb]
        y64, wn = orc.qgemv_f64(t, sub, r1 - r0, n_cols, X[toks])
        xn = np.linalg.norm(X[toks].astype(np.float64), axis=1)[:, None]
        ratio = np.abs(Y[toks][:, r0:r1] - y64) / (wn[None, :] * xn)
        worst = max(worst, float(ratio.max()))
    print("%s: max |delta| / (||w|| ||x||) = %.3e (bound %.0e, held to %.0e)" % (what, worst, REL_TOL, HELD), flush=True)
    assert np.isfinite(Y).all()
    assert worst <= HELD


CASES = [
    ("q4k_4096x4096", 12, 4096, 4096),
    ("q4k_11008x4096", 12, 11008, 4096),
    ("q6k_4096x11008", 14, 4096, 11008),
]


@pytest.mark.parametrize("name,t,rows,cols", CASES)
@pytest.mark.parametrize("M", [64, 512, 2048])
def test_prefill_shapes(ex, orc, name, t, rows, cols, M):
    from rustorch_amd import synth
    print("gemm", name, "M", M, flush=True)
    raw = synth.blocks(t, 31, 7, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    X = synth.normal(31, 100 + M, M * cols).reshape(M, cols)
    Y = ex.qgemm(w, X)
    assert Y.shape == (M, rows)
    rng = np.random.default_rng(M)
    toks = np.sort(rng.choice(M, size=min(M, 48), replace=False))
    starts = sorted(set([0, rows - 64] + [int(v) for v in rng.integers(0, rows - 64, 4)]))
    check(Y, [(s, s + 64) for s in starts], toks, raw, t, rows, cols, X, orc, "%s M=%d" % (name, M))


@pytest.mark.parametrize("t", [12, 14])
def test_ragged_and_scaled_inputs(ex, orc, t):
    from rustorch_amd import synth
    rows, cols = 1000, 1024                         # N not a multiple of the tile, several k splits
    raw = synth.blocks(t, 32, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    for M in (16, 17, 100, 300):
        print("gemm ragged type", t, "M", M, flush=True)
        X = synth.normal(32, M, M * cols).reshape(M, cols).copy()
        X[0] *= 3e5                                 # beyond the fp16 range before row scaling
        X[1] *= 1e-20
        X[2] = 0
        X[3, 5:] = 0                                # one non-zero element
        Y = ex.qgemm(w, X)
        y64, wn = orc.qgemv_f64(t, raw, rows, cols, X)
        xn = np.linalg.norm(X.astype(np.float64), axis=1)[:, None]
        xn[xn == 0] = 1
        ratio = np.abs(Y - y64) / (wn[None, :] * xn)
        held = HELD * np.sqrt(4096 / cols)          # the rounding noise of the fp16 operands averages as 1/sqrt(K)
        assert np.isfinite(Y).all() and ratio.max() <= held, (M, ratio.max())
        assert not Y[2].any()
        # a GEMM row is the GEMV of that token, to rounding of the two paths
        for m in (0, 4, M - 1):
            yv = ex.qgemv(w, X[m])
            assert np.all(np.abs(Y[m] - yv) <= 2 * held * wn * xn[m])


def test_other_formats_and_small_m_use_the_row_form(ex, orc):
    from rustorch_amd import synth
    for t, cols in ((8, 512), (2, 512), (12, 512)):
        raw = synth.blocks(t, 33, t, 96, cols)
        w = ex.upload_qweight(t, 96, cols, raw)
        for M in (1, 9, 40):
            X = synth.normal(33, M, M * cols).reshape(M, cols)
            y64, wn = orc.qgemv_f64(t, raw, 96, cols, X)
            xn = np.linalg.norm(X.astype(np.float64), axis=1)[:, None]
            assert (np.abs(ex.qgemm(w, X) - y64) / (wn[None, :] * xn)).max() <= HELD * np.sqrt(4096 / cols)


@pytest.mark.parametrize("t", [12, 14])
@pytest.mark.parametrize("rows,cols", [(4096, 4096), (100, 11008)])
def test_three_to_fifteen_rows_go_eight_at_a_time(ex, orc, t, rows, cols):
    """Fewer rows of X than the fused contraction's tiles take: the integer matrix-core GEMV, eight rows per launch, the
    remainder of one or two rows as passes of the one-row kernel (M = 9, 10)."""
    from rustorch_amd import synth
    print("gemm few rows", t, rows, cols, flush=True)
    raw = synth.blocks(t, 35, t, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    for M in (3, 8, 9, 10, 11, 15):
        X = synth.normal(35, M, M * cols).reshape(M, cols)
        y64, wn = orc.qgemv_f64(t, raw, rows, cols, X)
        xn = np.linalg.norm(X.astype(np.float64), axis=1)[:, None]
        worst = (np.abs(ex.qgemm(w, X) - y64) / (wn[None, :] * xn)).max()
        print("  M=%d: %.3e" % (M, worst), flush=True)
        assert worst <= 2e-5


@pytest.mark.parametrize("t", [8, 2, 3, 6, 7, 10, 11, 13, 1, 0])
def test_formats_without_a_fused_contraction(ex, orc, t):
    """From 32 rows of X on these formats go through the fp16 matrix-core kernel (F16 weights as they are, the others
    through an fp16 copy of the exact block decode): the benchmark's FFN shape, then ragged shapes with extreme rows."""
    from rustorch_amd import synth
    rows, cols, M = 4096, 11008 if t in (10, 11, 13) else 4096, 160
    print("hgemm type", t, rows, cols, "M", M, flush=True)
    raw = synth.blocks(t, 35, 7, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    X = synth.normal(35, 100 + M, M * cols).reshape(M, cols)
    Y = ex.qgemm(w, X)
    rng = np.random.default_rng(t)
    toks = np.sort(rng.choice(M, size=40, replace=False))
    starts = sorted(set([0, rows - 64] + [int(v) for v in rng.integers(0, rows - 64, 3)]))
    check(Y, [(s0, s0 + 64) for s0 in starts], toks, raw, t, rows, cols, X, orc, "type %d M=%d" % (t, M))
    rows, cols = 1000, 1024 if t not in (1, 0) else 960          # N not a multiple of the wave tile; K = 15 * 64 for plain rows
    raw = synth.blocks(t, 36, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    y_ref = None
    for M in (32, 33, 100, 300):
        X = synth.normal(36, M, M * cols).reshape(M, cols).copy()
        X[0] *= 3e5; X[1] *= 1e-20; X[2] = 0; X[3, 5:] = 0
        Y = ex.qgemm(w, X)
        y64, wn = orc.qgemv_f64(t, raw, rows, cols, X)
        xn = np.linalg.norm(X.astype(np.float64), axis=1)[:, None]
        xn[xn == 0] = 1
        ratio = np.abs(Y - y64) / (wn[None, :] * xn)
        held = HELD * np.sqrt(4096 / cols)
        assert np.isfinite(Y).all() and ratio.max() <= held, (M, ratio.max())
        assert not Y[2].any()


@pytest.mark.parametrize("t", [12, 14])
@pytest.mark.parametrize("rows,cols,M", [(36, 256, 40), (4, 512, 130), (260, 768, 65), (512, 2816, 96)])
def test_single_superblock_odd_counts_and_tiny_matrices(ex, orc, t, rows, cols, M):
    """One super-block per row (the pipeline's first and last body coincide), an odd number of super-blocks,
    fewer weight rows than one wave holds, M one past a tile."""
    from rustorch_amd import synth
    print("gemm edge type", t, rows, cols, "M", M, flush=True)
    raw = synth.blocks(t, 34, rows + cols, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    X = synth.normal(34, M, M * cols).reshape(M, cols)
    Y = ex.qgemm(w, X)
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, X)
    xn = np.linalg.norm(X.astype(np.float64), axis=1)[:, None]
    ratio = np.abs(Y - y64) / (wn[None, :] * xn)
    assert np.isfinite(Y).all() and ratio.max() <= HELD * np.sqrt(4096 / cols), ratio.max()
