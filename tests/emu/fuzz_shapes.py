"""Random shapes through the C-ABI, checked against the CPU oracle.  TEST INFRASTRUCTURE, meant for the emulated library
(tests/emu/build_emulated.py), where an access outside a buffer stops the run with an AddressSanitizer report:

    python tests/emu/build_emulated.py OUT_DIR --run tests/emu/fuzz_shapes.py [seed [rounds]]

Each round draws one case of each kind -- a GEMV (any format, 1..8 rows, ragged row counts, rows of one to several
passes), a grouped launch of several such problems, several weights against one batch (also from ready-made quantized
activations), a block decode, the greedy pick, the int8 affine product, a prefill contraction (rows on and off the matrix cores, ragged
tiles), the dense f32 product, the decode and prefill attention, RMSNorm / SwiGLU / RoPE -- sized so that the emulation
finishes a round in about a minute.  It prints every case before running it, so the last line names the culprit."""
import sys

import numpy as np

from oracle import oracle as orc
from rustorch_amd import synth
from rustorch_amd.executor import HipKernelExecutor

TYPES = [0, 1, 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14]
BLOCK = {0: 1, 1: 1, 2: 32, 3: 32, 6: 32, 7: 32, 8: 32, 9: 32, 10: 256, 11: 256, 12: 256, 13: 256, 14: 256}
TOL = 2e-5            # of ||w_row|| ||x||: what the GEMV tests hold the kernels to at the benchmark's row lengths
TOL_SHORT = 6e-5      # rows of a few blocks: one element's 15-bit rounding is not averaged away (the benchmark's bound is 1e-3)
TOL_GEMM = 3e-4       # the fp16 contractions (the emulation rounds after every fp16 operation)


def say(*a):
    print(*a, flush=True)


def cols_for(rng, t, big=False):
    unit = max(BLOCK[t], 32)
    return unit * int(rng.integers(1, (48 if big else 12) if unit == 256 else 40))


def gemv_case(ex, rng, i):
    t = int(rng.choice(TYPES)); rows = int(rng.integers(1, 300)); cols = cols_for(rng, t, big=rng.random() < 0.3); batch = int(rng.integers(1, 9))
    say("gemv type %d, %d x %d, batch %d" % (t, rows, cols, batch))
    raw = synth.blocks(t, 100 + i, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    x = synth.normal(100 + i, 2, batch * cols).reshape(batch, cols)
    y = np.atleast_2d(ex.qgemv(w, x if batch > 1 else x[0]))
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, x)
    ratio = np.abs(y - np.atleast_2d(y64)) / (wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None] + 1e-30)
    assert np.isfinite(y).all() and ratio.max() <= (TOL if cols >= 1024 else TOL_SHORT), ratio.max()
    w.free()


def grouped_case(ex, rng, i):
    n = int(rng.integers(2, 8))
    specs = [(int(rng.choice([2, 8, 12, 14])), int(rng.integers(1, 200))) for _ in range(n)]
    specs = [(t, r, cols_for(rng, t, big=rng.random() < 0.3)) for t, r in specs]
    say("grouped gemv", specs)
    ws, xs, ys, want = [], [], [], []
    for j, (t, r, c) in enumerate(specs):
        raw = synth.blocks(t, 200 + i, j, r, c)
        w = ex.upload_qweight(t, r, c, raw)
        x = synth.normal(200 + i, 50 + j, c)
        ws.append(w); xs.append(ex.to_device(x)); ys.append(ex.buffer(r * 4)); want.append(ex.qgemv(w, x))
    ex.qgemv_grouped_dev(ws, xs, ys)
    for y, wv in zip(ys, want):
        assert np.array_equal(y.download(np.float32), wv)
    for b in ws + xs + ys:
        b.free()


def gemm_case(ex, rng, i):
    t = int(rng.choice([12, 14, 12, 14, 13, 1, 8, 2])); rows = int(rng.integers(1, 70)) * 4; cols = 256 * int(rng.integers(1, 6))
    M = int(rng.choice([3, 9, 16, 17, 33, 64, 70, 130]))
    say("gemm type %d, %d x %d, M = %d" % (t, rows, cols, M))
    raw = synth.blocks(t, 300 + i, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    X = synth.normal(300 + i, 2, M * cols).reshape(M, cols)
    Y = ex.qgemm(w, X)
    y64, wn = orc.qgemv_f64(t, raw, rows, cols, X)
    ratio = np.abs(Y - y64) / (wn[None, :] * np.linalg.norm(X.astype(np.float64), axis=1)[:, None])
    assert np.isfinite(Y).all() and ratio.max() <= TOL_GEMM, ratio.max()
    w.free()


def dense_case(ex, rng, i):
    aligned = rng.random() < 0.6
    m, n, k = int(rng.integers(1, 200)), int(rng.integers(1, 50)) * (4 if aligned else 1), int(rng.integers(1, 40)) * (4 if aligned else 1)
    batch = int(rng.integers(1, 4))
    say("dense f32 batch %d, %d x %d x %d" % (batch, m, n, k))
    A = rng.standard_normal((batch, m, k)).astype(np.float32); B = rng.standard_normal((batch, k, n)).astype(np.float32)
    dA, dB, dC = ex.to_device(A), ex.to_device(B), ex.buffer(4 * batch * m * n)
    ex.matmul_f32_dev(dA, dB, dC, m, n, k, batch)
    got = dC.download(np.float32).reshape(batch, m, n)
    want = A.astype(np.float64) @ B.astype(np.float64)
    bound = 4 * np.sqrt(k) * 2.0 ** -24 * np.linalg.norm(A.astype(np.float64), axis=2)[:, :, None] * np.linalg.norm(B.astype(np.float64), axis=1)[:, None, :]
    assert np.all(np.abs(got - want) <= bound + 1e-30)
    for b in (dA, dB, dC):
        b.free()


def attention_case(ex, rng, i):
    hd = int(rng.choice([64, 128])); nh = int(rng.integers(1, 6)); n_pos = int(rng.integers(1, 300))
    say("decode attention %d heads of %d over %d positions" % (nh, hd, n_pos))
    q = synth.normal(400 + i, 1, nh * hd)
    kc = synth.normal(400 + i, 2, n_pos * nh * hd).astype(np.float16).view(np.uint16)
    vc = synth.normal(400 + i, 3, n_pos * nh * hd).astype(np.float16).view(np.uint16)
    got = ex.attn_decode(q, kc, vc, n_pos, nh, hd)
    want = orc.attn_decode(q, kc, vc, n_pos, nh, hd)
    assert np.allclose(got, want, rtol=2e-5, atol=1e-4)
    group = int(rng.choice([1, 1, 2, 4])); nkv = int(rng.integers(1, 4)); nh = nkv * group
    M = int(rng.integers(1, 70)); pos0 = int(rng.integers(0, 40))
    say("prefill attention %d heads over %d key / value heads of %d, %d queries from position %d" % (nh, nkv, hd, M, pos0))
    n_all = pos0 + M
    Q = synth.normal(410 + i, 1, M * nh * hd).reshape(M, nh * hd)
    kc = synth.normal(410 + i, 2, n_all * nkv * hd).astype(np.float16).view(np.uint16)
    vc = synth.normal(410 + i, 3, n_all * nkv * hd).astype(np.float16).view(np.uint16)
    got = ex.attn_causal(Q, kc, vc, pos0, nh, hd, nkv)
    want = np.stack([orc.attn_decode(Q[m], kc, vc, pos0 + m + 1, nh, hd, nkv) for m in range(M)])
    assert np.allclose(got, want, rtol=2e-5, atol=1e-4)


def small_ops_case(ex, rng, i):
    n = 32 * int(rng.integers(1, 400))
    say("rmsnorm / swiglu over %d elements" % n)
    x = synth.normal(500 + i, 1, n); g = synth.normal(500 + i, 2, n, 1.0, 0.01)
    assert np.allclose(ex.rmsnorm(x, g, 1e-5), orc.rmsnorm(x, g, 1e-5), rtol=1e-5, atol=1e-6)
    u = synth.normal(500 + i, 3, n)
    assert np.allclose(ex.swiglu(x, u), orc.swiglu(x, u), rtol=1e-5, atol=1e-6)
    nh = int(rng.integers(1, 9)); hd = int(rng.choice([64, 128])); pos = int(rng.integers(0, 5000))
    say("rope %d heads of %d at position %d" % (nh, hd, pos))
    v = synth.normal(510 + i, 1, nh * hd)
    assert np.allclose(ex.rope(v, nh, hd, pos, 10000.0), orc.rope(v, nh, hd, pos, 10000.0), rtol=1e-4, atol=1e-4)


def shared_x_case(ex, rng, i):
    """Several weights against one batch (the q / k / v and gate / up launches), also from ready-made quantized activations."""
    cols = 256 * int(rng.integers(1, 12)); batch = int(rng.integers(1, 9)); n = int(rng.integers(1, 8))
    specs = [(int(rng.choice([12, 14, 8, 2, 13])), int(rng.integers(1, 150))) for _ in range(n)]
    say("shared-x gemv, %d columns, batch %d:" % (cols, batch), specs)
    x = synth.normal(600 + i, 1, batch * cols).reshape(batch, cols)
    dx = ex.to_device(x)
    ws, ys, raws = [], [], []
    for j, (t, r) in enumerate(specs):
        raw = synth.blocks(t, 600 + i, 10 + j, r, cols)
        raws.append(raw); ws.append(ex.upload_qweight(t, r, cols, raw)); ys.append(ex.buffer(4 * batch * r))
    ex.qgemv_shared_x_dev(ws, dx, ys, batch)
    xn = np.linalg.norm(x.astype(np.float64), axis=1)[:, None]
    for (t, r), raw, y in zip(specs, raws, ys):
        y64, wn = orc.qgemv_f64(t, raw, r, cols, x)
        got = y.download(np.float32).reshape(batch, r)
        assert np.isfinite(got).all() and (np.abs(got - np.atleast_2d(y64)) / (wn[None, :] * xn)).max() <= TOL_SHORT
    if batch == 1:
        # the same launch from activations quantized once by their own kernel: one problem per weight
        xq = ex.buffer(ex.xq_bytes(cols))
        ex.quantize_act_dev([dx], [cols], [xq])
        ex.qgemv_xq_grouped_dev(ws, [xq] * n, ys)
        for (t, r), raw, y in zip(specs, raws, ys):
            y64, wn = orc.qgemv_f64(t, raw, r, cols, x)
            got = y.download(np.float32).reshape(1, r)
            assert (np.abs(got - np.atleast_2d(y64)) / (wn[None, :] * xn)).max() <= TOL_SHORT
        xq.free()
    for b in ws + ys + [dx]:
        b.free()


def misc_case(ex, rng, i):
    t = int(rng.choice(TYPES)); rows = int(rng.integers(1, 40)); cols = cols_for(rng, t)
    say("dequant type %d, %d x %d" % (t, rows, cols))
    raw = synth.blocks(t, 700 + i, 1, rows, cols)
    w = ex.upload_qweight(t, rows, cols, raw)
    assert np.array_equal(ex.dequant(w).view(np.uint32), orc.dequant(t, raw, rows, cols).view(np.uint32))
    w.free()
    n = int(rng.integers(1, 70000))
    say("argmax over %d" % n)
    v = synth.normal(700 + i, 2, n)
    v[int(rng.integers(0, n))] = v.max()              # a tie now and then: the lowest index wins
    assert ex.argmax(v) == orc.argmax(v)
    m, k, nn = int(rng.integers(1, 90)), int(rng.integers(1, 200)), int(rng.integers(1, 90))
    say("int8 affine matmul %d x %d x %d" % (m, k, nn))
    a = rng.integers(-128, 128, (m, k), dtype=np.int8); b = rng.integers(-128, 128, (k, nn), dtype=np.int8)
    za, zb = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
    got = ex.qmatmul_i8(a, 0.02, za, b, 0.03, zb)
    want = orc.qmatmul_i8(a, 0.02, za, b, 0.03, zb)
    assert np.array_equal(got[0], want[0]) and got[1:] == want[1:]


def main():
    seed = int(sys.argv[1]) if len(sys.argv) > 1 else 1
    rounds = int(sys.argv[2]) if len(sys.argv) > 2 else 10
    orc.load()
    rng = np.random.default_rng(seed)
    ex = HipKernelExecutor(0)
    say("device:", ex.device_info())
    for i in range(rounds):
        say("-- round %d of seed %d" % (i, seed))
        for case in (gemv_case, grouped_case, shared_x_case, gemm_case, dense_case, attention_case, small_ops_case, misc_case):
            case(ex, rng, 1000 * seed + i)
    ex.close()
    say("FUZZ OK: %d rounds" % rounds)


if __name__ == "__main__":
    main()
