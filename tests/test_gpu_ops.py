"""Decode-step operators on the GPU against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_rmsnorm(ex, orc):
    from rustorch_amd import synth
    print("rmsnorm", flush=True)
    for rows, n, eps in ((1, 4096, 1e-5), (8, 4096, 1e-5), (3, 100, 1e-8), (2, 11008, 1e-5)):
        x = synth.normal(1, rows, rows * n).reshape(rows, n) * 3
        g = synth.normal(1, 77, n, 1.0, 0.01)
        assert np.allclose(ex.rmsnorm(x, g, eps), orc.rmsnorm(x, g, eps), rtol=3e-6, atol=1e-7)
    assert np.array_equal(ex.rmsnorm(np.zeros(64, np.float32), np.ones(64, np.float32), 1e-5), np.zeros(64, np.float32))


def test_swiglu(ex, orc):
    from rustorch_amd import synth
    print("swiglu", flush=True)
    for n in (11008, 8 * 11008, 37):
        g = synth.normal(2, n, n) * 4; u = synth.normal(3, n, n)
        assert np.allclose(ex.swiglu(g, u), orc.swiglu(g, u), rtol=3e-6, atol=1e-7)
    g = np.array([0, 1, -1, 30, -30, 88, -88, 100, -100], dtype=np.float32)
    got = ex.swiglu(g, np.ones_like(g))
    assert np.allclose(got, orc.swiglu(g, np.ones_like(g)), rtol=3e-6, atol=1e-30) and np.isfinite(got).all()


def test_rope(ex, orc):
    from rustorch_amd import synth
    print("rope", flush=True)
    x = synth.normal(4, 1, 32 * 128)
    assert np.array_equal(ex.rope(x, 32, 128, 0, 10000.0), x)
    for pos in (1, 2, 127, 255, 4000):
        got, want = ex.rope(x, 32, 128, pos, 10000.0), orc.rope(x, 32, 128, pos, 10000.0)
        assert np.allclose(got, want, rtol=0, atol=4e-6 * np.abs(x).max() * max(1.0, pos / 256))
    x64 = synth.normal(4, 2, 4 * 64)
    assert np.allclose(ex.rope(x64, 4, 64, 9, 500000.0), orc.rope(x64, 4, 64, 9, 500000.0), atol=4e-6 * np.abs(x64).max())


def test_kv_append_and_attention(ex, orc):
    from rustorch_amd import synth
    print("attention", flush=True)
    for nh, hd, n_pos in ((32, 128, 1), (32, 128, 200), (32, 128, 256), (4, 64, 37), (2, 128, 1000)):
        row = nh * hd
        K = synth.normal(5, n_pos, n_pos * row).reshape(n_pos, row)
        V = synth.normal(6, n_pos, n_pos * row).reshape(n_pos, row) * 10
        q = synth.normal(7, n_pos, row)
        kc_h = np.zeros((n_pos, row), dtype=np.uint16); vc_h = np.zeros((n_pos, row), dtype=np.uint16)
        kc_d = ex.buffer(kc_h.nbytes); vc_d = ex.buffer(vc_h.nbytes)
        kc_d.zero(); vc_d.zero()
        pos_list = range(n_pos) if n_pos <= 40 else (0, 1, n_pos // 2, n_pos - 1)
        for p in range(n_pos):
            orc.kv_append(kc_h, K[p], p); orc.kv_append(vc_h, V[p], p)
        for p in pos_list:
            ex.kv_append(kc_d, K[p], p); ex.kv_append(vc_d, V[p], p)
        got_k = kc_d.download(np.uint16).reshape(n_pos, row)
        for p in pos_list:
            assert np.array_equal(got_k[p], kc_h[p])            # fp16 RNE, bit for bit
        got = ex.attn_decode(q, kc_h, vc_h, n_pos, nh, hd)
        want = orc.attn_decode(q, kc_h, vc_h, n_pos, nh, hd)
        assert np.allclose(got, want, rtol=2e-5, atol=2e-5 * np.abs(V).max())
    with np.errstate(over="ignore"):
        v = np.array([70000.0, -70000.0, 65504.0, 1e-9, 0.1, 1.00048828125, 1.00146484375, 0.0], dtype=np.float32)
        d = ex.buffer(16 * 2); d.zero()
        ex.kv_append(d, v, 1)
        assert np.array_equal(d.download(np.uint16)[8:], v.astype(np.float16).view(np.uint16))
        assert not d.download(np.uint16)[:8].any()


@pytest.mark.parametrize("nh,nkv,hd,pos0,m", [(4, 4, 64, 0, 37), (32, 32, 128, 0, 70), (8, 2, 128, 100, 45), (2, 1, 128, 1000, 33),
                                               (6, 3, 64, 31, 1), (3, 3, 128, 0, 129),
                                               # a batch that starts off a multiple of 32 among the first positions: the first tile
                                               # of a later wave lies wholly beyond the early queries
                                               (1, 1, 64, 24, 28), (6, 3, 128, 23, 41), (2, 2, 128, 3, 48), (4, 2, 64, 1, 95)])
def test_causal_attention_of_a_batch(ex, orc, nh, nkv, hd, pos0, m):
    """Row i of the batch (position pos0 + i) against the single-query oracle over cache rows [0, pos0 + i]."""
    from rustorch_amd import synth
    print("causal attention", nh, nkv, hd, pos0, m, flush=True)
    row, rowkv, n_pos = nh * hd, nkv * hd, pos0 + m
    K = synth.normal(15, n_pos, n_pos * rowkv).reshape(n_pos, rowkv)
    V = synth.normal(16, n_pos, n_pos * rowkv).reshape(n_pos, rowkv) * 10
    q = synth.normal(17, n_pos, m * row).reshape(m, row) * 3
    q[m // 2] *= 1e-6                                              # a query of tiny magnitude, and one of zeros
    if m > 2:
        q[1] = 0
    kc = K.astype(np.float16).view(np.uint16); vc = V.astype(np.float16).view(np.uint16)
    got = ex.attn_causal(q, kc, vc, pos0, nh, hd, nkv)
    assert got.shape == (m, row) and np.isfinite(got).all()
    for i in range(m):
        want = orc.attn_decode(q[i], kc, vc, pos0 + i + 1, nh, hd, nkv)
        assert np.allclose(got[i], want, rtol=2e-5, atol=2e-5 * np.abs(V).max()), "query %d" % i
    # a shorter batch over caches that end at its last position: same rows, bit for bit, and nothing is read past the end
    h = m // 2
    got2 = ex.attn_causal(q[:h + 1], kc[:pos0 + h + 1], vc[:pos0 + h + 1], pos0, nh, hd, nkv)
    assert np.array_equal(got2, got[:h + 1])


def test_causal_attention_rejects_bad_shapes(ex):
    from rustorch_amd import ShapeMismatch
    q = np.zeros((4, 2 * 64), np.float32); c = np.zeros((4, 2 * 64), np.uint16)
    with pytest.raises(ShapeMismatch):
        ex.attn_causal(q, c[:3], c, 0, 2, 64)                     # cache shorter than the positions
    with pytest.raises(ShapeMismatch):
        ex.attn_causal(q, c, c, 0, 3, 64)                         # row width does not match
    with pytest.raises(ShapeMismatch):
        ex.attn_causal(np.zeros((4, 3 * 96), np.float32), np.zeros((4, 3 * 96), np.uint16), np.zeros((4, 3 * 96), np.uint16), 0, 3, 96)


def test_attention_dominant_and_uniform_keys(ex, orc):
    nh, hd, n = 32, 128, 64
    row = nh * hd
    rng = np.random.default_rng(1)
    q = rng.standard_normal(row).astype(np.float32)
    V = rng.standard_normal((n, row)).astype(np.float32)
    vc = V.astype(np.float16).view(np.uint16)
    K = np.tile(rng.standard_normal(row).astype(np.float32), (n, 1))
    out = ex.attn_decode(q, K.astype(np.float16).view(np.uint16), vc, n, nh, hd)
    assert np.allclose(out, V.astype(np.float16).astype(np.float64).mean(axis=0), atol=2e-6)
    Kd = np.zeros((n, row), np.float32); Kd[41] = 30 * q
    out = ex.attn_decode(q, Kd.astype(np.float16).view(np.uint16), vc, n, nh, hd)
    assert np.allclose(out, V[41].astype(np.float16).astype(np.float32), atol=1e-5)
    # scores this large would overflow exp() without the max subtraction
    assert np.isfinite(out).all()


def test_add_and_argmax(ex, orc):
    from rustorch_amd import synth
    x = synth.normal(8, 1, 4096); y = synth.normal(8, 2, 4096)
    assert np.array_equal(ex.add(x, y), x + y)
    v = synth.normal(9, 1, 32000)
    assert ex.argmax(v) == orc.argmax(v) == int(np.argmax(v))
    v[[31999, 123, 20000]] = 50.0
    assert ex.argmax(v) == 123                               # ties: lowest index
    assert ex.argmax(np.full(5000, -3.0, np.float32)) == 0
    assert ex.argmax(np.array([1.0], np.float32)) == 0


def test_stream_read_probe_stays_inside_its_buffer(ex):
    """The bench's read probe touches whole 2 KB pieces of the range it is given and nothing else: ranges shorter than a
    piece, ragged ends and an offset range are all accepted; a range past the buffer is refused on the host."""
    from rustorch_amd import ShapeMismatch
    buf = ex.buffer(3 * 2048 + 100)
    buf.zero()
    for off, n in ((0, None), (0, 100), (16, 2048), (2048, 2 * 2048 + 100), (0, 0)):
        ex.stream_read_dev(buf, off, n)
    ex.synchronize()
    with pytest.raises(ShapeMismatch):
        ex.stream_read_dev(buf, 2048, 3 * 2048)
    buf.free()
