"""Pins the oracle's dense / decode-step functions: the reference's own known answers where it
has them, closed forms and invariants where it does not (RoPE, causal cache)."""
import numpy as np
import pytest

F32 = np.float32


def test_matmul_kat_from_reference(orc):
    # src/tensor/ops/matrix.rs:328-336: [[1,2],[3,4]] . [[5,6],[7,8]] = [19,22,43,50]; Linear stores W = B^T
    a = np.array([[1, 2], [3, 4]], dtype=F32)
    b = np.array([[5, 6], [7, 8]], dtype=F32)
    assert np.array_equal(orc.matmul_xwt(a, b.T.copy()).reshape(-1), np.array([19, 22, 43, 50], dtype=F32))


@pytest.mark.parametrize("t,cols", [(8, 128), (2, 96), (12, 512), (14, 768)])
def test_qgemv_is_dequant_then_sequential_matmul(orc, lib, t, cols):
    from rustorch_amd import synth
    rows = 37
    raw = synth.blocks(t, 5, 1, rows, cols)
    W = orc.dequant(t, raw, rows, cols)
    for m in (1, 3, 8, 19):
        x = synth.normal(5, 2, m * cols).reshape(m, cols)
        y = orc.qgemv(t, raw, rows, cols, x)
        assert np.array_equal(y, orc.matmul_xwt(x, W))           # same bits: same products, same order
        # hand-rolled sequential f32 sum for one output
        acc = F32(0)
        for k in range(cols):
            acc = F32(acc + F32(x[m - 1, k] * W[rows - 1, k]))
        assert y[m - 1, rows - 1] == acc
        y64, wn = orc.qgemv_f64(t, raw, rows, cols, x)
        assert np.allclose(y64, x.astype(np.float64) @ W.astype(np.float64).T, rtol=1e-12, atol=1e-12)
        assert np.allclose(wn, np.linalg.norm(W.astype(np.float64), axis=1))
        tol = 1e-5 * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]
        assert np.all(np.abs(y - y64) <= tol)
    onehot = np.zeros(cols, dtype=F32); onehot[cols // 3] = 1
    assert np.array_equal(orc.qgemv(t, raw, rows, cols, onehot), W[:, cols // 3])


def test_rmsnorm_formula_and_closed_forms(orc):
    # src/nn/normalization.rs:682-696: gamma * x / sqrt(mean(x^2) + eps), eps inside the root
    n = 64
    g = np.linspace(0.5, 1.5, n).astype(F32)
    for c, eps in ((3.0, 1e-5), (-0.25, 1e-8), (1e3, 1e-5)):
        y = orc.rmsnorm(np.full(n, c, F32), g, eps)
        assert np.allclose(y, g * c / np.sqrt(np.float64(c) ** 2 + eps), rtol=1e-6)
    assert np.array_equal(orc.rmsnorm(np.zeros(n, F32), g, 1e-5), np.zeros(n, F32))
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, n)).astype(F32)
    want = g * x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-5)
    assert np.allclose(orc.rmsnorm(x, g, 1e-5), want, rtol=2e-6, atol=1e-7)
    # eps matters: with eps comparable to mean square the output shrinks by sqrt(2)
    x1 = np.ones(n, F32)
    assert np.allclose(orc.rmsnorm(x1, np.ones(n, F32), 1.0), 1 / np.sqrt(2.0), rtol=1e-6)
    # scale invariance when eps -> 0
    assert np.allclose(orc.rmsnorm(x[0] * 7, g, 0.0), orc.rmsnorm(x[0], g, 0.0), rtol=1e-5)


def test_swiglu_values(orc):
    # src/nn/activation.rs:404-414: a * (b * sigmoid(b)) with a = up, b = gate
    gate = np.array([0.0, 1.0, -1.0, 20.0, -20.0, 3.5], dtype=F32)
    up = np.array([5.0, 2.0, 2.0, 1.0, 1.0, -4.0], dtype=F32)
    y = orc.swiglu(gate, up)
    assert y[0] == 0.0
    assert np.isclose(y[1], 2 * 0.7310586, rtol=1e-6)
    assert np.isclose(y[2], 2 * -0.26894143, rtol=1e-6)
    assert np.isclose(y[3], 20.0, rtol=1e-6) and abs(y[4]) < 1e-7
    g64 = gate.astype(np.float64)
    assert np.allclose(y, up * g64 / (1 + np.exp(-g64)), rtol=1e-6, atol=1e-9)
    # the gate is the activated operand: swapping operands changes the result
    assert not np.allclose(orc.swiglu(up, gate), y)


def test_rope_properties(orc):
    hd, nh, theta = 128, 3, 10000.0
    rng = np.random.default_rng(3)
    x = rng.standard_normal(nh * hd).astype(F32)
    assert np.array_equal(orc.rope(x, nh, hd, 0, theta), x)                      # pos 0 is the identity
    inv = orc.rope_inv_freq(hd, theta)
    assert inv[0] == 1.0 and np.isclose(inv[-1], theta ** (-(hd - 2) / hd), rtol=1e-6)
    assert np.allclose(inv, theta ** (-2.0 * np.arange(hd // 2) / hd), rtol=1e-6)
    y = orc.rope(x, nh, hd, 1, theta).reshape(nh, hd // 2, 2)
    xp = x.reshape(nh, hd // 2, 2)
    # pair 0 turns by exactly one radian at pos 1, counter-clockwise
    assert np.allclose(y[:, 0, 0], xp[:, 0, 0] * np.cos(1.0) - xp[:, 0, 1] * np.sin(1.0), atol=1e-6)
    assert np.allclose(y[:, 0, 1], xp[:, 0, 0] * np.sin(1.0) + xp[:, 0, 1] * np.cos(1.0), atol=1e-6)
    # pairs are interleaved neighbours (2i, 2i+1): norms of neighbour pairs are preserved
    for pos in (1, 17, 255):
        yp = orc.rope(x, nh, hd, pos, theta).reshape(nh, hd // 2, 2)
        assert np.allclose((yp ** 2).sum(-1), (xp ** 2).sum(-1), rtol=1e-5)
    # relative-position property: <R(m) q, R(n) k> = <R(m - n) q, k>
    q = rng.standard_normal(hd).astype(F32); k = rng.standard_normal(hd).astype(F32)
    for m, n in ((9, 4), (200, 137)):
        lhs = np.dot(orc.rope(q, 1, hd, m, theta).astype(np.float64), orc.rope(k, 1, hd, n, theta).astype(np.float64))
        rhs = np.dot(orc.rope(q, 1, hd, m - n, theta).astype(np.float64), k.astype(np.float64))
        assert np.isclose(lhs, rhs, rtol=1e-4, atol=1e-4)


def _cache(rows):
    return np.ascontiguousarray(np.asarray(rows, dtype=np.float32).astype(np.float16)).view(np.uint16)


def test_attention_properties(orc):
    nh, hd = 2, 64
    row = nh * hd
    rng = np.random.default_rng(5)
    q = rng.standard_normal(row).astype(F32)
    K = rng.standard_normal((6, row)).astype(F32); V = rng.standard_normal((6, row)).astype(F32)
    kc, vc = _cache(K), _cache(V)
    # one position: the output is fp16(v0) whatever the score
    assert np.array_equal(orc.attn_decode(q, kc, vc, 1, nh, hd), V[0].astype(np.float16).astype(F32))
    # identical keys: uniform weights -> mean of V
    ksame = _cache(np.tile(K[0], (6, 1)))
    out = orc.attn_decode(q, ksame, vc, 6, nh, hd)
    assert np.allclose(out, V.astype(np.float16).astype(np.float64).mean(axis=0), atol=1e-6)
    # one dominant key selects its V row
    Kd = np.zeros((6, row), dtype=F32); Kd[4] = 50 * q / np.linalg.norm(q)
    out = orc.attn_decode(q, _cache(Kd), vc, 6, nh, hd)
    assert np.allclose(out, V[4].astype(np.float16).astype(F32), atol=1e-4)
    # f64 brute force per head, scale 1/sqrt(head_dim), max-subtracted softmax
    out = orc.attn_decode(q, kc, vc, 5, nh, hd)
    Kh = K.astype(np.float16).astype(np.float64); Vh = V.astype(np.float16).astype(np.float64)
    for h in range(nh):
        sl = slice(h * hd, (h + 1) * hd)
        s = Kh[:5, sl] @ q[sl].astype(np.float64) / np.sqrt(hd)
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.isclose(p.sum(), 1.0)
        assert np.allclose(out[sl], p @ Vh[:5, sl], rtol=1e-5, atol=1e-6)
    # positions beyond n_pos are not read (causality of the cache)
    kc2, vc2 = kc.copy(), vc.copy(); kc2[5] = 0x7C00; vc2[5] = 0x7C00
    assert np.array_equal(orc.attn_decode(q, kc2, vc2, 5, nh, hd), out)


def test_grouped_query_attention_is_attention_over_repeated_kv_heads(orc):
    """Fewer key / value heads than query heads: query head h reads kv head h // group.  Expanding the cache by
    repeating every kv head `group` times must give the same numbers through the one-head-count routine."""
    nh, nkv, hd, npos = 8, 2, 64, 7
    rng = np.random.default_rng(9)
    q = rng.standard_normal(nh * hd).astype(F32)
    K = rng.standard_normal((npos, nkv, hd)).astype(F32); V = rng.standard_normal((npos, nkv, hd)).astype(F32)
    got = orc.attn_decode(q, _cache(K.reshape(npos, -1)), _cache(V.reshape(npos, -1)), npos, nh, hd, nkv)
    Kx = np.repeat(K, nh // nkv, axis=1).reshape(npos, -1); Vx = np.repeat(V, nh // nkv, axis=1).reshape(npos, -1)
    assert np.array_equal(got, orc.attn_decode(q, _cache(Kx), _cache(Vx), npos, nh, hd))
    # and one kv head per query head is the plain form
    assert np.array_equal(orc.attn_decode(q, _cache(Kx), _cache(Vx), npos, nh, hd, nh), orc.attn_decode(q, _cache(Kx), _cache(Vx), npos, nh, hd))


def test_kv_append_rounds_to_nearest_even(orc):
    v = np.array([1.0, 1.00048828125, 1.00146484375, 70000.0, -1e-8, 0.1], dtype=F32)
    cache = np.zeros((3, v.size), dtype=np.uint16)
    orc.kv_append(cache, v, 1)
    with np.errstate(over="ignore"):
        assert np.array_equal(cache[1], v.astype(np.float16).view(np.uint16))
    assert not cache[0].any() and not cache[2].any()


def test_argmax_ties_lowest_index(orc):
    assert orc.argmax(np.array([1, 5, 5, 2], dtype=F32)) == 1
    assert orc.argmax(np.array([-3, -3, -3], dtype=F32)) == 0
    assert orc.argmax(np.array([0, 1, 2, 9], dtype=F32)) == 3


def _tiny_model(orc, seed=3, n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=64, max_pos=16):
    from rustorch_amd import llama
    m = orc.OracleLlama(n_layers, hidden, n_heads, ffn, vocab, max_pos)
    tensors = list(llama.synthetic_tensors(seed, n_layers, hidden, ffn, vocab))
    for slot, layer, t, r, c, raw in tensors:
        m.set_tensor(slot, layer, t, r, c, raw)
    return m, tensors


def test_llama_token_by_token_equals_batched_prefix(orc, lib):
    # decode with a cache == causal attention over the prefix: feeding tokens one at a time
    # must give the logits of feeding them as one batch (same arithmetic per row).
    toks = [5, 17, 3, 60, 9, 9, 31]
    m1, _ = _tiny_model(orc)
    batched = m1.forward(toks, 0)
    m2, _ = _tiny_model(orc)
    stepwise = np.concatenate([m2.forward([t], i) for i, t in enumerate(toks)])
    assert np.array_equal(batched, stepwise)
    # split prefix: 4 tokens batched, 3 more continuing the same cache
    m3, _ = _tiny_model(orc)
    a = m3.forward(toks[:4], 0); b = m3.forward(toks[4:], 4)
    assert np.array_equal(np.concatenate([a, b]), batched)
    assert np.isfinite(batched).all() and np.ptp(batched) > 0


def test_llama_single_layer_against_numpy(orc, lib):
    # one layer, one token at position 0: attention output is fp16(v), everything else is plain algebra in f64
    from rustorch_amd import llama
    H, F, V, nh = 256, 256, 32, 2
    m = orc.OracleLlama(1, H, nh, F, V, 4)
    T = {}
    for slot, layer, t, r, c, raw in llama.synthetic_tensors(9, 1, H, F, V):
        m.set_tensor(slot, layer, t, r, c, raw)
        T[slot] = raw if t == 0 else orc.dequant(t, raw, r, c).astype(np.float64)
    tok = 7
    logits = m.forward([tok], 0)[0]

    def rms(x, g):
        return g.astype(np.float64) * x / np.sqrt((x ** 2).mean() + 1e-5)
    x = T["token_embd"][tok]
    h = rms(x, T["attn_norm"])
    v = (T["attn_v"] @ h).astype(np.float32).astype(np.float16).astype(np.float64)
    x = x + T["attn_output"] @ v
    h = rms(x, T["ffn_norm"])
    g, u = T["ffn_gate"] @ h, T["ffn_up"] @ h
    x = x + T["ffn_down"] @ (u * g / (1 + np.exp(-g)))
    want = T["output"] @ rms(x, T["output_norm"])
    assert np.allclose(logits, want, rtol=2e-3, atol=2e-3 * np.abs(want).max())
