"""The decode loop on the GPU against the oracle, teacher forced, logits per step.

Tolerance per logit: 1e-3 * ||w_row||_2 * ||x||_2 with w_row the output-head row and x the final normed
hidden state of the oracle (the benchmark's bound)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def build_pair(ex, orc, seed, n_layers, hidden, n_heads, ffn, vocab, max_pos, n_kv_heads=0):
    from rustorch_amd import llama
    gm = llama.HipLlama(ex, n_layers, hidden, n_heads, ffn, vocab, max_pos, n_kv_heads=n_kv_heads)
    om = orc.OracleLlama(n_layers, hidden, n_heads, ffn, vocab, max_pos, n_kv_heads=n_kv_heads)
    head = {}
    om.attn_norms = {}                                          # layer -> gamma, for stable_positions

    def sink(slot, layer, t, r, c, raw):
        om.set_tensor(slot, layer, t, r, c, raw)
        if slot == "output":
            head["wn"] = np.linalg.norm(orc.dequant(t, raw, r, c).astype(np.float64), axis=1)
        if slot == "attn_norm":
            om.attn_norms[layer] = np.array(raw, dtype=np.float32)
    llama.load_synthetic(gm, seed, sink)
    return gm, om, head["wn"]


def stable_positions(om, toks, want, tol, rel=3e-4, frac=0.02):
    """Positions at which the oracle itself is well conditioned.

    The tiny random models of this file have attention scores in the thousands, so a softmax is one-hot, and where two
    scores nearly tie an input change far below any kernel's rounding moves the attended row -- and the logits by many
    tolerances -- in the oracle just as on the GPU.  To tell those positions from real kernel errors the oracle is run a
    second and a third time with every attention-norm weight multiplied by 1 + rel * N(0, 1) (rel = 3e-4: ten times the relative
    rounding of the GPU's 15-bit activations): a position whose oracle logits move by more than `frac` of the tolerance in either run is
    ill conditioned and exempt from the bound on the maximum; every other position has to keep the bound itself.

    The filter depends on the oracle alone, so how much it leaves in is known without a device: 3 to 5 of the 26 checked
    positions of the grouped-query models, 13 and 20 of 42 of the long-context ones, 2 of 12 after the prefill passes.
    It is a small subset: what these tests state about every position is the typical-position bound (median and nine in
    ten inside the tolerance); the bound at every position without exemption is held by the full-size model test.  Each
    caller asserts the count it was written against, so the exemption cannot quietly grow to cover everything."""
    rng = np.random.default_rng(12345)
    n_layers = len(om.attn_norms)
    hidden = om.attn_norms[0].size
    ok = np.ones(len(toks), dtype=bool)
    for draw in range(2):                                       # two independent directions: a tie that one misses the other meets
        for l in range(n_layers):
            om.set_tensor("attn_norm", l, 0, 1, hidden, (om.attn_norms[l] * (1.0 + rel * rng.standard_normal(hidden))).astype(np.float32))
        moved = om.forward(toks, 0)
        ok &= (np.abs(moved - want) / tol).max(axis=1) <= frac
    for l in range(n_layers):
        om.set_tensor("attn_norm", l, 0, 1, hidden, om.attn_norms[l])
    return ok


def logit_tol(wn, hidden):
    # ||x||_2 of an RMS-normalised vector with gamma ~ 1 is sqrt(hidden)
    return 1e-3 * wn * np.sqrt(hidden)


@pytest.mark.parametrize("mode", [
    pytest.param(0, marks=pytest.mark.skip(reason="persistent step kernel switched off: GPU memory fault on first run, cause not found")),
    1, 2])
def test_small_model_teacher_forced(ex, orc, mode):
    from rustorch_amd import synth
    cfg = dict(n_layers=3, hidden=512, n_heads=4, ffn=1024, vocab=1000, max_pos=48)
    print("llama small", cfg, "mode", mode, flush=True)
    gm, om, wn = build_pair(ex, orc, 17, **cfg)
    gm.set_mode(mode)
    toks = synth.tokens(17, synth.TID_PROMPT, 40, cfg["vocab"])
    want = om.forward(toks, 0)                                  # [40, vocab]
    tol = logit_tol(wn, cfg["hidden"])
    worst = 0.0
    for p, t in enumerate(toks):
        pick = gm.step(int(t), p)
        got = gm.logits()
        err = np.abs(got - want[p])
        worst = max(worst, float((err / tol).max()))
        assert np.all(err <= tol), "position %d" % p
        assert pick == int(np.argmax(got))
        top2 = np.sort(want[p])[-2:]
        if top2[1] - top2[0] > 2 * tol.max():
            assert pick == orc.argmax(want[p])
    print("worst |delta| / tol over 40 positions: %.3e" % worst, flush=True)
    # prefill + continue gives the same logits as stepping
    gm.reset()
    gm.prefill(toks[:25], 0)
    assert np.all(np.abs(gm.logits() - want[24]) <= tol)
    gm.step(int(toks[25]), 25)
    assert np.all(np.abs(gm.logits() - want[25]) <= tol)


@pytest.mark.parametrize("mode", [
    pytest.param(0, marks=pytest.mark.skip(reason="persistent step kernel switched off: GPU memory fault on first run, cause not found")),
    1, 2])
def test_decode_loop_without_host_round_trips(ex, orc, mode):
    from rustorch_amd import synth, InvalidParameters, ShapeMismatch
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=300, max_pos=32)
    print("llama decode loop", cfg, "mode", mode, flush=True)
    gm, om, wn = build_pair(ex, orc, 23, **cfg)
    gm.set_mode(mode)
    prompt = synth.tokens(23, synth.TID_PROMPT, 8, cfg["vocab"])
    # greedy, stepping from the host
    picks = []
    tok = None
    for p, t in enumerate(prompt):
        tok = gm.step(int(t), p)
    first = tok
    for p in range(8, 20):
        picks.append(tok)
        tok = gm.step(int(tok), p)
    # the same 12 steps as one device-side loop after the same prefill
    gm.reset(); gm.prefill(prompt, 0)
    out = gm.decode(first, 8, 12)
    assert list(out[:-1]) == picks[1:] and out[-1] == tok
    # teacher forcing: feed `forced` regardless of the picks, picks still reported
    gm.reset(); gm.prefill(prompt, 0)
    forced = synth.tokens(23, 99, 12, cfg["vocab"])
    out_f = gm.decode(first, 8, 12, forced)
    seq = [first] + [int(v) for v in forced[:-1]]
    want = om.forward(np.concatenate([prompt, seq]).astype(np.int32), 0)[8:]
    tol = logit_tol(wn, cfg["hidden"])
    for i in range(12):
        top2 = np.sort(want[i])[-2:]
        if top2[1] - top2[0] > 2 * tol.max():
            assert out_f[i] == int(np.argmax(want[i]))
    with pytest.raises(InvalidParameters):
        gm.step(1, 5)                       # position must continue the cache
    with pytest.raises(InvalidParameters):
        gm.step(cfg["vocab"], 20)           # token outside the vocabulary
    with pytest.raises(ShapeMismatch):
        gm.decode(1, 20, 13)                # would run past max_pos


@pytest.mark.parametrize("n_heads,n_kv", [(8, 2), (4, 1), (4, 2)])
def test_grouped_query_attention_model(ex, orc, n_heads, n_kv):
    """Fewer key / value heads than query heads (k, v and the cache rows are n_kv * head_dim wide).

    Exact check: a model with one kv head per query head whose k / v matrices repeat the rows of each shared head
    computes the same thing, so stepping both on the GPU must give equal logits bit for bit.
    Against the oracle: these tiny random models have attention scores in the thousands (a one-hot softmax), and
    where two scores nearly tie the 16-bit activations pick the other row, for any head layout; so the bound is
    asked of the typical position (median a tenth of the tolerance, nine positions in ten inside it)."""
    from rustorch_amd import llama, synth, ShapeMismatch
    cfg = dict(n_layers=2, hidden=512, n_heads=n_heads, ffn=1024, vocab=500, max_pos=48)
    hd, group = cfg["hidden"] // n_heads, n_heads // n_kv
    print("llama gqa", cfg, "n_kv", n_kv, flush=True)
    gm, om, wn = build_pair(ex, orc, 31, n_kv_heads=n_kv, **cfg)
    twin = llama.HipLlama(ex, **cfg)
    rows = np.array([(h // group) * hd + d for h in range(n_heads) for d in range(hd)])
    for slot, layer, t, r, c, raw in llama.synthetic_tensors(31, cfg["n_layers"], cfg["hidden"], cfg["ffn"], cfg["vocab"], n_kv * hd):
        if slot in ("attn_k", "attn_v"):
            raw = np.ascontiguousarray(raw.view(np.uint8).reshape(r, -1)[rows]).reshape(-1)
            r = cfg["hidden"]
        twin.upload(slot, layer, t, r, c, raw)
    toks = synth.tokens(31, synth.TID_PROMPT, 40, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(wn, cfg["hidden"])
    stable = stable_positions(om, toks, want, tol)
    ratios, at = [], []
    for p, t in enumerate(toks[:24]):
        gm.step(int(t), p); twin.step(int(t), p)
        got = gm.logits()
        assert np.array_equal(got, twin.logits()), "position %d" % p
        ratios.append(float((np.abs(got - want[p]) / tol).max())); at.append(p)
    gm.reset()
    gm.prefill(toks[:30], 0)                                     # 30 tokens: the dense-contraction path
    ratios.append(float((np.abs(gm.logits() - want[29]) / tol).max())); at.append(29)
    out = gm.decode(int(toks[30]), 30, 9, toks[31:40])           # teacher forced continuation on the device
    ratios.append(float((np.abs(gm.logits() - want[38]) / tol).max())); at.append(38)
    ratios, ok = np.array(ratios), stable[np.array(at)]
    print("ratio to the tolerance: median %.3f, max %.2f, %d of %d above 1; well-conditioned positions: %d, max %.3f"
          % (np.median(ratios), ratios.max(), (ratios > 1).sum(), ratios.size, ok.sum(), ratios[ok].max() if ok.any() else 0.0), flush=True)
    assert np.median(ratios) <= 0.1 and (ratios <= 1).mean() >= 0.9
    assert ok.sum() >= 3, "the stability filter left %d positions in" % ok.sum()
    assert np.all(ratios[ok] <= 1.0), "positions %s" % [a for a, r, k in zip(at, ratios, ok) if k and r > 1.0]
    with pytest.raises(ShapeMismatch):                           # k must have n_kv * head_dim rows
        gm.upload("attn_k", 0, 12, 512, 512, synth.blocks(12, 1, 1, 512, 512))


@pytest.mark.parametrize("n_heads,n_kv", [(2, 2), (4, 2)])
def test_long_context_attention_split_over_workgroups(ex, orc, n_heads, n_kv):
    """From max_pos = 512 on the decode step spreads a head's positions over several workgroups and folds their
    partial softmax sums.  Same model, same cache, with max_pos below the switch: the single-workgroup kernel.
    The two differ only in the order of float additions inside the attention, so their logits agree far inside the
    tolerance; and both follow the oracle at the typical position (as in the grouped-query test)."""
    from rustorch_amd import llama, synth
    base = dict(n_layers=2, hidden=256, n_heads=n_heads, ffn=512, vocab=300)
    print("llama long context", base, "n_kv", n_kv, flush=True)
    split, om, wn = build_pair(ex, orc, 37, max_pos=600, n_kv_heads=n_kv, **base)       # 5 workgroups per head, 120 positions each
    single = llama.HipLlama(ex, max_pos=500, n_kv_heads=n_kv, **base)
    llama.load_synthetic(single, 37)
    toks = synth.tokens(37, synth.TID_PROMPT, 420, base["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(wn, base["hidden"])
    stable = stable_positions(om, toks, want, tol)
    ratios, between, at = [], [], []
    for n0 in (1, 112, 352):                      # the first steps, then across the chunk boundaries at 120 and 360
        split.reset(); single.reset()
        split.prefill(toks[:n0], 0); single.prefill(toks[:n0], 0)
        for p in range(n0, n0 + 14):
            split.step(int(toks[p]), p); single.step(int(toks[p]), p)
            a, b = split.logits(), single.logits()
            between.append(float((np.abs(a - b) / tol).max()))
            ratios.append(float((np.abs(a - want[p]) / tol).max())); at.append(p)
    ratios, between, ok = np.array(ratios), np.array(between), stable[np.array(at)]
    print("split vs single: max %.3f of the tolerance; split vs oracle: median %.3f, max %.2f; well-conditioned positions: %d of %d, max %.3f"
          % (between.max(), np.median(ratios), ratios.max(), ok.sum(), ok.size, ratios[ok].max() if ok.any() else 0.0), flush=True)
    assert between.max() <= 0.1
    # with hundreds of positions near-ties of the one-hot softmax are frequent: the typical position is held to the oracle,
    # and so is every position at which the oracle itself is well conditioned
    assert np.median(ratios) <= 0.2
    assert ok.sum() >= 10, "the stability filter left %d positions in" % ok.sum()
    assert np.all(ratios[ok] <= 1.0), "positions %s" % [a for a, r, k in zip(at, ratios, ok) if k and r > 1.0]


def test_70b_class_widths(ex, orc):
    """One layer with the widths of a 70B-class model (hidden 8192, 64 heads over 8 key / value heads, feed-forward
    28 672): rows whose staged activations exceed the default 64 KB of LDS, and a feed-forward wide enough for the
    1024-thread form of the fused pre-pass in the chained prefill."""
    from rustorch_amd import synth
    cfg = dict(n_layers=1, hidden=8192, n_heads=64, ffn=28672, vocab=256, max_pos=48)
    print("llama 70b-class widths", cfg, flush=True)
    gm, om, wn = build_pair(ex, orc, 43, n_kv_heads=8, **cfg)
    toks = synth.tokens(43, synth.TID_PROMPT, 40, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(wn, cfg["hidden"])
    ratios = []
    for p in range(8):
        gm.step(int(toks[p]), p)
        ratios.append(float((np.abs(gm.logits() - want[p]) / tol).max()))
    gm.reset()
    gm.prefill(toks[:36], 0)
    ratios.append(float((np.abs(gm.logits() - want[35]) / tol).max()))
    gm.step(int(toks[36]), 36)
    ratios.append(float((np.abs(gm.logits() - want[36]) / tol).max()))
    print("ratio to the tolerance: median %.3f, max %.2f" % (np.median(ratios), max(ratios)), flush=True)
    assert np.median(ratios) <= 0.1 and max(ratios) <= 1.0


def test_prefill_in_several_passes_and_calls(ex, orc):
    """A prompt longer than one pass of the batched prefill (512 tokens), the same prompt fed in two calls (the second
    starts at a position above zero) and token by token: the three device paths agree far inside the tolerance, and
    follow the oracle at the typical position."""
    from rustorch_amd import synth
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=300, max_pos=700)
    print("llama prefill passes", cfg, flush=True)
    gm, om, wn = build_pair(ex, orc, 41, **cfg)
    toks = synth.tokens(41, synth.TID_PROMPT, 560, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(wn, cfg["hidden"])
    n = 540                                                      # 512 + 28: two passes of the chained pipeline
    gm.prefill(toks[:n], 0)
    one_call = gm.logits().copy()
    gm.reset()
    gm.prefill(toks[:300], 0)
    gm.prefill(toks[300:n], 300)                                 # 240 tokens at positions 300 ..
    two_calls = gm.logits().copy()
    gm.reset()
    for p in range(n):
        gm.step(int(toks[p]), p)
    stepped = gm.logits().copy()
    d1 = float((np.abs(one_call - stepped) / tol).max()); d2 = float((np.abs(two_calls - stepped) / tol).max())
    r = float((np.abs(one_call - want[n - 1]) / tol).max())
    print("one call vs stepped %.3f, two calls vs stepped %.3f, vs oracle %.3f of the tolerance" % (d1, d2, r), flush=True)
    assert d1 <= 0.1 and d2 <= 0.1
    # the cache the passes left serves the decode steps that follow
    stable = stable_positions(om, toks, want, tol)
    ratios = []
    gm.reset(); gm.prefill(toks[:n], 0)
    for p in range(n, n + 12):
        gm.step(int(toks[p]), p)
        ratios.append(float((np.abs(gm.logits() - want[p]) / tol).max()))
    ratios, ok = np.array(ratios), stable[n:n + 12]
    print("steps after the passes: median %.3f, max %.2f; well-conditioned positions: %d of 12, max %.3f"
          % (np.median(ratios), ratios.max(), ok.sum(), ratios[ok].max() if ok.any() else 0.0), flush=True)
    assert np.median(ratios) <= 0.2
    assert ok.sum() >= 2, "the stability filter left %d positions in" % ok.sum()
    assert np.all(ratios[ok] <= 1.0)
    if stable[n - 1]:
        assert r <= 1.0


def test_short_prompts_take_the_batched_pass(ex, orc):
    """Prompts and tails of 3..15 tokens run the layer contractions eight rows at a time (one or two tokens go through
    the decode step): same logits as token by token, far inside the tolerance, and the cache they leave serves decode."""
    from rustorch_amd import synth
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=300, max_pos=64)
    print("llama short prompts", cfg, flush=True)
    gm, om, wn = build_pair(ex, orc, 43, **cfg)
    toks = synth.tokens(43, synth.TID_PROMPT, 40, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(wn, cfg["hidden"])
    for n in (2, 3, 7, 8, 11, 15, 17, 19):
        gm.reset()
        gm.prefill(toks[:n], 0)
        batched = gm.logits().copy()
        gm.step(int(toks[n]), n)
        after = gm.logits().copy()
        gm.reset()
        for p in range(n):
            gm.step(int(toks[p]), p)
        stepped = gm.logits().copy()
        d = float((np.abs(batched - stepped) / tol).max())
        r = float((np.abs(batched - want[n - 1]) / tol).max())
        r2 = float((np.abs(after - want[n]) / tol).max())
        print("  %2d tokens: vs stepped %.3f, vs oracle %.3f, next step vs oracle %.3f of the tolerance" % (n, d, r, r2), flush=True)
        # from 16 tokens on the fp16 operands of the fused contraction: another rounding than the decode step's
        assert d <= (0.25 if n < 16 else 1.0) and r <= 1.0 and r2 <= 1.0


@pytest.mark.parametrize("fmt", ["Q5_K", "Q8_0", "Q8_1", "Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q2_K", "Q3_K", "F16", "F32"])
def test_model_in_a_format_without_matrix_core_path(ex, orc, fmt):
    """All seven matrices of every layer in one format that the dense contraction does not serve.  Decode: the GEMV
    kernels (Q5_K: one row per step, gate and up as two problems of one launch followed by the separate SwiGLU).
    Prefill: from 32 tokens on the fp16 contraction over an fp16 copy kept with the model (second prompt: the copy is
    reused), from 16 the GEMV kernel run once per token as grid slices, below that token by token."""
    from rustorch_amd import llama, synth, GGMLType
    cfg = dict(n_layers=2, hidden=512, n_heads=4, ffn=1024, vocab=500, max_pos=44)
    print("llama uniform", fmt, cfg, flush=True)
    gm = llama.HipLlama(ex, **cfg)
    om = orc.OracleLlama(**cfg)
    head = {}
    for slot, layer, t, r, c, raw in llama.synthetic_tensors(29, cfg["n_layers"], cfg["hidden"], cfg["ffn"], cfg["vocab"]):
        if layer >= 0 and t != GGMLType.F32:
            t = getattr(GGMLType, fmt)
            raw = synth.blocks(t, 29, synth.layer_tid(layer, slot), r, c)
        gm.upload(slot, layer, t, r, c, raw)
        om.set_tensor(slot, layer, t, r, c, raw)
        if slot == "output":
            head["wn"] = np.linalg.norm(orc.dequant(t, raw, r, c).astype(np.float64), axis=1)
    toks = synth.tokens(29, synth.TID_PROMPT, 40, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(head["wn"], cfg["hidden"])
    ratios = []
    for p, t in enumerate(toks[:36]):
        gm.step(int(t), p)
        ratios.append(float((np.abs(gm.logits() - want[p]) / tol).max()))
    stepped = gm.logits().copy()
    gm.reset()
    gm.prefill(toks[:36], 0)                                    # fp16 contraction; the copies are made here
    batched = gm.logits().copy()
    ratios.append(float((np.abs(batched - want[35]) / tol).max()))
    # the fp16 contraction rounds weights and activations to fp16 (2^-11 each): further from the GEMV path than the fused
    # contraction is, still well inside the bound
    assert float((np.abs(batched - stepped) / tol).max()) <= 0.5
    gm.step(int(toks[36]), 36)                                  # the cache the batched path left serves the decode step
    ratios.append(float((np.abs(gm.logits() - want[36]) / tol).max()))
    gm.reset()
    gm.prefill(toks[:36], 0)                                    # the same prompt again: the copies are reused
    assert np.array_equal(gm.logits(), batched)
    gm.reset()
    gm.prefill(toks[:20], 0)                                    # 16..31 tokens: GEMV grid slices
    assert float((np.abs(gm.logits() - want[19]) / tol).max()) <= 1.0
    gm.reset()
    gm.prefill(toks[:10], 0)                                    # under 16 tokens: token by token
    assert float((np.abs(gm.logits() - want[9]) / tol).max()) <= 1.0
    ratios = np.array(ratios)
    print("ratio to the tolerance: median %.3f, max %.2f" % (np.median(ratios), ratios.max()), flush=True)
    assert np.median(ratios) <= 0.1 and (ratios <= 1).mean() >= 0.9


@pytest.mark.parametrize("fmts", [
    dict(attn_q="Q4_K", attn_k="Q8_0", attn_v="Q6_K", ffn_gate="Q4_K", ffn_up="Q5_K"),      # fused, fp16, fused contraction in one group
    dict(attn_q="Q5_K", attn_k="Q4_K", attn_v="Q4_K", ffn_gate="Q8_0", ffn_up="Q6_K"),      # fp16 first, then two that share a prepared X
    dict(attn_q="Q6_K", attn_k="F16", attn_v="Q4_0", attn_output="Q2_K", ffn_down="Q5_1")])
def test_prefill_with_mixed_formats_inside_a_group(ex, orc, fmts):
    """The matrices that meet one activation matrix (q / k / v; gate / up) in different formats: some take the fused
    matrix-core contraction, which shares a prepared copy of X in the workspace, some the fp16 contraction, which uses
    the same workspace for its own operands.  A batched prefill of 36 tokens has to give what feeding the tokens one by
    one gives, and both the oracle's logits."""
    from rustorch_amd import llama, synth, GGMLType
    cfg = dict(n_layers=2, hidden=512, n_heads=4, ffn=1024, vocab=400, max_pos=40)
    print("llama mixed formats", fmts, cfg, flush=True)
    gm = llama.HipLlama(ex, **cfg)
    om = orc.OracleLlama(**cfg)
    head = {}
    for slot, layer, t, r, c, raw in llama.synthetic_tensors(41, cfg["n_layers"], cfg["hidden"], cfg["ffn"], cfg["vocab"]):
        if slot in fmts:
            t = getattr(GGMLType, fmts[slot])
            raw = synth.blocks(t, 41, synth.layer_tid(layer, slot), r, c)
        gm.upload(slot, layer, t, r, c, raw)
        om.set_tensor(slot, layer, t, r, c, raw)
        if slot == "output":
            head["wn"] = np.linalg.norm(orc.dequant(t, raw, r, c).astype(np.float64), axis=1)
    toks = synth.tokens(41, synth.TID_PROMPT, 38, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(head["wn"], cfg["hidden"])
    for p, t in enumerate(toks[:36]):
        gm.step(int(t), p, want_token=False)
    stepped = gm.logits().copy()
    gm.reset()
    gm.prefill(toks[:36], 0)
    batched = gm.logits().copy()
    r_step, r_batch = float((np.abs(stepped - want[35]) / tol).max()), float((np.abs(batched - want[35]) / tol).max())
    between = float((np.abs(batched - stepped) / tol).max())
    print("position 35, ratio to the tolerance: token by token %.3f, batched %.3f, between the two %.3f" % (r_step, r_batch, between), flush=True)
    # the fp16 contraction rounds weights and activations to fp16: about half the bound at this size, the fused one a tenth
    assert np.isfinite(batched).all() and between <= 1.0 and r_batch <= 1.0 and r_step <= 0.2
    gm.step(int(toks[36]), 36)                                  # the cache the batched pass left serves the next step
    assert float((np.abs(gm.logits() - want[36]) / tol).max()) <= 1.0
    gm.close()


def test_graph_replay_equals_eager_launches(ex, orc):
    """Mode 2 replays the step from a captured graph.  Every replay is checked against the eager launches of mode 1:
    same kernels, same arguments, so logits and picks are equal bit for bit -- with eager work (a cache reset, a
    prefill through the other path, host reads) and synchronisations between the replays."""
    from rustorch_amd import synth
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=300, max_pos=40)
    gm, om, wn = build_pair(ex, orc, 29, **cfg)
    toks = synth.tokens(29, synth.TID_PROMPT, 30, cfg["vocab"])
    forced = synth.tokens(29, 77, 10, cfg["vocab"])

    def run(mode):
        gm.set_mode(mode)
        gm.reset()
        logits, picks = [], []
        for p, t in enumerate(toks[:14]):            # 14 steps: eager first, captured at the second, replayed 12 times
            picks.append(gm.step(int(t), p))
            logits.append(gm.logits().copy())        # a host read and a synchronisation between the replays
        out_a = gm.decode(int(toks[14]), 14, 8)      # the advancing form of the step: its own capture
        logits.append(gm.logits().copy())
        gm.reset()
        gm.prefill(toks[:20], 0)                     # 20 tokens: the batched path, eager kernels between the replays
        out_b = gm.decode(int(toks[20]), 20, 10, forced)
        logits.append(gm.logits().copy())
        return logits, picks, out_a, out_b

    l1, p1, a1, b1 = run(1)
    l2, p2, a2, b2 = run(2)
    l3, p3, a3, b3 = run(2)                          # graphs of the earlier run are still there: replays only
    for other in ((l2, p2, a2, b2), (l3, p3, a3, b3)):
        assert p1 == other[1] and list(a1) == list(other[2]) and list(b1) == list(other[3])
        for x, y in zip(l1, other[0]):
            assert np.array_equal(x, y)
    want = om.forward(toks[:14], 0)
    assert np.all(np.abs(l2[13] - want[13]) <= logit_tol(wn, cfg["hidden"]))


def test_incomplete_model_is_an_error(ex):
    from rustorch_amd import llama, InvalidParameters, ShapeMismatch, synth
    gm = llama.HipLlama(ex, 1, 256, 2, 256, 64, 8)
    with pytest.raises(InvalidParameters):
        gm.step(0, 0)
    with pytest.raises(ShapeMismatch):
        gm.upload("attn_q", 0, 12, 256, 512, synth.blocks(12, 1, 1, 256, 512))


def test_persistent_mode_is_refused_not_silently_replaced(ex):
    from rustorch_amd import llama, UnsupportedOperation
    gm = llama.HipLlama(ex, 1, 256, 2, 256, 64, 8)
    gm.set_mode(1)
    with pytest.raises(UnsupportedOperation):
        gm.set_mode(0)


def test_model_from_gguf_file_equals_direct_upload(ex, orc, tmp_path):
    """write a synthetic llama GGUF, load it through the container parser, compare with the oracle and with
    the model whose tensors were uploaded directly: same bytes on the device, so identical logits."""
    from rustorch_amd import llama, synth, InvalidParameters
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=128)
    print("llama from gguf", cfg, flush=True)
    p = tmp_path / "tiny.gguf"
    llama.write_synthetic_gguf(p, 31, context=24, **cfg)
    gf = llama.load_gguf(ex, p)
    assert (gf.cfg.n_layers, gf.cfg.hidden, gf.cfg.n_heads, gf.cfg.ffn, gf.cfg.vocab, gf.cfg.max_pos) == (2, 256, 2, 512, 128, 24)
    gm, om, wn = build_pair(ex, orc, 31, max_pos=24, **cfg)
    toks = synth.tokens(31, synth.TID_PROMPT, 10, cfg["vocab"])
    want = om.forward(toks, 0)
    tol = logit_tol(wn, cfg["hidden"])
    for pos, t in enumerate(toks):
        a, b = gf.step(int(t), pos), gm.step(int(t), pos)
        la, lb = gf.logits(), gm.logits()
        assert a == b and np.array_equal(la, lb)
        assert np.all(np.abs(la - want[pos]) <= tol)
    # a training context beyond what the attention kernels hold is capped, an explicit one is taken as given
    llama.write_synthetic_gguf(tmp_path / "long.gguf", 31, context=131072, **cfg)
    gl = llama.load_gguf(ex, tmp_path / "long.gguf")
    assert gl.cfg.max_pos == 16000
    gl.close()
    gl = llama.load_gguf(ex, tmp_path / "long.gguf", max_pos=600)
    assert gl.cfg.max_pos == 600
    gl.close()
    # a file without the block count is an error, not a guess
    from rustorch_amd import gguf
    w = gguf.GGUFWriter()
    w.add_kv("general.architecture", gguf.VT_STRING, "llama")
    w.write(tmp_path / "empty.gguf")
    with pytest.raises(InvalidParameters):
        llama.load_gguf(ex, tmp_path / "empty.gguf")


def test_generate_greedy_and_sampled(ex, orc):
    from rustorch_amd import llama, synth
    from rustorch_amd.sampling import SamplingConfig
    cfg = dict(n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=200, max_pos=40)
    print("llama generate", cfg, flush=True)
    gm, om, wn = build_pair(ex, orc, 41, **cfg)
    prompt = [int(t) for t in synth.tokens(41, synth.TID_PROMPT, 6, cfg["vocab"])]
    greedy = llama.generate(gm, prompt, 10)
    assert len(greedy) == 10
    # the host-sampled loop with top_k = 1 walks the same path as the device-side greedy loop
    gm.reset()
    again = llama.generate(gm, prompt, 10, SamplingConfig(temperature=0.7, top_k=1, repetition_penalty=1.0000001))
    assert again == greedy
    # a seeded draw is reproducible, stays inside the vocabulary and stops at the end-of-sequence token
    runs = []
    for _ in range(2):
        gm.reset()
        runs.append(llama.generate(gm, prompt, 12, SamplingConfig.with_top_k(5, 0.9), rng=np.random.default_rng(7)))
    assert runs[0] == runs[1] and all(0 <= t < cfg["vocab"] for t in runs[0])
    gm.reset()
    stop = llama.generate(gm, prompt, 10, eos_token=greedy[3])
    assert stop == greedy[:greedy.index(greedy[3]) + 1]
    # never past the cache: 6 prompt tokens leave 35 positions
    gm.reset()
    assert len(llama.generate(gm, prompt, 1000)) == cfg["max_pos"] - len(prompt) + 1
