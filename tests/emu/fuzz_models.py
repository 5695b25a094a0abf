"""Random small Llama-shaped models through the model object of the C-ABI, against the CPU oracle.  TEST INFRASTRUCTURE for
the emulated library (an access outside a buffer stops the run with an AddressSanitizer report):

    python tests/emu/build_emulated.py OUT_DIR --run tests/emu/fuzz_models.py [seed [cases]]

A case draws the widths (head size 64 or 128, grouped-query layouts, feed-forward width), a format per matrix slot (so
the q / k / v and gate / up groups mix formats with and without a matrix-core path), a context length (from 512 on the
decode attention splits a head's positions over workgroups) and a way to cut a prompt into prefill calls (lengths that
take the batched pass, the grid-slice pass and the token-by-token pass, starting off multiples of 32), then steps a few
tokens.  After every call the logits must be finite and within a loose multiple of
the benchmark's bound of the oracle's -- the tiny models are ill conditioned in places, so this hunts for faults, NaNs and
gross errors, not for the last bit -- and a second model fed token by token must agree with the first.  Last, a random
number of sequences (1..8) is decoded side by side against the same weights (rt_hip_llama_batch_*), some of them starting
late or sitting steps out, each against the oracle's forward of that sequence alone."""
import sys

import numpy as np

from oracle import oracle as orc
from rustorch_amd import GGMLType, llama, synth
from rustorch_amd.executor import HipKernelExecutor

MATRIX_FORMATS = ["Q4_K", "Q6_K", "Q8_0", "Q4_0", "Q5_K", "Q2_K", "Q3_K", "Q4_1", "Q5_0", "Q5_1", "Q8_1", "F16", "F32"]
LOOSE = 8.0          # multiples of 1e-3 * ||w_row|| * sqrt(hidden)


def say(*a):
    print(*a, flush=True)


def one_case(ex, rng, seed):
    hd = int(rng.choice([64, 128])); n_kv = int(rng.choice([1, 2, 4])); group = int(rng.choice([1, 1, 2]))
    nh = n_kv * group
    while (nh * hd) % 256:
        nh *= 2
    n_kv = nh // group
    hidden = nh * hd
    ffn = 256 * int(rng.integers(1, 5)); vocab = int(rng.integers(40, 200)); n_layers = int(rng.integers(1, 3))
    n_tok = int(rng.integers(20, 60)); max_pos = n_tok + 4
    if rng.random() < 0.3:
        max_pos = int(rng.integers(512, 700))      # from 512 positions on the decode attention is split over several workgroups
    kind = rng.random()
    uniform = kind < 0.35
    k_quants = 0.35 <= kind < 0.6       # Q4_K / Q6_K throughout, as the common 4-bit files are: several sequences then take the fused step
    fmts = {}
    base = str(rng.choice(MATRIX_FORMATS))
    for slot in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"):
        if k_quants:
            fmts[slot] = str(rng.choice(["Q4_K", "Q6_K"]))
        else:
            fmts[slot] = base if uniform else str(rng.choice(MATRIX_FORMATS[:6] if rng.random() < 0.7 else MATRIX_FORMATS))
    cfg = dict(n_layers=n_layers, hidden=hidden, n_heads=nh, ffn=ffn, vocab=vocab, max_pos=max_pos)
    say("model", cfg, "kv heads", n_kv, "formats", fmts, "tokens", n_tok)
    gm = llama.HipLlama(ex, n_kv_heads=n_kv, **cfg)
    g2 = llama.HipLlama(ex, n_kv_heads=n_kv, **cfg)
    om = orc.OracleLlama(n_kv_heads=n_kv, **cfg)
    wn = None
    norms = []
    for slot, layer, t, r, c, raw in llama.synthetic_tensors(seed, n_layers, hidden, ffn, vocab, n_kv * hd):
        if slot in ("attn_norm", "ffn_norm", "output_norm"):
            norms.append((slot, layer, t, r, c, np.array(raw, dtype=np.float32)))
        if slot in fmts:
            t = getattr(GGMLType, fmts[slot])
            raw = synth.blocks(t, seed, synth.layer_tid(layer, slot), r, c)
        for m in (gm, g2):
            m.upload(slot, layer, t, r, c, raw)
        om.set_tensor(slot, layer, t, r, c, raw)
        if slot == "output":
            wn = np.linalg.norm(orc.dequant(t, raw, r, c).astype(np.float64), axis=1)
    tol = 1e-3 * wn * np.sqrt(hidden)
    toks = synth.tokens(seed, synth.TID_PROMPT, n_tok, vocab)
    want = om.forward(toks, 0)

    def oracle_movement(sequence, reference, positions):
        """How far the oracle's own logits move, in bounds, at `positions` when every norm weight changes in the fourth digit:
        the measure of how well conditioned the case is there (a near-tie of attention scores moves them by many bounds)."""
        prng = np.random.default_rng(seed)
        worst_move = 0.0
        for _ in range(2):
            for slot, layer, t, r, c, w in norms:
                om.set_tensor(slot, layer, t, r, c, (w * (1.0 + 1e-4 * prng.standard_normal(w.size))).astype(np.float32))
            moved = om.forward(sequence, 0)
            worst_move = max(worst_move, max(float((np.abs(moved[q] - reference[q]) / tol).max()) for q in positions))
        for slot, layer, t, r, c, w in norms:
            om.set_tensor(slot, layer, t, r, c, w)
        return worst_move

    # the prompt in a few prefill calls of random lengths, the rest token by token
    cuts, p = [], 0
    while p < n_tok - 4 and len(cuts) < 3:
        n = int(rng.choice([1, 2, 3, 5, 16, 17, 20, 32, 33, 40]))
        n = min(n, n_tok - 4 - p)
        cuts.append((p, n)); p += n
    say("prefill calls (pos0, n):", cuts, "then steps from", p)
    worst = 0.0
    checked = []
    for pos0, n in cuts:
        gm.prefill(toks[pos0:pos0 + n], pos0)
        lg = gm.logits()
        assert np.isfinite(lg).all(), "prefill at %d of %d tokens left non-finite logits" % (pos0, n)
        worst = max(worst, float((np.abs(lg - want[pos0 + n - 1]) / tol).max()))
        checked.append(pos0 + n - 1)
    for q in range(p, min(p + 3, n_tok)):
        gm.step(int(toks[q]), q)
        lg = gm.logits()
        assert np.isfinite(lg).all(), "step at %d left non-finite logits" % q
        worst = max(worst, float((np.abs(lg - want[q]) / tol).max()))
        checked.append(q)
    last = min(p + 3, n_tok) - 1
    # the same tokens one by one through the other model: the two ways of filling the cache must agree
    for q in range(last + 1):
        g2.step(int(toks[q]), q, want_token=False)
    worst2 = float((np.abs(g2.logits() - want[last]) / tol).max())
    between = float((np.abs(g2.logits() - gm.logits()) / tol).max())
    say("   worst |delta| / bound: calls %.3f, token by token %.3f, between the two %.3f" % (worst, worst2, between))
    if not (worst <= LOOSE and worst2 <= LOOSE and between <= LOOSE):
        # a gross error, or a case that is ill conditioned at a checked position?  The oracle against itself tells
        move = oracle_movement(toks, want, checked)
        say("   beyond the loose bound; the oracle's own logits move by %.2f bounds there under a 1e-4 perturbation of its norm weights" % move)
        assert max(worst, worst2, between) <= max(LOOSE, 4.0 * move), "beyond what the case's conditioning explains"
    # several sequences side by side against the same weights
    n_seq = int(rng.integers(1, 9)); steps = int(rng.integers(3, 7))
    seqs = [synth.tokens(seed, 500 + i, steps, vocab) for i in range(n_seq)]
    wants = [om.forward(sq, 0) for sq in seqs]
    start = [int(rng.integers(0, 3)) if i else 0 for i in range(n_seq)]      # sequence 0 always runs; the others may start late
    b = llama.HipLlamaBatch(gm, n_seq, steps + 1)
    fed = [0] * n_seq
    worst3, step = 0.0, 0
    while min(fed) < steps:
        toks_b, pos_b = [], []
        for i in range(n_seq):
            idle = fed[i] >= steps or step < start[i] or (i and rng.random() < 0.15)
            toks_b.append(-1 if idle else int(seqs[i][fed[i]])); pos_b.append(fed[i])
        if all(t < 0 for t in toks_b):
            toks_b[0] = int(seqs[0][min(fed[0], steps - 1)]) if fed[0] < steps else -1
            if toks_b[0] < 0:
                i = int(np.argmin(fed)); toks_b[i] = int(seqs[i][fed[i]])
        picks = b.step(toks_b, pos_b)
        lg = b.logits()
        for i in range(n_seq):
            if toks_b[i] < 0:
                assert picks[i] == -1
                continue
            assert np.isfinite(lg[i]).all(), "batch step left non-finite logits for sequence %d" % i
            assert picks[i] == int(np.argmax(lg[i]))
            worst3 = max(worst3, float((np.abs(lg[i] - wants[i][fed[i]]) / tol).max()))
            fed[i] += 1
        step += 1
    say("   %d sequences side by side, %d steps each (in %d batch steps): worst |delta| / bound %.3f" % (n_seq, steps, step, worst3))
    if worst3 > LOOSE:
        move = max(oracle_movement(sq, w, range(steps)) for sq, w in zip(seqs, wants))
        say("   beyond the loose bound; the oracle's own logits move by %.2f bounds under a 1e-4 perturbation of its norm weights" % move)
        assert worst3 <= max(LOOSE, 4.0 * move), "beyond what the case's conditioning explains"
    b.close()
    gm.close(); g2.close()


def main():
    seed = int(sys.argv[1]) if len(sys.argv) > 1 else 1
    cases = int(sys.argv[2]) if len(sys.argv) > 2 else 5
    orc.load()
    rng = np.random.default_rng(seed)
    ex = HipKernelExecutor(0)
    for i in range(cases):
        say("-- case %d of seed %d" % (i, seed))
        one_case(ex, rng, 100 * seed + i)
    ex.close()
    say("FUZZ OK: %d cases" % cases)


if __name__ == "__main__":
    main()
