"""End-to-end configuration at its full size (32 layers, hidden 4096, FFN 11008, vocab 32000; a 128-token prompt and the
128 tokens of the oracle's greedy continuation) against golden logits of the CPU oracle for every one of the 256 positions
(tests/golden/llama7b_golden.npz, written by tests/golden/make_llama7b_golden.py).

Tolerance per logit: 1e-3 * ||w_row||_2 * ||x||_2, with ||x||_2 of the RMS-normalised final hidden state taken
as sqrt(hidden) (gamma ~ 1 + N(0, 0.01)).

What can be asked of every position and what cannot.  A random-init model of this size has attention scores in the
thousands: a softmax is close to one-hot, and where two scores nearly tie in some head, a change of the inputs far below
any kernel's rounding moves the attended row and the logits by several tolerances -- in the oracle itself.  The golden file
records this (`moved`: the oracle run again with its norm weights perturbed by 1e-5 .. 1e-4, see make_llama7b_golden.py):
the typical position moves by 0.001 to 0.005 of the tolerance, nine in ten by less than 0.02, and in every draw two to
five of the 256 positions move by 1 to 9 tolerances -- not the same positions from draw to draw.  An implementation with
another rounding than the oracle's is one more such draw.  So the bound is held
  * at the typical position far inside (median <= 0.05 of the tolerance, nine in ten <= 0.25), and
  * as a maximum at all but at most MAX_OUTLIERS of the 256 positions (a draw of the oracle against itself shows up to 5),
and the positions that exceed it are reported together with what the oracle's own draws did there.  Single-position checks
(the prefill's last logits, the device loop's last logits) are asserted unless that position is sensitive in a stored
draw or in this run's own stepping pass."""
import os
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# RT_LLAMA_GOLDEN names another file of the same layout (make_llama7b_golden.py --small: a small model, to try this test's
# own code where the full size is out of reach)
GOLD = Path(os.environ.get("RT_LLAMA_GOLDEN") or Path(__file__).resolve().parent / "golden" / "llama7b_golden.npz")
SENSITIVE_ABOVE = 0.25  # a position counts as sensitive when a conditioning draw moved the oracle's logits by more (in tolerances)
MAX_OUTLIERS = 10       # of 256 positions that may exceed the tolerance in one pass (the oracle against itself: 1 to 5 per draw)


def test_full_size_model_matches_oracle_golden(ex):
    from rustorch_amd import llama
    g = np.load(GOLD)
    seed, nl, h, nh, f, v = (int(x) for x in g["config"])
    toks, n_prompt, ids = g["tokens"], int(g["n_prompt"]), g["ids"]
    n_pos = toks.size
    print("llama 7B-shaped: %d layers, hidden %d, ffn %d, vocab %d, %d prompt + %d continuation positions, %d sampled logits + %d largest per position"
          % (nl, h, f, v, n_prompt, n_pos - n_prompt, ids.size, g["top_ids"].shape[1]), flush=True)
    gm = llama.HipLlama(ex, nl, h, nh, f, v, n_pos)
    nbytes = llama.load_synthetic(gm, seed)
    if (nl, h, f, v) == (32, 4096, 11008, 32000):
        assert nbytes == 32 * 129_785_856 + 139_264_000 + 107_520_000
    tol_ids = 1e-3 * g["id_norm"] * np.sqrt(h)
    tol_top = 1e-3 * g["top_norm"] * np.sqrt(h)                 # [n_pos, n_top]
    moved = g["moved"].max(axis=0)                               # worst movement of the oracle's own logits per position, over the stored draws
    sensitive = moved > SENSITIVE_ABOVE
    print("oracle's own conditioning draws (perturbations %s): median movement %.4f of the tolerance, positions above %.2f: %s"
          % (g["perturb"].tolist(), float(np.median(g["moved"])), SENSITIVE_ABOVE, [(int(p), round(float(moved[p]), 2)) for p in np.nonzero(sensitive)[0]]), flush=True)

    def ratio(p, got):
        """logits of position p at the sampled ids and at the oracle's largest: the worst ratio to the tolerance"""
        assert np.isfinite(got).all()
        r1 = np.abs(got[ids].astype(np.float64) - g["logits"][p]) / tol_ids
        r2 = np.abs(got[g["top_ids"][p]].astype(np.float64) - g["top_vals"][p]) / tol_top[p]
        return float(max(r1.max(), r2.max()))

    def hold(ratios, positions, what):
        """The statement of the module docstring over one pass of positions."""
        ratios = np.asarray(ratios)
        out = [(int(p), round(float(r), 2), round(float(moved[p]), 2)) for p, r in zip(positions, ratios) if r > 1.0]
        print("%s, %d positions: median %.4f, nine in ten below %.4f, max %.3f of the tolerance; above it (position, ratio, oracle's own movement): %s"
              % (what, ratios.size, np.median(ratios), np.quantile(ratios, 0.9), ratios.max(), out), flush=True)
        assert np.median(ratios) <= 0.05 and np.quantile(ratios, 0.9) <= 0.25, what
        assert len(out) <= MAX_OUTLIERS * ratios.size / 256 + 1, "%s: %d positions outside the tolerance: %s" % (what, len(out), out)

    def check_pick(p, pick, got, r):
        assert pick == int(np.argmax(got))
        top_vals = g["top_vals"][p]
        if r <= 1.0 and top_vals[0] - top_vals[1] > 2 * tol_top[p].max():     # logits inside the tolerance and no near-tie: the oracle's pick
            assert pick == int(g["top_ids"][p][0]), "position %d" % p

    # (a) every position one step at a time, teacher forced: the decode kernels at positions 0..255
    stepped = np.zeros(n_pos)
    for p in range(n_pos):
        pick = gm.step(int(toks[p]), p)
        got = gm.logits()
        stepped[p] = ratio(p, got)
        check_pick(p, pick, got, stepped[p])
    hold(stepped, range(n_pos), "stepping")
    sensitive = sensitive | (stepped > SENSITIVE_ABOVE)          # this run's own evidence counts too

    def single(p, got, what):
        r = ratio(p, got)
        print("%s: position %d, |delta| / tol = %.3e%s" % (what, p, r, " (sensitive position: reported only)" if sensitive[p] else ""), flush=True)
        assert sensitive[p] or r <= 1.0, what
        return r

    # (b) the configuration's own sequence of calls: the prompt in one prefill (dense contractions on the matrix cores),
    # then the continuation -- once with a host round trip per step (logits of every position compared), once as the
    # device-side loop (picks compared) -- with separate launches (mode 1) and replayed from a captured graph (mode 2)
    forced = np.concatenate([toks[n_prompt + 1:], [0]]).astype(np.int32)      # token fed after step i of the loop
    for mode in (1, 2):
        gm.set_mode(mode)
        gm.reset()
        gm.prefill(toks[:n_prompt], 0)
        single(n_prompt - 1, gm.logits(), "mode %d, prefill of %d tokens" % (mode, n_prompt))
        after = []
        for p in range(n_prompt, n_pos):
            pick = gm.step(int(toks[p]), p)
            got = gm.logits()
            after.append(ratio(p, got))
            check_pick(p, pick, got, after[-1])
        hold(after, range(n_prompt, n_pos), "mode %d, steps after the prefill" % mode)
        gm.reset()
        gm.prefill(toks[:n_prompt], 0)
        picks = gm.decode(int(toks[n_prompt]), n_prompt, n_pos - n_prompt, forced)
        last = gm.logits()
        single(n_pos - 1, last, "mode %d, device loop of %d steps, last logits" % (mode, n_pos - n_prompt))
        wrong = []
        for i, pick in enumerate(picks):
            p = n_prompt + i
            top_vals = g["top_vals"][p]
            if after[i] <= 1.0 and top_vals[0] - top_vals[1] > 2 * tol_top[p].max() and int(pick) != int(g["top_ids"][p][0]):
                wrong.append(p)
        assert not wrong, "mode %d, device loop: picks differ from the oracle's at %s" % (mode, wrong)
        assert int(picks[-1]) == int(np.argmax(last))
    gm.close()
