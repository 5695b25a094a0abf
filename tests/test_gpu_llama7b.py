"""End-to-end configuration at its full size (32 layers, hidden 4096, FFN 11008, vocab 32000) against golden
logits of the CPU oracle (tests/golden/llama7b_golden.npz, written by tests/golden/make_llama7b_golden.py).

Tolerance per logit: 1e-3 * ||w_row||_2 * ||x||_2, with ||x||_2 of the RMS-normalised final hidden state taken
as sqrt(hidden) (gamma ~ 1 + N(0, 0.01)); the run also reports how far inside that bound the kernels stay."""
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = Path(__file__).resolve().parent / "golden" / "llama7b_golden.npz"


def test_full_size_model_matches_oracle_golden(ex):
    from rustorch_amd import llama
    g = np.load(GOLD)
    seed, nl, h, nh, f, v = (int(x) for x in g["config"])
    toks, rows, want, wn = g["tokens"], g["rows"], g["logits"], g["row_norm"]
    print("llama 7B-shaped: %d layers, hidden %d, ffn %d, vocab %d, %d positions, %d sampled logits" % (nl, h, f, v, toks.size, rows.size), flush=True)
    gm = llama.HipLlama(ex, nl, h, nh, f, v, 32)
    nbytes = llama.load_synthetic(gm, seed)
    assert nbytes == 32 * 129_785_856 + 139_264_000 + 107_520_000
    tol = 1e-3 * wn * np.sqrt(h)
    worst = 0.0
    for p, t in enumerate(toks):
        pick = gm.step(int(t), p)
        got = gm.logits()
        assert np.isfinite(got).all()
        err = np.abs(got[rows].astype(np.float64) - want[p])
        worst = max(worst, float((err / tol).max()))
        assert np.all(err <= tol), "position %d: max |delta|/tol = %.3f" % (p, (err / tol).max())
        assert pick == int(np.argmax(got))
        top_ids, top_vals = g["top_ids"][p], g["top_vals"][p]
        if top_vals[0] - top_vals[1] > 2 * tol.max():
            assert pick == int(top_ids[0])
    print("worst |delta| / tol over %d positions: %.3e" % (toks.size, worst), flush=True)
    # prefill of the same prefix (16 tokens or more: the dense-contraction path on the matrix cores) leaves the
    # logits of its last token, and stepping on from its cache reproduces the next position
    gm.reset()
    gm.prefill(toks[:-1], 0)
    err = np.abs(gm.logits()[rows].astype(np.float64) - want[-2])
    print("prefill of %d tokens: max |delta| / tol = %.3e" % (toks.size - 1, float((err / tol).max())), flush=True)
    assert np.all(err <= tol)
    gm.step(int(toks[-1]), toks.size - 1)
    err = np.abs(gm.logits()[rows].astype(np.float64) - want[-1])
    print("step after prefill: max |delta| / tol = %.3e" % float((err / tol).max()), flush=True)
    assert np.all(err <= tol)
    gm.close()
