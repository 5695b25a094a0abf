"""Several sequences decoded side by side against one model (rt_hip_llama_batch_*): per step and sequence the logits against
the oracle's forward of that sequence alone and against the single-sequence decode step on the device; sequences at
different positions (idle steps, a slot reset and refilled); the generate loop for several prompts; refused arguments.

The file sorts after the other GPU tests: the entry points here have not been on a device before."""
import numpy as np
import pytest

from test_gpu_llama import build_pair, logit_tol

pytestmark = pytest.mark.gpu

CFG = dict(n_layers=2, hidden=512, n_heads=4, ffn=1024, vocab=500, max_pos=40)


def sequences(seed, n_seq, length, vocab):
    from rustorch_amd import synth
    return [synth.tokens(seed, 300 + i, length, vocab) for i in range(n_seq)]


@pytest.mark.parametrize("n_seq,n_kv", [(1, 0), (2, 0), (3, 0), (8, 0), (5, 2)])
def test_batch_steps_match_the_oracle_and_the_single_sequence_step(ex, orc, n_seq, n_kv):
    """n_seq = 1, 2: the one-row GEMV kernel per row; from 3 on Q4_K / Q6_K go through the matrix-core small-batch kernel."""
    from rustorch_amd import llama
    print("batch decode", CFG, "sequences", n_seq, "kv heads", n_kv, flush=True)
    gm, om, wn = build_pair(ex, orc, 61, n_kv_heads=n_kv, **CFG)
    seqs = sequences(61, n_seq, 12, CFG["vocab"])
    want = [om.forward(s, 0) for s in seqs]                    # per sequence [12, vocab]
    tol = logit_tol(wn, CFG["hidden"])
    single = []
    for s in seqs:                                              # the single-sequence step on the device, for comparison
        gm.reset()
        rows = []
        for p, t in enumerate(s):
            gm.step(int(t), p)
            rows.append(gm.logits().copy())
        single.append(np.stack(rows))
    b = llama.HipLlamaBatch(gm, n_seq, 16)
    ratios, between = [], []
    for p in range(12):
        picks = b.step([int(s[p]) for s in seqs], [p] * n_seq)
        got = b.logits()
        assert np.isfinite(got).all()
        for i in range(n_seq):
            assert picks[i] == int(np.argmax(got[i]))
            ratios.append(float((np.abs(got[i] - want[i][p]) / tol).max()))
            between.append(float((np.abs(got[i] - single[i][p]) / tol).max()))
    ratios, between = np.array(ratios), np.array(between)
    print("batch vs oracle: median %.3f, max %.2f of the tolerance; batch vs single-sequence step: median %.4f, max %.3f"
          % (np.median(ratios), ratios.max(), np.median(between), between.max()), flush=True)
    # the typical position is held to the oracle (tiny random models have one-hot softmaxes with near-ties, as in test_gpu_llama.py),
    # and the two device paths -- which differ only in the order of float additions -- to each other
    assert np.median(ratios) <= 0.1 and (ratios <= 1).mean() >= 0.9
    assert np.median(between) <= 0.05 and (between <= 1).mean() >= 0.9
    b.close()
    gm.close()


def test_three_sequences_on_a_small_model(ex, orc):
    """The whole step once at a size the CPU emulation of the library finishes in seconds: three rows, so the Q4_K / Q6_K
    matrices take the matrix-core small-batch kernel."""
    from rustorch_amd import llama
    cfg = dict(n_layers=1, hidden=256, n_heads=2, ffn=256, vocab=64, max_pos=8)
    gm, om, wn = build_pair(ex, orc, 59, **cfg)
    seqs = sequences(59, 3, 4, cfg["vocab"])
    want = [om.forward(s, 0) for s in seqs]
    tol = logit_tol(wn, cfg["hidden"])
    b = llama.HipLlamaBatch(gm, 3, 4)
    ratios = []
    for p in range(4):
        picks = b.step([int(s[p]) for s in seqs], [p] * 3)
        got = b.logits()
        assert np.isfinite(got).all() and all(picks[i] == int(np.argmax(got[i])) for i in range(3))
        ratios += [float((np.abs(got[i] - want[i][p]) / tol).max()) for i in range(3)]
    print("small model, three sequences: median %.3f, max %.2f of the tolerance" % (np.median(ratios), max(ratios)), flush=True)
    assert np.median(ratios) <= 0.1 and np.mean(np.array(ratios) <= 1) >= 0.9
    b.close()
    gm.close()


def test_sequences_at_different_positions_and_refilled_slots(ex, orc):
    """Sequence 1 starts three steps after sequence 0 (idle steps), sequence 2 is reset in mid-run and takes a new prompt: every
    sequence's logits are those of that sequence fed alone."""
    from rustorch_amd import llama, InvalidParameters
    gm, om, wn = build_pair(ex, orc, 67, **CFG)
    s0, s1, s2, s3 = sequences(67, 4, 10, CFG["vocab"])
    b = llama.HipLlamaBatch(gm, 3, 16)
    alone = llama.HipLlamaBatch(gm, 3, 16)                     # the same sequences, each in a batch where the others idle
    tol = logit_tol(wn, CFG["hidden"])

    def fed_alone(seq, upto):
        alone.reset()
        for p in range(upto + 1):
            alone.step([int(seq[p]), -1, -1], [p, 0, 0])
        return alone.logits()[0]

    worst = 0.0
    for step in range(10):
        toks, pos = [int(s0[step]), -1, -1], [step, 0, 0]
        if step >= 3:
            toks[1], pos[1] = int(s1[step - 3]), step - 3
        if step < 5:
            toks[2], pos[2] = int(s2[step]), step
        else:
            if step == 5:
                b.reset(2)                                       # the slot takes a new prompt
            toks[2], pos[2] = int(s3[step - 5]), step - 5
        picks = b.step(toks, pos)
        got = b.logits()
        assert picks[1] == -1 if step < 3 else picks[1] >= 0
        for i, (seq, p) in enumerate(((s0, step), (s1, step - 3), (s2 if step < 5 else s3, step if step < 5 else step - 5))):
            if p < 0:
                continue
            ref = fed_alone(seq, p)
            worst = max(worst, float((np.abs(got[i] - ref) / tol).max()))
    print("sequences side by side vs each alone: max %.4f of the tolerance" % worst, flush=True)
    assert worst <= 0.05                                         # the same kernels on the same rows: only the row's place in the batch differs
    with pytest.raises(InvalidParameters):
        b.step([1, 1, 1], [10, 7, 4])                            # sequence 2 has been fed 5 tokens since its reset
    with pytest.raises(InvalidParameters):
        b.step([-1, -1, -1], [0, 0, 0])
    b.close(); alone.close()
    gm.close()


def test_prompt_of_one_sequence_through_the_prefill_passes(ex, orc):
    """A sequence's prompt in one prefill call (the model's batched passes, writing that sequence's cache) while another
    sequence is in mid-run: the prompt's last logits and the steps that follow agree with the same tokens fed step by step and
    with the oracle, and the other sequence is undisturbed."""
    from rustorch_amd import llama, InvalidParameters, ShapeMismatch
    gm, om, wn = build_pair(ex, orc, 69, **CFG)
    s0, s1 = sequences(69, 2, 30, CFG["vocab"])
    want0, want1 = om.forward(s0, 0), om.forward(s1, 0)
    tol = logit_tol(wn, CFG["hidden"])
    b, ref = llama.HipLlamaBatch(gm, 2, 32), llama.HipLlamaBatch(gm, 2, 32)
    for p in range(4):                                           # sequence 0 runs four steps on its own first
        b.step([int(s0[p]), -1], [p, 0]); ref.step([int(s0[p]), -1], [p, 0])
    b.prefill(1, s1[:20], 0)                                     # 20 tokens: the dense-contraction pass
    for p in range(20):
        ref.step([-1, int(s1[p])], [0, p])
    r_pf = float((np.abs(b.logits()[1] - want1[19]) / tol).max())
    d_pf = float((np.abs(b.logits()[1] - ref.logits()[1]) / tol).max())
    ratios, between = [], []
    for k in range(6):                                           # both sequences go on together
        toks, pos = [int(s0[4 + k]), int(s1[20 + k])], [4 + k, 20 + k]
        b.step(toks, pos); ref.step(toks, pos)
        got, other = b.logits(), ref.logits()
        assert np.array_equal(got[0], other[0])                  # sequence 0 never met the prefill: the same bits as without it
        ratios.append(float((np.abs(got[1] - want1[20 + k]) / tol).max()))
        between.append(float((np.abs(got[1] - other[1]) / tol).max()))
        ratios.append(float((np.abs(got[0] - want0[4 + k]) / tol).max()))
    print("prefill of 20 tokens into sequence 1: %.3f of the tolerance against the oracle, %.3f against step by step; the steps after: "
          "median %.3f max %.2f against the oracle, max %.3f against step by step" % (r_pf, d_pf, np.median(ratios), max(ratios), max(between)), flush=True)
    assert np.median(ratios + [r_pf]) <= 0.1 and d_pf <= 0.5 and np.median(between) <= 0.1
    with pytest.raises(ShapeMismatch):
        b.prefill(0, s0[:2], 10)                                 # fewer than three tokens go through step
    with pytest.raises(InvalidParameters):
        b.prefill(0, s0[:5], 3)                                  # sequence 0 has been fed 10 tokens
    with pytest.raises(ShapeMismatch):
        b.prefill(0, s0[10:30].tolist() + [1, 2, 3], 10)         # past the end of the cache
    b.close(); ref.close()
    gm.close()


def test_generate_for_several_prompts(ex, orc):
    """Greedy generation for three prompts of different lengths: what a manual loop over batch steps yields, end-of-sequence and
    the token budget honoured per sequence."""
    from rustorch_amd import llama, synth
    gm, om, wn = build_pair(ex, orc, 71, **CFG)
    prompts = [list(synth.tokens(71, 400, 5, CFG["vocab"])), list(synth.tokens(71, 401, 2, CFG["vocab"])), list(synth.tokens(71, 402, 8, CFG["vocab"]))]
    b = llama.HipLlamaBatch(gm, 3, 24)
    out = b.generate(prompts, 6)
    assert [len(o) for o in out] == [6, 6, 6]
    # the same by hand, one sequence per batch slot with the others idle (prompts of four tokens or more: all but the last
    # token in one prefill call, as generate does)
    for i, prompt in enumerate(prompts):
        b.reset()
        toks, pos, pick = list(prompt), 0, None
        if len(toks) >= 4:
            b.prefill(i, toks[:-1], 0)
            pos = len(toks) - 1
        gen = []
        while len(gen) < 6:
            t = toks[pos] if pos < len(toks) else gen[-1]
            step = [-1, -1, -1]; step[i] = int(t)
            pick = int(b.step(step, [pos if j == i else 0 for j in range(3)])[i])
            pos += 1
            if pos >= len(toks):
                gen.append(pick)
        assert gen == out[i], "sequence %d" % i
    eos = out[0][2]
    stopped = b.generate(prompts, 6, eos_token=eos)
    assert stopped[0] == out[0][:out[0].index(eos) + 1]
    short = llama.HipLlamaBatch(gm, 3, 9)                       # the longest prompt leaves room for two new tokens
    assert [len(o) for o in short.generate(prompts, 6)] == [5, 6, 2]
    # sampling on the host from each sequence's own row of logits: a greedy configuration that has to take that way (a
    # repetition penalty, here one that changes nothing) repeats the device's picks; a seeded draw repeats itself
    from rustorch_amd.sampling import SamplingConfig
    assert b.generate(prompts, 6, config=SamplingConfig(temperature=0.0, top_k=1, repetition_penalty=1.0 + 1e-12)) == out
    warm = SamplingConfig(temperature=0.9, top_k=20, top_p=0.95, repetition_penalty=1.1)
    drawn = b.generate(prompts, 6, config=warm, rng=np.random.default_rng(5))
    assert drawn == b.generate(prompts, 6, config=warm, rng=np.random.default_rng(5))
    assert [len(o) for o in drawn] == [6, 6, 6] and all(0 <= t < CFG["vocab"] for o in drawn for t in o)
    b.close(); short.close()
    gm.close()


def test_batch_arguments_are_checked(ex, orc):
    from rustorch_amd import llama, InvalidParameters, ShapeMismatch
    gm, om, wn = build_pair(ex, orc, 73, **CFG)
    for n_seq, max_pos in ((0, 8), (9, 8), (2, 0), (2, 9000)):
        with pytest.raises(ShapeMismatch):
            llama.HipLlamaBatch(gm, n_seq, max_pos)
    b = llama.HipLlamaBatch(gm, 2, 4)
    with pytest.raises(InvalidParameters):
        b.step([1, CFG["vocab"]], [0, 0])
    with pytest.raises(InvalidParameters):
        b.step([1, 1], [1, 0])
    with pytest.raises(ShapeMismatch):
        b.step([1, 1, 1], [0, 0, 0])
    for p in range(4):
        b.step([1, 2], [p, p])
    with pytest.raises(ShapeMismatch):
        b.step([1, 2], [4, 4])                                   # past the end of the caches
    with pytest.raises(InvalidParameters):
        b.reset(2)
    b.close()
    gm.close()
