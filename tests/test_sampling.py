"""Host-side sampling against the reference's own tests (example-cli/src/model/sampling.rs:298-447) and the
properties its functions state."""
import numpy as np
import pytest

from rustorch_amd import InvalidParameters
from rustorch_amd.sampling import (SamplingConfig, apply_repetition_penalty, apply_temperature, apply_top_k_to_probs,
                                   apply_top_p_to_probs, multinomial_sample, sample_token, softmax)


def test_reference_configs():
    c = SamplingConfig()
    assert (c.temperature, c.top_k, c.top_p) == (1.0, None, None)
    c.validate()
    g = SamplingConfig.greedy()
    assert (g.temperature, g.top_k) == (0.0, 1) and g.is_greedy
    g.validate()
    k = SamplingConfig.with_top_k(50, 0.8)
    assert (k.temperature, k.top_k) == (0.8, 50)
    n = SamplingConfig.nucleus(0.9, 0.7)
    assert (n.temperature, n.top_p) == (0.7, 0.9)
    for bad in (SamplingConfig(temperature=-1.0), SamplingConfig(top_k=0), SamplingConfig(top_p=1.5), SamplingConfig(repetition_penalty=-0.1)):
        with pytest.raises(InvalidParameters):
            bad.validate()


def test_reference_softmax():
    p = softmax([1.0, 2.0, 3.0])
    assert abs(p.sum() - 1.0) < 1e-6 and p[0] < p[1] < p[2]
    assert np.allclose(softmax([1000.0, 1000.0]), [0.5, 0.5])          # max subtraction keeps it finite


def test_reference_top_k():
    f = apply_top_k_to_probs([0.1, 0.4, 0.3, 0.2], 2)
    assert (f > 0).sum() == 2 and abs(f.sum() - 1.0) < 1e-6
    assert np.allclose(f, [0, 0.4 / 0.7, 0.3 / 0.7, 0])
    assert np.allclose(apply_top_k_to_probs([0.1, 0.9], 0), [0.1, 0.9]) and np.allclose(apply_top_k_to_probs([0.1, 0.9], 5), [0.1, 0.9])


def test_reference_top_p():
    f = apply_top_p_to_probs([0.5, 0.3, 0.15, 0.05], 0.8)
    assert abs(f.sum() - 1.0) < 1e-6
    assert np.allclose(f, [0.5 / 0.8, 0.3 / 0.8, 0, 0])                # 0.5 + 0.3 reaches 0.8: two tokens kept
    assert np.allclose(apply_top_p_to_probs([0.5, 0.5], 1.0), [0.5, 0.5]) and np.allclose(apply_top_p_to_probs([0.5, 0.5], 0.0), [0.5, 0.5])
    g = apply_top_p_to_probs([0.4, 0.35, 0.25], 0.5)                   # 0.4 < 0.5 -> the second one is needed too
    assert (g > 0).sum() == 2


def test_reference_multinomial_and_greedy():
    rng = np.random.default_rng(1)
    draws = [multinomial_sample([0.25, 0.25, 0.25, 0.25], rng) for _ in range(400)]
    assert min(draws) >= 0 and max(draws) < 4 and len(set(draws)) == 4
    assert multinomial_sample([0.0, 0.0, 1.0], rng) == 2
    logits = np.array([0.1, 2.0, 2.0, -1.0])
    assert sample_token(logits, SamplingConfig.greedy()) == 1          # tie -> lowest index, as the device argmax
    assert sample_token(logits, SamplingConfig(temperature=0.0)) == 1
    assert sample_token(np.zeros((1, 100)), SamplingConfig(), rng=rng) in range(100)


def test_temperature_and_penalty():
    x = np.array([1.0, -2.0, 3.0])
    assert np.array_equal(apply_temperature(x, 1.0), x) and np.array_equal(apply_temperature(x, 0.0), x)
    assert np.allclose(apply_temperature(x, 0.5), [2.0, -4.0, 6.0])
    assert np.allclose(apply_repetition_penalty(x, [0, 1, 1, 7], 2.0), [0.5, -4.0, 3.0])
    assert np.array_equal(apply_repetition_penalty(x, [], 2.0), x) and np.array_equal(apply_repetition_penalty(x, [0], 1.0), x)
    # sharper temperature concentrates the draw on the mode; top_k=2 never leaves the two best tokens
    rng = np.random.default_rng(3)
    logits = np.array([0.0, 1.0, 2.0, 3.0])
    cold = [sample_token(logits, SamplingConfig(temperature=0.05), rng=rng) for _ in range(50)]
    assert set(cold) == {3}
    picks = {sample_token(logits, SamplingConfig.with_top_k(2, 1.0), rng=rng) for _ in range(200)}
    assert picks == {2, 3}
    picks = {sample_token(logits, SamplingConfig.nucleus(0.6, 1.0), rng=rng) for _ in range(200)}
    assert picks == {3}                                                 # p(3) = 0.644 alone reaches 0.6
