"""Sampling of the next token from a logits row, on the host.

Mirrors example-cli/src/model/sampling.rs of the reference: `SamplingConfig` with its constructors and
`validate` (:8-80), `softmax` (:118-132), temperature scaling (:135-151), `apply_top_k_to_probs` (:154-181),
`apply_top_p_to_probs` (:201-240), `multinomial_sample` (:258-274) and the repetition penalty the reference
only sketches in a comment (:283-288).  The reference's `sample_token` itself is a stub that returns
vocab/2 (:84-115); `sample_token` here does what that stub's comments list, in that order.  Greedy
(temperature 0 or top_k 1) is the device-side argmax of the decode loop: ties resolve to the lowest index.
All arithmetic is float64, as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

from .errors import InvalidParameters


@dataclass
class SamplingConfig:
    temperature: float = 1.0
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    repetition_penalty: float = 1.0

    @classmethod
    def greedy(cls) -> "SamplingConfig":
        return cls(temperature=0.0, top_k=1)

    @classmethod
    def with_top_k(cls, k: int, temperature: float) -> "SamplingConfig":
        return cls(temperature=temperature, top_k=k)

    @classmethod
    def nucleus(cls, p: float, temperature: float) -> "SamplingConfig":
        return cls(temperature=temperature, top_p=p)

    def validate(self) -> None:
        if self.temperature < 0.0:
            raise InvalidParameters("Temperature must be non-negative")
        if self.top_k is not None and self.top_k == 0:
            raise InvalidParameters("top_k must be positive")
        if self.top_p is not None and not (0.0 <= self.top_p <= 1.0):
            raise InvalidParameters("top_p must be between 0.0 and 1.0")
        if self.repetition_penalty < 0.0:
            raise InvalidParameters("Repetition penalty must be non-negative")

    @property
    def is_greedy(self) -> bool:
        return self.temperature == 0.0 or self.top_k == 1


def softmax(logits) -> np.ndarray:
    x = np.asarray(logits, dtype=np.float64)
    e = np.exp(x - x.max())
    return e / e.sum()


def apply_temperature(logits, temperature: float) -> np.ndarray:
    x = np.asarray(logits, dtype=np.float64)
    if temperature == 0.0 or temperature == 1.0:
        return x.copy()
    return x / temperature


def _descending(probs: np.ndarray) -> np.ndarray:
    # stable: equal probabilities keep index order, as the reference's stable sort does
    return np.argsort(-probs, kind="stable")


def apply_top_k_to_probs(probs, k: int) -> np.ndarray:
    p = np.asarray(probs, dtype=np.float64)
    if k == 0 or k >= p.size:
        return p.copy()
    out = np.zeros_like(p)
    keep = _descending(p)[:k]
    out[keep] = p[keep]
    s = out.sum()
    return out / s if s > 0.0 else out


def apply_top_p_to_probs(probs, p_keep: float) -> np.ndarray:
    p = np.asarray(probs, dtype=np.float64)
    if p_keep <= 0.0 or p_keep >= 1.0:
        return p.copy()
    order = _descending(p)
    cum = np.cumsum(p[order])
    hit = np.nonzero(cum >= p_keep)[0]
    cutoff = int(hit[0]) + 1 if hit.size else p.size       # smallest set whose cumulative probability reaches p
    out = np.zeros_like(p)
    out[order[:cutoff]] = p[order[:cutoff]]
    s = out.sum()
    return out / s if s > 0.0 else out


def apply_repetition_penalty(logits, previous_tokens: Sequence[int], penalty: float) -> np.ndarray:
    x = np.asarray(logits, dtype=np.float64).copy()
    if penalty == 1.0 or len(previous_tokens) == 0:
        return x
    for t in set(int(t) for t in previous_tokens):
        if 0 <= t < x.size:
            x[t] = x[t] / penalty if x[t] > 0 else x[t] * penalty
    return x


def multinomial_sample(probs, rng: np.random.Generator) -> int:
    r = rng.random()
    cum = np.cumsum(np.asarray(probs, dtype=np.float64))
    hit = np.nonzero(r < cum)[0]
    return int(hit[0]) if hit.size else int(cum.size - 1)       # fallback: last index


def sample_token(logits, config: SamplingConfig, previous_tokens: Sequence[int] = (), rng: Optional[np.random.Generator] = None) -> int:
    """Repetition penalty -> temperature -> softmax -> top-k -> top-p -> multinomial draw; greedy configurations
    return the arg-max (lowest index on ties)."""
    config.validate()
    x = apply_repetition_penalty(np.asarray(logits, dtype=np.float64).reshape(-1), previous_tokens, config.repetition_penalty)
    if config.is_greedy:
        return int(np.argmax(x))
    probs = softmax(apply_temperature(x, config.temperature))
    if config.top_k is not None:
        probs = apply_top_k_to_probs(probs, config.top_k)
    if config.top_p is not None:
        probs = apply_top_p_to_probs(probs, config.top_p)
    return multinomial_sample(probs, rng if rng is not None else np.random.default_rng())
