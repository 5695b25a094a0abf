"""Inference timing in the reference CLI's vocabulary: `InferenceTimer`
(example-cli/src/metrics/timing.rs:111-199) and `MetricsCollector` with its targets
(example-cli/src/metrics/mod.rs:9-118: time to first token < 200 ms, > 20 tokens/s, memory < 1.5x model size)."""
from __future__ import annotations

import time
from dataclasses import dataclass, field


class InferenceTimer:
    def __init__(self):
        self.ttft = None            # seconds
        self.token_times = []       # seconds since start, one per generated token
        self.total_time = None
        self._t0 = None
        self._first_done = False

    def start(self) -> None:
        self._t0 = time.perf_counter()
        self._first_done = False

    def mark_first_token(self) -> None:
        if self._t0 is not None and not self._first_done:
            self.ttft = time.perf_counter() - self._t0
            self._first_done = True

    def mark_token(self) -> None:
        if self._t0 is not None:
            self.token_times.append(time.perf_counter() - self._t0)

    def end(self) -> None:
        if self._t0 is not None:
            self.total_time = time.perf_counter() - self._t0
            self._t0 = None

    def ttft_ms(self):
        return None if self.ttft is None else self.ttft * 1e3

    def total_ms(self):
        return None if self.total_time is None else self.total_time * 1e3

    def tokens_per_sec(self):
        if not self.total_time or self.total_time <= 0:
            return None
        return len(self.token_times) / self.total_time

    def avg_token_time_ms(self):
        """timing.rs:188-194 averages the recorded stamps themselves (times since start, not differences)."""
        if not self.token_times:
            return None
        return sum(self.token_times) * 1e3 / len(self.token_times)


@dataclass
class MetricsCollector:
    ttft: float | None = None               # ms
    tokens_per_sec: float | None = None
    total_time: float | None = None         # ms
    memory_usage: int | None = None         # bytes
    gpu_memory_usage: int | None = None
    model_size: int | None = None
    backend: str | None = None
    custom: dict = field(default_factory=dict)

    def set_ttft(self, ms): self.ttft = float(ms)
    def set_tokens_per_sec(self, v): self.tokens_per_sec = float(v)
    def set_total_time(self, ms): self.total_time = float(ms)
    def set_memory_usage(self, b): self.memory_usage = int(b)
    def set_gpu_memory_usage(self, b): self.gpu_memory_usage = int(b)
    def set_model_size(self, b): self.model_size = int(b)
    def set_backend(self, name): self.backend = str(name)
    def add_custom(self, key, value): self.custom[str(key)] = float(value)

    def memory_efficiency(self):
        if self.model_size is not None and self.memory_usage:
            return self.model_size / self.memory_usage
        return None

    def meets_ttft_target(self) -> bool:
        return self.ttft is not None and self.ttft < 200.0

    def meets_tps_target(self) -> bool:
        return self.tokens_per_sec is not None and self.tokens_per_sec > 20.0

    def meets_memory_target(self) -> bool:
        if self.model_size is None or self.memory_usage is None:
            return False
        return self.memory_usage < int(self.model_size * 1.5)

    def meets_all_targets(self) -> bool:
        return self.meets_ttft_target() and self.meets_tps_target() and self.meets_memory_target()
