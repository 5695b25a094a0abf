"""Host-side driver of the decode loop: what the CLI's `InferenceEngine`
(example-cli/src/model/inference.rs:91-211 in the reference) does once per
token, on top of the `rt_hip_llama_*` entry points."""
from __future__ import annotations

import ctypes as C
from typing import Callable, Iterable

import numpy as np

from . import _lib, synth
from .executor import HipKernelExecutor
from .gguf import GGMLType

SLOT = {"token_embd": 0, "output": 1, "output_norm": 2, "attn_q": 10, "attn_k": 11, "attn_v": 12, "attn_output": 13,
        "ffn_gate": 14, "ffn_up": 15, "ffn_down": 16, "attn_norm": 17, "ffn_norm": 18}


class HipLlama:
    def __init__(self, ex: HipKernelExecutor, n_layers: int, hidden: int, n_heads: int, ffn: int, vocab: int,
                 max_pos: int, rms_eps: float = 1e-5, rope_theta: float = 10000.0):
        self.ex = ex
        self.cfg = _lib.LlamaConfig(n_layers, hidden, n_heads, ffn, vocab, max_pos, rms_eps, rope_theta)
        self.h = C.c_void_p()
        _lib.check(ex.lib.rt_hip_llama_create(ex.ctx, C.byref(self.cfg), C.byref(self.h)), ex.ctx)

    def upload(self, slot: str, layer: int, ggml_type: int, n_rows: int, n_cols: int, raw: np.ndarray) -> None:
        raw = np.ascontiguousarray(raw)
        _lib.check(self.ex.lib.rt_hip_llama_upload_tensor(self.ex.ctx, self.h, SLOT[slot], layer, int(ggml_type), n_rows,
                                                          n_cols, C.c_void_p(raw.ctypes.data), raw.nbytes), self.ex.ctx)

    def set_mode(self, mode: int) -> None:
        """1 = one launch per operator group (default); 0 = one persistent launch per token (switched off in this build)."""
        _lib.check(self.ex.lib.rt_hip_llama_set_mode(self.ex.ctx, self.h, mode), self.ex.ctx)

    def reset(self) -> None:
        _lib.check(self.ex.lib.rt_hip_llama_reset(self.ex.ctx, self.h), self.ex.ctx)

    def step(self, token: int, pos: int, want_token: bool = True) -> int | None:
        nxt = C.c_int(-1)
        _lib.check(self.ex.lib.rt_hip_llama_step(self.ex.ctx, self.h, token, pos, C.byref(nxt) if want_token else None), self.ex.ctx)
        return int(nxt.value) if want_token else None

    def prefill(self, tokens: Iterable[int], pos0: int = 0) -> None:
        t = np.ascontiguousarray(np.asarray(list(tokens), dtype=np.int32))
        _lib.check(self.ex.lib.rt_hip_llama_prefill(self.ex.ctx, self.h, t.ctypes.data_as(_lib.c_int_p), t.size, pos0), self.ex.ctx)

    def logits(self) -> np.ndarray:
        out = np.empty(self.cfg.vocab, dtype=np.float32)
        _lib.check(self.ex.lib.rt_hip_llama_logits(self.ex.ctx, self.h, C.c_void_p(out.ctypes.data)), self.ex.ctx)
        return out

    def decode(self, first_token: int, pos0: int, n_steps: int, forced=None) -> np.ndarray:
        out = np.empty(n_steps, dtype=np.int32)
        f = None
        if forced is not None:
            f = np.ascontiguousarray(np.asarray(forced, dtype=np.int32))
            assert f.size >= n_steps
        _lib.check(self.ex.lib.rt_hip_llama_decode(self.ex.ctx, self.h, first_token, pos0, n_steps,
                                                   f.ctypes.data_as(_lib.c_int_p) if f is not None else None,
                                                   out.ctypes.data_as(_lib.c_int_p)), self.ex.ctx)
        return out

    def close(self) -> None:
        if self.h and self.ex.ctx:
            self.ex.lib.rt_hip_llama_destroy(self.ex.ctx, self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def synthetic_tensors(seed: int, n_layers: int, hidden: int, ffn: int, vocab: int):
    """Yield (slot, layer, ggml type, n_rows, n_cols, raw) of a random-init Llama: token embedding Q8_0,
    q/k/o/gate/up Q4_K, v/down and the output head Q6_K, RMSNorm weights f32 ~ 1 + N(0, 0.01)."""
    yield ("token_embd", -1, GGMLType.Q8_0, vocab, hidden, synth.blocks(GGMLType.Q8_0, seed, synth.TID_TOK_EMBD, vocab, hidden))
    yield ("output", -1, GGMLType.Q6_K, vocab, hidden, synth.blocks(GGMLType.Q6_K, seed, synth.TID_OUTPUT, vocab, hidden))
    yield ("output_norm", -1, GGMLType.F32, 1, hidden, synth.normal(seed, synth.TID_OUT_NORM, hidden, 1.0, 0.01))
    for l in range(n_layers):
        for slot, t, r, c in synth.layer_tensor_specs(hidden, ffn):
            yield (slot, l, t, r, c, synth.blocks(t, seed, synth.layer_tid(l, slot), r, c))
        yield ("attn_norm", l, GGMLType.F32, 1, hidden, synth.normal(seed, synth.layer_tid(l, "attn_norm"), hidden, 1.0, 0.01))
        yield ("ffn_norm", l, GGMLType.F32, 1, hidden, synth.normal(seed, synth.layer_tid(l, "ffn_norm"), hidden, 1.0, 0.01))


def load_synthetic(model: HipLlama, seed: int, sink: Callable | None = None) -> int:
    """Upload a synthetic model; `sink(slot, layer, type, n_rows, n_cols, raw)` sees every tensor too. Returns weight bytes."""
    c = model.cfg
    total = 0
    for slot, layer, t, r, cc, raw in synthetic_tensors(seed, c.n_layers, c.hidden, c.ffn, c.vocab):
        model.upload(slot, layer, t, r, cc, raw)
        if sink is not None:
            sink(slot, layer, t, r, cc, raw)
        if t != GGMLType.F32:
            total += raw.nbytes
    return total
