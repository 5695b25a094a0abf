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
                 max_pos: int, rms_eps: float = 1e-5, rope_theta: float = 10000.0, n_kv_heads: int = 0):
        """n_kv_heads: key / value heads of grouped-query attention (0 = n_heads)."""
        self.ex = ex
        self.cfg = _lib.LlamaConfig(n_layers, hidden, n_heads, ffn, vocab, max_pos, rms_eps, rope_theta, n_kv_heads)
        self.kv_dim = (n_kv_heads or n_heads) * (hidden // n_heads)
        self.h = C.c_void_p()
        _lib.check(ex.lib.rt_hip_llama_create(ex.ctx, C.byref(self.cfg), C.byref(self.h)), ex.ctx)

    def upload(self, slot: str, layer: int, ggml_type: int, n_rows: int, n_cols: int, raw: np.ndarray) -> None:
        raw = np.ascontiguousarray(raw)
        _lib.check(self.ex.lib.rt_hip_llama_upload_tensor(self.ex.ctx, self.h, SLOT[slot], layer, int(ggml_type), n_rows,
                                                          n_cols, C.c_void_p(raw.ctypes.data), raw.nbytes), self.ex.ctx)

    def set_mode(self, mode: int) -> None:
        """1 = one launch per operator group (default); 2 = the same launches replayed from a captured graph;
        0 = one persistent launch per token (switched off in this build)."""
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


class HipLlamaBatch:
    """Up to 8 sequences decoded side by side against one model's weights (rt_hip_llama_batch_*): each sequence has its own
    cache and position, a step feeds one token per sequence and streams every weight matrix once for all of them."""

    def __init__(self, model: HipLlama, n_seq: int, max_pos: int):
        self.model, self.ex, self.n_seq, self.max_pos = model, model.ex, n_seq, max_pos
        self.h = C.c_void_p()
        _lib.check(self.ex.lib.rt_hip_llama_batch_create(self.ex.ctx, model.h, n_seq, max_pos, C.byref(self.h)), self.ex.ctx)

    def reset(self, seq: int = -1) -> None:
        """Forget sequence `seq` (its slot can take a new prompt), or every sequence."""
        _lib.check(self.ex.lib.rt_hip_llama_batch_reset(self.ex.ctx, self.h, seq), self.ex.ctx)

    def step(self, tokens, positions, want_tokens: bool = True):
        """tokens[i] at positions[i] for every sequence i (a negative token leaves the sequence idle for the step);
        returns the greedy picks (-1 for idle sequences), or None."""
        t = np.ascontiguousarray(np.asarray(tokens, dtype=np.int32))
        p = np.ascontiguousarray(np.asarray(positions, dtype=np.int32))
        if t.shape != (self.n_seq,) or p.shape != (self.n_seq,):
            from .errors import ShapeMismatch
            raise ShapeMismatch("batch step: %d tokens and %d positions for %d sequences" % (t.size, p.size, self.n_seq))
        out = np.empty(self.n_seq, dtype=np.int32)
        _lib.check(self.ex.lib.rt_hip_llama_batch_step(self.ex.ctx, self.h, t.ctypes.data_as(_lib.c_int_p), p.ctypes.data_as(_lib.c_int_p),
                                                       out.ctypes.data_as(_lib.c_int_p) if want_tokens else None), self.ex.ctx)
        return out if want_tokens else None

    def prefill(self, seq: int, tokens, pos0: int = 0) -> None:
        """Three or more tokens of one sequence through the model's batched prefill passes, into that sequence's cache."""
        t = np.ascontiguousarray(np.asarray(list(tokens), dtype=np.int32))
        _lib.check(self.ex.lib.rt_hip_llama_batch_prefill(self.ex.ctx, self.h, seq, t.ctypes.data_as(_lib.c_int_p), t.size, pos0), self.ex.ctx)

    def logits(self) -> np.ndarray:
        out = np.empty((self.n_seq, self.model.cfg.vocab), dtype=np.float32)
        _lib.check(self.ex.lib.rt_hip_llama_batch_logits(self.ex.ctx, self.h, C.c_void_p(out.ctypes.data)), self.ex.ctx)
        return out

    def generate(self, prompts, max_new_tokens: int, eos_token: int | None = None, config=None, rng=None):
        """The generate loop (inference.rs:135-192) for n_seq prompts at once: feeds the prompts (a shorter prompt starts
        generating while longer ones are still being fed), stops a sequence at eos_token, after max_new_tokens or at the end
        of its cache, and leaves finished sequences idle while the others go on.  Greedy by default (the pick is made on the
        device); with a sampling configuration (sampling.rs:8-80) that is not greedy, every step's logits are read back and
        each live sequence draws on the host from its own row, with its own history for the repetition penalty.  Returns
        the generated ids per sequence."""
        from .sampling import SamplingConfig, sample_token
        config = config or SamplingConfig.greedy()
        config.validate()
        on_host = not (config.is_greedy and config.repetition_penalty == 1.0)
        prompts = [list(map(int, p)) for p in prompts]
        if len(prompts) != self.n_seq or any(len(p) == 0 for p in prompts):
            from .errors import ShapeMismatch
            raise ShapeMismatch("generate: %d non-empty prompts wanted" % self.n_seq)
        self.reset()
        out = [[] for _ in prompts]
        done = [False] * self.n_seq
        cur = [p[0] for p in prompts]
        pos = [0] * self.n_seq
        for i, p in enumerate(prompts):                      # all but the last prompt token in one prefill call where that is 3 tokens or more
            if 4 <= len(p) <= self.max_pos:
                self.prefill(i, p[:-1], 0)
                pos[i], cur[i] = len(p) - 1, p[-1]
        while True:
            for i in range(self.n_seq):
                done[i] = done[i] or pos[i] >= self.max_pos
            if all(done):
                break
            picks = self.step([-1 if done[i] else cur[i] for i in range(self.n_seq)], pos, want_tokens=not on_host)
            rows = self.logits() if on_host else None
            for i in range(self.n_seq):
                if done[i]:
                    continue
                pos[i] += 1
                if pos[i] < len(prompts[i]):
                    cur[i] = prompts[i][pos[i]]                      # still feeding the prompt
                    continue
                tok = int(sample_token(rows[i], config, prompts[i] + out[i], rng)) if on_host else int(picks[i])
                out[i].append(tok)
                cur[i] = tok
                if (eos_token is not None and tok == eos_token) or len(out[i]) >= max_new_tokens:
                    done[i] = True
        return out

    def close(self) -> None:
        if self.h and self.ex.ctx:
            self.ex.lib.rt_hip_llama_batch_destroy(self.ex.ctx, self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def synthetic_tensors(seed: int, n_layers: int, hidden: int, ffn: int, vocab: int, kv_dim: int | None = None):
    """Yield (slot, layer, ggml type, n_rows, n_cols, raw) of a random-init Llama: token embedding Q8_0,
    q/k/o/gate/up Q4_K, v/down and the output head Q6_K, RMSNorm weights f32 ~ 1 + N(0, 0.01)."""
    yield ("token_embd", -1, GGMLType.Q8_0, vocab, hidden, synth.blocks(GGMLType.Q8_0, seed, synth.TID_TOK_EMBD, vocab, hidden))
    yield ("output", -1, GGMLType.Q6_K, vocab, hidden, synth.blocks(GGMLType.Q6_K, seed, synth.TID_OUTPUT, vocab, hidden))
    yield ("output_norm", -1, GGMLType.F32, 1, hidden, synth.normal(seed, synth.TID_OUT_NORM, hidden, 1.0, 0.01))
    for l in range(n_layers):
        for slot, t, r, c in synth.layer_tensor_specs(hidden, ffn, kv_dim):
            yield (slot, l, t, r, c, synth.blocks(t, seed, synth.layer_tid(l, slot), r, c))
        yield ("attn_norm", l, GGMLType.F32, 1, hidden, synth.normal(seed, synth.layer_tid(l, "attn_norm"), hidden, 1.0, 0.01))
        yield ("ffn_norm", l, GGMLType.F32, 1, hidden, synth.normal(seed, synth.layer_tid(l, "ffn_norm"), hidden, 1.0, 0.01))


def load_synthetic(model: HipLlama, seed: int, sink: Callable | None = None) -> int:
    """Upload a synthetic model; `sink(slot, layer, type, n_rows, n_cols, raw)` sees every tensor too. Returns weight bytes."""
    c = model.cfg
    total = 0
    for slot, layer, t, r, cc, raw in synthetic_tensors(seed, c.n_layers, c.hidden, c.ffn, c.vocab, model.kv_dim):
        model.upload(slot, layer, t, r, cc, raw)
        if sink is not None:
            sink(slot, layer, t, r, cc, raw)
        if t != GGMLType.F32:
            total += raw.nbytes
    return total


# ---- GGUF model files: llama tensor names and metadata keys -> the upload slots above

_GLOBAL_NAMES = {"token_embd.weight": "token_embd", "output.weight": "output", "output_norm.weight": "output_norm"}
_LAYER_NAMES = {"attn_q": "attn_q", "attn_k": "attn_k", "attn_v": "attn_v", "attn_output": "attn_output", "ffn_gate": "ffn_gate",
                "ffn_up": "ffn_up", "ffn_down": "ffn_down", "attn_norm": "attn_norm", "ffn_norm": "ffn_norm"}


def gguf_tensor_name(slot: str, layer: int) -> str:
    return "%s.weight" % slot if layer < 0 else "blk.%d.%s.weight" % (layer, slot)


def write_synthetic_gguf(path, seed: int, n_layers: int, hidden: int, n_heads: int, ffn: int, vocab: int, context: int,
                         rms_eps: float = 1e-5, rope_theta: float = 10000.0, n_kv_heads: int = 0) -> None:
    """A random-init Llama as a GGUF v3 file (same tensors as `synthetic_tensors`), so the file path can be
    exercised without a downloaded model."""
    from . import gguf
    w = gguf.GGUFWriter()
    w.add_kv("general.architecture", gguf.VT_STRING, "llama")
    w.add_kv("general.name", gguf.VT_STRING, "synthetic-llama-seed-%d" % seed)
    w.add_kv("llama.block_count", gguf.VT_UINT32, n_layers)
    w.add_kv("llama.context_length", gguf.VT_UINT32, context)
    w.add_kv("llama.embedding_length", gguf.VT_UINT32, hidden)
    w.add_kv("llama.feed_forward_length", gguf.VT_UINT32, ffn)
    w.add_kv("llama.attention.head_count", gguf.VT_UINT32, n_heads)
    w.add_kv("llama.attention.head_count_kv", gguf.VT_UINT32, n_kv_heads or n_heads)
    w.add_kv("llama.attention.layer_norm_rms_epsilon", gguf.VT_FLOAT32, rms_eps)
    w.add_kv("llama.rope.freq_base", gguf.VT_FLOAT32, rope_theta)
    for slot, layer, t, r, c, raw in synthetic_tensors(seed, n_layers, hidden, ffn, vocab, (n_kv_heads or n_heads) * (hidden // n_heads)):
        dims = (c,) if t == GGMLType.F32 else (c, r)
        w.add_tensor(gguf_tensor_name(slot, layer), t, dims, raw)
    w.write(path)


def load_gguf(ex: HipKernelExecutor, path, max_pos: int | None = None) -> HipLlama:
    """Build a device model from a llama-architecture GGUF file: hyper-parameters from the metadata keys,
    every tensor's raw bytes uploaded as stored (what the reference's `load_gguf` stub,
    example-cli/src/model/loader.rs:55-59, leaves open)."""
    from . import gguf
    from .errors import InvalidParameters, UnsupportedOperation
    with gguf.GGUFLoader(path) as g:
        arch = g.get_metadata("general.architecture")
        if arch is None or arch.as_str() != "llama":
            raise UnsupportedOperation("load_gguf: architecture %r is not llama" % (arch.as_str() if arch else None))

        def need_u32(key):
            v = g.get_metadata(key)
            if v is None or v.as_u32() is None:
                raise InvalidParameters("load_gguf: metadata key %s missing or not an unsigned integer" % key)
            return v.as_u32()

        def opt_f32(key, default):
            v = g.get_metadata(key)
            return default if v is None or v.as_f32() is None else float(v.as_f32())

        n_layers, hidden = need_u32("llama.block_count"), need_u32("llama.embedding_length")
        ffn, n_heads = need_u32("llama.feed_forward_length"), need_u32("llama.attention.head_count")
        kv = g.get_metadata("llama.attention.head_count_kv")
        n_kv = n_heads if kv is None or kv.as_u32() is None else kv.as_u32()
        if n_kv == 0 or n_heads % n_kv != 0:
            raise InvalidParameters("load_gguf: head_count_kv=%d does not divide head_count=%d" % (n_kv, n_heads))
        emb = g.find_tensor("token_embd.weight")
        if emb is None or emb.n_dims != 2:
            raise InvalidParameters("load_gguf: token_embd.weight missing or not 2-D")
        vocab = emb.dims[1]
        ctx = g.get_metadata("llama.context_length")
        if max_pos is None:
            # the file's training context, capped at what the attention kernels hold per head (16 000 positions)
            max_pos = min(ctx.as_u32() if ctx is not None and ctx.as_u32() else 2048, 16000)
        model = HipLlama(ex, n_layers, hidden, n_heads, ffn, vocab, max_pos, opt_f32("llama.attention.layer_norm_rms_epsilon", 1e-5),
                         opt_f32("llama.rope.freq_base", 10000.0), n_kv)
        try:
            wanted = [(s, -1) for s in ("token_embd", "output", "output_norm")] + [(s, l) for l in range(n_layers) for s in _LAYER_NAMES]
            for slot, layer in wanted:
                name = gguf_tensor_name(slot, layer)
                t = g.find_tensor(name)
                if t is None and slot == "output":
                    t, name = emb, "token_embd.weight"          # tied embeddings: the head reuses the embedding matrix
                if t is None:
                    raise InvalidParameters("load_gguf: tensor %s missing" % name)
                raw = g.load_tensor_data(name)
                if slot.endswith("norm"):
                    model.upload(slot, layer, GGMLType.F32, 1, t.n_cols, g.load_f32(name))
                else:
                    model.upload(slot, layer, t.ggml_type, t.n_rows, t.n_cols, raw)
        except Exception:
            model.close()
            raise
        return model


def generate(model: HipLlama, prompt: Iterable[int], max_new_tokens: int, config=None, eos_token: int | None = None,
             rng=None, pos0: int = 0, on_token: Callable[[int], None] | None = None) -> list[int]:
    """Prompt in, new tokens out: the loop of `InferenceEngine::generate_with_gpt`
    (example-cli/src/model/inference.rs:135-192) -- forward, logits of the last position, pick, stop at the
    end-of-sequence token or at max_new_tokens.  Greedy configurations run entirely on the device
    (`rt_hip_llama_decode`); anything else reads the logits back each step and samples on the host."""
    from .sampling import SamplingConfig, sample_token
    config = config or SamplingConfig.greedy()
    config.validate()
    toks = [int(t) for t in prompt]
    if not toks:
        raise ValueError("generate: empty prompt")
    room = model.cfg.max_pos - (pos0 + len(toks)) + 1
    n_new = min(max_new_tokens, room)
    if n_new <= 0:
        return []
    if len(toks) > 1:
        model.prefill(toks[:-1], pos0)
    pos = pos0 + len(toks) - 1
    if config.is_greedy and config.repetition_penalty == 1.0:
        # the first token comes back on its own (the caller's time to first token), the rest in one device-side loop
        out = [int(model.step(toks[-1], pos))]
        if on_token is not None:
            on_token(out[0])
        if n_new > 1 and out[0] != eos_token:
            rest = [int(t) for t in model.decode(out[0], pos + 1, n_new - 1)]
            if eos_token is not None and eos_token in rest:
                rest = rest[:rest.index(eos_token) + 1]
            if on_token is not None:
                for t in rest:
                    on_token(t)
            out += rest
        return out
    out: list[int] = []
    cur = toks[-1]
    for _ in range(n_new):
        model.step(cur, pos, want_token=False)
        cur = sample_token(model.logits(), config, toks + out, rng)
        out.append(cur)
        if on_token is not None:
            on_token(cur)
        pos += 1
        if eos_token is not None and cur == eos_token:
            break
    return out
