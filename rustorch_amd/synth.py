"""Seeded synthetic GGUF payloads of the benchmark configurations (host only).

A tensor is a pure function of (seed, tensor_id); the generator lives in the
native library (`rt_synth_*`).  Scale ranges follow the benchmark
configurations: Q8_0 d in [1e-4, 2e-3], Q4_0 d in [1e-3, 2e-2], Q4_K d and
dmin in [1e-3, 1e-2]; Q6_K uses the Q4_K range (its range is not specified).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .gguf import GGMLType

D_RANGE = {
    GGMLType.Q8_0: (1e-4, 2e-3),
    GGMLType.Q8_1: (1e-4, 2e-3),
    GGMLType.Q4_0: (1e-3, 2e-2),
    GGMLType.Q4_1: (1e-3, 2e-2),      # offsets m are drawn from -8 * this range (Q5_1: -16 *)
    GGMLType.Q5_0: (5e-4, 1e-2),
    GGMLType.Q5_1: (5e-4, 1e-2),
    GGMLType.Q2_K: (1e-3, 1e-2),
    GGMLType.Q3_K: (1e-3, 1e-2),
    GGMLType.Q4_K: (1e-3, 1e-2),
    GGMLType.Q5_K: (1e-3, 1e-2),
    GGMLType.Q6_K: (1e-3, 1e-2),
}

# Llama-7B layer shapes (n_rows = output features, n_cols = input features)
LLAMA7B = dict(n_layers=32, hidden=4096, n_heads=32, ffn=11008, vocab=32000, rms_eps=1e-5, rope_theta=10000.0)


DENSE_STD = 0.02      # unquantized synthetic matrices: N(0, DENSE_STD^2), rounded to the storage type


def blocks(ggml_type: int, seed: int, tensor_id: int, n_rows: int, n_cols: int, d_range=None) -> np.ndarray:
    """Raw GGUF payload (uint8) of an n_rows x n_cols tensor."""
    t = GGMLType(int(ggml_type))
    if t in (GGMLType.F16, GGMLType.F32):
        w = normal(seed, tensor_id, n_rows * n_cols, 0.0, DENSE_STD)
        return np.ascontiguousarray(w.astype(np.float16 if t == GGMLType.F16 else np.float32)).view(np.uint8)
    lo, hi = d_range if d_range is not None else D_RANGE[t]
    n_blocks = n_rows * (n_cols // t.block_elems())
    out = np.empty(n_blocks * t.type_size(), dtype=np.uint8)
    _lib.check(_lib.load().rt_synth_blocks(int(t), seed, tensor_id, n_blocks, lo, hi, C.c_void_p(out.ctypes.data)))
    return out


def normal(seed: int, tensor_id: int, n: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _lib.check(_lib.load().rt_synth_normal_f32(seed, tensor_id, n, mean, std, C.c_void_p(out.ctypes.data)))
    return out


def tokens(seed: int, tensor_id: int, n: int, vocab: int) -> np.ndarray:
    out = np.empty(n, dtype=np.int32)
    _lib.check(_lib.load().rt_synth_tokens(seed, tensor_id, n, vocab, C.c_void_p(out.ctypes.data)))
    return out


# tensor ids: global tensors 1..9, layer l slot s -> 100 * (l + 1) + s
TID_TOK_EMBD, TID_OUTPUT, TID_OUT_NORM, TID_PROMPT, TID_X = 1, 2, 3, 4, 5
LAYER_SLOTS = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down", "attn_norm", "ffn_norm")


def layer_tid(layer: int, slot: str) -> int:
    return 100 * (layer + 1) + LAYER_SLOTS.index(slot)


def layer_tensor_specs(hidden: int, ffn: int, kv_dim: int | None = None):
    """(slot, ggml type, n_rows, n_cols) of one decoder layer: q, k, o, gate, up are Q4_K; v and down are Q6_K.
    kv_dim = n_kv_heads * head_dim rows of k and v (default: hidden, one key / value head per query head)."""
    kv_dim = hidden if kv_dim is None else kv_dim
    return [
        ("attn_q", GGMLType.Q4_K, hidden, hidden),
        ("attn_k", GGMLType.Q4_K, kv_dim, hidden),
        ("attn_v", GGMLType.Q6_K, kv_dim, hidden),
        ("attn_output", GGMLType.Q4_K, hidden, hidden),
        ("ffn_gate", GGMLType.Q4_K, ffn, hidden),
        ("ffn_up", GGMLType.Q4_K, ffn, hidden),
        ("ffn_down", GGMLType.Q6_K, hidden, ffn),
    ]


def layer_weight_bytes(hidden: int, ffn: int) -> int:
    return sum(t.row_bytes(c) * r for _, t, r, c in layer_tensor_specs(hidden, ffn))
