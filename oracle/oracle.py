"""ctypes wrapper of the CPU oracle (oracle/rt_oracle.c).

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the bench's cpu_baseline leg
load this; the product (rustorch_amd, librustorch_hip) never does.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "liboracle.so"

_lib = None


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "liboracle.so"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB.exists():
        build()
    lib = C.CDLL(str(LIB))
    vp, sz, i, f = C.c_void_p, C.c_size_t, C.c_int, C.c_float
    sig = {
        "orc_h2f": (C.c_float, [C.c_uint16]),
        "orc_f2h": (C.c_uint16, [C.c_float]),
        "orc_block_elems": (i, [i]), "orc_block_bytes": (i, [i]), "orc_row_bytes": (sz, [i, sz]),
        "orc_dequant": (i, [i, vp, sz, sz, vp]),
        "orc_dequant_nt": (i, [i, vp, sz, sz, vp, i]),
        "orc_matmul_xwt": (None, [vp, vp, vp, sz, sz, sz, i]),
        "orc_qmatmul_i8": (C.c_float, [vp, C.c_float, i, vp, C.c_float, i, sz, sz, sz, vp]),
        "orc_qgemv": (i, [i, vp, sz, sz, vp, sz, vp, i]),
        "orc_qgemm": (i, [i, vp, sz, sz, vp, sz, vp, i]),
        "orc_qgemv_f64": (i, [i, vp, sz, sz, vp, sz, vp, vp, i]),
        "orc_rmsnorm": (None, [vp, vp, sz, f, sz, vp]),
        "orc_swiglu": (None, [vp, vp, sz, vp]),
        "orc_rope_inv_freq": (None, [i, f, vp]),
        "orc_rope": (None, [vp, i, i, i, vp]),
        "orc_kv_append": (None, [vp, vp, sz, sz]),
        "orc_attn_decode": (None, [vp, vp, vp, i, i, i, vp]),
        "orc_attn_decode_gqa": (None, [vp, vp, vp, i, i, i, i, vp]),
        "orc_llama_set_kv_heads": (i, [vp, i]),
        "orc_argmax": (i, [vp, sz]),
        "orc_add": (None, [vp, vp, sz]),
        "orc_llama_create": (vp, [i, i, i, i, i, i, f, f, i]),
        "orc_llama_destroy": (None, [vp]),
        "orc_llama_set_tensor": (i, [vp, i, i, i, vp, sz, sz]),
        "orc_llama_forward": (i, [vp, vp, i, i, vp, i]),
        "orc_num_threads": (i, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _raw(a) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


def h2f(h: int) -> float:
    return float(load().orc_h2f(int(h)))


def f2h(x: float) -> int:
    return int(load().orc_f2h(float(x)))


def num_threads() -> int:
    return int(load().orc_num_threads())


def dequant(ggml_type: int, raw, n_rows: int, n_cols: int, nthreads: int = 0) -> np.ndarray:
    raw = _raw(raw)
    out = np.empty((n_rows, n_cols), dtype=np.float32)
    if load().orc_dequant_nt(int(ggml_type), _p(raw), n_rows, n_cols, _p(out), nthreads or num_threads()) != 0:
        raise ValueError("oracle: bad type/shape")
    return out


def matmul_xwt(x: np.ndarray, w: np.ndarray, nthreads: int = 0) -> np.ndarray:
    """y = x . w^T with one sequential f32 k-sum per output (dense reference path)."""
    x = np.ascontiguousarray(x, dtype=np.float32); w = np.ascontiguousarray(w, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    y = np.empty((x2.shape[0], w.shape[0]), dtype=np.float32)
    load().orc_matmul_xwt(_p(x2), _p(w), _p(y), x2.shape[0], w.shape[0], w.shape[1], nthreads or num_threads())
    return y[0] if x.ndim == 1 else y


def qmatmul_i8(a: np.ndarray, scale_a: float, zp_a: int, b: np.ndarray, scale_b: float, zp_b: int):
    """Per-tensor affine int8 matmul (operations.rs:195-260): returns (int8 [m,n], output scale, zero point 0)."""
    a = np.ascontiguousarray(a, dtype=np.int8); b = np.ascontiguousarray(b, dtype=np.int8)
    m, k = a.shape
    k2, n = b.shape
    if k != k2:
        raise ValueError("oracle: inner dimensions differ")
    out = np.empty((m, n), dtype=np.int8)
    scale = load().orc_qmatmul_i8(_p(a), scale_a, zp_a, _p(b), scale_b, zp_b, m, n, k, _p(out))
    return out, float(scale), 0


def qgemv(ggml_type: int, raw, n_rows: int, n_cols: int, x: np.ndarray, nthreads: int = 0) -> np.ndarray:
    raw = _raw(raw)
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    y = np.empty((x2.shape[0], n_rows), dtype=np.float32)
    if load().orc_qgemm(int(ggml_type), _p(raw), n_rows, n_cols, _p(x2), x2.shape[0], _p(y), nthreads or num_threads()) != 0:
        raise ValueError("oracle: bad type/shape")
    return y[0] if x.ndim == 1 else y


def qgemv_f64(ggml_type: int, raw, n_rows: int, n_cols: int, x: np.ndarray, nthreads: int = 0):
    """(y in f64 accumulation, ||w_row||_2 per row)."""
    raw = _raw(raw)
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    y = np.empty((x2.shape[0], n_rows), dtype=np.float64)
    wn = np.empty(n_rows, dtype=np.float64)
    if load().orc_qgemv_f64(int(ggml_type), _p(raw), n_rows, n_cols, _p(x2), x2.shape[0], _p(y), _p(wn), nthreads or num_threads()) != 0:
        raise ValueError("oracle: bad type/shape")
    return (y[0] if x.ndim == 1 else y), wn


def rmsnorm(x: np.ndarray, gamma: np.ndarray, eps: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32); gamma = np.ascontiguousarray(gamma, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    y = np.empty_like(x2)
    load().orc_rmsnorm(_p(x2), _p(gamma), x2.shape[1], eps, x2.shape[0], _p(y))
    return y.reshape(x.shape)


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    gate = np.ascontiguousarray(gate, dtype=np.float32); up = np.ascontiguousarray(up, dtype=np.float32)
    out = np.empty_like(gate)
    load().orc_swiglu(_p(gate), _p(up), gate.size, _p(out))
    return out


def rope_inv_freq(head_dim: int, theta: float) -> np.ndarray:
    out = np.empty(head_dim // 2, dtype=np.float32)
    load().orc_rope_inv_freq(head_dim, theta, _p(out))
    return out


def rope(x: np.ndarray, n_heads: int, head_dim: int, pos: int, theta: float) -> np.ndarray:
    out = np.array(x, dtype=np.float32, copy=True).reshape(-1)
    inv = rope_inv_freq(head_dim, theta)
    load().orc_rope(_p(out), n_heads, head_dim, pos, _p(inv))
    return out.reshape(np.shape(x))


def kv_append(cache_u16: np.ndarray, v: np.ndarray, pos: int) -> None:
    v = np.ascontiguousarray(v, dtype=np.float32)
    load().orc_kv_append(_p(cache_u16), _p(v), pos, v.size)


def attn_decode(q: np.ndarray, kc_u16: np.ndarray, vc_u16: np.ndarray, n_pos: int, n_heads: int, head_dim: int,
                n_kv_heads: int = 0) -> np.ndarray:
    """n_kv_heads (0 = n_heads): cache rows hold that many heads; query head h reads head h // (n_heads // n_kv_heads)."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    kc_u16 = np.ascontiguousarray(kc_u16); vc_u16 = np.ascontiguousarray(vc_u16)
    out = np.empty(n_heads * head_dim, dtype=np.float32)
    load().orc_attn_decode_gqa(_p(q), _p(kc_u16), _p(vc_u16), n_pos, n_heads, n_kv_heads or n_heads, head_dim, _p(out))
    return out


def argmax(v: np.ndarray) -> int:
    v = np.ascontiguousarray(v, dtype=np.float32)
    return int(load().orc_argmax(_p(v), v.size))


SLOT = {"token_embd": 0, "output": 1, "output_norm": 2, "attn_q": 10, "attn_k": 11, "attn_v": 12, "attn_output": 13,
        "ffn_gate": 14, "ffn_up": 15, "ffn_down": 16, "attn_norm": 17, "ffn_norm": 18}


class OracleLlama:
    """CPU decode loop over borrowed raw tensors (keeps references so the buffers outlive the model)."""

    def __init__(self, n_layers, hidden, n_heads, ffn, vocab, max_pos, eps=1e-5, theta=10000.0, nthreads=0, n_kv_heads=0):
        self.vocab = vocab
        self.keep = []
        self.h = C.c_void_p(load().orc_llama_create(n_layers, hidden, n_heads, ffn, vocab, max_pos, eps, theta, nthreads or num_threads()))
        if n_kv_heads and load().orc_llama_set_kv_heads(self.h, n_kv_heads) != 0:
            raise ValueError("oracle: n_kv_heads must divide n_heads")

    def set_tensor(self, slot, layer, ggml_type, n_rows, n_cols, raw):
        raw = np.ascontiguousarray(raw)
        self.keep.append(raw)
        rc = load().orc_llama_set_tensor(self.h, SLOT[slot], layer, int(ggml_type), _p(raw), n_rows, n_cols)
        if rc != 0:
            raise ValueError("oracle: bad tensor slot/layer")

    def forward(self, tokens, pos0: int, last_only: bool = False) -> np.ndarray:
        t = np.ascontiguousarray(np.asarray(tokens, dtype=np.int32))
        out = np.empty((1 if last_only else t.size, self.vocab), dtype=np.float32)
        rc = load().orc_llama_forward(self.h, _p(t), t.size, pos0, _p(out), 1 if last_only else 0)
        if rc != 0:
            raise ValueError("oracle llama forward failed (%d)" % rc)
        return out

    def close(self):
        if self.h:
            load().orc_llama_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
