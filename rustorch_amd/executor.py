"""Host-side mirror of the reference's per-vendor executor for `DeviceType::Hip`.

`HipKernelExecutor` is the sibling of `CudaKernelExecutor`
(src/gpu/cuda_kernels.rs:201-283 in the reference): `new(device_id)`, a
blocking `matmul_f32(a, b, c, m, n, k)` on host slices, plus the quantized
entry points the `hip` arm of `OptimizedOps::qmatmul`
(src/quantization/hardware/mod.rs:25-46) and a GGUF-aware `Linear` would call.
Every method forwards to the C ABI; numpy arrays stand in for Rust slices.
"""
from __future__ import annotations

import ctypes as C
from typing import Sequence

import numpy as np

from . import _lib
from .errors import InvalidParameters, ShapeMismatch
from .gguf import GGMLType


def device_count() -> int:
    return int(_lib.load().rt_hip_device_count())


def is_available() -> bool:
    """`DeviceType::Hip(0).is_available()` (src/gpu/mod.rs:429-486)."""
    return device_count() > 0


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _f32(a, name: str) -> np.ndarray:
    arr = np.ascontiguousarray(a, dtype=np.float32)
    if arr.size == 0:
        raise ShapeMismatch("%s is empty" % name)
    return arr


class DeviceBuffer:
    """Resident device memory, the `GpuBuffer<T>` idiom (src/gpu/memory_ops/buffer.rs:22-48)."""

    def __init__(self, ex: "HipKernelExecutor", nbytes: int):
        self.ex = ex
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _lib.check(ex.lib.rt_hip_malloc(ex.ctx, self.nbytes, C.byref(p)), ex.ctx)
        self.ptr = p

    @classmethod
    def from_host(cls, ex: "HipKernelExecutor", a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(ex, a.nbytes)
        buf.upload(a)
        return buf

    def upload(self, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        if a.nbytes > self.nbytes:
            raise ShapeMismatch("upload of %d bytes into a buffer of %d" % (a.nbytes, self.nbytes))
        _lib.check(self.ex.lib.rt_hip_memcpy_h2d(self.ex.ctx, self.ptr, _ptr(a), a.nbytes), self.ex.ctx)

    def download(self, dtype, count: int | None = None) -> np.ndarray:
        dt = np.dtype(dtype)
        n = self.nbytes // dt.itemsize if count is None else int(count)
        out = np.empty(n, dtype=dt)
        _lib.check(self.ex.lib.rt_hip_memcpy_d2h(self.ex.ctx, _ptr(out), self.ptr, out.nbytes), self.ex.ctx)
        return out

    def zero(self) -> None:
        _lib.check(self.ex.lib.rt_hip_memset_dev(self.ex.ctx, self.ptr, 0, self.nbytes), self.ex.ctx)

    def free(self) -> None:
        if self.ptr:
            self.ex.lib.rt_hip_free(self.ex.ctx, self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            if self.ex.ctx:
                self.free()
        except Exception:
            pass


class QWeight:
    """A GGUF tensor resident in HBM as its raw blocks, rows = output features (Linear stores W as [out, in])."""

    def __init__(self, ex: "HipKernelExecutor", handle: C.c_void_p, ggml_type: GGMLType, n_rows: int, n_cols: int,
                 nbytes: int):
        self.ex, self.handle, self.ggml_type = ex, handle, ggml_type
        self.n_rows, self.n_cols, self.nbytes = n_rows, n_cols, nbytes

    def free(self) -> None:
        if self.handle:
            self.ex.lib.rt_hip_qweight_free(self.ex.ctx, self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            if self.ex.ctx:
                self.free()
        except Exception:
            pass


class Event:
    def __init__(self, ex: "HipKernelExecutor"):
        self.ex = ex
        p = C.c_void_p()
        _lib.check(ex.lib.rt_hip_event_create(ex.ctx, C.byref(p)), ex.ctx)
        self.h = p

    def record(self) -> None:
        _lib.check(self.ex.lib.rt_hip_event_record(self.ex.ctx, self.h), self.ex.ctx)

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        _lib.check(self.ex.lib.rt_hip_event_elapsed_ms(self.ex.ctx, self.h, stop.h, C.byref(ms)), self.ex.ctx)
        return float(ms.value)

    def __del__(self):
        try:
            if self.ex.ctx and self.h:
                self.ex.lib.rt_hip_event_destroy(self.ex.ctx, self.h)
        except Exception:
            pass


class HipKernelExecutor:
    """`HipKernelExecutor::new(device_id)`; dropped by `close()` or garbage collection."""

    def __init__(self, device_id: int = 0):
        self.lib = _lib.load()
        self.ctx = C.c_void_p()
        self.device_id = device_id
        _lib.check(self.lib.rt_hip_create(device_id, C.byref(self.ctx)), None)

    # -- lifetime
    def close(self) -> None:
        if self.ctx:
            self.lib.rt_hip_destroy(self.ctx)
            self.ctx = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def synchronize(self) -> None:
        _lib.check(self.lib.rt_hip_synchronize(self.ctx), self.ctx)

    def device_info(self) -> dict:
        info = _lib.DevInfo()
        _lib.check(self.lib.rt_hip_device_info(self.device_id, C.byref(info)), None)
        return {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
                "wavefront_size": info.wavefront_size, "hbm_bytes": info.hbm_bytes,
                "lds_bytes_per_block": info.lds_bytes_per_block}

    # -- code-path switches (rt_hip_set_option): process-wide, read at every launch
    OPT_GEMV_LEAN = 1
    OPT_DENSE_MFMA = 2

    def set_option(self, option: int, value: int) -> None:
        _lib.check(self.lib.rt_hip_set_option(self.ctx, int(option), int(value)), self.ctx)

    def get_option(self, option: int) -> int:
        v = C.c_int(0)
        _lib.check(self.lib.rt_hip_get_option(self.ctx, int(option), C.byref(v)), self.ctx)
        return v.value

    def event(self) -> Event:
        return Event(self)

    def buffer(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, a: np.ndarray) -> DeviceBuffer:
        return DeviceBuffer.from_host(self, a)

    # -- dense f32: CudaKernelExecutor::matmul_f32(a, b, c, m, n, k)
    def matmul_f32(self, a, b, c: np.ndarray, m: int, n: int, k: int) -> None:
        a = _f32(a, "a"); b = _f32(b, "b")
        if a.size != m * k or b.size != k * n or c.size != m * n:
            raise ShapeMismatch("matmul_f32: slices of %d, %d, %d elements for m=%d n=%d k=%d" % (a.size, b.size, c.size, m, n, k))
        if c.dtype != np.float32 or not c.flags.c_contiguous:
            raise InvalidParameters("matmul_f32: c must be a contiguous float32 array")
        _lib.check(self.lib.rt_hip_matmul_f32(self.ctx, _ptr(a), _ptr(b), _ptr(c), m, n, k), self.ctx)

    def stream_read_dev(self, buf: DeviceBuffer, offset: int = 0, nbytes: int | None = None) -> None:
        """Measurement aid: one pass of plain reads over buf[offset : offset + nbytes] in the GEMV's access shape
        (rt_hip_stream_read_dev); offset a multiple of 16."""
        n = buf.nbytes - offset if nbytes is None else int(nbytes)
        if offset < 0 or n < 0 or offset + n > buf.nbytes:
            raise ShapeMismatch("stream_read_dev: bytes %d .. %d of a buffer of %d" % (offset, offset + n, buf.nbytes))
        _lib.check(self.lib.rt_hip_stream_read_dev(self.ctx, C.c_void_p(buf.ptr.value + offset), n), self.ctx)

    def matmul_f32_dev(self, a: DeviceBuffer, b: DeviceBuffer, c: DeviceBuffer, m: int, n: int, k: int, batch: int = 1) -> None:
        """c[i] = a[i] . b[i] for i < batch on resident buffers (gpu_matmul / gpu_batch_matmul / gpu_matvec with n = 1,
        src/gpu/matrix_ops.rs:562-595); enqueues only."""
        if a.nbytes < 4 * batch * m * k or b.nbytes < 4 * batch * k * n or c.nbytes < 4 * batch * m * n:
            raise ShapeMismatch("matmul_f32_dev: buffers of %d, %d, %d bytes for batch=%d m=%d n=%d k=%d" % (a.nbytes, b.nbytes, c.nbytes, batch, m, n, k))
        _lib.check(self.lib.rt_hip_matmul_f32_dev(self.ctx, a.ptr, b.ptr, c.ptr, m, n, k, batch), self.ctx)

    # -- per-tensor affine int8 tensors: QuantizedOps::qmatmul (src/quantization/operations.rs:195-260)
    def qmatmul_i8(self, a, scale_a: float, zero_point_a: int, b, scale_b: float, zero_point_b: int):
        """(int8 [m, n], output scale = scale_a * scale_b, output zero point = 0)."""
        a = np.ascontiguousarray(a); b = np.ascontiguousarray(b)
        if a.dtype != np.int8 or b.dtype != np.int8:
            raise InvalidParameters("qmatmul_i8: operands must be int8 arrays")
        if a.ndim != 2 or b.ndim != 2:
            raise InvalidParameters("qmatmul_i8: only 2D matrix multiplication is supported")      # operations.rs:218-223
        if a.shape[1] != b.shape[0]:
            raise ShapeMismatch("qmatmul_i8: expected %d rows in b, got %d" % (a.shape[1], b.shape[0]))
        out = np.empty((a.shape[0], b.shape[1]), dtype=np.int8)
        sc, zp = C.c_float(), C.c_int()
        _lib.check(self.lib.rt_hip_qmatmul_i8(self.ctx, _ptr(a), float(scale_a), int(zero_point_a), _ptr(b), float(scale_b), int(zero_point_b),
                                              a.shape[0], b.shape[1], a.shape[1], _ptr(out), C.byref(sc), C.byref(zp)), self.ctx)
        return out, float(sc.value), int(zp.value)

    # -- quantized weights
    def upload_qweight(self, ggml_type: int, n_rows: int, n_cols: int, raw: np.ndarray | bytes) -> QWeight:
        raw = np.frombuffer(raw, dtype=np.uint8) if isinstance(raw, (bytes, bytearray, memoryview)) else np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        h = C.c_void_p()
        _lib.check(self.lib.rt_hip_qweight_upload(self.ctx, int(ggml_type), n_rows, n_cols, _ptr(raw), raw.nbytes, C.byref(h)), self.ctx)
        return QWeight(self, h, GGMLType(int(ggml_type)), n_rows, n_cols, raw.nbytes)

    def dequant(self, w: QWeight) -> np.ndarray:
        out = np.empty((w.n_rows, w.n_cols), dtype=np.float32)
        _lib.check(self.lib.rt_hip_dequant(self.ctx, w.handle, _ptr(out)), self.ctx)
        return out

    def qgemv(self, w: QWeight, x) -> np.ndarray:
        """y[batch, n_rows] = x[batch, n_cols] . dequant(W)^T for batch 1..8 (a 1-D x gives a 1-D y)."""
        x = _f32(x, "x")
        one_d = x.ndim == 1
        x2 = x.reshape(1, -1) if one_d else x
        if x2.ndim != 2 or x2.shape[1] != w.n_cols:
            raise ShapeMismatch("qgemv: x has shape %s, weight is %d x %d" % (x.shape, w.n_rows, w.n_cols))
        y = np.empty((x2.shape[0], w.n_rows), dtype=np.float32)
        _lib.check(self.lib.rt_hip_qgemv(self.ctx, w.handle, _ptr(x2), _ptr(y), x2.shape[0]), self.ctx)
        return y[0] if one_d else y

    def qgemm(self, w: QWeight, X) -> np.ndarray:
        """Y[M, n_rows] = X[M, n_cols] . dequant(W)^T (prefill)."""
        X = _f32(X, "X")
        if X.ndim != 2 or X.shape[1] != w.n_cols:
            raise ShapeMismatch("qgemm: X has shape %s, weight is %d x %d" % (X.shape, w.n_rows, w.n_cols))
        Y = np.empty((X.shape[0], w.n_rows), dtype=np.float32)
        _lib.check(self.lib.rt_hip_qgemm(self.ctx, w.handle, _ptr(X), X.shape[0], _ptr(Y)), self.ctx)
        return Y

    def qlinear(self, w: QWeight, x) -> np.ndarray:
        """`Linear::forward` without bias (src/nn/linear.rs:150-182): GEMV up to 8 rows, GEMM beyond."""
        x = _f32(x, "x")
        rows = 1 if x.ndim == 1 else x.shape[0]
        return self.qgemv(w, x) if rows <= 8 else self.qgemm(w, x)

    # -- device-pointer forms
    def qgemv_dev(self, w: QWeight, x: DeviceBuffer, y: DeviceBuffer, batch: int = 1) -> None:
        _lib.check(self.lib.rt_hip_qgemv_dev(self.ctx, w.handle, x.ptr, y.ptr, batch), self.ctx)

    def qgemm_dev(self, w: QWeight, x: DeviceBuffer, m: int, y: DeviceBuffer) -> None:
        _lib.check(self.lib.rt_hip_qgemm_dev(self.ctx, w.handle, x.ptr, m, y.ptr), self.ctx)

    def qgemv_grouped_dev(self, ws: Sequence[QWeight], xs: Sequence[DeviceBuffer], ys: Sequence[DeviceBuffer]) -> None:
        n = len(ws)
        if not (n == len(xs) == len(ys)):
            raise InvalidParameters("grouped GEMV: %d weights, %d inputs, %d outputs" % (n, len(xs), len(ys)))
        arr = C.c_void_p * n
        wa = arr(*[w.handle for w in ws]); xa = arr(*[x.ptr for x in xs]); ya = arr(*[y.ptr for y in ys])
        _lib.check(self.lib.rt_hip_qgemv_grouped_dev(self.ctx, n, wa, xa, ya), self.ctx)

    def qgemv_shared_x_dev(self, ws: Sequence[QWeight], x: DeviceBuffer, ys: Sequence[DeviceBuffer], batch: int) -> None:
        """Several weights against one activation batch (q / k / v, gate / up): ys[i] = x[batch, n_cols] . dequant(ws[i])^T."""
        n = len(ws)
        if n != len(ys):
            raise InvalidParameters("shared-x GEMV: %d weights, %d outputs" % (n, len(ys)))
        arr = C.c_void_p * n
        wa = arr(*[w.handle for w in ws]); ya = arr(*[y.ptr for y in ys])
        _lib.check(self.lib.rt_hip_qgemv_shared_x_dev(self.ctx, n, wa, x.ptr, ya, batch), self.ctx)

    def xq_bytes(self, n_cols: int) -> int:
        return int(self.lib.rt_hip_xq_bytes(n_cols))

    def quantize_act_dev(self, xs: Sequence[DeviceBuffer], n_cols: Sequence[int], xqs: Sequence[DeviceBuffer]) -> None:
        n = len(xs)
        arr = C.c_void_p * n
        xa = arr(*[x.ptr for x in xs]); qa = arr(*[q.ptr for q in xqs]); ka = (C.c_size_t * n)(*n_cols)
        _lib.check(self.lib.rt_hip_quantize_act_dev(self.ctx, n, xa, ka, qa), self.ctx)

    def qgemv_xq_grouped_dev(self, ws: Sequence[QWeight], xqs: Sequence[DeviceBuffer], ys: Sequence[DeviceBuffer]) -> None:
        n = len(ws)
        arr = C.c_void_p * n
        wa = arr(*[w.handle for w in ws]); qa = arr(*[q.ptr for q in xqs]); ya = arr(*[y.ptr for y in ys])
        _lib.check(self.lib.rt_hip_qgemv_xq_grouped_dev(self.ctx, n, wa, qa, ya), self.ctx)

    def qgemv_describe(self, ws: Sequence[QWeight], batch: int = 1) -> str:
        """The kernel a grouped launch over these weights would run and how it would be cut (rt_hip_qgemv_describe)."""
        n = len(ws)
        wa = (C.c_void_p * n)(*[w.handle for w in ws])
        buf = C.create_string_buffer(256)
        _lib.check(self.lib.rt_hip_qgemv_describe(self.ctx, n, wa, batch, buf, len(buf)), self.ctx)
        return buf.value.decode()

    # -- decode-step operators (host arrays in, host arrays out; each call goes through device buffers)
    def rmsnorm(self, x, gamma, eps: float) -> np.ndarray:
        x = _f32(x, "x"); gamma = _f32(gamma, "gamma")
        x2 = x.reshape(1, -1) if x.ndim == 1 else x
        if x2.shape[-1] != gamma.size:
            raise ShapeMismatch("rmsnorm: x rows of %d, gamma of %d" % (x2.shape[-1], gamma.size))
        dx, dg = self.to_device(x2), self.to_device(gamma)
        dy = self.buffer(x2.nbytes)
        _lib.check(self.lib.rt_hip_rmsnorm_dev(self.ctx, dx.ptr, dg.ptr, dy.ptr, x2.shape[0], x2.shape[1], eps), self.ctx)
        return dy.download(np.float32).reshape(x.shape)

    def swiglu(self, gate, up) -> np.ndarray:
        gate = _f32(gate, "gate"); up = _f32(up, "up")
        if gate.shape != up.shape:
            raise ShapeMismatch("swiglu: gate %s vs up %s" % (gate.shape, up.shape))
        dg, du = self.to_device(gate), self.to_device(up)
        do = self.buffer(gate.nbytes)
        _lib.check(self.lib.rt_hip_swiglu_dev(self.ctx, dg.ptr, du.ptr, do.ptr, gate.size), self.ctx)
        return do.download(np.float32).reshape(gate.shape)

    def rope(self, x, n_heads: int, head_dim: int, pos: int, theta: float) -> np.ndarray:
        x = _f32(x, "x")
        if x.size != n_heads * head_dim:
            raise ShapeMismatch("rope: %d elements for %d heads of %d" % (x.size, n_heads, head_dim))
        dx = self.to_device(x)
        _lib.check(self.lib.rt_hip_rope_dev(self.ctx, dx.ptr, n_heads, head_dim, pos, theta), self.ctx)
        return dx.download(np.float32).reshape(x.shape)

    def attn_decode(self, q, kcache_f16: np.ndarray, vcache_f16: np.ndarray, n_pos: int, n_heads: int, head_dim: int) -> np.ndarray:
        q = _f32(q, "q")
        row = n_heads * head_dim
        if q.size != row or kcache_f16.size < n_pos * row or vcache_f16.size < n_pos * row:
            raise ShapeMismatch("attn_decode: operand sizes do not match n_pos=%d n_heads=%d head_dim=%d" % (n_pos, n_heads, head_dim))
        dq = self.to_device(q)
        dk = self.to_device(np.ascontiguousarray(kcache_f16).view(np.uint16))
        dv = self.to_device(np.ascontiguousarray(vcache_f16).view(np.uint16))
        do = self.buffer(row * 4)
        _lib.check(self.lib.rt_hip_attn_decode_dev(self.ctx, dq.ptr, dk.ptr, dv.ptr, n_pos, n_heads, head_dim, do.ptr), self.ctx)
        return do.download(np.float32)

    def attn_causal(self, q, kcache_f16: np.ndarray, vcache_f16: np.ndarray, pos0: int, n_heads: int, head_dim: int,
                    n_kv_heads: int = 0) -> np.ndarray:
        """q[n_queries, n_heads * head_dim]: row m sits at position pos0 + m and attends cache rows [0, pos0 + m]."""
        q = _f32(q, "q")
        row, rowkv = n_heads * head_dim, (n_kv_heads or n_heads) * head_dim
        if q.ndim != 2 or q.shape[1] != row or q.shape[0] == 0:
            raise ShapeMismatch("attn_causal: q must be [n_queries, %d]" % row)
        n_pos = pos0 + q.shape[0]
        if kcache_f16.size < n_pos * rowkv or vcache_f16.size < n_pos * rowkv:
            raise ShapeMismatch("attn_causal: the caches hold fewer than %d rows of %d" % (n_pos, rowkv))
        dq = self.to_device(q)
        dk = self.to_device(np.ascontiguousarray(kcache_f16).view(np.uint16))
        dv = self.to_device(np.ascontiguousarray(vcache_f16).view(np.uint16))
        do = self.buffer(q.size * 4)
        _lib.check(self.lib.rt_hip_attn_causal_dev(self.ctx, dq.ptr, dk.ptr, dv.ptr, pos0, q.shape[0], n_heads, n_kv_heads, head_dim, do.ptr), self.ctx)
        return do.download(np.float32).reshape(q.shape)

    def kv_append(self, cache: DeviceBuffer, v, pos: int) -> None:
        v = _f32(v, "v")
        dv = self.to_device(v)
        _lib.check(self.lib.rt_hip_kv_append_dev(self.ctx, cache.ptr, dv.ptr, pos, v.size), self.ctx)
        self.synchronize()

    def add(self, x, y) -> np.ndarray:
        x = _f32(x, "x"); y = _f32(y, "y")
        if x.shape != y.shape:
            raise ShapeMismatch("add: %s vs %s" % (x.shape, y.shape))
        dx, dy = self.to_device(x), self.to_device(y)
        _lib.check(self.lib.rt_hip_add_dev(self.ctx, dx.ptr, dy.ptr, x.size), self.ctx)
        return dx.download(np.float32).reshape(x.shape)

    def add_dev(self, x: DeviceBuffer, y: DeviceBuffer, n: int) -> None:
        """x[i] += y[i] for n f32 values, both resident on the device."""
        _lib.check(self.lib.rt_hip_add_dev(self.ctx, x.ptr, y.ptr, n), self.ctx)

    def argmax(self, v) -> int:
        v = _f32(v, "v")
        dv = self.to_device(v)
        do = self.buffer(4)
        _lib.check(self.lib.rt_hip_argmax_dev(self.ctx, dv.ptr, v.size, do.ptr), self.ctx)
        return int(do.download(np.int32)[0])
