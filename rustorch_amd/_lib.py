"""ctypes binding of librustorch_hip.so (the declarations of include/rustorch_hip.h)."""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

from . import errors

_PKG = Path(__file__).resolve().parent
# RUSTORCH_HIP_LIBRARY names another build of the same library (a differently tuned or instrumented one)
LIB_PATH = Path(os.environ["RUSTORCH_HIP_LIBRARY"]) if os.environ.get("RUSTORCH_HIP_LIBRARY") else _PKG / "librustorch_hip.so"

c_void_pp = C.POINTER(C.c_void_p)
c_float_p = C.POINTER(C.c_float)
c_int_p = C.POINTER(C.c_int)


class DevInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int),
                ("wavefront_size", C.c_int), ("hbm_bytes", C.c_size_t), ("lds_bytes_per_block", C.c_size_t)]


class LlamaConfig(C.Structure):
    _fields_ = [("n_layers", C.c_int), ("hidden", C.c_int), ("n_heads", C.c_int), ("ffn", C.c_int),
                ("vocab", C.c_int), ("max_pos", C.c_int), ("rms_eps", C.c_float), ("rope_theta", C.c_float),
                ("n_kv_heads", C.c_int)]


# name -> (restype, argtypes); the keys are exactly the RT_HIP_API symbols of the header
SIGNATURES = {
    "rt_hip_device_count": (C.c_int, []),
    "rt_hip_device_info": (C.c_int, [C.c_int, C.POINTER(DevInfo)]),
    "rt_hip_create": (C.c_int, [C.c_int, c_void_pp]),
    "rt_hip_destroy": (C.c_int, [C.c_void_p]),
    "rt_hip_synchronize": (C.c_int, [C.c_void_p]),
    "rt_hip_last_error": (C.c_char_p, [C.c_void_p]),
    "rt_hip_type_block_bytes": (C.c_size_t, [C.c_int]),
    "rt_hip_type_block_elems": (C.c_size_t, [C.c_int]),
    "rt_hip_malloc": (C.c_int, [C.c_void_p, C.c_size_t, c_void_pp]),
    "rt_hip_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_memcpy_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rt_hip_memcpy_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rt_hip_memset_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t]),
    "rt_hip_event_create": (C.c_int, [C.c_void_p, c_void_pp]),
    "rt_hip_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, c_float_p]),
    "rt_hip_event_destroy": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_set_option": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "rt_hip_get_option": (C.c_int, [C.c_void_p, C.c_int, c_int_p]),
    "rt_hip_stream_read_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "rt_hip_matmul_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]),
    "rt_hip_matmul_f32_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]),
    "rt_hip_qmatmul_i8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_void_p, C.c_float, C.c_int, C.c_size_t, C.c_size_t,
                                    C.c_size_t, C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_int)]),
    "rt_hip_qweight_upload": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, c_void_pp]),
    "rt_hip_qweight_wrap_dev": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, c_void_pp]),
    "rt_hip_qweight_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_dequant": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "rt_hip_dequant_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "rt_hip_qgemv": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]),
    "rt_hip_qgemv_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]),
    "rt_hip_qgemv_grouped_dev": (C.c_int, [C.c_void_p, C.c_int, c_void_pp, c_void_pp, c_void_pp]),
    "rt_hip_qgemv_shared_x_dev": (C.c_int, [C.c_void_p, C.c_int, c_void_pp, C.c_void_p, c_void_pp, C.c_int]),
    "rt_hip_xq_bytes": (C.c_size_t, [C.c_size_t]),
    "rt_hip_quantize_act_dev": (C.c_int, [C.c_void_p, C.c_int, c_void_pp, C.POINTER(C.c_size_t), c_void_pp]),
    "rt_hip_qgemv_xq_grouped_dev": (C.c_int, [C.c_void_p, C.c_int, c_void_pp, c_void_pp, c_void_pp]),
    "rt_hip_qgemv_describe": (C.c_int, [C.c_void_p, C.c_int, c_void_pp, C.c_int, C.c_char_p, C.c_size_t]),
    "rt_hip_qgemm": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rt_hip_qgemm_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rt_hip_rmsnorm_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_float]),
    "rt_hip_swiglu_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rt_hip_rope_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float]),
    "rt_hip_kv_append_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]),
    "rt_hip_attn_decode_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "rt_hip_attn_causal_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "rt_hip_add_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rt_hip_argmax_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rt_hip_llama_create": (C.c_int, [C.c_void_p, C.POINTER(LlamaConfig), c_void_pp]),
    "rt_hip_llama_destroy": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_llama_upload_tensor": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t]),
    "rt_hip_llama_reset": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_llama_set_mode": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "rt_hip_llama_step": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, c_int_p]),
    "rt_hip_llama_prefill": (C.c_int, [C.c_void_p, C.c_void_p, c_int_p, C.c_int, C.c_int]),
    "rt_hip_llama_logits": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "rt_hip_llama_decode": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, c_int_p, c_int_p]),
    "rt_hip_llama_batch_create": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, c_void_pp]),
    "rt_hip_llama_batch_destroy": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rt_hip_llama_batch_reset": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "rt_hip_llama_batch_step": (C.c_int, [C.c_void_p, C.c_void_p, c_int_p, c_int_p, c_int_p]),
    "rt_hip_llama_batch_prefill": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, c_int_p, C.c_int, C.c_int]),
    "rt_hip_llama_batch_logits": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "rt_synth_blocks": (C.c_int, [C.c_int, C.c_uint64, C.c_uint64, C.c_size_t, C.c_float, C.c_float, C.c_void_p]),
    "rt_synth_normal_f32": (C.c_int, [C.c_uint64, C.c_uint64, C.c_size_t, C.c_float, C.c_float, C.c_void_p]),
    "rt_synth_tokens": (C.c_int, [C.c_uint64, C.c_uint64, C.c_size_t, C.c_int, C.c_void_p]),
}

_lib = None


def load() -> C.CDLL:
    """Load the native library; there is no fallback when it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            "%s is missing: build it with `python -m rustorch_amd.build` (hipcc, gfx950). "
            "rustorch_amd has no CPU fallback." % LIB_PATH)
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, ctx=None) -> None:
    """Raise the exception class that matches a non-zero status."""
    if rc == 0:
        return
    msg = load().rt_hip_last_error(ctx)
    text = msg.decode("utf-8", "replace") if msg else "status %d" % rc
    raise errors.BY_CODE.get(rc, errors.RusTorchHipError)(text)
