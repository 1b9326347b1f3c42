"""ctypes binding of libmimir_mi355x.so, the C ABI of include/mimir_mi355x.h.

This is the same binding a Go host makes with purego (Dlopen + RegisterFunc):
symbols are looked up by name and called with plain pointers and integers.
The library is built ahead of time by mimir_amd.build; loading fails loudly
when it is missing, and there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libmimir_mi355x.so")

OK = 0
ERR_OUT_OF_MEMORY, ERR_SHAPE, ERR_DTYPE, ERR_INDEX, ERR_INTERNAL = 2, 0x1001, 0x1002, 0x1003, 0x1005
F32, I32, BF16, F16, Q8_0, Q4_K, Q6_K, Q4_0 = 1, 2, 3, 4, 5, 6, 7, 8

_vp, _i64, _int, _sz = C.c_void_p, C.c_int64, C.c_int, C.c_size_t

# name -> (restype, argtypes): every symbol include/mimir_mi355x.h declares.
SYMBOLS = {
    "mi355x_init": (C.c_uint32, [_int]),
    "mi355x_last_error": (_sz, [C.c_char_p, _sz]),
    "mi355x_block_size": (_int, [_int]),
    "mi355x_block_bytes": (_int, [_int]),
    "mi355x_bytes": (_i64, [_int, _i64]),
    "mi355x_alloc": (C.c_uint32, [C.POINTER(_vp), _sz]),
    "mi355x_free": (C.c_uint32, [_vp]),
    "mi355x_upload": (C.c_uint32, [_vp, _vp, _sz, _vp]),
    "mi355x_download": (C.c_uint32, [_vp, _vp, _sz, _vp]),
    "mi355x_sync": (C.c_uint32, [_vp]),
    "mi355x_qgemv": (C.c_uint32, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "mi355x_qgemv_noalloc": (C.c_uint32, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "mi355x_act_bytes": (_sz, [_int, _i64]),
    "mi355x_convert_act": (C.c_uint32, [_int, _vp, _i64, _i64, _i64, _vp, _vp]),
    "mi355x_qgemv_act": (C.c_uint32, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_qgemv_act_add": (C.c_uint32, [_int, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_qgemv_act_multi": (C.c_uint32, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _vp]),
    "mi355x_qgemv_act_swiglu": (C.c_uint32, [_int, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_dequant": (C.c_uint32, [_int, _vp, _i64, _i64, _vp, _int, _vp]),
    "mi355x_gather_rows": (C.c_uint32, [_int, _vp, _i64, _i64, _vp, _i64, _vp, _vp]),
    "mi355x_rmsnorm": (C.c_uint32, [_vp, _vp, _vp, _i64, _i64, C.c_double, _vp]),
    "mi355x_rope": (C.c_uint32, [_vp, _vp, _i64, _i64, _int, _int, _int, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _vp]),
    "mi355x_kv_write": (C.c_uint32, [_vp, _vp, _int, _i64, _int, _i64, _int, _i64, _i64, _i64, _i64, _i64, _vp]),
    "mi355x_attention": (C.c_uint32, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _i64, _i64, _int, _int,
                                      C.c_double, _int, _i64, _vp]),
    "mi355x_swiglu": (C.c_uint32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_add": (C.c_uint32, [_vp, _vp, _vp, _i64, _vp]),
    "mi355x_argmax": (C.c_uint32, [_vp, _i64, _i64, _vp, _vp]),
    "mi355x_llama_create": (C.c_uint32, [_vp, C.POINTER(_vp)]),
    "mi355x_llama_destroy": (C.c_uint32, [_vp]),
    "mi355x_llama_set_tensor": (C.c_uint32, [_vp, C.c_char_p, _int, _vp, _i64]),
    "mi355x_llama_set_rope_factors": (C.c_uint32, [_vp, _vp, C.c_int32]),
    "mi355x_llama_finalize": (C.c_uint32, [_vp, _i64]),
    "mi355x_llama_reset": (C.c_uint32, [_vp]),
    "mi355x_llama_set_cache": (C.c_uint32, [_vp, C.c_int32, _vp, _vp, _i64]),
    "mi355x_llama_cache_len": (_i64, [_vp]),
    "mi355x_llama_logits": (C.c_uint32, [_vp, _vp, _i64, _int, _vp]),
    "mi355x_llama_generate": (C.c_uint32, [_vp, _vp, _i64, _i64, _vp, _vp]),
    "mi355x_tune": (C.c_uint32, [C.c_char_p, _int]),
    "mi355x_backend_last_error": (_sz, [C.c_char_p, _sz]),
    "mi355x_backend_open": (C.c_uint32, [_int, _vp]),
    "mi355x_backend_close": (C.c_uint32, [_vp]),
    "mi355x_backend_alloc": (C.c_uint32, [_vp, _int, _i64, _vp]),
    "mi355x_backend_free": (C.c_uint32, [_vp, _vp]),
    "mi355x_backend_upload": (C.c_uint32, [_vp, _vp, _vp, _sz]),
    "mi355x_backend_download": (C.c_uint32, [_vp, _vp, _sz, _vp]),
    "mi355x_backend_sync": (C.c_uint32, [_vp]),
    "mi355x_backend_run": (C.c_uint32, [_vp, _vp, _vp, _int, _vp, _int]),
    "mi355x_batch_new": (C.c_uint32, [_vp, _int, _vp, _vp, _vp, _vp, _vp]),
    "mi355x_batch_free": (C.c_uint32, [_vp]),
    "mi355x_backend_run_batch": (C.c_uint32, [_vp, _vp]),
    "mi355x_backend_graph_replays": (_i64, [_vp]),
    "mi355x_qgemm_bf16": (C.c_uint32, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "mi355x_attention_d": (C.c_uint32, [_vp, _vp]),
    "mi355x_stream_release": (C.c_uint32, [_vp]),
    "mi355x_last_kernel": (C.c_uint32, [_vp, _sz]),
    "mi355x_timed_begin": (C.c_uint32, [_int]),
    "mi355x_timed_end": (C.c_uint32, [_vp, _vp]),
    "mi355x_gemv_stamps": (C.c_uint32, [_vp]),
    "mi355x_stream_read": (C.c_uint32, [_vp, _sz, _vp, _int, _int, _vp]),
}


class LlamaConfig(C.Structure):
    """mi355x_llama_config."""
    _fields_ = [(n, C.c_int32) for n in ("embed", "hidden", "layers", "heads", "kv_heads", "head_dim", "rope_dim", "vocab", "context",
                                          "interleaved", "cache_dtype", "batch")] + [(n, C.c_double) for n in ("rope_base", "rope_scale", "eps")]


class AttentionDesc(C.Structure):
    """mi355x_attention_desc."""
    _fields_ = [(n, C.c_void_p) for n in ("q", "k", "v", "mask", "out", "lse")] + \
               [("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3), ("out_strides", C.c_int64 * 3),
                ("mask_strides", C.c_int64 * 4)] + [(n, C.c_int64) for n in ("B", "Q", "K", "causal_offset")] + [("scale", C.c_double)] + \
               [(n, C.c_int32) for n in ("kv_dtype", "H", "HK", "D", "DV", "causal")]


class Mi355xError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"[{status:#x}] {message}")
        self.status = status


_lib = None


def load() -> C.CDLL:
    """Loads the library and declares every symbol; raises if it is not built."""
    global _lib
    if _lib is None:
        path = os.environ.get("MIMIR_MI355X_LIB") or LIB_PATH  # as the reference's loaders take a path from the environment
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is not built: run `python -m mimir_amd.build`")
        lib = C.CDLL(path)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is missing
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def last_error() -> str:
    buf = C.create_string_buffer(1024)
    load().mi355x_last_error(buf, 1024)
    return buf.value.decode(errors="replace")


def check(status: int) -> None:
    if status != OK:
        raise Mi355xError(status, last_error())
