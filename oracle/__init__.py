"""ctypes binding of the CPU oracle (oracle/mimir_oracle.c).

TEST INFRASTRUCTURE: only tests, the smoke check and the benchmark's
cpu_baseline leg import this package, and only as the checker. Nothing under
mimir_amd/ may import it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "build", "libmimir_oracle.so")

# dtype codes, shared with include/mimir_mi355x.h
F32, I32, BF16, F16, Q8_0, Q4_K, Q6_K, Q4_0 = 1, 2, 3, 4, 5, 6, 7, 8
QUANT = (Q8_0, Q4_K, Q6_K, Q4_0)
NAMES = {F32: "f32", I32: "i32", BF16: "bf16", F16: "f16", Q8_0: "q8_0", Q4_K: "q4_K", Q6_K: "q6_K", Q4_0: "q4_0"}
ROPE_NONE, ROPE_LINEAR, ROPE_LLAMA3 = 0, 1, 2


def build(force: bool = False) -> str:
    """Compiles the oracle with the committed Makefile; returns the library path."""
    src = os.path.join(_HERE, "mimir_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        path = os.environ.get("MIMIR_ORACLE_LIB")  # another build of the same source, e.g. `make -C oracle asan`
        if not path:
            if not os.path.exists(_LIB_PATH):
                build()
            path = _LIB_PATH
        _lib = C.CDLL(path)
        _declare(_lib)
    return _lib


def _declare(l):
    i64, f32p, u8p, u16p, vp = C.c_int64, C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_uint16), C.c_void_p
    l.mo_bf16_to_f32.restype = C.c_float; l.mo_bf16_to_f32.argtypes = [C.c_uint16]
    l.mo_f16_to_f32.restype = C.c_float; l.mo_f16_to_f32.argtypes = [C.c_uint16]
    l.mo_f32_to_bf16.restype = C.c_uint16; l.mo_f32_to_bf16.argtypes = [C.c_float]
    l.mo_f32_to_f16.restype = C.c_uint16; l.mo_f32_to_f16.argtypes = [C.c_float]
    for n in ("mo_f16_to_f32_n", "mo_bf16_to_f32_n"):
        getattr(l, n).restype = None; getattr(l, n).argtypes = [vp, vp, i64]
    for n in ("mo_f32_to_f16_n", "mo_f32_to_bf16_n"):
        getattr(l, n).restype = None; getattr(l, n).argtypes = [vp, vp, i64]
    l.mo_block_size.restype = C.c_int; l.mo_block_size.argtypes = [C.c_int]
    l.mo_block_bytes.restype = C.c_int; l.mo_block_bytes.argtypes = [C.c_int]
    l.mo_dequantize.restype = None; l.mo_dequantize.argtypes = [C.c_int, vp, i64, vp]
    l.mo_dequant_at.restype = C.c_float; l.mo_dequant_at.argtypes = [C.c_int, vp, i64]
    l.mo_dequantize_to.restype = None; l.mo_dequantize_to.argtypes = [C.c_int, vp, i64, vp, C.c_int]
    l.mo_gather_rows.restype = C.c_int; l.mo_gather_rows.argtypes = [C.c_int, vp, i64, i64, vp, i64, vp]
    l.mo_quantize_row.restype = None; l.mo_quantize_row.argtypes = [vp, vp, i64, C.c_int, C.c_int]
    for n in ("mo_qdot_q8_0", "mo_qdot_q4k", "mo_qdot_q6k", "mo_qdot_q8_0_simd"):
        getattr(l, n).restype = C.c_float; getattr(l, n).argtypes = [i64, vp, vp]
    l.mo_has_simd.restype = C.c_int
    l.mo_dot.restype = C.c_float; l.mo_dot.argtypes = [vp, vp, i64]
    l.mo_sgemv.restype = None; l.mo_sgemv.argtypes = [vp, vp, vp, i64, i64, i64, C.c_int]
    l.mo_qmatmul.restype = C.c_int; l.mo_qmatmul.argtypes = [C.c_int, vp, vp, vp, i64, i64, i64, i64, C.c_int, C.c_int]
    l.mo_q4_0_matmul_f32.restype = C.c_int; l.mo_q4_0_matmul_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, C.c_int]
    l.mo_q4_0_matmul_bf16.restype = C.c_int; l.mo_q4_0_matmul_bf16.argtypes = [vp, vp, vp, i64, i64, i64, C.c_int]
    l.mo_rmsnorm.restype = None; l.mo_rmsnorm.argtypes = [vp, vp, vp, i64, i64, C.c_double]
    l.mo_rope_angles.restype = None
    l.mo_rope_angles.argtypes = [C.c_int, C.c_double, C.c_int, vp, vp, i64, i64, vp, vp]
    l.mo_rope_apply.restype = None
    l.mo_rope_apply.argtypes = [vp, vp, i64, i64, C.c_int, C.c_int, C.c_int, vp, vp]
    l.mo_attention.restype = None
    l.mo_attention.argtypes = [vp, vp, vp, C.c_int, vp, vp] + [i64] * 13 + [C.c_double, C.c_int, i64, vp, i64, i64]
    l.mo_silu_mul.restype = None; l.mo_silu_mul.argtypes = [vp, vp, vp, i64]
    l.mo_argmax.restype = C.c_int32; l.mo_argmax.argtypes = [vp, i64]
    l.mo_stream_sum.restype = C.c_double; l.mo_stream_sum.argtypes = [vp, i64, C.c_int]
    l.mo_num_threads.restype = C.c_int
    del f32p, u8p, u16p


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ---- numpy-level helpers -------------------------------------------------

def block_size(dt: int) -> int:
    return lib().mo_block_size(dt)


def block_bytes(dt: int) -> int:
    return lib().mo_block_bytes(dt)


def f16_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16); out = np.empty(h.shape, np.float32)
    lib().mo_f16_to_f32_n(_p(h), _p(out), h.size); return out


def f32_to_f16(f) -> np.ndarray:
    f = _c(f, np.float32); out = np.empty(f.shape, np.uint16)
    lib().mo_f32_to_f16_n(_p(f), _p(out), f.size); return out


def bf16_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16); out = np.empty(h.shape, np.float32)
    lib().mo_bf16_to_f32_n(_p(h), _p(out), h.size); return out


def f32_to_bf16(f) -> np.ndarray:
    f = _c(f, np.float32); out = np.empty(f.shape, np.uint16)
    lib().mo_f32_to_bf16_n(_p(f), _p(out), f.size); return out


def dequantize(dt: int, data, out_dt: int = F32) -> np.ndarray:
    """All elements of the blocks in data (uint8), flat."""
    data = _c(data, np.uint8).reshape(-1)
    bb, bs = block_bytes(dt), block_size(dt)
    assert data.size % bb == 0
    nb = data.size // bb
    out = np.empty(nb * bs, np.float32 if out_dt == F32 else np.uint16)
    lib().mo_dequantize_to(dt, _p(data), nb, _p(out), out_dt)
    return out


def dequant_at(dt: int, data, i: int) -> float:
    data = _c(data, np.uint8).reshape(-1)
    return lib().mo_dequant_at(dt, _p(data), i)


def gather_rows(dt: int, table, rows: int, k: int, idx) -> np.ndarray:
    table = _c(table, np.uint8).reshape(-1); idx = _c(idx, np.int32).reshape(-1)
    out = np.empty((idx.size, k), np.float32)
    if lib().mo_gather_rows(dt, _p(table), rows, k, _p(idx), idx.size, _p(out)) != 0:
        raise IndexError("index out of range")
    return out


def quantize_row(x, bs: int, sums: bool) -> np.ndarray:
    x = _c(x, np.float32).reshape(-1)
    stride = 4 + bs + (32 if sums else 0)
    out = np.zeros(x.size // bs * stride, np.uint8)
    lib().mo_quantize_row(_p(out), _p(x), x.size, bs, int(sums))
    return out


def qdot(dt: int, w, xq, simd: bool = False) -> float:
    w = _c(w, np.uint8).reshape(-1); xq = _c(xq, np.uint8).reshape(-1)
    nb = w.size // block_bytes(dt)
    fn = {Q8_0: lib().mo_qdot_q8_0_simd if simd else lib().mo_qdot_q8_0, Q4_K: lib().mo_qdot_q4k, Q6_K: lib().mo_qdot_q6k}[dt]
    return fn(nb, _p(w), _p(xq))


def dot(a, b) -> float:
    a = _c(a, np.float32).reshape(-1); b = _c(b, np.float32).reshape(-1)
    return lib().mo_dot(_p(a), _p(b), a.size)


def sgemv(w, x, threads: int = 0) -> np.ndarray:
    """x [m, k] . w[n, k]^T in float32 with the portable dot's order."""
    w = _c(w, np.float32); x = _c(x, np.float32)
    n, k = w.shape; x2 = x.reshape(-1, k)
    out = np.empty((x2.shape[0], n), np.float32)
    lib().mo_sgemv(_p(w), _p(x2), _p(out), x2.shape[0], n, k, threads)
    return out.reshape(x.shape[:-1] + (n,))


def qmatmul(dt: int, w, x, n: int, k: int, simd: bool = False, threads: int = 0) -> np.ndarray:
    """x [..., k] by the transpose of quantized w [n, k], as the reference CPU
    computes it: int8 activations for Q8_0/Q4_K/Q6_K, the float32 product of
    the dequantized weights for Q4_0."""
    w = _c(w, np.uint8).reshape(-1); x = _c(x, np.float32)
    assert w.size == n * k // block_size(dt) * block_bytes(dt), (w.size, n, k)
    x2 = x.reshape(-1, k)
    out = np.empty((x2.shape[0], n), np.float32)
    if dt == Q4_0:
        rc = lib().mo_q4_0_matmul_f32(_p(w), _p(x2), _p(out), x2.shape[0], n, k, k, threads)
    else:
        rc = lib().mo_qmatmul(dt, _p(w), _p(x2), _p(out), x2.shape[0], n, k, k, int(simd), threads)
    if rc != 0:
        raise ValueError(f"oracle qmatmul failed: {rc}")
    return out.reshape(x.shape[:-1] + (n,))


def q4_0_matmul_bf16(w, x_bf16, n: int, k: int, threads: int = 0) -> np.ndarray:
    w = _c(w, np.uint8).reshape(-1); x = _c(x_bf16, np.uint16).reshape(-1, k)
    out = np.empty((x.shape[0], n), np.uint16)
    rc = lib().mo_q4_0_matmul_bf16(_p(w), _p(x), _p(out), x.shape[0], n, k, threads)
    if rc != 0:
        raise ValueError(f"oracle q4_0 bf16 matmul failed: {rc}")
    return out


def rmsnorm(x, w, eps: float) -> np.ndarray:
    x = _c(x, np.float32); d = x.shape[-1]
    out = np.empty_like(x)
    wp = _p(_c(w, np.float32)) if w is not None else None
    lib().mo_rmsnorm(_p(x), wp, _p(out), x.size // d, d, eps)
    return out


def rope_angles(dim: int, base: float, offset: int, n: int, scaling: int = ROPE_NONE, params=(), freq_factors=None):
    cos = np.empty((n, dim // 2), np.float32); sin = np.empty((n, dim // 2), np.float32)
    p = (C.c_double * 4)(*(list(params) + [0.0] * (4 - len(params))))
    ff = _c(freq_factors, np.float32) if freq_factors is not None else None
    lib().mo_rope_angles(dim, base, scaling, C.cast(p, C.c_void_p), _p(ff) if ff is not None else None, offset, n, _p(cos), _p(sin))
    return cos, sin


def rope_apply(x, cos, sin, dim: int, interleaved: bool) -> np.ndarray:
    """x [..., S, head_dim]; cos/sin [S, dim/2]."""
    x = _c(x, np.float32); s, hd = x.shape[-2], x.shape[-1]
    out = np.empty_like(x)
    cos = _c(cos, np.float32); sin = _c(sin, np.float32)
    lib().mo_rope_apply(_p(x), _p(out), x.size // (s * hd), s, hd, dim, int(interleaved), _p(cos), _p(sin))
    return out


def attention(q, k, v, scale: float, causal: bool = False, causal_offset: int = 0, mask=None, kv_dt: int = F32,
              k_len: int | None = None):
    """q [B,H,Q,D]; k [B,HK,Kcap,D]; v [B,HK,Kcap,DV] (float32, or uint16 bits
    when kv_dt is F16). Attends to the first k_len positions (default all).
    Returns (out [B,H,Q,DV], lse [B,H,Q])."""
    q = _c(q, np.float32)
    kd = np.float32 if kv_dt == F32 else np.uint16
    k = _c(k, kd); v = _c(v, kd)
    B, H, Q, D = q.shape
    _, HK, cap, _ = k.shape
    DV = v.shape[-1]
    K = cap if k_len is None else k_len
    out = np.empty((B, H, Q, DV), np.float32); lse = np.empty((B, H, Q), np.float32)
    mb = mh = 0; mp = None
    if mask is not None:
        mask = _c(mask, np.float32)
        assert mask.shape[-2:] == (Q, K), mask.shape
        m4 = mask.reshape((1,) * (4 - mask.ndim) + mask.shape)
        mh = Q * K if m4.shape[1] != 1 else 0
        mb = (m4.shape[1] * Q * K) if m4.shape[0] != 1 else 0
        mp = _p(mask)
    lib().mo_attention(_p(q), _p(k), _p(v), kv_dt, _p(out), _p(lse), B, H, HK, Q, K, D, DV,
                       HK * cap * D, cap * D, D, HK * cap * DV, cap * DV, DV,
                       scale, int(causal), causal_offset, mp, mb, mh)
    return out, lse


def silu_mul(g, u) -> np.ndarray:
    g = _c(g, np.float32); u = _c(u, np.float32); out = np.empty_like(g)
    lib().mo_silu_mul(_p(g), _p(u), _p(out), g.size); return out


def argmax(logits) -> int:
    l = _c(logits, np.float32).reshape(-1)
    return int(lib().mo_argmax(_p(l), l.size))
