"""The reference's operator interface for the quantized path, from Python: the
names and meanings of backend.Backend, Kernel, View and Batch
(backend/backend.go:131-180, view.go:23-165, batch.go:22-52) over the library's
mi355x_backend_* entry points. Tests written against this read like the
reference's kernel tests (backend/internal/kerneltest)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from . import capi

MAX_RANK, MAX_INPUTS = 8, 4
OP_CAST, OP_GATHER, OP_QMATMUL, OP_ATTENTION = 1, 2, 3, 4


class _CView(C.Structure):
    _fields_ = [("rank", C.c_int32), ("shape", C.c_int64 * MAX_RANK), ("strides", C.c_int64 * MAX_RANK), ("offset", C.c_int64)]


class _CKernel(C.Structure):
    _fields_ = [("op", C.c_int32), ("dtype", C.c_int32), ("rank", C.c_int32), ("shape", C.c_int64 * MAX_RANK), ("n_in", C.c_int32),
                ("in_", _CView * MAX_INPUTS), ("axis", C.c_int32), ("scale", C.c_double), ("causal", C.c_int32), ("causal_offset", C.c_int64)]


@dataclass
class View:
    """How a kernel reads a buffer: shape, strides and offset in elements."""
    shape: list
    strides: list
    offset: int = 0

    @staticmethod
    def contiguous(shape) -> "View":
        strides, s = [0] * len(shape), 1
        for i in range(len(shape) - 1, -1, -1):
            strides[i] = s
            s *= shape[i]
        return View(list(shape), strides, 0)

    def size(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def is_contiguous(self) -> bool:
        want = 1
        for i in range(len(self.shape) - 1, -1, -1):
            if self.shape[i] == 1:
                continue
            if self.shape[i] == 0:
                return True
            if self.strides[i] != want:
                return False
            want *= self.shape[i]
        return True

    def permute(self, perm) -> "View":
        return View([self.shape[p] for p in perm], [self.strides[p] for p in perm], self.offset)

    def expand(self, shape) -> "View":
        strides = [0 if self.shape[i] == 1 and shape[i] != 1 else self.strides[i] for i in range(len(shape))]
        return View(list(shape), strides, self.offset)

    def shrink(self, ranges) -> "View":
        out = View([hi - lo for lo, hi in ranges], list(self.strides), self.offset)
        for i, (lo, hi) in enumerate(ranges):
            if hi - lo > 0:
                out.offset += lo * self.strides[i]
        return out

    def indices(self) -> np.ndarray:
        """The element index of every position, shaped like the view (for oracles)."""
        idx = np.full(self.shape, self.offset, np.int64)
        for d, (n, s) in enumerate(zip(self.shape, self.strides)):
            shp = [1] * len(self.shape)
            shp[d] = n
            idx = idx + (np.arange(n, dtype=np.int64) * s).reshape(shp)
        return idx


@dataclass
class Kernel:
    op: int
    dtype: int
    shape: list
    ins: list  # of View
    axis: int = 0
    scale: float = 0.0
    causal: bool = False
    causal_offset: int = 0

    def _c(self) -> _CKernel:
        k = _CKernel()
        k.op, k.dtype, k.rank, k.n_in = self.op, self.dtype, len(self.shape), len(self.ins)
        for i, d in enumerate(self.shape):
            k.shape[i] = d
        for j, v in enumerate(self.ins):
            k.in_[j].rank, k.in_[j].offset = len(v.shape), v.offset
            for i, (d, s) in enumerate(zip(v.shape, v.strides)):
                k.in_[j].shape[i], k.in_[j].strides[i] = d, s
        k.axis, k.scale, k.causal, k.causal_offset = self.axis, self.scale, int(self.causal), self.causal_offset
        return k


class BackendError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"{message} (0x{code:x})")
        self.code = code


@dataclass
class Buffer:
    handle: int
    dtype: int
    len: int
    nbytes: int


class Batch:
    def __init__(self, backend: "Backend", kernels, outs, ins):
        self.backend = backend
        n = len(kernels)
        ck = (_CKernel * n)(*[k._c() for k in kernels])
        lists = []

        def ptrs(bufs):
            arr = (C.c_void_p * max(len(bufs), 1))(*[b.handle for b in bufs])
            lists.append(arr)
            return C.cast(arr, C.POINTER(C.c_void_p))

        co = (C.POINTER(C.c_void_p) * n)(*[ptrs(o) for o in outs])
        ci = (C.POINTER(C.c_void_p) * n)(*[ptrs(i) for i in ins])
        no = (C.c_int * n)(*[len(o) for o in outs])
        ni = (C.c_int * n)(*[len(i) for i in ins])
        h = C.c_void_p()
        backend._check(backend.lib.mi355x_batch_new(ck, n, co, no, ci, ni, C.byref(h)))
        self.handle = h

    def close(self):
        if self.handle:
            self.backend.lib.mi355x_batch_free(self.handle)
            self.handle = None


class Backend:
    """backend.Backend and backend.Batcher."""

    def __init__(self, device: int = 0):
        self.lib = capi.load()
        h = C.c_void_p()
        self._check(self.lib.mi355x_backend_open(device, C.byref(h)))
        self._h = h

    def _check(self, code: int):
        if code:
            buf = C.create_string_buffer(1024)
            self.lib.mi355x_backend_last_error(buf, 1024)
            raise BackendError(code, buf.value.decode(errors="replace"))

    def name(self) -> str:
        return "mi355x"

    def close(self):
        if self._h:
            self.lib.mi355x_backend_close(self._h)
            self._h = None

    def alloc(self, dtype: int, n: int) -> Buffer:
        h = C.c_void_p()
        self._check(self.lib.mi355x_backend_alloc(self._h, dtype, n, C.byref(h)))
        bs, bb = self.lib.mi355x_block_size(dtype), self.lib.mi355x_block_bytes(dtype)
        return Buffer(h.value, dtype, n, n // bs * bb)

    def free(self, b: Buffer):
        self.lib.mi355x_backend_free(self._h, b.handle)

    def upload(self, dst: Buffer, src):
        raw = np.ascontiguousarray(src).view(np.uint8).reshape(-1)
        self._check(self.lib.mi355x_backend_upload(self._h, dst.handle, raw.ctypes.data, raw.size))

    def download(self, src: Buffer, nbytes: int | None = None) -> np.ndarray:
        out = np.empty(src.nbytes if nbytes is None else nbytes, np.uint8)
        self._check(self.lib.mi355x_backend_download(self._h, out.ctypes.data, out.size, src.handle))
        return out

    def run(self, k: Kernel, outs, ins):
        ck = k._c()
        o = (C.c_void_p * max(len(outs), 1))(*[b.handle for b in outs])
        i = (C.c_void_p * max(len(ins), 1))(*[b.handle for b in ins])
        self._check(self.lib.mi355x_backend_run(self._h, C.byref(ck), o, len(outs), i, len(ins)))

    def run_batch(self, b: Batch):
        self._check(self.lib.mi355x_backend_run_batch(self._h, b.handle))

    def sync(self):
        self._check(self.lib.mi355x_backend_sync(self._h))

    def graph_replays(self) -> int:
        return self.lib.mi355x_backend_graph_replays(self._h)
