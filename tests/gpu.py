"""Plumbing of the GPU tests: device memory and streams come from torch, and
every compute call goes through the C ABI with raw pointers."""
import ctypes as C
import sys

import numpy as np
import torch

from mimir_amd import capi

_ready = False


def lib():
    global _ready
    l = capi.load()
    if not _ready:
        capi.check(l.mi355x_init(0))
        _ready = True
    return l


def say(msg):
    """Names the case before the GPU step, flushed, so a fault can be placed."""
    print(f"[gpu] {msg}", flush=True)
    sys.stdout.flush()


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def dev_bytes_at(raw: np.ndarray, offset: int) -> tuple[torch.Tensor, int]:
    """raw bytes placed `offset` bytes into a fresh device buffer; returns the
    buffer (keep it alive) and the address of the first byte of raw."""
    buf = torch.empty(raw.size + offset + 64, dtype=torch.uint8, device="cuda:0")
    buf[offset:offset + raw.size] = torch.from_numpy(np.ascontiguousarray(raw)).to("cuda:0")
    return buf, buf.data_ptr() + offset


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def sync():
    capi.check(lib().mi355x_sync(stream()))


def qgemv(dt, w_ptr, x: torch.Tensor, n: int, k: int) -> np.ndarray:
    x2 = x.reshape(-1, k)
    m = x2.shape[0]
    y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(lib().mi355x_qgemv(dt, w_ptr, x2.data_ptr(), y.data_ptr(), m, n, k, x2.stride(0) if m > 1 else k, stream()))
    sync()
    return y.cpu().numpy().reshape(tuple(x.shape[:-1]) + (n,))


def dequant(dt, w_ptr, first: int, n: int, out_dt=capi.F32) -> np.ndarray:
    tdt = torch.float32 if out_dt == capi.F32 else torch.int16
    out = torch.zeros(n, dtype=tdt, device="cuda:0")
    capi.check(lib().mi355x_dequant(dt, w_ptr, first, n, out.data_ptr(), out_dt, stream()))
    sync()
    r = out.cpu().numpy()
    return r if out_dt == capi.F32 else r.view(np.uint16)


def convert_act(dt, x: torch.Tensor, k: int) -> np.ndarray:
    """The converted activations of the rows of x, as raw bytes [m, act_bytes]."""
    l = lib()
    x2 = x.reshape(-1, k)
    m = x2.shape[0]
    nbytes = l.mi355x_act_bytes(dt, k)
    assert nbytes > 0
    act = torch.zeros((m, nbytes), dtype=torch.uint8, device="cuda:0")
    capi.check(l.mi355x_convert_act(dt, x2.data_ptr(), m, k, x2.stride(0) if m > 1 else k, act.data_ptr(), stream()))
    sync()
    return act.cpu().numpy()


def qgemv_act(dt, w_ptr, x: torch.Tensor, n: int, k: int) -> np.ndarray:
    """The two-step product: convert once, multiply."""
    l = lib()
    x2 = x.reshape(-1, k)
    m = x2.shape[0]
    act = torch.zeros((m, l.mi355x_act_bytes(dt, k)), dtype=torch.uint8, device="cuda:0")
    y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(l.mi355x_convert_act(dt, x2.data_ptr(), m, k, x2.stride(0) if m > 1 else k, act.data_ptr(), stream()))
    capi.check(l.mi355x_qgemv_act(dt, w_ptr, act.data_ptr(), y.data_ptr(), m, n, k, stream()))
    sync()
    return y.cpu().numpy().reshape(tuple(x.shape[:-1]) + (n,))
