"""Pins the oracle's half conversions (backend/cpu/half.go:37-102) against
library routines: numpy.float16 over every binary16 pattern, numpy/torch
rounding on sampled float32 including ties, subnormals and NaN payloads."""
import numpy as np
import torch

import oracle as O


def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    got = O.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    # NaNs keep sign and payload, shifted into the float32 fraction.
    exp = ((bits[nan].astype(np.uint32) & 0x8000) << 16) | 0x7f800000 | ((bits[nan].astype(np.uint32) & 0x3ff) << 13)
    assert np.array_equal(got.view(np.uint32)[nan], exp)


def _samples():
    rng = np.random.default_rng(1)
    u = rng.integers(0, 2**32, 400000, dtype=np.uint64).astype(np.uint32)
    # every binary16 value, and the midpoints between neighbours (ties)
    h = np.arange(0x7c00, dtype=np.uint16)
    hv = h.view(np.float16).astype(np.float64)
    mids = ((hv[:-1] + hv[1:]) / 2).astype(np.float32)
    near = np.concatenate([mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    edge = np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0x7f800001, 0xffc12345, 0x477fe000, 0x477ff000,
                     0x33000000, 0x33000001, 0x32ffffff, 0x00000001, 0x807fffff], dtype=np.uint32)
    f = np.concatenate([u.view(np.float32), near, -near, hv.astype(np.float32), edge.view(np.float32)])
    return f


def test_f32_to_f16_matches_numpy():
    f = _samples()
    got = O.f32_to_f16(f)
    with np.errstate(over="ignore", invalid="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    # half.go:84-86: sign | 0x7e00 | payload top 9 bits
    b = f.view(np.uint32)[nan]
    exp = ((b >> 16) & 0x8000).astype(np.uint16) | 0x7e00 | ((b >> 13) & 0x1ff).astype(np.uint16)
    assert np.array_equal(got[nan], exp)


def test_f32_to_bf16_matches_torch():
    f = _samples()
    got = O.f32_to_bf16(f)
    nan = np.isnan(f)
    want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[~nan], want[~nan])
    b = f.view(np.uint32)[nan]
    assert np.array_equal(got[nan], ((b >> 16) | 0x40).astype(np.uint16))
    # widening is exact
    assert np.array_equal(O.bf16_to_f32(got[~nan]).view(np.uint32), got[~nan].astype(np.uint32) << 16)


def test_scalar_entry_points_agree_with_array_ones():
    l = O.lib()
    for bits in (0, 1, 0x3c00, 0x8001, 0x7bff, 0x7c00, 0xfc00, 0x0400, 0x03ff):
        assert l.mo_f16_to_f32(bits) == O.f16_to_f32(np.array([bits], np.uint16))[0]
    for v in (0.0, 1.0, -2.5, 65504.0, 65520.0, 1e-8, 6e-8, 3.0e-5):
        assert l.mo_f32_to_f16(v) == O.f32_to_f16(np.array([v], np.float32))[0]
        assert l.mo_f32_to_bf16(v) == O.f32_to_bf16(np.array([v], np.float32))[0]
