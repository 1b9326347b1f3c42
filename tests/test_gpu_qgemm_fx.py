"""The Q4_0 product of many rows of float32 x on the int8 matrix cores (mi355x_qgemv from enough rows on),
against the oracle's float32 product with dequantized weights (io/mim/dtype.go:118-123,
backend/cpu/gemv.go:73-104; bound asked for: 1e-3 relative) and against the row kernels, whose
fixed-point arithmetic it shares: same integers and scales per block of x, another order of the float32
additions. Bounds go with sum |x||w| because random scales span binary16's range."""
import numpy as np
import pytest
import torch

import oracle as O
from mimir_amd import capi
from tests import gpu
from tests.helpers import bench_blocks, random_blocks

pytestmark = pytest.mark.gpu


def both(raw, x, n, k):
    """(matrix cores, row kernels) for the same product."""
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    out = []
    try:
        for rows in (1, 1 << 30):  # a threshold of 1 row, or none
            capi.check(l.mi355x_tune(b"q4_0.fx_rows", rows))
            out.append(gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k))
    finally:
        capi.check(l.mi355x_tune(b"q4_0.fx_rows", 0))
    return out


def magnitude(raw, x, n, k):
    with np.errstate(invalid="ignore"):  # rows with NaN or infinities have no bound (and are compared as NaN)
        return np.abs(x).astype(np.float64) @ np.abs(O.dequantize(O.Q4_0, raw).reshape(n, k)).astype(np.float64).T


@pytest.mark.parametrize("m,n,k", [(1, 5, 128), (32, 64, 128), (40, 100, 256), (33, 65, 384), (130, 70, 1280), (129, 200, 4096 + 128),
                                   (512, 300, 4096)])
def test_matches_the_oracle_and_the_row_kernels(m, n, k):
    rng = np.random.default_rng(m + n + k)
    raw = random_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[m // 2, :32] = 0  # a block of zeros: scale 0
    gpu.say(f"q4_0 fx gemm M={m} N={n} K={k}")
    got, rows = both(raw, x, n, k)
    mag = magnitude(raw, x, n, k)
    assert np.all(np.abs(got - O.qmatmul(O.Q4_0, raw, x, n, k)) <= 2e-6 * mag + 1e-30)
    assert np.all(np.abs(got - rows) <= 1e-6 * mag + 1e-30)


def test_blocks_of_x_at_the_ends_of_the_fixed_point_range():
    """Every element of a block at the block's largest magnitude, every nibble 0 or 15: the largest integer
    sums a block can reach (32 * 8 * 7829367, just below 2^31), with and without cancellation."""
    m, n, k = 32, 64, 256
    raw = np.zeros((n * k // 32, 18), np.uint8)
    raw[:, :2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    raw[0::2, 2:] = 0x00  # n = 0: -8
    raw[1::2, 2:] = 0xFF  # n = 15: +7
    raw = raw.reshape(-1)
    x = np.full((m, k), 3.25, np.float32)
    x[1::2] *= -1
    x[:, 1::2] *= np.where(np.arange(m)[:, None] % 3 == 0, -1.0, 1.0).astype(np.float32)
    gpu.say("q4_0 fx gemm extremes")
    got, rows = both(raw, x, n, k)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    assert np.all(np.abs(got - want) <= 2e-6 * magnitude(raw, x, n, k))
    assert np.all(np.abs(got - rows) <= 1e-6 * magnitude(raw, x, n, k))


def test_rows_with_nan_and_inf():
    m, n, k = 40, 70, 512
    rng = np.random.default_rng(4)
    raw = random_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[3, 300] = np.nan
    x[9, 10] = np.inf
    gpu.say("q4_0 fx gemm nan")
    got, rows = both(raw, x, n, k)
    assert np.isnan(got[3]).all() and np.isnan(got[9]).all() and np.array_equal(np.isnan(got), np.isnan(rows))
    ok = ~np.isnan(got)
    assert np.all(np.abs(got - rows)[ok] <= 1e-6 * magnitude(raw, x, n, k)[ok] + 1e-30)


def test_prompt_shapes_pick_the_matrix_cores_by_themselves():
    """512 rows of x by 4096 x 4096 weights: the library's own choice, within 1e-4 of max(1, |want|)."""
    m, n, k = 512, 4096, 4096
    rng = np.random.default_rng(2)
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    gpu.say("q4_0 fx gemm 512 x 4096 x 4096")
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    lo, hi = 1000, 1256
    want = O.qmatmul(O.Q4_0, raw.reshape(n, -1)[lo:hi].reshape(-1), x, hi - lo, k)
    assert np.all(np.abs(got[:, lo:hi] - want) <= 1e-4 * np.maximum(1, np.abs(want)))
