"""The Q4_0 product of two to fifteen rows of x (the decoding step of a batch of sequences), which
reads W once for eight rows on the int8 matrix cores, against the oracle's float32 product with the
dequantized weights (io/mim/dtype.go:118-123, backend/cpu/gemv.go:73-104; bound 1e-3) and against
the one-row kernel, whose integers it shares."""
import numpy as np
import pytest
import torch

import oracle as O
from mimir_amd import capi
from tests import gpu
from tests.helpers import bench_blocks, random_blocks

pytestmark = pytest.mark.gpu


def per_row(l, raw_ptr, x, n, k):
    """The same rows one at a time through the one-row kernel."""
    capi.check(l.mi355x_tune(b"q4_0.rows_path", 1))
    try:
        return gpu.qgemv(O.Q4_0, raw_ptr, x, n, k)
    finally:
        capi.check(l.mi355x_tune(b"q4_0.rows_path", 0))


@pytest.mark.parametrize("m,n,k", [(2, 32, 64), (8, 40, 128), (5, 203, 4096 + 64), (8, 515, 4096), (3, 70, 14336), (9, 64, 512),
                                   (15, 33, 1024), (8, 1, 64), (29, 100, 512), (40, 64, 4096 + 64)])
def test_rows_kernel_matches_oracle_and_one_row_kernel(m, n, k):
    rng = np.random.default_rng(m * 1000 + n + k)
    raw = random_blocks(rng, O.Q4_0, n * k)  # scales of either sign, zero and subnormal
    x = (rng.normal(size=(m, k)) * np.exp(rng.normal(size=(m, 1)) * 3)).astype(np.float32)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    gpu.say(f"q4_0 rows kernel M={m} N={n} K={k}")
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    w = O.dequantize(O.Q4_0, raw).reshape(n, k).astype(np.float64)
    mag = np.abs(x.astype(np.float64)) @ np.abs(w).T  # what the rounding errors scale with
    assert np.all(np.abs(got - want) <= 2e-6 * mag + 1e-30)
    if m >= 16:  # the cost model may prefer the tiled kernel at this size: ask for the rows kernel
        capi.check(gpu.lib().mi355x_tune(b"q4_0.rows_max", 1000))
        try:
            got2 = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
        finally:
            capi.check(gpu.lib().mi355x_tune(b"q4_0.rows_max", 0))
        assert np.all(np.abs(got2 - want) <= 2e-6 * mag + 1e-30)
    one = per_row(gpu.lib(), ptr, gpu.dev(x), n, k)
    assert np.all(np.abs(got - one) <= 1e-6 * mag + 1e-30)  # the same integers, another order of float32 additions


def test_rows_kernel_at_the_model_shapes():
    """Bench-generated weights at the 8B shapes, eight rows: within the path's 1e-3 of the oracle."""
    rng = np.random.default_rng(3)
    for n, k in ((1024, 4096), (4096, 14336)):
        raw = bench_blocks(rng, O.Q4_0, n * k)
        x = rng.normal(size=(8, k)).astype(np.float32)
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        gpu.say(f"q4_0 rows kernel 8 x {n}x{k}")
        got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
        want = O.qmatmul(O.Q4_0, raw, x, n, k)
        assert np.all(np.abs(got - want) <= 1e-3 * np.maximum(1.0, np.abs(want)))
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-5


def test_rows_kernel_special_values_and_strided_rows():
    """Zero, tiny, huge and subnormal blocks of x; an infinity or a NaN makes its row NaN and leaves
    the other rows alone; rows of x further apart than K."""
    rng = np.random.default_rng(11)
    n, k, m = 40, 512, 4
    raw = bench_blocks(rng, O.Q4_0, n * k)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[0, 0:32] = 0
    x[1, 32:64] *= 1e-36
    x[2, 64:96] *= 1e30
    x[3, 96:128] = np.float32(1e-42)
    gpu.say("q4_0 rows kernel special values")
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want).max(axis=1, keepdims=True))
    x[1, 200] = np.inf
    x[2, 300] = np.nan
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all()
    assert np.all(np.abs(got[[0, 3]] - want[[0, 3]]) <= 1e-5 * np.abs(want).max())
    wide = torch.zeros((m, k + 8), device="cuda:0")
    xs = rng.normal(size=(m, k)).astype(np.float32)
    wide[:, :k] = gpu.dev(xs)
    gpu.say("q4_0 rows kernel strided rows")
    got = gpu.qgemv(O.Q4_0, ptr, wide[:, :k], n, k)
    want = O.qmatmul(O.Q4_0, raw, xs, n, k)
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want).max())
