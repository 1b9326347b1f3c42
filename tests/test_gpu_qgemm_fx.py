"""The Q4_0 product of many rows of float32 x on the int8 matrix cores (mi355x_qgemv from enough rows on),
against the oracle's float32 product with dequantized weights (io/mim/dtype.go:118-123,
backend/cpu/gemv.go:73-104; bound asked for: 1e-3 relative) and against the row kernels, whose
fixed-point arithmetic it shares: same integers and scales per block of x, another order of the float32
additions. Bounds go with sum |x||w| because random scales span binary16's range."""
import ctypes

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


@pytest.mark.parametrize("m,kernel", [(512, "qgemm_q4_0_fx_kernel"), (2048, "qgemm_q4_0_fx16_kernel: 16 x 16 tiles of 128 x 256")])
def test_prompt_shapes_pick_the_matrix_cores_by_themselves(m, kernel):
    """512 and 2048 rows of x by 4096 x 4096 weights: the library's own choice (the int8 form, and from where its
    pass over W pays the binary16 one), within 1e-4 of max(1, |want|)."""
    n, k = 4096, 4096
    rng = np.random.default_rng(2)
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    gpu.say(f"q4_0 fx gemm {m} x 4096 x 4096")
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    assert last_kernel() == kernel
    lo, hi = 1000, 1256
    want = O.qmatmul(O.Q4_0, raw.reshape(n, -1)[lo:hi].reshape(-1), x, hi - lo, k)
    assert np.all(np.abs(got[:, lo:hi] - want) <= 1e-4 * np.maximum(1, np.abs(want)))


def last_kernel():
    buf = ctypes.create_string_buffer(200)
    capi.check(gpu.lib().mi355x_last_kernel(buf, 200))
    return buf.value.decode()


def pairs_and_int8(raw, x_dev, n, k):
    """The same product from 256 rows on in its two forms: 12-bit digit pairs on the binary16 matrix cores (the
    library's choice for large products; "q4_0.fx_pairs" = 2 asks for it whatever the shape), and the int8 form
    ("q4_0.fx_pairs" = 0). Returns both and the kernels that ran."""
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    out, ran = [], []
    try:
        capi.check(l.mi355x_tune(b"q4_0.fx_rows", 1))
        for pairs in (2, 0):
            capi.check(l.mi355x_tune(b"q4_0.fx_pairs", pairs))
            out.append(gpu.qgemv(O.Q4_0, ptr, x_dev, n, k))
            ran.append(last_kernel())
    finally:
        capi.check(l.mi355x_tune(b"q4_0.fx_pairs", 1))
        capi.check(l.mi355x_tune(b"q4_0.fx_rows", 0))
    return out[0], out[1], ran


@pytest.mark.parametrize("m,n,k,tiles", [(40, 100, 256, "1 x 1"), (256, 64, 128, "2 x 1"), (300, 520, 256, "3 x 3"), (1000, 1030, 1152, "8 x 5"), (2047, 700, 768, "16 x 3"),
                                         (512, 4096, 4096, "4 x 16"), (257, 129, 14336, "3 x 1")])
def test_digit_pairs_on_the_binary16_matrix_cores_give_the_int8_form_its_bits(m, n, k, tiles):
    """Rows and columns that do not fill the last tiles, one and many blocks of K; scales of either sign, zero and
    subnormal; rows of x of very different magnitude, a block of zeros, a tiny and a huge block, a NaN and an
    infinity: every bit of the result equal, NaNs in the same places."""
    rng = np.random.default_rng(m + n + k)
    raw = random_blocks(rng, O.Q4_0, n * k)
    x = (rng.normal(size=(m, k)) * np.exp(rng.normal(size=(m, 1)) * 3)).astype(np.float32)
    x[m // 2, :32] = 0
    x[1, 32:64] *= 1e-36
    x[2, 64:96] *= 1e30
    x[3, 96:128] = np.float32(1e-42)
    x[5, k - 1] = np.nan
    x[m - 1, 7] = np.inf
    gpu.say(f"q4_0 fx gemm, digit pairs, M={m} N={n} K={k}")
    got, int8, ran = pairs_and_int8(raw, gpu.dev(x), n, k)
    assert ran == [f"qgemm_q4_0_fx16_kernel: {tiles} tiles of 128 x 256", "qgemm_q4_0_fx_kernel"]
    assert np.isnan(got[5]).all() and np.isnan(got[m - 1]).all() and not np.isnan(got[:5]).any()
    assert np.array_equal(got.view(np.uint32), int8.view(np.uint32))
    if m * n * k <= 1 << 30:  # the larger ones rest on the int8 form, which the tests above hold to the oracle
        ok = ~np.isnan(got)
        want = O.qmatmul(O.Q4_0, raw, x, n, k)
        assert np.all(np.abs(got - want)[ok] <= 2e-6 * magnitude(raw, x, n, k)[ok] + 1e-30)


def test_digit_pairs_at_the_ends_of_the_fixed_point_range_and_rows_further_apart_than_k():
    """Every element of a block at the block's largest magnitude, every nibble 0 or 15: both digits and their sums at
    their extremes (d1 = 2048, block sums of 32 * 8 * 2048), with and without cancellation; rows of x 8 floats
    further apart than K."""
    m, n, k = 260, 130, 256
    raw = np.zeros((n * k // 32, 18), np.uint8)
    raw[:, :2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    raw[0::2, 2:] = 0x00  # n = 0: -8
    raw[1::2, 2:] = 0xFF  # n = 15: +7
    raw = raw.reshape(-1)
    x = np.full((m, k), 3.25, np.float32)
    x[1::2] *= -1
    x[:, 1::2] *= np.where(np.arange(m)[:, None] % 3 == 0, -1.0, 1.0).astype(np.float32)
    wide = torch.zeros((m, k + 8), device="cuda:0")
    wide[:, :k] = gpu.dev(x)
    gpu.say("q4_0 fx gemm, digit pairs, extremes")
    got, int8, ran = pairs_and_int8(raw, wide[:, :k], n, k)
    assert ran[0].startswith("qgemm_q4_0_fx16_kernel") and ran[1] == "qgemm_q4_0_fx_kernel"
    assert np.array_equal(got.view(np.uint32), int8.view(np.uint32))
    assert np.all(np.abs(got - O.qmatmul(O.Q4_0, raw, x, n, k)) <= 2e-6 * magnitude(raw, x, n, k))
