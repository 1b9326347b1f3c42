"""The prompt-sized Q4_0 product with bfloat16 activations on the matrix cores,
through the C ABI, against the oracle's restatement of Tensor.MatMulT for a
half x and a block-quantized w (tensor/quant.go:45-48): float32 product over
dequantized weights, one rounding to bfloat16.

The device sums in another order (each weight as two bfloat16 halves on the
matrix cores), so its float32 result differs from the oracle's in the last bits, and its bfloat16 result differs where such a difference crosses a
rounding boundary: by one unit in the last place of bfloat16, at a small share of
the outputs. The float32 output is held to 1e-4 of max(1, |want|) at K = 4096 (the
bound asked for is 1e-3)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as O
from mimir_amd import capi
from tests import gpu
from tests.helpers import bench_blocks, random_blocks

pytestmark = pytest.mark.gpu


def bf16_bits(a):
    return O.f32_to_bf16(np.ascontiguousarray(a, np.float32))


def qgemm(w_raw, x_bits, n, k, out_dt=capi.BF16, x_stride=None, w_offset=0):
    l = gpu.lib()
    m = x_bits.shape[0]
    wbuf, wp = gpu.dev_bytes_at(w_raw, w_offset)
    xs = k if x_stride is None else x_stride
    xbuf = torch.zeros(m * xs + 8, dtype=torch.int16, device="cuda:0")
    xbuf[: m * xs].view(m, xs)[:, :k] = torch.from_numpy(x_bits.view(np.int16)).to("cuda:0")
    if out_dt == capi.BF16:
        y = torch.full((m, n), -1, dtype=torch.int16, device="cuda:0")
    else:
        y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(l.mi355x_qgemm_bf16(capi.Q4_0, wp, xbuf.data_ptr(), y.data_ptr(), m, n, k, xs, out_dt, gpu.stream()))
    gpu.sync()
    out = y.cpu().numpy()
    return out.view(np.uint16) if out_dt == capi.BF16 else out


def reference_f32(w_raw, x_bits, n, k):
    """The float32 sums before the rounding: the oracle's product of float32
    activations with the dequantized weights."""
    return O.qmatmul(O.Q4_0, w_raw, O.bf16_to_f32(x_bits), n, k)


def f32_bound(w_raw, x_bits, n, k):
    """2e-6 of sum_k |x| |w|: random scales span binary16's range, so terms of
    very different size cancel, and the error of a float32 sum goes with the
    size of its terms, not of its result (the reference's own sum is as far
    from the exact one)."""
    wf = np.abs(O.dequantize(O.Q4_0, w_raw).reshape(n, k).astype(np.float64))
    mag = np.abs(O.bf16_to_f32(x_bits).astype(np.float64)) @ wf.T
    return np.maximum(2e-6 * mag, 1e-30)


def check_f32(got32, want_f32, bound, what=""):
    err = np.abs(got32.astype(np.float64) - want_f32)
    worst = float((err / bound).max())
    assert worst <= 1.0, (what, worst, float(err.max()))


def check_bf16(got, want_bits, bound):
    """Equal, or apart by one bfloat16 step (the float32 sums differ in their
    last bits, which now and then straddle a rounding boundary) plus what the
    float32 sums themselves may differ by; few outputs differ at all."""
    g = O.bf16_to_f32(got).astype(np.float64); w = O.bf16_to_f32(want_bits).astype(np.float64)
    differ = got != want_bits
    ulp = np.maximum(np.abs(w), 2.0 ** -116) * 2.0 ** -7
    over = np.abs(g - w) - (ulp * 1.01 + 2 * bound)
    assert np.all(over[differ] <= 0), float(over[differ].max())
    assert differ.mean() <= 0.01, float(differ.mean())


@pytest.mark.parametrize("m,n,k", [(64, 128, 256), (32, 128, 512), (70, 200, 768), (1, 130, 4096), (200, 384, 1024), (129, 257, 1280), (33, 65, 96), (40, 130, 192),
                                   (250, 12790, 512)])  # the last: 128-row tiles
def test_small_and_ragged_shapes(m, n, k):
    rng = np.random.default_rng(m * 7 + n)
    w = random_blocks(rng, O.Q4_0, n * k)
    x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say(f"qgemm_bf16 {m}x{k} by {n}x{k}")
    want_f32 = reference_f32(w, x, n, k)
    got32 = qgemm(w, x, n, k, capi.F32)
    bound = f32_bound(w, x, n, k)
    check_f32(got32, want_f32, bound)
    got = qgemm(w, x, n, k)
    check_bf16(got, O.q4_0_matmul_bf16(w, x, n, k), bound)
    # strided rows of x, weights at another address (K = 96 and 192 take the general route: K must be whole panels of 256)
    got2 = qgemm(w, x, n, k, x_stride=k + 24, w_offset=32)
    assert np.array_equal(got2, got)


def test_general_route_for_other_shapes_and_agreement():
    """Rows of x that are not 16-byte aligned go through the decode kernels; both
    routes agree on a shape both take."""
    l = gpu.lib()
    rng = np.random.default_rng(3)
    m, n, k = 9, 70, 96
    w = random_blocks(rng, O.Q4_0, n * k); x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say("qgemm_bf16 general route, rows of x 99 apart")
    want_f32 = reference_f32(w, x, n, k)
    got32 = qgemm(w, x, n, k, capi.F32, x_stride=k + 3)
    bound = f32_bound(w, x, n, k)
    check_f32(got32, want_f32, bound)
    check_bf16(qgemm(w, x, n, k, x_stride=k + 3), O.q4_0_matmul_bf16(w, x, n, k), bound)
    m, n, k = 40, 256, 256
    w = random_blocks(rng, O.Q4_0, n * k); x = bf16_bits(rng.normal(size=(m, k)))
    fast = qgemm(w, x, n, k, capi.F32)
    try:
        capi.check(l.mi355x_tune(b"qgemm.path", 1))
        slow = qgemm(w, x, n, k, capi.F32)
    finally:
        capi.check(l.mi355x_tune(b"qgemm.path", 0))
    check_f32(fast, slow, f32_bound(w, x, n, k))


def test_special_values():
    """Zero, subnormal and negative scales; activations that span the range of
    bfloat16; an infinity and a NaN stay in their own rows."""
    rng = np.random.default_rng(4)
    m, n, k = 64, 128, 128
    w = random_blocks(rng, O.Q4_0, n * k).reshape(-1, 18)
    for i, bits in enumerate([0x0000, 0x8000, 0x0001, 0x83ff, 0xbc00, 0x7bff]):
        w[i::7, 0] = bits & 0xff; w[i::7, 1] = bits >> 8
    w = w.reshape(-1)
    xf = rng.normal(size=(m, k)).astype(np.float32)
    xf[1] *= 1e-30; xf[2] *= 1e20; xf[3, 5] = 0.0; xf[4] = 0.0
    x = bf16_bits(xf)
    # keep the largest scale out of the huge row's way: its sums must stay finite for the comparison
    gpu.say("qgemm_bf16 special values")
    want_f32 = reference_f32(w, x, n, k)
    got32 = qgemm(w, x, n, k, capi.F32)
    assert np.isfinite(want_f32).all() and np.isfinite(got32).all()
    check_f32(got32, want_f32, f32_bound(w, x, n, k))
    xf[5, 7] = np.inf; xf[6, 9] = np.nan
    got32 = qgemm(w, bf16_bits(xf), n, k, capi.F32)
    assert not np.isfinite(got32[5]).any() and np.isnan(got32[6]).all()
    assert np.array_equal(got32[:5], qgemm(w, x, n, k, capi.F32)[:5])


@pytest.mark.parametrize("n", [4096, 14336])
def test_prefill_shapes(n):
    """M = 512 tokens at the 8B model's shapes, weights and activations as the
    configurations draw them. The oracle takes a band of output columns (rows of
    W) at N = 14336 to stay within seconds; M = 2048 (which takes the exact form's
    other kernel) is checked against the oracle too, and row for row against
    itself, rows being independent."""
    rng = np.random.default_rng(0)
    m, k = 512, 4096
    w = bench_blocks(rng, O.Q4_0, n * k)
    x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say(f"qgemm_bf16 512x4096 by {n}x4096")
    got = qgemm(w, x, n, k)
    got32 = qgemm(w, x, n, k, capi.F32)
    lo, hi = (0, n) if n == 4096 else (5000, 7048)
    wb = w.reshape(n, -1)[lo:hi].reshape(-1)
    want_f32 = reference_f32(wb, x, hi - lo, k)
    err = np.abs(got32[:, lo:hi] - want_f32)
    # two float32 sums of 4096 terms in different orders; the bound asked for is 1e-3
    assert np.all(err <= 1e-4 * np.maximum(1, np.abs(want_f32))), float(err.max())
    check_bf16(got[:, lo:hi], O.q4_0_matmul_bf16(wb, x, hi - lo, k), 1e-4 * np.maximum(1, np.abs(want_f32)))
    if n == 4096:
        gpu.say("qgemm_bf16 2048x4096 by 4096x4096")
        x4 = np.concatenate([x, x[::-1], x, x[::-1]], axis=0)
        got4 = qgemm(w, x4, n, k)
        # rows are independent: the same row of x gives the same bits wherever it stands among the 2048
        assert np.array_equal(got4[512:1024], got4[:512][::-1]) and np.array_equal(got4[1024:1536], got4[:512]) and np.array_equal(got4[1536:], got4[512:1024])
        # 2048 rows take the exact form's other kernel (the weights' integers from a panel): the same sums in another order
        assert last_kernel().startswith("qgemm_q4_0_blocks_kernel")
        check_bf16(got4[:512], O.q4_0_matmul_bf16(w, x, n, k), 1e-4 * np.maximum(1, np.abs(want_f32)))


def test_prefill_shape_2048_by_14336():
    """The shape the prompt-sized product's figures are quoted on: M = 2048 tokens by N = 14336, K = 4096,
    weights and activations as the configurations draw them. The oracle takes two bands of 256 output columns,
    one of them across a tile boundary of every tile height, over all 2048 rows; the exact form (float32 sums and
    their bfloat16 rounding) and the form with weights rounded to binary16."""
    rng = np.random.default_rng(3)
    m, n, k = 2048, 14336, 4096
    w = bench_blocks(rng, O.Q4_0, n * k)
    x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say("qgemm_bf16 2048x4096 by 14336x4096")
    got = qgemm(w, x, n, k)
    got32 = qgemm(w, x, n, k, capi.F32)
    # the exact form's cut of this shape: a wide and a narrow tile a compute unit
    assert last_kernel() == "qgemm_q4_0_blocks_kernel: 8 x 32 tiles of 256 x 256, 8 x 32 tiles of 256 x 192"
    with binary16_weights():
        gpu.say("qgemm_bf16 2048x4096 by 14336x4096, binary16 weights")
        half32 = qgemm(w, x, n, k, capi.F32)
    for lo in (0, 9088 - 128):
        hi = lo + 256
        wb = w.reshape(n, -1)[lo:hi].reshape(-1)
        want_f32 = reference_f32(wb, x, hi - lo, k)
        err = np.abs(got32[:, lo:hi] - want_f32)
        assert np.all(err <= 1e-4 * np.maximum(1, np.abs(want_f32))), (lo, float(err.max()))
        check_bf16(got[:, lo:hi], O.q4_0_matmul_bf16(wb, x, hi - lo, k), 1e-4 * np.maximum(1, np.abs(want_f32)))
        check_binary16_form(wb, x, hi - lo, k, half32[:, lo:hi])


def test_tall_tiles():
    """M = 2048 by N = 6144 takes the 256-row tiles: a band of columns against
    the oracle, and ragged edges (M = 2000, N = 6100) against the same rows and
    columns of the whole product."""
    rng = np.random.default_rng(21)
    m, n, k = 2048, 6144, 1024
    w = bench_blocks(rng, O.Q4_0, n * k)
    x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say("qgemm_bf16 2048x1024 by 6144x1024")
    got32 = qgemm(w, x, n, k, capi.F32)
    lo, hi = 3000, 3512
    wb = w.reshape(n, -1)[lo:hi].reshape(-1)
    want_f32 = reference_f32(wb, x, hi - lo, k)
    err = np.abs(got32[:, lo:hi] - want_f32)
    assert np.all(err <= 1e-4 * np.maximum(1, np.abs(want_f32))), float(err.max())
    got = qgemm(w, x, n, k)
    check_bf16(got[:, lo:hi], O.q4_0_matmul_bf16(wb, x, hi - lo, k), 1e-4 * np.maximum(1, np.abs(want_f32)))
    gpu.say("qgemm_bf16 2000x1024 by 6100x1024")
    part = qgemm(w.reshape(n, -1)[:6100].reshape(-1), x[:2000], 6100, k)
    assert np.array_equal(part, got[:2000, :6100])


def test_errors():
    l = gpu.lib()
    z = torch.zeros(4096, dtype=torch.int16, device="cuda:0")
    p = z.data_ptr()
    assert l.mi355x_qgemm_bf16(capi.F16, p, p, p, 2, 32, 64, 64, capi.BF16, gpu.stream()) == capi.ERR_DTYPE
    assert l.mi355x_qgemm_bf16(capi.Q4_K, p, p, p, 2, 32, 64, 64, capi.BF16, gpu.stream()) == capi.ERR_INTERNAL  # K not in blocks of 256
    assert l.mi355x_qgemm_bf16(capi.Q4_0, p, p, p, 2, 32, 64, 64, capi.F16, gpu.stream()) == capi.ERR_DTYPE
    assert l.mi355x_qgemm_bf16(capi.Q4_0, p, p, p, 2, 32, 48, 48, capi.BF16, gpu.stream()) == capi.ERR_INTERNAL
    assert l.mi355x_qgemm_bf16(capi.Q4_0, p, p, p, 2, 32, 64, 32, capi.BF16, gpu.stream()) == capi.ERR_SHAPE
    capi.check(l.mi355x_qgemm_bf16(capi.Q4_0, p, p, p, 0, 32, 64, 64, capi.BF16, gpu.stream()))


# ---- the approximate form: weights rounded once to binary16 ("qgemm.f16" = 1) ----

class binary16_weights:
    """Switches mi355x_qgemm_bf16's Q4_0 matrix-core kernel to its binary16 form and back."""

    def __enter__(self):
        capi.check(gpu.lib().mi355x_tune(b"qgemm.f16", 1))

    def __exit__(self, *exc):
        capi.check(gpu.lib().mi355x_tune(b"qgemm.f16", 0))


def scales_within_binary16(rng, n_elems, top=8188.0):
    """Random Q4_0 blocks whose scales span binary16's range up to what eight times
    the scale still fits (subnormal scales and both signs included)."""
    w = random_blocks(rng, O.Q4_0, n_elems).reshape(-1, 18)
    d = w[:, :2].copy().view(np.float16).reshape(-1)
    big = np.abs(d.astype(np.float32)) > top
    d[big] = (d[big].astype(np.float32) / 16).astype(np.float16)
    w[:, :2] = d.view(np.uint8).reshape(-1, 2)
    return w.reshape(-1)


def rounded_weights(w_raw, n, k):
    """What the kernel multiplies with: (n - 8) * d rounded once, to nearest even, to
    binary16 (the product is exact in float32, so numpy's float16 cast is that rounding)."""
    b = w_raw.reshape(-1, 18)
    d = b[:, :2].copy().view(np.float16).astype(np.float32)
    q = np.concatenate([b[:, 2:] & 15, b[:, 2:] >> 4], axis=1).astype(np.float32) - 8
    with np.errstate(over="ignore"):
        return (q * d).astype(np.float16).astype(np.float64).reshape(n, k)


def check_binary16_form(w, x, n, k, got32):
    xf = O.bf16_to_f32(x).astype(np.float64)
    w16 = rounded_weights(w, n, k)
    bound = f32_bound(w, x, n, k)
    # the kernel's own arithmetic: exact products of x with the rounded weights, float32 sums
    check_f32(got32, xf @ w16.T, bound, "against the rounded weights")
    # and how far that is from the reference: 2^-11 of every term (2^-25 for subnormal weights)
    want = reference_f32(w, x, n, k)
    wf = np.abs(O.dequantize(O.Q4_0, w).reshape(n, k).astype(np.float64))
    slack = np.abs(xf) @ (np.maximum(wf * 2.0 ** -11, 2.0 ** -25)).T
    check_f32(got32, want, bound + slack, "against the reference")


@pytest.mark.parametrize("m,n,k", [(64, 128, 256), (70, 200, 768), (1, 130, 4096), (200, 384, 1024), (129, 257, 1280), (300, 3200, 512),
                                   (250, 12790, 512)])  # the last: 128-row tiles
def test_binary16_form_small_and_ragged_shapes(m, n, k):
    rng = np.random.default_rng(m * 11 + n)
    w = scales_within_binary16(rng, n * k)
    x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say(f"qgemm_bf16, binary16 weights, {m}x{k} by {n}x{k}")
    with binary16_weights():
        got32 = qgemm(w, x, n, k, capi.F32)
        got = qgemm(w, x, n, k)
        got2 = qgemm(w, x, n, k, capi.F32, x_stride=k + 24, w_offset=32)
    check_binary16_form(w, x, n, k, got32)
    assert np.array_equal(got2, got32)
    assert np.array_equal(got, O.f32_to_bf16(got32))  # one rounding of the same float32 sums


class binary16_weights_in_tiles:
    """The binary16 form kept on the one launch whose tiles convert W for themselves, whatever the shape."""

    def __enter__(self):
        capi.check(gpu.lib().mi355x_tune(b"qgemm.f16", 2))

    def __exit__(self, *exc):
        capi.check(gpu.lib().mi355x_tune(b"qgemm.f16", 0))


def last_kernel():
    buf = ctypes.create_string_buffer(200)
    capi.check(gpu.lib().mi355x_last_kernel(buf, 200))
    return buf.value.decode()


@pytest.mark.parametrize("m,n,k,tiles", [
    (2048, 14336, 256, "8 x 32 tiles of 256 x 256, 8 x 32 tiles of 256 x 192"),  # the quoted shape's cut: a wide and a narrow tile a compute unit
    (1024, 12288, 256, "4 x 0 tiles of 256 x 256, 4 x 64 tiles of 256 x 192"),
    (2047, 6200, 768, "8 x 25 tiles of 256 x 256, 8 x 0 tiles of 256 x 192"),   # ragged both ways
    (1300, 10241, 256, "6 x 41 tiles of 256 x 256, 6 x 0 tiles of 256 x 192"),
    (1024, 8100, 512, "8 x 32 tiles of 128 x 256, 8 x 0 tiles of 256 x 192"),   # too few wide tiles for the device
])
def test_binary16_form_through_the_panel(m, n, k, tiles):
    """From 1024 rows of x on, where its tiles keep the device busy, W is first written once as a binary16 panel
    and the product is a plain one from LDS (two launches). Every kind of tile; shapes that fill their tiles and
    shapes whose last tiles are ragged both ways; scales over binary16's range; rows of x apart and W at an offset.
    The same weights as the tile kernel's, bit for bit, so the two routes differ by the order of the float32 sums only."""
    rng = np.random.default_rng(m + 3 * n + k)
    w = scales_within_binary16(rng, n * k)
    xf = rng.normal(size=(m, k)).astype(np.float32)
    xf[5] *= 2.0 ** 90
    xf[6] *= 2.0 ** -90
    xf[7] = 0
    x = bf16_bits(xf)
    gpu.say(f"qgemm_bf16, binary16 weights through the panel, {m}x{k} by {n}x{k}")
    with binary16_weights():
        got32 = qgemm(w, x, n, k, capi.F32)
        got = qgemm(w, x, n, k)
        got2 = qgemm(w, x, n, k, capi.F32, x_stride=k + 24, w_offset=32)
        assert last_kernel() == "hgemm_f16_nt_kernel: " + tiles
    check_binary16_form(w, x, n, k, got32)
    assert np.array_equal(got2, got32)
    assert np.array_equal(got, O.f32_to_bf16(got32))  # one rounding of the same float32 sums
    assert np.all(got32[7] == 0)
    gpu.say(f"qgemm_bf16, binary16 weights in tiles, {m}x{k} by {n}x{k}")
    with binary16_weights_in_tiles():
        tiles32 = qgemm(w, x, n, k, capi.F32)
    check_f32(got32, tiles32.astype(np.float64), 2 * f32_bound(w, x, n, k), "panel route against the tile kernel")


@pytest.mark.parametrize("m,n,k,panel", [(64, 256, 512, False), (1024, 8192, 256, True)])
def test_binary16_form_rows_of_any_range(m, n, k, panel):
    """Each row of x is scaled by a power of two of its own before it becomes binary16:
    rows near float32's largest and smallest magnitudes, a row of zeros, a row with one
    element 2^20 above the others and a row of bfloat16 subnormals come out as exactly
    as rows of ordinary size; a row holding an infinity or a NaN has no finite results
    and leaves the other rows alone. In the tile kernel and through the panel."""
    rng = np.random.default_rng(5)
    w = bench_blocks(rng, O.Q4_0, n * k)
    xf = rng.normal(size=(m, k)).astype(np.float32)
    xf[1] *= 2.0 ** 100
    xf[2] *= 2.0 ** -100
    xf[3] = 0
    xf[4, 7] = 2.0 ** 20
    xf[5] *= 2.0 ** -130
    xf[6] *= 2.0 ** 120
    xf[7] *= 2.0 ** -110
    x = bf16_bits(xf)
    bad = x.copy()
    bad[8, 3] = 0x7f80   # +Inf
    bad[9, 5] = 0x7fc0   # NaN
    gpu.say("qgemm_bf16, binary16 weights, rows of extreme ranges")
    with binary16_weights():
        got32 = qgemm(w, x, n, k, capi.F32)
        assert last_kernel().startswith("hgemm_f16_nt_kernel") == panel
        got_bad = qgemm(w, bad, n, k, capi.F32)
    check_binary16_form(w, x, n, k, got32)
    assert np.all(got32[3] == 0)
    assert not np.any(np.isfinite(got_bad[8])) and np.all(np.isnan(got_bad[9]))
    keep = np.ones(m, bool); keep[[8, 9]] = False
    assert np.array_equal(got_bad[keep], got32[keep])


@pytest.mark.parametrize("n", [4096, 14336])
def test_binary16_form_prefill_shapes(n):
    """The configurations' shapes and draws: off by 2^-11 of every term at most, which at
    K = 4096 is some 2e-4 of the results' root mean square and less than 2e-3 of it for
    the worst of a million outputs (held to 3e-4 and 2e-3); the bfloat16 result is the one
    rounding of the float32 one. M = 2048 takes the 256-row tiles."""
    rng = np.random.default_rng(0)
    m, k = 2048, 4096
    w = bench_blocks(rng, O.Q4_0, n * k)
    x = bf16_bits(rng.normal(size=(m, k)))
    gpu.say(f"qgemm_bf16, binary16 weights, 2048x4096 by {n}x4096")
    with binary16_weights():
        got32 = qgemm(w, x, n, k, capi.F32)
        got = qgemm(w, x, n, k)
    assert np.array_equal(got, O.f32_to_bf16(got32))
    lo, hi = 5000 % n, 5000 % n + 512
    wb = w.reshape(n, -1)[lo:hi].reshape(-1)
    rows = slice(0, m, 4)
    check_binary16_form(wb, x[rows], hi - lo, k, got32[rows, lo:hi])
    want = reference_f32(wb, x[rows], hi - lo, k).astype(np.float64)
    err = got32[rows, lo:hi] - want
    size = np.sqrt(np.mean(want ** 2))
    print(f"binary16 weights, N={n}: rms error {np.sqrt(np.mean(err ** 2)) / size:.2e}, worst {np.abs(err).max() / size:.2e} of the rms result")
    assert np.sqrt(np.mean(err ** 2)) <= 3e-4 * size and np.abs(err).max() <= 2e-3 * size


@pytest.mark.parametrize("m,n,k,tiles", [(300, 515, 512, "3 x 3 tiles of 128 x 256, 3 x 0 tiles of 256 x 192"),
                                         (1000, 1030, 1280, "8 x 5 tiles of 128 x 256, 8 x 0 tiles of 256 x 192"),
                                         (2047, 6200, 768, "8 x 25 tiles of 256 x 256, 8 x 0 tiles of 256 x 192"),
                                         (2047, 9000, 256, "8 x 25 tiles of 256 x 256, 8 x 14 tiles of 256 x 192"),  # the last narrow tile ragged
                                         (1024, 12288, 256, "4 x 0 tiles of 256 x 256, 4 x 64 tiles of 256 x 192"),
                                         (512, 14336, 256, "4 x 56 tiles of 128 x 256, 4 x 0 tiles of 256 x 192")])
def test_exact_form_from_the_panel_of_integers(m, n, k, tiles):
    """The exact form's second kernel (W's integers n - 8 once as a bfloat16 panel, block sums on the matrix cores, one
    FMA per block with the block's scale), asked for whatever the shape: against the oracle within the bound of the
    first, and against the first (the same exact products, other float32 sums); rows of x further apart than K, W at
    another address, tiles that the edges do not fill; both output dtypes, the bfloat16 one the rounding of
    the float32 one."""
    rng = np.random.default_rng(m + n + k)
    w = random_blocks(rng, O.Q4_0, n * k)
    x = bf16_bits(rng.normal(size=(m, k)) * np.exp(rng.normal(size=(m, 1)) * 2))
    l = gpu.lib()
    try:
        capi.check(l.mi355x_tune(b"qgemm.blocks", 2))
        gpu.say(f"qgemm_bf16, exact form from the panel, M={m} N={n} K={k}")
        got32 = qgemm(w, x, n, k, capi.F32, x_stride=k + 8)
        assert last_kernel() == "qgemm_q4_0_blocks_kernel: " + tiles
        got = qgemm(w, x, n, k, x_stride=k + 8)
        moved = qgemm(w, x, n, k, capi.F32, w_offset=16)
        capi.check(l.mi355x_tune(b"qgemm.blocks", 0))
        tile32 = qgemm(w, x, n, k, capi.F32)
        assert last_kernel().startswith("qgemm_q4_0_kernel")
    finally:
        capi.check(l.mi355x_tune(b"qgemm.blocks", 1))
    bound = f32_bound(w, x, n, k)
    assert np.array_equal(moved, got32)
    assert np.array_equal(got, bf16_bits(got32))
    check_f32(got32, tile32.astype(np.float64), 2 * bound, "against the tile kernel")
    if m * n * k <= 1 << 30:
        check_f32(got32, reference_f32(w, x, n, k), bound, "against the oracle")
    else:
        lo, hi = n - 300, n  # the last columns, across the edge tile
        wb = w.reshape(n, -1)[lo:hi].reshape(-1)
        check_f32(got32[:, lo:hi], reference_f32(wb, x, hi - lo, k), bound[:, lo:hi], "against the oracle")


def test_exact_form_from_the_panel_rows_with_nan_and_inf():
    m, n, k = 300, 260, 512
    rng = np.random.default_rng(8)
    w = random_blocks(rng, O.Q4_0, n * k)
    xf = rng.normal(size=(m, k)).astype(np.float32)
    clean = bf16_bits(xf)
    xf[5, 7] = np.inf; xf[6, 9] = np.nan
    l = gpu.lib()
    try:
        capi.check(l.mi355x_tune(b"qgemm.blocks", 2))
        gpu.say("qgemm_bf16, exact form from the panel, nan and inf")
        got32 = qgemm(w, bf16_bits(xf), n, k, capi.F32)
        base = qgemm(w, clean, n, k, capi.F32)
    finally:
        capi.check(l.mi355x_tune(b"qgemm.blocks", 1))
    assert not np.isfinite(got32[5]).any() and np.isnan(got32[6]).all()
    keep = np.ones(m, bool); keep[[5, 6]] = False
    assert np.array_equal(got32[keep], base[keep])
