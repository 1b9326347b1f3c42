"""Parity of the HIP path with the oracle, through the C ABI, on a real
MI355X: dequantization bit for bit, products within the stated tolerance.

Tolerances: dequantized weights 0 (bit-exact). Products: the conformance rule
of the reference, |got - want| <= tol * max(1, |want|), with tol = 1e-3 (the
bar this build is given for GEMV outputs) and, for Q4_0, also 1e-4 on inputs
the reference's own GPU conformance cases use (kerneltest/quant.go:142)."""
import os

import numpy as np
import pytest
import torch

import oracle as O
from mimir_amd import capi
from mimir_amd.mimfile import golden_cases
from tests import gpu
from tests.helpers import bench_blocks, bits_equal, check_close, exact_rows, random_blocks, rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-3


@pytest.mark.parametrize("dt", [O.Q8_0, O.Q4_K, O.Q6_K, O.Q4_0])
@pytest.mark.parametrize("out_dt", [O.F32, O.BF16, O.F16])
def test_dequantize_bit_exact(dt, out_dt):
    rng = np.random.default_rng(100 + dt)
    n = 10 * 1280  # kerneltest/quant.go:85: 9+1 rows of 1280
    raw = random_blocks(rng, dt, n)
    gpu.say(f"dequant dt={dt} out={out_dt} n={n}")
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    got = gpu.dequant(dt, ptr, 0, n, out_dt)
    want = O.dequantize(dt, raw, out_dt)
    assert bits_equal(got, want) if out_dt == O.F32 else np.array_equal(got, want)
    # rows 1..9: a view that starts a row in (the "shrunk" case)
    got = gpu.dequant(dt, ptr, 1280, 9 * 1280, out_dt)
    assert np.array_equal(got.view(np.uint32 if out_dt == O.F32 else np.uint16), want[1280:].view(np.uint32 if out_dt == O.F32 else np.uint16))


def test_dequantize_golden(golden_dir):
    cases = golden_cases(os.path.join(golden_dir, "quant.mim"))
    for kind, dt in (("q8_0", O.Q8_0), ("q4_K", O.Q4_K), ("q6_K", O.Q6_K)):
        c = cases[f"{kind}_dequantize"]
        raw = c["in"][-1].data.reshape(-1)
        gpu.say(f"golden dequant {kind}")
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        got = gpu.dequant(dt, ptr, 0, c["out"].data.size)
        assert bits_equal(got, c["out"].data.reshape(-1))


@pytest.mark.parametrize("dt", [O.Q8_0, O.Q4_K, O.Q6_K, O.Q4_0])
def test_gather_rows(dt):
    rng = np.random.default_rng(200 + dt)
    k = 1280
    raw = random_blocks(rng, dt, 10 * k)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    l = gpu.lib()
    for idx, ok in (([2, 0, 9], True), ([2, 10, 0], False)):  # kerneltest/quant.go:97
        gpu.say(f"gather dt={dt} idx={idx}")
        ti = gpu.dev(np.array(idx, np.int32))
        out = torch.zeros((3, k), dtype=torch.float32, device="cuda:0")
        capi.check(l.mi355x_gather_rows(dt, ptr, 10, k, ti.data_ptr(), 3, out.data_ptr(), gpu.stream()))
        st = l.mi355x_sync(gpu.stream())
        if ok:
            assert st == 0
            assert bits_equal(out.cpu().numpy(), O.gather_rows(dt, raw, 10, k, idx))
        else:
            assert st == capi.ERR_INDEX
            assert l.mi355x_sync(gpu.stream()) == 0  # the error is reported once


# ---- products ---------------------------------------------------------------

Q4_SHAPES = [  # (N, K): the decode shapes of an 8B Llama, and ragged ones
    (14336, 4096), (4096, 14336), (4096, 4096), (1024, 4096),
    (9, 1280), (1, 32), (5, 64), (130, 2048 + 32), (257, 4096 + 64), (33, 17 * 32), (3, 16384 + 256),
]


@pytest.mark.parametrize("n,k", Q4_SHAPES)
def test_q4_0_gemv_matches_oracle(n, k):
    rng = np.random.default_rng(n * 31 + k)
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    gpu.say(f"q4_0 gemv N={n} K={k}")
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    check_close(got, want, TOL, f"q4_0 {n}x{k}")
    assert rel_l2(got, want) < 1e-5


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336), (6144, 4096), (257, 4096 + 64), (1000, 128), (7, 8192), (512, 64),
                                 (40, 24576), (3, 65536), (70000, 256)])  # rows past what the whole-chip kernel stages; very many rows
def test_q4_0_gemv_both_launch_shapes_agree(n, k):
    """One row of float32 x goes to the kernel with a workgroup per compute unit (x digits in registers, rows in chunks
    of 64 pairs of blocks); "q4_0.stream" = 1 keeps it on the finer-grained launch. Same integers and the same float32
    operation per block in both: each within the oracle's bound, and equal to each other to the order of a row's sums."""
    rng = np.random.default_rng(n + 7 * k)
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    got = {}
    try:
        for off in (0, 1):
            capi.check(l.mi355x_tune(b"q4_0.stream", off))
            gpu.say(f"q4_0 gemv N={n} K={k}, whole-chip kernel {'off' if off else 'on'}")
            got[off] = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
            check_close(got[off], want, TOL, f"q4_0 {n}x{k} stream off={off}")
    finally:
        capi.check(l.mi355x_tune(b"q4_0.stream", 0))
    scale = np.abs(want).max()
    assert np.abs(got[0] - got[1]).max() <= 4e-6 * scale


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336), (4096, 4096), (1024, 4096), (6144, 4096), (1000, 4096), (300, 8192), (50, 2048)])
def test_q4_0_gemv_fed_through_lds_gives_the_same_bits(n, k):
    """"q4_0.stream" = 3 selects the whole-chip kernel's variant whose weights reach LDS by loads that write it directly,
    requested by wavefronts that do nothing else (slower on this device, kept for measurement). Same integers, same
    float32 operations in the same order as the default whole-chip kernel: the same bits from float32 x, and from
    converted x where the default is that kernel's order too, for any number of feeding wavefronts and rows under way."""
    rng = np.random.default_rng(3 * n + k)
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    base = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    base_act = gpu.qgemv_act(O.Q4_0, ptr, gpu.dev(x), n, k)
    check_close(base, want, TOL)
    try:
        capi.check(l.mi355x_tune(b"q4_0.stream", 3))
        for feeders, window in ((8, 3), (2, 20), (5, 1)):
            capi.check(l.mi355x_tune(b"q4_0.feeders", feeders))
            capi.check(l.mi355x_tune(b"q4_0.feed_window", window))
            gpu.say(f"q4_0 gemv N={n} K={k} fed through LDS by {feeders} wavefronts, {window} rows under way")
            assert bits_equal(gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k), base)
            got_act = gpu.qgemv_act(O.Q4_0, ptr, gpu.dev(x), n, k)
            if k <= 4096:
                assert bits_equal(got_act, base_act)
            else:  # converted x of longer rows is otherwise multiplied by the finer-grained launch, which adds a row's blocks in another order
                assert np.abs(got_act - base_act).max() <= 4e-6 * np.abs(want).max()
    finally:
        capi.check(l.mi355x_tune(b"q4_0.stream", 0))
        capi.check(l.mi355x_tune(b"q4_0.feeders", 8))
        capi.check(l.mi355x_tune(b"q4_0.feed_window", 3))


def test_q4_0_gemv_clock_readings():
    """mi355x_gemv_stamps: five readings of the 100 MHz clock per workgroup of the whole-chip kernel, in order, the launch
    a few microseconds long; NULL stops it (the buffer is then left alone)."""
    rng = np.random.default_rng(2)
    n, k = 14336, 4096
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    stamps = torch.zeros(5 * 1024, dtype=torch.int64, device="cuda:0")
    gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    try:
        capi.check(l.mi355x_gemv_stamps(stamps.data_ptr()))
        gpu.say("q4_0 gemv with clock readings")
        got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    finally:
        capi.check(l.mi355x_gemv_stamps(None))
    check_close(got, O.qmatmul(O.Q4_0, raw, x, n, k), TOL)
    s = stamps.cpu().numpy().reshape(-1, 5)
    s = s[s[:, 0] != 0]
    assert 64 <= len(s) <= 512
    assert np.all(np.diff(s, axis=1) >= 0)
    assert 100 <= s[:, 4].max() - s[:, 0].min() <= 10000  # 1 us to 100 us in ticks of 10 ns
    stamps.zero_()
    gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    assert int(stamps.abs().sum()) == 0


def test_q4_0_gemv_random_scales_and_unaligned_start():
    """Weights that start a row into a buffer, 18 bytes past a 256-byte
    boundary (kerneltest/quant.go:89-92), with scales of either sign,
    subnormal and zero; activations the int8 path would keep exactly."""
    rng = np.random.default_rng(5)
    n, k = 9, 1280
    raw = random_blocks(rng, O.Q4_0, (n + 1) * k)
    row = k // 32 * 18
    for m, shape in ((1, (k,)), (1, (1, k)), (6, (2, 3, k))):
        x = exact_rows(rng, O.Q4_0, m, k).reshape(shape)
        gpu.say(f"q4_0 gemv shrunk rows, x shape {shape}")
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        got = gpu.qgemv(O.Q4_0, ptr + row, gpu.dev(x), n, k)
        want = O.qmatmul(O.Q4_0, raw[row:], x, n, k)
        check_close(got, want, 1e-4, f"q4_0 shrunk {shape}")


@pytest.mark.parametrize("rows,cols,waves", [(1, 1, 1), (2, 1, 4), (4, 1, 8), (2, 1, 8), (4, 1, 2), (1, 2, 4), (2, 2, 8), (4, 2, 2)])
def test_q4_0_fixed_point_kernel_every_launch_shape(rows, cols, waves):
    rng = np.random.default_rng(9)
    n, k = 203, 4096 + 64 * 3
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    try:
        for key, v in ((b"q4_0.path", 2), (b"q4_0.rows", rows), (b"q4_0.cols", cols), (b"q4_0.waves", waves)):
            capi.check(l.mi355x_tune(key, v))
        gpu.say(f"q4_0 fixed-point gemv plan R={rows} PC={cols} waves={waves}")
        got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
        check_close(got, want, TOL)
        assert rel_l2(got, want) < 1e-5
    finally:
        for key in (b"q4_0.path", b"q4_0.rows", b"q4_0.cols", b"q4_0.waves"):
            capi.check(l.mi355x_tune(key, 0))


def test_q4_0_fixed_point_kernel_special_values():
    """Blocks of x that are all zero, tiny, huge, or hold an infinity or a NaN:
    zeros contribute nothing, and a non-finite block makes its rows NaN, as a
    float product does (Inf - Inf or 0 * Inf)."""
    rng = np.random.default_rng(10)
    n, k = 40, 512
    raw = bench_blocks(rng, O.Q4_0, n * k)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    x = rng.normal(size=k).astype(np.float32)
    x[0:32] = 0
    x[32:64] *= 1e-36
    x[64:96] *= 1e30
    x[96:128] = np.float32(1e-42)  # subnormal
    gpu.say("q4_0 fixed-point gemv special values")
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    x[200] = np.inf
    got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    assert np.isnan(got).all()
    x[200] = np.nan
    assert np.isnan(gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)).all()


@pytest.mark.parametrize("m", [1, 8, 64])
def test_q4_0_fixed_point_outliers_inside_a_block(m):
    """The fixed-point kernels keep 24 bits per block of 32 activations, not per element: an element
    10^6 times its neighbours takes the block's scale, and the neighbours keep what is left of the 24 bits.
    The error per element is at most 2^-23 of the block's largest magnitude (half a unit of a grid of 7829367
    steps, and the rounding of the scaling), so the result is within 2^-23 * sum_b amax_b * sum_{e in b} |w_e| of the float32 product's exact
    value, whatever the weights are. Three cases a float32 product would keep exactly and this one cannot:
    the outlier's own weight is zero (nibble 8), so that only the neighbours count; every other weight is
    zero, so that only the outlier counts; and random weights. Each is held to that bound plus the float32
    product's own 2e-6 * sum |x| |w|, and to the conformance rule tol * max(1, |want|) with tol 1e-3 where
    the bound itself is inside it. One row of x (v_dot8), eight (int8 matrix cores, W read once) and 64
    (the tiled kernel)."""
    rng = np.random.default_rng(31 + m)
    n, k = 64, 4096
    nb = k // 32
    base = bench_blocks(rng, O.Q4_0, n * k).reshape(n, nb, 18)
    x = rng.normal(size=(m, k)).astype(np.float32)
    pos = rng.integers(0, 32, nb)  # the outlier's place in each block
    x.reshape(m, nb, 32)[:, np.arange(nb), pos] *= np.float32(1e6)

    def with_nibbles(blocks, e, value):
        """Sets the nibble of element e[b] of block b of every row to value."""
        out = blocks.copy()
        for b in range(nb):
            byte, high = 2 + (e[b] % 16), e[b] >= 16
            col = out[:, b, byte]
            out[:, b, byte] = (col & 0x0f) | (value << 4) if high else (col & 0xf0) | value
        return out

    zeros = np.full((n, nb, 18), 0x88, np.uint8); zeros[:, :, :2] = base[:, :, :2]  # every weight (8 - 8) * d
    only = zeros.copy()
    for b in range(nb):  # only the outlier's weight is not zero
        byte, high = 2 + (pos[b] % 16), pos[b] >= 16
        only[:, b, byte] = base[:, b, byte] & (0xf0 if high else 0x0f) | (0x08 if high else 0x80)
    cases = {"outlier's weight zero": with_nibbles(base, pos, 8), "only the outlier's weight": only, "random weights": base}
    for name, blocks in cases.items():
        raw = blocks.reshape(-1)
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        gpu.say(f"q4_0 fixed-point outliers in every block, m={m}: {name}")
        got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
        want = O.qmatmul(O.Q4_0, raw, x, n, k)
        wf = np.abs(O.dequantize(O.Q4_0, raw).reshape(n, nb, 32).astype(np.float64))
        amax = np.abs(x.reshape(m, nb, 32)).max(2).astype(np.float64)                        # [m, nb]
        fixed = 2.0 ** -23 * np.einsum("mb,nb->mn", amax, wf.sum(2))                         # the fixed-point grid
        f32 = 2e-6 * np.einsum("mbe,nbe->mn", np.abs(x.reshape(m, nb, 32)).astype(np.float64), wf)  # float32 sums in two orders
        err = np.abs(got.astype(np.float64) - want)
        assert np.all(err <= fixed + f32 + 1e-30), (name, float((err / (fixed + f32 + 1e-30)).max()))
        inside = fixed + f32 <= 1e-3 * np.maximum(1, np.abs(want))
        assert np.all(err[inside] <= 1e-3 * np.maximum(1, np.abs(want[inside]))), name
        if name == "only the outlier's weight":  # the outliers are exact in 24 bits: nothing is lost at all beyond float32's sums
            assert np.all(err <= f32 + 1e-30), float((err / (f32 + 1e-30)).max())
        if name == "outlier's weight zero":
            # what a float32 product keeps and this one loses: the neighbours' low bits, at most the bound above,
            # which here is about 1e-1 of the result (the neighbours are 1e-6 of their block's scale)
            print(f"[outliers m={m}] worst error {err.max():.3e}, bound {float((fixed + f32).max()):.3e}, largest |want| {np.abs(want).max():.3e}")
        # "q4_0.path" = 1, the float32 kernel, does not keep the reference's exactness on such a block either: it takes the
        # offset out as sum n x - 8 sum x, two sums that hold the outlier and cancel. It is held to that formulation's own
        # bound, float32 rounding of the terms |x| (n + 8) d, which is where it lands (nothing larger goes unnoticed).
        try:
            capi.check(gpu.lib().mi355x_tune(b"q4_0.path", 1))
            gpu.say(f"q4_0 float32 kernel on the same case, m={m}: {name}")
            got32 = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
        finally:
            capi.check(gpu.lib().mi355x_tune(b"q4_0.path", 0))
        d = np.abs(O.f16_to_f32(blocks[:, :, :2].copy().view(np.uint16).reshape(n, nb)).astype(np.float64))  # [n, nb]
        offset_terms = 8.0 * np.einsum("mb,nb->mn", np.abs(x.reshape(m, nb, 32)).astype(np.float64).sum(2), d)
        f32_offset = f32 + 2e-6 * 2 * offset_terms
        err32 = np.abs(got32.astype(np.float64) - want)
        assert np.all(err32 <= f32_offset + 1e-30), (name, float((err32 / (f32_offset + 1e-30)).max()))
        if name != "outlier's weight zero":
            assert np.all(err32 <= np.maximum(1e-3 * np.maximum(1, np.abs(want)), f32)), (name, float(err32.max()))


def test_q4_0_gemv_without_lds_staging():
    rng = np.random.default_rng(6)
    n, k = 64, 4096
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    try:
        capi.check(l.mi355x_tune(b"q4_0.no_lds", 1))
        capi.check(l.mi355x_tune(b"q4_0.path", 1))
        gpu.say("q4_0 gemv no-lds path")
        check_close(gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k), want, TOL)
    finally:
        capi.check(l.mi355x_tune(b"q4_0.no_lds", 0))
        capi.check(l.mi355x_tune(b"q4_0.path", 0))


@pytest.mark.parametrize("rows,cols,waves", [(1, 1, 1), (2, 1, 4), (4, 2, 8), (7, 2, 8), (8, 2, 2), (4, 4, 4), (2, 7, 8), (1, 7, 1), (16, 1, 2)])
def test_q4_0_gemv_every_launch_shape(rows, cols, waves):
    rng = np.random.default_rng(7)
    n, k = 203, 4096 + 32 * 5
    raw = bench_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    l = gpu.lib()
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(O.Q4_0, raw, x, n, k)
    try:
        for key, v in ((b"q4_0.path", 1), (b"q4_0.rows", rows), (b"q4_0.cols", cols), (b"q4_0.waves", waves)):
            capi.check(l.mi355x_tune(key, v))
        gpu.say(f"q4_0 gemv plan R={rows} C={cols} waves={waves}")
        check_close(gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k), want, TOL)
    finally:
        for key in (b"q4_0.path", b"q4_0.rows", b"q4_0.cols", b"q4_0.waves"):
            capi.check(l.mi355x_tune(key, 0))


def test_q4_0_gemv_linearity_at_full_size():
    """Size-independent property at the benchmark's shape: the product is
    linear in x, and a one-hot x picks a column of the dequantized W."""
    rng = np.random.default_rng(8)
    n, k = 14336, 4096
    raw = bench_blocks(rng, O.Q4_0, n * k)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    a = rng.normal(size=k).astype(np.float32); b = rng.normal(size=k).astype(np.float32)
    gpu.say("q4_0 gemv linearity 14336x4096")
    ya, yb, yab = (gpu.qgemv(O.Q4_0, ptr, gpu.dev(v), n, k) for v in (a, b, a + b))
    assert np.abs(yab - (ya + yb)).max() <= 1e-4 * max(1, np.abs(yab).max())
    e = np.zeros(k, np.float32); e[1234] = 1
    col = gpu.qgemv(O.Q4_0, ptr, gpu.dev(e), n, k)
    wcol = O.dequantize(O.Q4_0, raw).reshape(n, k)[:, 1234]
    assert np.abs(col - wcol).max() <= 1e-6 * np.abs(wcol).max()  # a few float32 roundings of the scales
    l = gpu.lib()
    try:  # the float32 kernel multiplies by exactly 1: the column itself
        capi.check(l.mi355x_tune(b"q4_0.path", 1))
        assert bits_equal(gpu.qgemv(O.Q4_0, ptr, gpu.dev(e), n, k), wcol)
    finally:
        capi.check(l.mi355x_tune(b"q4_0.path", 0))


@pytest.mark.parametrize("m,n,k", [(2, 100, 4096), (5, 257, 1280), (8, 4096, 4096), (11, 64, 14336), (37, 130, 256)])
def test_q4_0_gemv_of_several_rows_reads_w_once_and_gives_each_row_its_own_bits(m, n, k):
    """The batch kernel multiplies a workgroup's rows of W with up to eight rows of x (as many as fit the
    LDS); every row of x meets the same lanes and reductions as alone, so the results equal the one-row
    kernel's bit for bit, whatever M leaves for the last group. (The library picks it for long rows of x.)"""
    l = gpu.lib()
    rng = np.random.default_rng(m * n + k)
    raw = random_blocks(rng, O.Q4_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    gpu.say(f"q4_0 gemv batch M={m} N={n} K={k}")
    try:
        capi.check(l.mi355x_tune(b"q4_0.batch_off", 2))  # the batch kernel whatever the shape
        got = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
        capi.check(l.mi355x_tune(b"q4_0.batch_off", 1))  # the one-row kernel
        rows = gpu.qgemv(O.Q4_0, ptr, gpu.dev(x), n, k)
    finally:
        capi.check(l.mi355x_tune(b"q4_0.batch_off", 0))
    assert np.array_equal(got, rows)
    # random scales span binary16's range: the bound goes with the size of the terms, not of the result
    mag = np.abs(x).astype(np.float64) @ np.abs(O.dequantize(O.Q4_0, raw).reshape(n, k)).astype(np.float64).T
    assert np.all(np.abs(got - O.qmatmul(O.Q4_0, raw, x, n, k)) <= 2e-6 * mag + 1e-30)


def test_q4_0_fused_products():
    """The fused products of a decoding step against the oracle's separate
    ones: residual add, three matrices in one launch, SwiGLU of gate and up."""
    rng = np.random.default_rng(31)
    l = gpu.lib()
    k, m = 4096, 3
    x = rng.normal(size=(m, k)).astype(np.float32)
    xd = gpu.dev(x)
    act = torch.zeros((m, l.mi355x_act_bytes(capi.Q4_0, k)), dtype=torch.uint8, device="cuda:0")
    capi.check(l.mi355x_convert_act(capi.Q4_0, xd.data_ptr(), m, k, k, act.data_ptr(), gpu.stream()))
    ns = (4096, 1024, 1022)
    raws = [bench_blocks(rng, O.Q4_0, n * k) for n in ns]
    bufs = [gpu.dev_bytes_at(r, 0) for r in raws]
    wants = [O.qmatmul(O.Q4_0, r, x, n, k) for r, n in zip(raws, ns)]
    gpu.say("q4_0 multi: q, k, v in one launch")
    y = torch.full((m, sum(ns)), float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(l.mi355x_qgemv_act_multi(capi.Q4_0, bufs[0][1], bufs[1][1], bufs[2][1], ns[0], ns[1], ns[2], act.data_ptr(), y.data_ptr(), m, k, gpu.stream()))
    gpu.sync()
    check_close(y.cpu().numpy(), np.concatenate(wants, axis=1), TOL)
    y2 = torch.full((m, ns[0] + ns[1]), float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(l.mi355x_qgemv_act_multi(capi.Q4_0, bufs[0][1], bufs[1][1], None, ns[0], ns[1], 0, act.data_ptr(), y2.data_ptr(), m, k, gpu.stream()))
    gpu.sync()
    assert bits_equal(y2.cpu().numpy(), y.cpu().numpy()[:, :ns[0] + ns[1]])
    gpu.say("q4_0 add: product plus residual, in place")
    resid = rng.normal(size=(m, ns[0])).astype(np.float32)
    rd = gpu.dev(resid)
    capi.check(l.mi355x_qgemv_act_add(capi.Q4_0, bufs[0][1], act.data_ptr(), rd.data_ptr(), rd.data_ptr(), m, ns[0], k, gpu.stream()))
    gpu.sync()
    check_close(rd.cpu().numpy(), wants[0] + resid, TOL)
    gpu.say("q4_0 swiglu: gate and up, 14336 and a ragged 1023")
    for n in (14336, 1023):
        g_raw, u_raw = bench_blocks(rng, O.Q4_0, n * k), bench_blocks(rng, O.Q4_0, n * k)
        gb, ub = gpu.dev_bytes_at(g_raw, 0), gpu.dev_bytes_at(u_raw, 0)
        out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
        capi.check(l.mi355x_qgemv_act_swiglu(capi.Q4_0, gb[1], ub[1], act.data_ptr(), out.data_ptr(), m, n, k, gpu.stream()))
        gpu.sync()
        want = O.silu_mul(O.qmatmul(O.Q4_0, g_raw, x, n, k), O.qmatmul(O.Q4_0, u_raw, x, n, k))
        got = out.cpu().numpy()
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    assert l.mi355x_qgemv_act_multi(capi.Q8_0, bufs[0][1], None, None, 4, 0, 0, act.data_ptr(), y.data_ptr(), m, k, gpu.stream()) == capi.ERR_DTYPE


# ---- Q8_0: the int8-activation product of the CPU backend -------------------

def _unpack_q8_act(raw, k):
    """The device's converted row (q[2][nbp] of 16 bytes, then float scales) as
    quantizeRow's blocks: f32 d | int8 q[32]."""
    nb = k // 32; nbp = nb | 1
    q = raw[:2 * nbp * 16].reshape(2, nbp, 16)
    d = raw[2 * nbp * 16:2 * nbp * 16 + 4 * nb].view(np.float32)
    out = np.zeros((nb, 36), np.uint8)
    out[:, :4] = d.view(np.uint8).reshape(nb, 4)
    out[:, 4:20] = q[0, :nb]
    out[:, 20:36] = q[1, :nb]
    return out.reshape(-1)


def test_q8_activation_rounding_is_bit_exact():
    """quantizeRow on the device against the oracle's, byte for byte: normal
    values, ties under an amax of 127, tiny and huge magnitudes, zeros, an
    infinity and a NaN (backend/cpu/quant_test.go:523-558)."""
    rng = np.random.default_rng(17)
    bs, nblk = 32, 64
    x = np.empty(nblk * bs, np.float32)
    for b in range(nblk):
        v = x[b * bs:(b + 1) * bs]
        if b % 4 == 0:
            v[:] = rng.random(bs, dtype=np.float32) * 2 - 1
        elif b % 4 == 1:
            v[:] = (rng.integers(0, 254, bs) - 127) / 2
            v[0] = 127
        elif b % 4 == 2:
            v[:] = rng.normal(size=bs) * 1e-30
        else:
            v[:] = rng.normal(size=bs) * 1e30
    x[7 * bs:8 * bs] = 0
    x[5 * bs + 3] = np.inf
    x[9 * bs] = np.nan
    gpu.say("q8 convert_act vs quantize_row")
    got = _unpack_q8_act(gpu.convert_act(O.Q8_0, gpu.dev(x), x.size)[0], x.size).reshape(nblk, 36)
    want = O.quantize_row(x, 32, False).reshape(nblk, 36)
    for b in range(nblk):
        gd, wd = got[b, :4].view(np.float32)[0], want[b, :4].view(np.float32)[0]
        assert (np.isnan(gd) and np.isnan(wd)) or got[b, :4].tobytes() == want[b, :4].tobytes(), b
        assert np.array_equal(got[b, 4:], want[b, 4:]), b


def test_q8_0_gemv_baseline_config():
    """W 4096 x 4096 int8 uniform in [-127, 127], one binary16 scale |N(0, 0.02)|
    per block, x ~ N(0, 1), seed 0, against the CPU path (int8 activations)."""
    rng = np.random.default_rng(0)
    n = k = 4096
    raw = bench_blocks(rng, O.Q8_0, n * k)
    x = rng.normal(size=(1, k)).astype(np.float32)
    gpu.say("q8_0 gemv 4096x4096")
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q8_0, raw, x, n, k)
    check_close(got, want, TOL, "q8_0 4096x4096")
    assert rel_l2(got, want) < 1e-6  # only the order of the blocks' additions differs
    assert np.array_equal(got, gpu.qgemv_act(O.Q8_0, ptr, gpu.dev(x), n, k))  # the two-step entry is the same product


@pytest.mark.parametrize("n,k,offset", [(9, 1280, 0), (9, 1280, 2), (7, 32 * 5, 0), (1, 32, 0), (300, 4096 + 96, 0), (64, 14336, 0), (5, 32768, 2)])
def test_q8_0_gemv_shapes(n, k, offset):
    """Ragged shapes, an odd number of blocks, and a W that is only 2-byte
    aligned (the single-block path)."""
    rng = np.random.default_rng(n * 7 + k + offset)
    raw = random_blocks(rng, O.Q8_0, n * k)
    for m, shape in ((1, (k,)), (6, (2, 3, k))):
        x = rng.normal(size=shape).astype(np.float32)
        gpu.say(f"q8_0 gemv N={n} K={k} offset={offset} x{shape}")
        buf, ptr = gpu.dev_bytes_at(raw, offset)
        got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
        want = O.qmatmul(O.Q8_0, raw, x, n, k)
        # Same integers, same per-block roundings; only the order of the blocks'
        # float32 additions differs, so the error scales with sum |w||x|.
        mag = np.abs(x.reshape(-1, k)).astype(np.float64) @ np.abs(O.dequantize(O.Q8_0, raw).reshape(n, k)).astype(np.float64).T
        assert np.all(np.abs(got.reshape(-1, n) - want.reshape(-1, n)) <= 2e-6 * mag + 1e-30), f"q8_0 {n}x{k}+{offset}"


def test_q8_0_gemv_golden_and_exact_rows(golden_dir):
    c = golden_cases(os.path.join(golden_dir, "quant.mim"))["q8_0_matmul"]
    x, raw = c["in"][0].data, c["in"][1].data.reshape(-1)
    n, k = c["in"][1].shape[0], c["in"][1].shape[1] // 34 * 32
    gpu.say("q8_0 golden matmul")
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
    assert np.all(np.abs(got - c["out"].data) <= 1e-5 + 1e-5 * np.abs(c["out"].data))  # tensor/quant_test.go:321
    # kerneltest/quant.go:113-139: rows 1..9 of a 10-row table, exact activations, Tol 1e-4 against the CPU
    rng = np.random.default_rng(13)
    n, k = 9, 1280
    raw = random_blocks(rng, O.Q8_0, (n + 1) * k)
    row = k // 32 * 34
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    for shape in ((k,), (1, k), (2, 3, k)):
        x = exact_rows(rng, O.Q8_0, int(np.prod(shape[:-1])), k).reshape(shape)
        got = gpu.qgemv(O.Q8_0, ptr + row, gpu.dev(x), n, k)
        check_close(got, O.qmatmul(O.Q8_0, raw[row:], x, n, k), 1e-4)


def test_q8_0_gemv_nan_and_inf_blocks():
    """A block of x that holds a NaN or an infinity makes every product NaN
    (backend/cpu/qmatmul.go:205-207)."""
    rng = np.random.default_rng(3)
    n, k = 16, 256
    raw = bench_blocks(rng, O.Q8_0, n * k)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    x = rng.normal(size=k).astype(np.float32)
    for bad in (np.inf, -np.inf, np.nan):
        x2 = x.copy(); x2[77] = bad
        got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x2), n, k)
        want = O.qmatmul(O.Q8_0, raw, x2, n, k)
        assert np.isnan(got).all() and np.isnan(want).all()


def test_q8_0_lm_head_shape_sampled():
    """The output projection of an 8B model, 128256 x 4096 (558 MB), against
    the oracle on every row."""
    rng = np.random.default_rng(11)
    n, k = 128256, 4096
    raw = bench_blocks(rng, O.Q8_0, n * k)
    x = rng.normal(size=k).astype(np.float32)
    gpu.say("q8_0 gemv lm_head 128256x4096")
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q8_0, raw, x, n, k, simd=True)
    check_close(got, want, 1e-4, "lm_head")
    assert O.argmax(got) == O.argmax(want)


@pytest.mark.parametrize("m,n,k", [(11, 203, 4096 + 64), (2, 70, 128), (16, 9, 1280), (8, 7000, 4096)])
def test_q8_0_rows_of_x_share_one_pass_over_w(m, n, k):
    """Several rows of x against Q8_0 weights read once: every sum is formed as the one-row kernel forms it,
    so the results are its bits, row by row."""
    rng = np.random.default_rng(m + n + k)
    raw = random_blocks(rng, O.Q8_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    gpu.say(f"q8_0 rows kernel M={m} N={n} K={k}")
    got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
    want = O.qmatmul(O.Q8_0, raw, x, n, k)
    w = O.dequantize(O.Q8_0, raw).reshape(n, k).astype(np.float64)
    mag = np.abs(x.astype(np.float64)) @ np.abs(w).T  # what the rounding errors of the float32 sums scale with
    assert np.all(np.abs(got - want) <= 2e-6 * mag + 1e-30)
    xd = gpu.dev(x)
    one = np.stack([gpu.qgemv(O.Q8_0, ptr, xd[i], n, k) for i in range(m)])
    assert bits_equal(got, one)


@pytest.mark.parametrize("m,n,k", [(8, 203, 4096), (2, 32, 256), (5, 1000, 1280), (8, 33, 14336), (3, 1, 512)])
def test_q8_0_rows_on_the_matrix_cores(m, n, k):
    """Two to eight rows of x against Q8_0 weights on the int8 matrix cores (the head of a batch's decoding
    step; forced here for small matrices too): the CPU's integer lane sums, float32 sums of a row's
    blocks in another order, so close to the oracle and to the one-row kernel, not their bits."""
    l = gpu.lib()
    rng = np.random.default_rng(3 * m + n + k)
    raw = random_blocks(rng, O.Q8_0, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[0, :32] = 0
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    try:
        capi.check(l.mi355x_tune(b"q8_0.mfma", 1))
        gpu.say(f"q8_0 matrix-core rows kernel M={m} N={n} K={k}")
        got = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
        capi.check(l.mi355x_tune(b"q8_0.mfma", 2))
        rows = gpu.qgemv(O.Q8_0, ptr, gpu.dev(x), n, k)
    finally:
        capi.check(l.mi355x_tune(b"q8_0.mfma", 0))
    want = O.qmatmul(O.Q8_0, raw, x, n, k)
    w = O.dequantize(O.Q8_0, raw).reshape(n, k).astype(np.float64)
    mag = np.abs(x.astype(np.float64)) @ np.abs(w).T
    assert np.all(np.abs(got - want) <= 2e-6 * mag + 1e-30)
    assert np.all(np.abs(got - rows) <= 2e-6 * mag + 1e-30)


# ---- Q4_K / Q6_K -------------------------------------------------------------

@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_kquant_activation_rounding_is_bit_exact(dt):
    rng = np.random.default_rng(21)
    k = 256 * 6
    x = rng.normal(size=k).astype(np.float32)
    x[256:512] = 0
    x[512:768] = (rng.integers(0, 254, 256) - 127) / 2; x[512] = 127  # ties
    x[1300] = np.nan
    gpu.say(f"kquant convert_act dt={dt}")
    raw = gpu.convert_act(dt, gpu.dev(x), k)[0]
    nsb = k // 256
    want = O.quantize_row(x, 256, True).reshape(nsb, 292)
    assert np.array_equal(raw[:nsb * 256].reshape(nsb, 256), want[:, 4:260])
    assert np.array_equal(raw[nsb * 256:nsb * 288].reshape(nsb, 32), want[:, 260:292])
    gd, wd = raw[nsb * 288:nsb * 292].view(np.float32), want[:, :4].copy().view(np.float32).reshape(-1)
    assert np.array_equal(np.isnan(gd), np.isnan(wd)) and np.array_equal(gd[~np.isnan(gd)], wd[~np.isnan(wd)])


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("n,k,offset", [(9, 1280, 0), (5, 256, 2), (33, 256 * 17, 0), (300, 4096, 0)])
def test_kquant_gemv_matches_oracle(dt, n, k, offset):
    rng = np.random.default_rng(n + k + dt)
    raw = random_blocks(rng, dt, n * k)
    for shape in ((k,), (2, 3, k)):
        x = rng.normal(size=shape).astype(np.float32)
        gpu.say(f"kquant gemv dt={dt} N={n} K={k} offset={offset} x{shape}")
        buf, ptr = gpu.dev_bytes_at(raw, offset)
        got = gpu.qgemv(dt, ptr, gpu.dev(x), n, k)
        want = O.qmatmul(dt, raw, x, n, k)
        assert bits_equal(got, want)  # integer sums, and the float32 operations of qdotQ4KGo / qdotQ6KGo in their order
        assert np.array_equal(got, gpu.qgemv_act(dt, ptr, gpu.dev(x), n, k))


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_kquant_gemv_every_launch_shape(dt):
    """The kernels that stage x in LDS, at every count of rows per wavefront, and the ones that
    read it from global memory all give the CPU's bits."""
    l = gpu.lib()
    rng = np.random.default_rng(77 + dt)
    for n, k in ((37, 256 * 56), (130, 256 * 9), (16, 256)):
        raw = random_blocks(rng, dt, n * k)
        x = rng.normal(size=(3, k)).astype(np.float32)
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        want = O.qmatmul(dt, raw, x, n, k)
        results = []
        try:
            for key, v in ((b"kquant.rows", 1), (b"kquant.rows", 2), (b"kquant.rows", 4), (b"kquant.path", 1)):
                gpu.say(f"kquant gemv dt={dt} N={n} K={k} {key.decode()}={v}")
                capi.check(l.mi355x_tune(key, v))
                results.append(gpu.qgemv(dt, ptr, gpu.dev(x), n, k))
        finally:
            capi.check(l.mi355x_tune(b"kquant.rows", 0))
            capi.check(l.mi355x_tune(b"kquant.path", 0))
        for r in results:
            assert bits_equal(r, want)


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_kquant_gemv_single_row_rounds_x_in_the_product(dt):
    """One row of x against a small matrix is one launch whose workgroups round x themselves: the
    same bits as the two-launch form (taken when x is not 16-byte aligned) and as the CPU, with
    zero super-blocks, ties and a NaN in x."""
    rng = np.random.default_rng(5 + dt)
    for n, k in ((37, 256 * 56), (515, 256 * 16), (2, 256)):
        raw = random_blocks(rng, dt, n * k)
        x = rng.normal(size=k).astype(np.float32)
        x[:256] = 0
        x[k - 256:] = (rng.integers(0, 254, 256) - 127) / 2; x[k - 1] = 127
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        for poison in (False, True):
            if poison: x[k // 2] = np.nan
            want = O.qmatmul(dt, raw, x, n, k)
            xd = gpu.dev(np.concatenate([np.zeros(1, np.float32), x]))
            gpu.say(f"kquant single row dt={dt} N={n} K={k} nan={poison}")
            one = gpu.qgemv(dt, ptr, gpu.dev(x), n, k)
            two = gpu.qgemv(dt, ptr, xd[1:], n, k)
            assert bits_equal(one, want) and bits_equal(two, want)


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("m,n,k", [(2, 33, 256), (5, 100, 512), (8, 203, 4096), (11, 64, 256 * 9), (20, 31, 256 * 56), (40, 130, 1024),
                                   (3, 40, 256 * 37), (4, 33, 256 * 70), (9, 300, 256 * 33)])
def test_kquant_rows_of_x_share_one_pass_over_w_on_the_matrix_cores(dt, m, n, k):
    """Rows of x, eight at a time, against Q4_K or Q6_K weights read once on the int8 matrix cores (the decoding
    step of a batch; forced here beyond the rows it is chosen for): the CPU's integer sums, and its float32
    operations in its order, so the oracle's bits and those of the one-row kernels. x holds a zero
    super-block, ties and, in one row, a NaN. Rows of up to 32 super-blocks keep their partial sums in
    LDS, longer ones (to 64) in registers, handed from wavefront to wavefront; beyond that LDS again, or
    another kernel where it has no room."""
    l = gpu.lib()
    rng = np.random.default_rng(dt + 7 * m + n + k)
    raw = random_blocks(rng, dt, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[0, :256] = 0
    x[1, k - 256:] = (rng.integers(0, 254, 256) - 127) / 2; x[1, k - 1] = 127
    if m > 2: x[m - 1, k // 2] = np.nan
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(dt, raw, x, n, k)
    try:
        capi.check(l.mi355x_tune(b"kquant.mfma_rows", 2))
        gpu.say(f"kquant matrix-core rows kernel dt={dt} M={m} N={n} K={k}")
        got = gpu.qgemv(dt, ptr, gpu.dev(x), n, k)
        got_act = gpu.qgemv_act(dt, ptr, gpu.dev(x), n, k)
        capi.check(l.mi355x_tune(b"kquant.mfma_rows", 1))
        rows = gpu.qgemv(dt, ptr, gpu.dev(x), n, k)
    finally:
        capi.check(l.mi355x_tune(b"kquant.mfma_rows", 0))
    assert bits_equal(got, want) and bits_equal(got_act, want) and bits_equal(rows, want)


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_kquant_rows_kernel_at_the_largest_integer_sums(dt):
    """Every quant and scale at its largest magnitude with x at +-127 per super-block (backend/cpu/quant_test.go:164-204), through the
    kernel that reads W once per eight rows of x: its 24-bit multiplies and int32 sums hold what the CPU's int32 arithmetic holds."""
    l = gpu.lib()
    m, n, k = 11, 64, 256 * 40
    bb = O.block_bytes(dt)
    raw = np.zeros(n * k // 256 * bb, np.uint8).reshape(-1, bb)
    if dt == O.Q4_K:
        raw[:, 4:16] = 0xFF          # every scale and min 63
        raw[:, 16:144] = 0xFF        # every quant 15
        raw[:, 0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
        raw[:, 2:4] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
        raw[1::2, 16:144] = 0        # and every quant 0
    else:
        raw[:, 0:192] = 0xFF         # every quant 63 (31 after the offset)
        raw[1::2, 0:192] = 0         # every quant 0 (-32)
        raw[:, 192:208] = 0x80       # every scale -128
        raw[2::3, 192:208] = 0x7F    # or 127
        raw[:, 208:210] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    raw = raw.reshape(-1)
    x = np.where(np.arange(m * k).reshape(m, k) % 3 == 0, -127.0, 127.0).astype(np.float32)
    x[1::2] = 127.0
    buf, ptr = gpu.dev_bytes_at(raw, 0)
    want = O.qmatmul(dt, raw, x, n, k)
    try:
        capi.check(l.mi355x_tune(b"kquant.mfma_rows", 2))
        for key, v in ((b"kquant.mfma_rows_waves", 0), (b"kquant.mfma_rows_waves", 1)):  # partial sums in registers (K = 10240), then in LDS
            capi.check(l.mi355x_tune(key, v))
            gpu.say(f"kquant rows kernel extremes dt={dt} {key.decode()}={v}")
            assert bits_equal(gpu.qgemv(dt, ptr, gpu.dev(x), n, k), want)
    finally:
        capi.check(l.mi355x_tune(b"kquant.mfma_rows", 0))
        capi.check(l.mi355x_tune(b"kquant.mfma_rows_waves", 0))


def test_kquant_gemv_golden_and_exact_rows(golden_dir):
    cases = golden_cases(os.path.join(golden_dir, "quant.mim"))
    for kind, dt in (("q4_K", O.Q4_K), ("q6_K", O.Q6_K)):
        c = cases[f"{kind}_matmul"]
        x, raw = c["in"][0].data, c["in"][1].data.reshape(-1)
        n, k = c["in"][1].shape[0], c["in"][1].shape[1] // O.block_bytes(dt) * 256
        gpu.say(f"{kind} golden matmul")
        buf, ptr = gpu.dev_bytes_at(raw, 0)
        got = gpu.qgemv(dt, ptr, gpu.dev(x), n, k)
        assert np.all(np.abs(got - c["out"].data) <= 1e-5 + 1e-5 * np.abs(c["out"].data))
        rng = np.random.default_rng(13)
        n2, k2 = 9, 1280
        raw2 = random_blocks(rng, dt, (n2 + 1) * k2)
        row = k2 // 256 * O.block_bytes(dt)
        buf2, ptr2 = gpu.dev_bytes_at(raw2, 0)
        for shape in ((k2,), (1, k2), (2, 3, k2)):
            xx = exact_rows(rng, dt, int(np.prod(shape[:-1])), k2).reshape(shape)
            check_close(gpu.qgemv(dt, ptr2 + row, gpu.dev(xx), n2, k2), O.qmatmul(dt, raw2[row:], xx, n2, k2), 1e-4)


def test_qgemv_argument_errors():
    l = gpu.lib()
    x = torch.zeros(64, device="cuda:0"); y = torch.zeros(4, device="cuda:0"); w = torch.zeros(1024, dtype=torch.uint8, device="cuda:0")
    assert l.mi355x_qgemv(capi.F32, w.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 4, 64, 64, 0) == capi.ERR_DTYPE
    assert l.mi355x_qgemv(capi.Q4_0, w.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 4, 48, 48, 0) == capi.ERR_INTERNAL  # K not whole blocks (qmatmul.go:329-332)
    assert "blocks of 32" in capi.last_error()
    assert l.mi355x_qgemv(capi.Q4_0, w.data_ptr(), x.data_ptr(), y.data_ptr(), 0, 4, 64, 64, 0) == 0  # empty output
    y.fill_(7)
    assert l.mi355x_qgemv(capi.Q4_0, w.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 4, 0, 0, 0) == 0    # K = 0: zeros
    gpu.sync()
    assert not y.cpu().numpy().any()
