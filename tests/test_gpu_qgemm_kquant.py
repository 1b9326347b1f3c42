"""The Q4_K / Q6_K product for many rows of x on the matrix cores, against the oracle's
qmatmul (backend/cpu/qmatmul.go:148-200, 310-405). It runs every output through the CPU's float32
operations in the CPU's order on exact integer sums, so the comparison is for equal bits, the
property the reference claims for its own tiles (backend/cpu/qtile.go:51-54)."""
import numpy as np
import pytest

import oracle as O
from mimir_amd import capi
from tests import gpu
from tests.helpers import bits_equal, exact_rows, random_blocks

pytestmark = pytest.mark.gpu


@pytest.fixture
def matrix_cores():
    """The library picks the faster kernel by shape; these tests are about one of them."""
    l = gpu.lib()
    capi.check(l.mi355x_tune(b"kquant.path", 3))
    yield
    capi.check(l.mi355x_tune(b"kquant.path", 0))


def product(dt, raw, x, n, k, offset=0):
    buf, ptr = gpu.dev_bytes_at(raw, offset)
    return gpu.qgemv(dt, ptr, gpu.dev(x), n, k)


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("m,n,k", [(8, 5, 256), (33, 64, 1280), (130, 100, 512), (256, 64, 256), (300, 200, 768),
                                   (129, 65, 256 * 17), (512, 2048, 1024)])
def test_matches_the_cpu_bit_for_bit(dt, m, n, k, matrix_cores):
    rng = np.random.default_rng(m + n + k + dt)
    raw = random_blocks(rng, dt, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[m // 2, 256 * (k // 512):256 * (k // 512) + 256] = 0  # a super-block of zeros: scale 0
    gpu.say(f"kquant gemm dt={dt} M={m} N={n} K={k}")
    got = product(dt, raw, x, n, k)
    want = O.qmatmul(dt, raw, x, n, k)
    assert bits_equal(got, want)


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_extreme_quants_and_scales(dt, matrix_cores):
    """Every quant and scale at its largest magnitude with x at +-127 per super-block: the largest integer sums
    the planes and the sums of x can reach (backend/cpu/quant_test.go:164-204)."""
    m, n, k = 40, 64, 512
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
    gpu.say(f"kquant gemm extremes dt={dt}")
    assert bits_equal(product(dt, raw, x, n, k), O.qmatmul(dt, raw, x, n, k))


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_rows_with_nan_and_inf(dt, matrix_cores):
    m, n, k = 16, 70, 768
    rng = np.random.default_rng(5)
    raw = random_blocks(rng, dt, n * k)
    x = rng.normal(size=(m, k)).astype(np.float32)
    x[3, 300] = np.nan
    x[9, 10] = np.inf
    gpu.say(f"kquant gemm nan dt={dt}")
    got, want = product(dt, raw, x, n, k), O.qmatmul(dt, raw, x, n, k)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(got[3]).all() and np.isnan(got[9]).all()
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))


def test_q6_k_from_a_2_byte_aligned_start_and_q4_k_from_a_misaligned_one(matrix_cores):
    m, n, k = 64, 96, 1024
    rng = np.random.default_rng(6)
    x = rng.normal(size=(m, k)).astype(np.float32)
    raw = random_blocks(rng, O.Q6_K, n * k)
    gpu.say("kquant gemm q6_K offset 2")
    assert bits_equal(product(O.Q6_K, raw, x, n, k, offset=2), O.qmatmul(O.Q6_K, raw, x, n, k))
    # Q4_K away from 16-byte alignment goes to the row-by-row kernels, which give the same bits.
    raw = random_blocks(rng, O.Q4_K, n * k)
    gpu.say("kquant gemm q4_K offset 2")
    assert bits_equal(product(O.Q4_K, raw, x, n, k, offset=2), O.qmatmul(O.Q4_K, raw, x, n, k))


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
def test_few_rows_on_the_matrix_cores_and_many_on_the_row_kernels(dt):
    """Whichever kernel the shape would not pick by itself still gives the CPU's bits."""
    l = gpu.lib()
    n, k = 130, 256 * 9
    rng = np.random.default_rng(8)
    raw = random_blocks(rng, dt, n * k)
    x = exact_rows(rng, dt, 3, k)
    want = O.qmatmul(dt, raw, x, n, k)
    try:
        gpu.say(f"kquant gemm dt={dt} forced for 3 rows")
        capi.check(l.mi355x_tune(b"kquant.path", 3))
        assert bits_equal(product(dt, raw, x, n, k), want)
        gpu.say(f"kquant gemv dt={dt} forced for 40 rows")
        capi.check(l.mi355x_tune(b"kquant.path", 2))
        x2 = rng.normal(size=(40, k)).astype(np.float32)
        assert bits_equal(product(dt, raw, x2, n, k), O.qmatmul(dt, raw, x2, n, k))
    finally:
        capi.check(l.mi355x_tune(b"kquant.path", 0))


@pytest.mark.parametrize("dt", [O.Q4_K, O.Q6_K])
@pytest.mark.parametrize("m", [512, 11])
def test_prompt_sized_products_take_the_matrix_cores_and_bf16_rounds_once(dt, m):
    """Left to itself the library sends a prompt-sized product to the matrix cores (the CPU's bits), and
    mi355x_qgemm_bf16 is the reference's sequence for a half x: cast to float32, product, one rounding
    (tensor/quant.go:45-48). Eleven rows take the kernel that reads W once per eight rows of x, from
    bfloat16 rows too."""
    import torch
    n, k = 1024, 2048
    rng = np.random.default_rng(31 + dt)
    raw = random_blocks(rng, dt, n * k)
    xb = O.f32_to_bf16(rng.normal(size=(m, k)).astype(np.float32))
    xf = O.bf16_to_f32(xb)
    want = O.qmatmul(dt, raw, xf, n, k)
    gpu.say(f"kquant gemm dt={dt} default dispatch")
    assert bits_equal(product(dt, raw, xf, n, k), want)
    l = gpu.lib()
    wbuf, wp = gpu.dev_bytes_at(raw, 0)
    xd = torch.from_numpy(xb.view(np.int16)).to("cuda:0")
    for out_dt in (capi.BF16, capi.F32):
        y = torch.zeros((m, n), dtype=torch.int16 if out_dt == capi.BF16 else torch.float32, device="cuda:0")
        gpu.say(f"qgemm_bf16 dt={dt} out={out_dt}")
        capi.check(l.mi355x_qgemm_bf16(dt, wp, xd.data_ptr(), y.data_ptr(), m, n, k, k, out_dt, gpu.stream()))
        gpu.sync()
        got = y.cpu().numpy()
        if out_dt == capi.BF16:
            assert np.array_equal(got.view(np.uint16), O.f32_to_bf16(want))
        else:
            assert bits_equal(got, want)
