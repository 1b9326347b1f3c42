"""mi355x_qgemv_noalloc, the entry point that allocates nothing, against mi355x_qgemv: the same kernels
over a fixed scratch block, so the results must be the same bits (and within the product's bound of
the oracle). Two calls in a row per case, the second with a smaller input, since the block keeps the
last call's contents. That nothing is allocated is shown twice: the device's free memory does not move
across the calls, and the calls are made under stream capture on a stream the library has never seen
(where an allocation is refused, the library's growing scratch included), then replayed from the graph."""
import numpy as np
import pytest
import torch

import oracle as O
from mimir_amd import capi
from tests import gpu, helpers

pytestmark = pytest.mark.gpu

DT = {"q4_0": (capi.Q4_0, O.Q4_0), "q8_0": (capi.Q8_0, O.Q8_0), "q4_K": (capi.Q4_K, O.Q4_K), "q6_K": (capi.Q6_K, O.Q6_K)}

# (M, N, K): twelve rows (every dtype converts them into the block: Q4_0 and Q8_0 do so from nine rows on, the
# K-quants from two), then three, then one
CASES = ((12, 384, 2048), (3, 160, 512), (1, 96, 256))


def _blocks(rng, name, odt, n, k):
    # scales as the configurations draw them for the dtypes whose float32 sums differ in order from the oracle's
    return helpers.bench_blocks(rng, odt, n * k) if name in ("q4_0", "q8_0") else helpers.random_blocks(rng, odt, n * k)


def _both(dt, w, x, n, k):
    l = gpu.lib()
    m = x.shape[0]
    ys = []
    for fn in (l.mi355x_qgemv, l.mi355x_qgemv_noalloc):
        y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
        capi.check(fn(dt, w.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, k, gpu.stream()))
        gpu.sync()
        ys.append(y.cpu().numpy())
    return ys


@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4_K", "q6_K"])
def test_noalloc_equals_qgemv_twice_second_smaller(name):
    dt, odt = DT[name]
    rng = np.random.default_rng(7)
    # the first call fills more of the block than the second reads
    for (m, n, k) in CASES:
        raw = _blocks(rng, name, odt, n, k)
        x = rng.normal(size=(m, k)).astype(np.float32)
        gpu.say(f"qgemv_noalloc {name} M={m} N={n} K={k}")
        w, xd = gpu.dev(raw), gpu.dev(x)
        got, got_fixed = _both(dt, w, xd, n, k)
        assert np.array_equal(got.view(np.uint32), got_fixed.view(np.uint32))
        want = O.qmatmul(odt, raw, x, n, k)
        tol = 1e-3 if name == "q4_0" else 1e-4 if name == "q8_0" else 1e-5  # the K-quant kernels give the oracle's bits
        assert np.all(np.abs(got_fixed - want) <= tol * np.maximum(1, np.abs(want)))


@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4_K", "q6_K"])
def test_noalloc_allocates_nothing(name):
    """Free device memory is the same before and after; and the calls succeed under stream capture on a fresh
    stream, where hipMalloc is refused (so a route back to the library's growing scratch would fail there), the
    graph's replays giving the bits of the eager mi355x_qgemv."""
    dt, odt = DT[name]
    l = gpu.lib()
    rng = np.random.default_rng(11)
    prepared = []
    for (m, n, k) in CASES:
        raw = _blocks(rng, name, odt, n, k)
        x = rng.normal(size=(m, k)).astype(np.float32)
        w, xd = gpu.dev(raw), gpu.dev(x)
        want = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
        capi.check(l.mi355x_qgemv(dt, w.data_ptr(), xd.data_ptr(), want.data_ptr(), m, n, k, k, gpu.stream()))  # also loads the kernels
        y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
        prepared.append((m, n, k, w, xd, y, want))
    gpu.sync()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for (m, n, k, w, xd, y, want) in prepared:
        gpu.say(f"qgemv_noalloc {name} M={m} N={n} K={k}: free memory")
        capi.check(l.mi355x_qgemv_noalloc(dt, w.data_ptr(), xd.data_ptr(), y.data_ptr(), m, n, k, k, gpu.stream()))
    gpu.sync()
    assert torch.cuda.mem_get_info()[0] == free_before
    for (_, _, _, _, _, y, want) in prepared:
        assert torch.equal(y.view(torch.int32), want.view(torch.int32))
        y.fill_(float("nan"))
    fresh = torch.cuda.Stream()  # the library holds no scratch for it
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    gpu.say(f"qgemv_noalloc {name}: under stream capture")
    with torch.cuda.stream(fresh):
        with torch.cuda.graph(graph, stream=fresh):
            for (m, n, k, w, xd, y, want) in prepared:
                capi.check(l.mi355x_qgemv_noalloc(dt, w.data_ptr(), xd.data_ptr(), y.data_ptr(), m, n, k, k, fresh.cuda_stream))
        for replay in range(2):
            graph.replay()
            fresh.synchronize()
            # the last case is the block's current content; every case's result was written by its own replayed launch
            for (_, _, _, _, _, y, want) in prepared:
                assert torch.equal(y.view(torch.int32), want.view(torch.int32)), replay
                y.fill_(float("nan"))
            fresh.synchronize()


def test_noalloc_rejects_what_the_block_cannot_hold():
    l = gpu.lib()
    k, n, m = 4096, 32, 300  # 300 rows of q8_0 activations: 4608 bytes each, more than 1 MiB
    w = torch.zeros(n * k // 32 * 34, dtype=torch.uint8, device="cuda:0")
    x = torch.zeros((m, k), dtype=torch.float32, device="cuda:0")
    y = torch.zeros((m, n), dtype=torch.float32, device="cuda:0")
    st = l.mi355x_qgemv_noalloc(capi.Q8_0, w.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, k, gpu.stream())
    assert st == capi.ERR_SHAPE and "fixed scratch" in capi.last_error()
    # and the growing entry point takes the same call
    capi.check(l.mi355x_qgemv(capi.Q8_0, w.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, k, gpu.stream()))
    gpu.sync()
