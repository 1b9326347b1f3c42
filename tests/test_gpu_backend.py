"""The Backend mirror against the oracle, case for case as the reference's
kernel tests build them (backend/internal/kerneltest/quant.go:82-161, run by
kerneltest.Check, kerneltest.go:77-125): dequantize through contiguous, shrunk
and transposed views into float32, bfloat16 and binary16; gather as an
embedding reads rows, and with a row out of range; products by rows 1 to 9 of a
10-row table from x of shapes [K], [1, K], [2, 3, K] and [3, K] read transposed.
Q4_0 runs the same cases. Then attention as OpAttention lays its output out,
CheckRun's refusals, buffer ownership, and a batch that becomes a graph."""
import numpy as np
import pytest

import oracle as O
from mimir_amd import capi
from mimir_amd.backend import (OP_ATTENTION, OP_CAST, OP_GATHER, OP_QMATMUL, Backend, BackendError, Batch, Kernel, View)
from tests import gpu
from tests.helpers import bench_blocks, bits_equal, check_close, exact_rows, random_blocks

pytestmark = pytest.mark.gpu

DT = {O.Q8_0: capi.Q8_0, O.Q4_K: capi.Q4_K, O.Q6_K: capi.Q6_K, O.Q4_0: capi.Q4_0}
N, K = 9, 1280  # 40 sub-blocks of 32 values a row


@pytest.fixture(scope="module")
def be():
    gpu.lib()
    b = Backend(0)
    yield b
    b.close()


def f32_buffer(be, a):
    a = np.ascontiguousarray(a, np.float32)
    buf = be.alloc(capi.F32, a.size)
    be.upload(buf, a)
    return buf


def quant_buffer(be, rng, odt, n):
    raw = random_blocks(rng, odt, n)
    buf = be.alloc(DT[odt], n)
    be.upload(buf, raw)
    return buf, raw


def out_f32(be, buf):
    be.sync()
    return be.download(buf).view(np.float32)


@pytest.mark.parametrize("odt", [O.Q8_0, O.Q4_K, O.Q6_K, O.Q4_0])
def test_dequantize_through_views(be, odt):
    rng = np.random.default_rng(13)
    w, raw = quant_buffer(be, rng, odt, (N + 1) * K)
    full = O.dequantize(odt, raw)
    assert bits_equal(be.download(w), raw)  # Download returns the uploaded bytes unchanged
    allv = View.contiguous([N + 1, K])
    views = {"contiguous": allv, "shrunk": allv.shrink([(1, N + 1), (0, K)]), "transposed": allv.permute([1, 0])}
    for name, v in views.items():
        for to in (capi.F32, capi.BF16, capi.F16):
            if to != capi.F32 and name != "contiguous":
                continue
            gpu.say(f"dequantize/{odt}/{to}/{name}")
            out = be.alloc(to, v.size())
            be.run(Kernel(OP_CAST, to, v.shape, [v]), [out], [w])
            be.sync()
            want = full[v.indices().reshape(-1)]
            got = be.download(out)
            if to == capi.F32:
                assert bits_equal(got.view(np.float32), want)
            elif to == capi.BF16:
                assert np.array_equal(got.view(np.uint16), O.f32_to_bf16(want))
            else:
                assert np.array_equal(got.view(np.uint16), O.f32_to_f16(want))
            be.free(out)


@pytest.mark.parametrize("odt", [O.Q8_0, O.Q4_K, O.Q6_K, O.Q4_0])
def test_gather_rows_and_out_of_range(be, odt):
    rng = np.random.default_rng(14)
    w, raw = quant_buffer(be, rng, odt, (N + 1) * K)
    full = O.dequantize(odt, raw).reshape(N + 1, K)
    allv = View.contiguous([N + 1, K])
    vi = View([3, K], [1, 0])  # one index a row, as Embedding.Forward expands it
    ib = be.alloc(capi.I32, 3)
    out = be.alloc(capi.F32, 3 * K)
    k = Kernel(OP_GATHER, capi.F32, [3, K], [allv, vi], axis=0)
    gpu.say(f"gather/{odt}/rows")
    be.upload(ib, np.array([2, 0, 9], np.int32))
    be.run(k, [out], [w, ib])
    assert bits_equal(out_f32(be, out), full[[2, 0, 9]].reshape(-1))
    # the same lookup through views the fast route does not take: the table read transposed, on axis 1
    tv = allv.permute([1, 0])
    vi2 = View([K, 3], [0, 1])
    out2 = be.alloc(capi.F32, 3 * K)
    be.run(Kernel(OP_GATHER, capi.F32, [K, 3], [tv, vi2], axis=1), [out2], [w, ib])
    assert bits_equal(out_f32(be, out2).reshape(K, 3), full[[2, 0, 9]].T)
    gpu.say(f"gather/{odt}/out of range")
    be.upload(ib, np.array([2, 10, 0], np.int32))
    be.run(k, [out], [w, ib])
    with pytest.raises(BackendError) as e:
        be.sync()
    assert e.value.code == capi.ERR_INDEX
    be.sync()  # reported once


@pytest.mark.parametrize("odt", [O.Q8_0, O.Q4_K, O.Q6_K, O.Q4_0])
def test_qmatmul_cases(be, odt):
    rng = np.random.default_rng(15)
    w, raw = quant_buffer(be, rng, odt, (N + 1) * K)
    rows = View.contiguous([N + 1, K]).shrink([(1, N + 1), (0, K)])
    wrows = raw.reshape(N + 1, -1)[1:].reshape(-1)
    for shape in ([K], [1, K], [2, 3, K]):
        m = int(np.prod(shape[:-1], dtype=np.int64))
        x = exact_rows(rng, odt, m, K)
        gpu.say(f"qmatmul/{odt}/{shape}")
        out = be.alloc(capi.F32, m * N)
        be.run(Kernel(OP_QMATMUL, capi.F32, shape[:-1] + [N], [View.contiguous(shape), rows]), [out], [f32_buffer(be, x), w])
        check_close(out_f32(be, out), O.qmatmul(odt, wrows, x, N, K), 1e-4, f"qmatmul {shape}")
    x = exact_rows(rng, odt, 3, K)
    gpu.say(f"qmatmul/{odt}/transposed")
    out = be.alloc(capi.F32, 3 * N)
    be.run(Kernel(OP_QMATMUL, capi.F32, [3, N], [View.contiguous([K, 3]).permute([1, 0]), rows]), [out], [f32_buffer(be, x.T.copy()), w])
    check_close(out_f32(be, out), O.qmatmul(odt, wrows, x, N, K), 1e-4, "qmatmul transposed")
    # rows of x a stride apart (a shrunk view), and an empty product
    xs = exact_rows(rng, odt, 4, 2 * K)
    out = be.alloc(capi.F32, 4 * N)
    be.run(Kernel(OP_QMATMUL, capi.F32, [4, N], [View.contiguous([4, 2 * K]).shrink([(0, 4), (K, 2 * K)]), rows]), [out], [f32_buffer(be, xs), w])
    check_close(out_f32(be, out), O.qmatmul(odt, wrows, xs[:, K:].copy(), N, K), 1e-4, "qmatmul shrunk x")
    empty = be.alloc(capi.F32, 0)
    be.run(Kernel(OP_QMATMUL, capi.F32, [0, N], [View.contiguous([0, K]), rows]), [empty], [f32_buffer(be, np.zeros(4)), w])
    be.sync()


def test_attention_output_layout(be):
    """The result [B, H, Q, D] followed by the logsumexp [B, H, Q] in one
    output, queries and keys through shrunk views, grouped heads, a causal
    offset, binary16 keys and values."""
    rng = np.random.default_rng(16)
    B, H, HK, Q, Kn, D, cap = 2, 4, 2, 3, 11, 64, 16
    q = rng.normal(size=(B, H, Q, D)).astype(np.float32)
    kf = rng.normal(size=(B, HK, cap, D)).astype(np.float32); vf = rng.normal(size=(B, HK, cap, D)).astype(np.float32)
    for kv_dt, odt in ((capi.F32, O.F32), (capi.F16, O.F16)):
        kk, vv = (kf, vf) if kv_dt == capi.F32 else (O.f32_to_f16(kf), O.f32_to_f16(vf))
        qb = f32_buffer(be, q)
        kb = be.alloc(kv_dt, kk.size); be.upload(kb, kk)
        vb = be.alloc(kv_dt, vv.size); be.upload(vb, vv)
        kview = View.contiguous([B, HK, cap, D]).shrink([(0, B), (0, HK), (0, Kn), (0, D)])
        out = be.alloc(capi.F32, B * H * Q * (D + 1))
        gpu.say(f"attention through the backend, keys of dtype {kv_dt}")
        be.run(Kernel(OP_ATTENTION, capi.F32, [B * H * Q * (D + 1)], [View.contiguous([B, H, Q, D]), kview, kview], scale=0.125, causal=True,
                      causal_offset=Kn - Q), [out], [qb, kb, vb])
        got = out_f32(be, out)
        wo, wl = O.attention(q, kk, vv, 0.125, causal=True, causal_offset=Kn - Q, kv_dt=odt, k_len=Kn)
        check_close(got[: B * H * Q * D], wo, 1e-5, "attention")
        check_close(got[B * H * Q * D:], wl, 1e-5, "logsumexp")


def test_attention_mask_value_width_and_no_keys(be):
    """OpAttention's other inputs (backend/op.go:117-129): the additive mask In[3] [B, H, Q, K], here expanded over
    the heads with stride 0 and holding -Inf entries; values of another width than the keys; and K = 0, where
    every row is zeros and -Inf and the key buffers are never read (NewAttentionShape allows it)."""
    rng = np.random.default_rng(26)
    B, H, HK, Q, Kn, D, DV = 2, 4, 2, 3, 19, 32, 48
    q = rng.normal(size=(B, H, Q, D)).astype(np.float32)
    kf = rng.normal(size=(B, HK, Kn, D)).astype(np.float32); vf = rng.normal(size=(B, HK, Kn, DV)).astype(np.float32)
    mask = rng.normal(size=(B, 1, Q, Kn)).astype(np.float32)
    mask[rng.random(mask.shape) < 0.25] = -np.inf
    mask[1, 0, 2, :] = -np.inf
    qb, kb, vb, mb = f32_buffer(be, q), f32_buffer(be, kf), f32_buffer(be, vf), f32_buffer(be, mask)
    out = be.alloc(capi.F32, B * H * Q * (DV + 1))
    mview = View.contiguous([B, 1, Q, Kn]).expand([B, H, Q, Kn])
    gpu.say("attention through the backend with a mask and values of another width")
    be.run(Kernel(OP_ATTENTION, capi.F32, [B * H * Q * (DV + 1)], [View.contiguous([B, H, Q, D]), View.contiguous([B, HK, Kn, D]),
                                                                    View.contiguous([B, HK, Kn, DV]), mview], scale=0.2, causal=True, causal_offset=Kn - Q),
           [out], [qb, kb, vb, mb])
    got = out_f32(be, out)
    wo, wl = O.attention(q, kf, vf, 0.2, causal=True, causal_offset=Kn - Q, mask=mask)
    check_close(got[: B * H * Q * DV], wo, 1e-5, "attention")
    check_close(got[B * H * Q * DV:], wl, 1e-5, "logsumexp")
    # a mask of the wrong shape, and one that is not float32
    for bad_view, bad_buf, code in ((View.contiguous([B, H, Q, Kn + 1]), f32_buffer(be, np.zeros(B * H * Q * (Kn + 1))), capi.ERR_SHAPE),):
        with pytest.raises(BackendError) as e:
            be.run(Kernel(OP_ATTENTION, capi.F32, [B * H * Q * (DV + 1)], [View.contiguous([B, H, Q, D]), View.contiguous([B, HK, Kn, D]),
                                                                            View.contiguous([B, HK, Kn, DV]), bad_view]), [out], [qb, kb, vb, bad_buf])
        assert e.value.code == code
    # no keys: views [B, HK, 0, D] over buffers of one element
    empty = be.alloc(capi.F32, 0)
    out0 = be.alloc(capi.F32, B * H * Q * (D + 1))
    be.upload(out0, np.full(B * H * Q * (D + 1), np.nan, np.float32))
    gpu.say("attention through the backend without keys")
    be.run(Kernel(OP_ATTENTION, capi.F32, [B * H * Q * (D + 1)], [View.contiguous([B, H, Q, D]), View.contiguous([B, HK, 0, D]),
                                                                   View.contiguous([B, HK, 0, D])], scale=0.2, causal=True), [out0], [qb, empty, empty])
    got = out_f32(be, out0)
    assert not got[: B * H * Q * D].any() and np.all(got[B * H * Q * D:] == -np.inf)


def test_recorded_batch_survives_scratch_growth(be):
    """A batch that has become a graph keeps the scratch blocks it was recorded with: calls that outgrow the
    library's scratch afterwards (activations and attention partials) must leave the graph's replays right."""
    rng = np.random.default_rng(27)
    l = gpu.lib()
    k, n, B, H, HK, D, cap = 1024, 64, 1, 8, 2, 64, 512
    wraw = bench_blocks(rng, O.Q8_0, n * k)
    w = be.alloc(capi.Q8_0, n * k); be.upload(w, wraw)
    x = rng.normal(size=(2, k)).astype(np.float32)
    q = rng.normal(size=(B, H, 1, D)).astype(np.float32)
    kf = rng.normal(size=(B, HK, cap, D)).astype(np.float32); vf = rng.normal(size=(B, HK, cap, D)).astype(np.float32)
    xb, qb, kb, vb = f32_buffer(be, x), f32_buffer(be, q), f32_buffer(be, kf), f32_buffer(be, vf)
    y = be.alloc(capi.F32, 2 * n); a = be.alloc(capi.F32, B * H * (D + 1))
    ks = [Kernel(OP_QMATMUL, capi.F32, [2, n], [View.contiguous([2, k]), View.contiguous([n, k])]),
          Kernel(OP_ATTENTION, capi.F32, [B * H * (D + 1)], [View.contiguous([B, H, 1, D]), View.contiguous([B, HK, cap, D]), View.contiguous([B, HK, cap, D])],
                 scale=0.125)]
    batch = Batch(be, ks, [[y], [a]], [[xb, w], [qb, kb, vb]])
    want_y = O.qmatmul(O.Q8_0, wraw, x, n, k)
    wo, wl = O.attention(q, kf, vf, 0.125)

    def check(tag):
        be.upload(y, np.full(2 * n, np.nan, np.float32)); be.upload(a, np.full(B * H * (D + 1), np.nan, np.float32))
        gpu.say(f"recorded batch, {tag}")
        be.run_batch(batch)
        check_close(out_f32(be, y).reshape(2, n), want_y, 1e-4, tag)  # float32 sums of a row's blocks in another order
        got = out_f32(be, a)
        check_close(got[: B * H * D], wo, 1e-5, tag); check_close(got[B * H * D:], wl, 1e-5, tag)

    before = be.graph_replays()
    for it in range(3):
        check(f"run {it}")
    assert be.graph_replays() - before == 2
    # outgrow both blocks on the backend's stream: 2000 rows of converted activations (2.3 MB) and the partials of 256 query rows
    big_m, big_q = 2000, 256
    bx = f32_buffer(be, rng.normal(size=(big_m, k)).astype(np.float32)); by = be.alloc(capi.F32, big_m * n)
    be.run(Kernel(OP_QMATMUL, capi.F32, [big_m, n], [View.contiguous([big_m, k]), View.contiguous([n, k])]), [by], [bx, w])
    bq = f32_buffer(be, rng.normal(size=(B, H, big_q, D)).astype(np.float32)); bo = be.alloc(capi.F32, B * H * big_q * (D + 1))
    be.run(Kernel(OP_ATTENTION, capi.F32, [B * H * big_q * (D + 1)], [View.contiguous([B, H, big_q, D]), View.contiguous([B, HK, cap, D]),
                                                                       View.contiguous([B, HK, cap, D])], scale=0.125), [bo], [bq, kb, vb])
    be.sync()
    for it in range(2):
        check(f"replay {it} after the scratch grew")
    assert be.graph_replays() - before == 4
    batch.close()


def test_check_run_and_ownership(be):
    rng = np.random.default_rng(17)
    w, _ = quant_buffer(be, rng, O.Q8_0, 4 * 64)
    x = f32_buffer(be, np.ones(64))
    out = be.alloc(capi.F32, 4)
    wv, xv = View.contiguous([4, 64]), View.contiguous([64])
    good = Kernel(OP_QMATMUL, capi.F32, [4], [xv, wv])
    be.run(good, [out], [x, w]); be.sync()

    def refused(code, k, outs, ins):
        with pytest.raises(BackendError) as e:
            be.run(k, outs, ins)
        assert e.value.code == code, e.value

    refused(capi.ERR_INTERNAL, good, [out], [x])                                   # buffers for views
    refused(capi.ERR_INTERNAL, good, [out, out], [x, w])                           # outputs
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [5], [xv, wv]), [out], [x, w])   # output of another size
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F16, [4], [xv, wv]), [out], [x, w])   # output of another dtype
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [4], [View([64], [2]), wv]), [out], [x, w])  # view outside its buffer
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [4], [View([64], [-1], 0), wv]), [out], [x, w])
    big = be.alloc(capi.Q8_0, 8 * 64)
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [4], [xv, View([4, 64], [64, 1], 16)]), [out], [x, big])      # weights off a block boundary
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [4], [xv, View([4, 64], [128, 1], 0)]), [out], [x, big])      # weights not contiguous
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [4], [View.contiguous([32]), wv]), [out], [x, w])             # K of x and of the weights differ
    # an input that is also the output
    xo = be.alloc(capi.F32, 64)
    refused(capi.ERR_INTERNAL, Kernel(OP_QMATMUL, capi.F32, [64], [View.contiguous([64]), View.contiguous([64, 64])]), [xo], [xo, be.alloc(capi.Q8_0, 64 * 64)])
    # an operation that is not on this path
    refused(capi.ERR_INTERNAL, Kernel(OP_CAST, capi.F16, [64], [xv]), [be.alloc(capi.F16, 64)], [x])
    # allocation: negative, not whole blocks, unknown dtype
    for dt, n, code in ((capi.F32, -1, capi.ERR_SHAPE), (capi.Q8_0, 33, capi.ERR_SHAPE), (99, 4, capi.ERR_DTYPE)):
        with pytest.raises(BackendError) as e:
            be.alloc(dt, n)
        assert e.value.code == code
    # upload and download sizes
    with pytest.raises(BackendError) as e:
        be.upload(x, np.ones(63, np.float32))
    assert e.value.code == capi.ERR_SHAPE
    with pytest.raises(BackendError) as e:
        be.download(x, 100)
    assert e.value.code == capi.ERR_SHAPE
    # a freed buffer, freed twice, and another backend's buffer
    be.free(out); be.free(out)
    refused(capi.ERR_DTYPE, good, [out], [x, w])
    other = Backend(0)
    try:
        theirs = other.alloc(capi.F32, 4)
        refused(capi.ERR_DTYPE, good, [theirs], [x, w])
        with pytest.raises(BackendError) as e:
            be.upload(theirs, np.zeros(4, np.float32))
        assert e.value.code == capi.ERR_DTYPE
    finally:
        other.close()
    # a buffer of less than four bytes holds its element
    tiny = be.alloc(capi.F16, 1)
    be.upload(tiny, np.array([0x3c00], np.uint16))
    assert be.download(tiny).view(np.uint16)[0] == 0x3c00


def test_batch_becomes_a_graph(be):
    """A schedule of three kernels (embedding lookup, product from a strided
    view, product) run five times with new inputs uploaded in between: the
    second run records it, later runs replay it, every run matches the
    oracle."""
    rng = np.random.default_rng(18)
    rows, k, n = 16, 256, 48
    table, traw = quant_buffer(be, rng, O.Q8_0, rows * k)
    w1, w1raw = quant_buffer(be, rng, O.Q4_0, 2 * k * k)
    w2, w2raw = quant_buffer(be, rng, O.Q8_0, n * 2 * k)
    ib = be.alloc(capi.I32, 3)
    emb = be.alloc(capi.F32, 3 * k); h = be.alloc(capi.F32, 3 * 2 * k); y = be.alloc(capi.F32, 3 * n)
    ks = [Kernel(OP_GATHER, capi.F32, [3, k], [View.contiguous([rows, k]), View([3, k], [1, 0])], axis=0),
          Kernel(OP_QMATMUL, capi.F32, [3, 2 * k], [View.contiguous([k, 3]).permute([1, 0]), View.contiguous([2 * k, k])]),
          Kernel(OP_QMATMUL, capi.F32, [3, n], [View.contiguous([3, 2 * k]), View.contiguous([n, 2 * k])])]
    # the second kernel reads emb as if it were stored [k, 3]: a strided view that has to be gathered first
    batch = Batch(be, ks, [[emb], [h], [y]], [[table, ib], [emb, w1], [h, w2]])
    full = O.dequantize(O.Q8_0, traw).reshape(rows, k)
    before = be.graph_replays()
    for it in range(5):
        idx = rng.integers(0, rows, 3).astype(np.int32)
        be.upload(ib, idx)
        gpu.say(f"batch run {it}")
        be.run_batch(batch)
        got = out_f32(be, y).reshape(3, n)
        e = full[idx].reshape(-1).reshape(k, 3).T.copy()  # what the strided view reads
        hh = O.qmatmul(O.Q4_0, w1raw, e, 2 * k, k)
        want = O.qmatmul(O.Q8_0, w2raw, hh, n, 2 * k)
        check_close(got, want, 2e-3, f"batch run {it}")  # int8 rounding of h on both sides: a step function of float32 sums
    assert be.graph_replays() - before == 4
    batch.close()
