"""Parity of the decode-step kernels with the oracle and with the reference's
golden attention.mim, through the C ABI, on a real MI355X.

Tolerances: the reference's own for these ops, atol 1e-5 + rtol 1e-4
(nn/transformer_test.go:139); RoPE, the KV write, SwiGLU's operations and
argmax are compared bit for bit where the arithmetic order is fixed."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import oracle as O
from mimir_amd import capi
from mimir_amd.mimfile import golden_cases
from tests import gpu
from tests.helpers import bits_equal

pytestmark = pytest.mark.gpu
ATOL, RTOL = 1e-5, 1e-4


def close(got, want, what=""):
    assert got.shape == want.shape, (got.shape, want.shape)
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf]), f"{what}: infinities differ"
    err = np.abs(got[~inf].astype(np.float64) - want[~inf])
    assert np.all(err <= ATOL + RTOL * np.abs(want[~inf])), f"{what}: worst {err.max():.3e}"


@pytest.fixture(scope="module")
def cases(golden_dir):
    return golden_cases(os.path.join(golden_dir, "attention.mim"))


def rmsnorm(x, w, eps):
    l = gpu.lib()
    xd = gpu.dev(x); y = torch.empty_like(xd)
    wd = gpu.dev(w) if w is not None else None
    d = x.shape[-1]
    capi.check(l.mi355x_rmsnorm(xd.data_ptr(), wd.data_ptr() if wd is not None else None, y.data_ptr(), x.size // d, d, eps, gpu.stream()))
    gpu.sync()
    return y.cpu().numpy()


def test_rmsnorm(cases):
    gpu.say("rmsnorm golden + 8B shape")
    c = cases["rms_norm"]
    close(rmsnorm(c["in"][0].data, c["in"][1].data, 1e-6), c["out"].data)
    c = cases["rms_norm_default_eps"]
    close(rmsnorm(c["in"][0].data, c["in"][1].data, 2.0 ** -23), c["out"].data)
    rng = np.random.default_rng(0)
    x = rng.normal(size=(8, 4096)).astype(np.float32) * 3; w = rng.normal(1, 0.02, 4096).astype(np.float32)
    got = rmsnorm(x, w, 1e-5)
    want = O.rmsnorm(x, w, 1e-5)
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()  # only the order of the sum of squares differs
    assert np.abs(rmsnorm(x, None, 1e-5) - O.rmsnorm(x, None, 1e-5)).max() <= 2e-6 * 4


def rope(x, cos, sin, dim, inter, offset, table_len=None):
    """x [..., S, head_dim] contiguous."""
    l = gpu.lib()
    s, hd = x.shape[-2], x.shape[-1]
    xd = gpu.dev(x); y = torch.empty_like(xd)
    cd, sd = gpu.dev(cos), gpu.dev(sin)
    capi.check(l.mi355x_rope(xd.data_ptr(), y.data_ptr(), x.size // (s * hd), s, hd, dim, int(inter), s * hd, hd, s * hd, hd,
                             cd.data_ptr(), sd.data_ptr(), cos.shape[0], offset, gpu.stream()))
    gpu.sync()
    return y.cpu().numpy()


@pytest.mark.parametrize("name,dim,inter,off,scaling,params", [
    ("rope_neox", 8, False, 3, O.ROPE_NONE, ()),
    ("rope_interleaved", 8, True, 3, O.ROPE_NONE, ()),
    ("rope_partial_scaled", 8, False, 2, O.ROPE_LLAMA3, (8, 1, 4, 64)),
])
def test_rope_golden(cases, name, dim, inter, off, scaling, params):
    c = cases[name]
    x = c["in"][0].data
    n = off + x.shape[-2]
    cos, sin = O.rope_angles(dim, 10000.0, 0, n, scaling, params)  # the whole table; the kernel reads rows off..
    gpu.say(name)
    got = rope(x, cos, sin, dim, inter, off)
    close(got, c["out"].data)
    assert bits_equal(got, O.rope_apply(x, cos[off:], sin[off:], dim, inter))


def test_rope_decode_shape_bit_exact_and_strided():
    """40 heads of 128 features at position 2048 of a table for theta 500000,
    interleaved; and q read in place from a [S, heads * dim] product (position
    stride heads * dim, head stride dim)."""
    rng = np.random.default_rng(1)
    cos, sin = O.rope_angles(128, 500000.0, 0, 2100)
    x = rng.normal(size=(40, 1, 128)).astype(np.float32)
    gpu.say("rope decode shape")
    assert bits_equal(rope(x, cos, sin, 128, True, 2048), O.rope_apply(x, cos[2048:2049], sin[2048:2049], 128, True))
    S, H, D = 5, 4, 128
    tok_major = rng.normal(size=(S, H * D)).astype(np.float32)
    l = gpu.lib()
    xd = gpu.dev(tok_major); cd, sd = gpu.dev(cos), gpu.dev(sin)
    capi.check(l.mi355x_rope(xd.data_ptr(), xd.data_ptr(), H, S, D, D, 1, D, H * D, D, H * D, cd.data_ptr(), sd.data_ptr(), 2100, 7, gpu.stream()))
    gpu.sync()
    heads_major = tok_major.reshape(S, H, D).transpose(1, 0, 2).copy()
    want = O.rope_apply(heads_major, cos[7:12], sin[7:12], D, True).transpose(1, 0, 2).reshape(S, H * D)
    assert bits_equal(xd.cpu().numpy(), want)
    assert l.mi355x_rope(xd.data_ptr(), xd.data_ptr(), H, S, D, D, 1, D, H * D, D, H * D, cd.data_ptr(), sd.data_ptr(), 2100, 2098, gpu.stream()) == capi.ERR_SHAPE


def test_kv_write_casts_like_the_reference():
    rng = np.random.default_rng(2)
    B, KVH, S, D, cap, pos = 2, 8, 3, 128, 64, 5
    src = (rng.normal(size=(B, KVH, S, D)) * np.array([1e-6, 1, 300, 70000])[rng.integers(0, 4, (B, KVH, S, D))]).astype(np.float32)
    l = gpu.lib()
    sd = gpu.dev(src)
    for dt, tdt in ((capi.F16, torch.int16), (capi.F32, torch.float32)):
        cache = torch.zeros((B, KVH, cap, D), dtype=tdt, device="cuda:0")
        gpu.say(f"kv_write dt={dt}")
        capi.check(l.mi355x_kv_write(sd.data_ptr(), cache.data_ptr(), dt, B, KVH, S, D, cap, pos, KVH * S * D, S * D, D, gpu.stream()))
        gpu.sync()
        got = cache.cpu().numpy()
        if dt == capi.F16:
            got = got.view(np.uint16)
            assert np.array_equal(got[:, :, pos:pos + S], O.f32_to_f16(src))  # round to nearest even, overflow to infinity
        else:
            assert bits_equal(got[:, :, pos:pos + S], src)
        assert not got[:, :, :pos].any() and not got[:, :, pos + S:].any()
    assert l.mi355x_kv_write(sd.data_ptr(), cache.data_ptr(), capi.F32, B, KVH, S, D, cap, cap - 2, KVH * S * D, S * D, D, gpu.stream()) == capi.ERR_SHAPE


def attention(q, k, v, scale, causal=False, offset=0, kv_dt=capi.F32, k_len=None, want_lse=True, mask=None):
    """q [B,H,Q,D], k [B,HK,cap,D] and v [B,HK,cap,DV] contiguous numpy (uint16 bits for F16); mask broadcastable
    to [B,H,Q,K] (dimensions of size 1 are read with stride 0)."""
    l = gpu.lib()
    B, H, Q, D = q.shape
    HK, cap, DV = k.shape[1], k.shape[2], v.shape[3]
    K = cap if k_len is None else k_len
    qd = gpu.dev(q)
    kd = gpu.dev(k.view(np.int16) if kv_dt == capi.F16 else k); vd = gpu.dev(v.view(np.int16) if kv_dt == capi.F16 else v)
    out = torch.full((B, H, Q, DV), float("nan"), dtype=torch.float32, device="cuda:0")
    lse = torch.full((B, H, Q), float("nan"), dtype=torch.float32, device="cuda:0")
    arr = lambda *a: (C.c_int64 * len(a))(*a)
    md, ms = None, None
    if mask is not None:
        m4 = np.ascontiguousarray(mask, np.float32).reshape((1,) * (4 - np.ndim(mask)) + np.shape(mask))
        md = gpu.dev(m4)
        ms = arr(*[0 if m4.shape[i] == 1 else int(np.prod(m4.shape[i + 1:])) for i in range(4)])
    capi.check(l.mi355x_attention(qd.data_ptr(), arr(H * Q * D, Q * D, D), kd.data_ptr(), arr(HK * cap * D, cap * D, D), vd.data_ptr(),
                                  arr(HK * cap * DV, cap * DV, DV), kv_dt, md.data_ptr() if md is not None else None, ms,
                                  out.data_ptr(), arr(H * Q * DV, Q * DV, DV), lse.data_ptr() if want_lse else None, B, H, HK, Q, K, D, DV,
                                  scale, int(causal), offset, gpu.stream()))
    gpu.sync()
    # the same call with its arguments in one structure (mi355x_attention_d) gives the same bits
    out2, lse2 = torch.full_like(out, float("nan")), torch.full_like(lse, float("nan"))
    d = capi.AttentionDesc()
    d.q, d.k, d.v, d.out, d.lse = qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out2.data_ptr(), (lse2.data_ptr() if want_lse else None)
    d.mask = md.data_ptr() if md is not None else None
    d.q_strides[:] = [H * Q * D, Q * D, D]
    d.k_strides[:] = [HK * cap * D, cap * D, D]
    d.v_strides[:] = [HK * cap * DV, cap * DV, DV]
    d.out_strides[:] = [H * Q * DV, Q * DV, DV]
    if ms is not None:
        d.mask_strides[:] = list(ms)
    d.B, d.Q, d.K, d.causal_offset, d.scale = B, Q, K, offset, scale
    d.kv_dtype, d.H, d.HK, d.D, d.DV, d.causal = kv_dt, H, HK, D, DV, int(causal)
    capi.check(l.mi355x_attention_d(C.byref(d), gpu.stream()))
    gpu.sync()
    assert torch.equal(out.view(torch.int32), out2.view(torch.int32))
    if want_lse:
        assert torch.equal(lse.view(torch.int32), lse2.view(torch.int32))
    return out.cpu().numpy(), lse.cpu().numpy()


def test_attention_golden_mask(cases):
    """The reference's masked case (nn/transformer_test.go:36-38): an additive float mask as In[3]."""
    c = cases["sdpa_mask"]
    q, k, v, mask = (t.data for t in c["in"][:4])
    gpu.say(f"sdpa_mask q={q.shape} mask={mask.shape}")
    out, lse = attention(q, k, v, 1 / np.sqrt(q.shape[-1]), mask=mask)
    close(out, c["out"].data, "sdpa_mask")
    _, wl = O.attention(q, k, v, 1 / np.sqrt(q.shape[-1]), mask=mask)
    close(lse, wl, "sdpa_mask lse")


@pytest.mark.parametrize("B,H,HK,Q,K,D,DV", [(2, 4, 2, 5, 37, 16, 24), (1, 8, 2, 1, 300, 64, 128), (1, 3, 1, 7, 70, 128, 8), (2, 32, 8, 1, 129, 128, 128)])
def test_attention_mask_and_value_width(B, H, HK, Q, K, D, DV):
    """Values of another width than the keys, and an additive mask with -Inf entries (whole rows among them),
    per head, broadcast over heads, and broadcast over batch and heads; with and without causality."""
    rng = np.random.default_rng(B * 100 + K)
    q = rng.normal(size=(B, H, Q, D)).astype(np.float32)
    k = rng.normal(size=(B, HK, K, D)).astype(np.float32); v = rng.normal(size=(B, HK, K, DV)).astype(np.float32)
    scale = 1 / np.sqrt(D)
    full = rng.normal(size=(B, H, Q, K)).astype(np.float32)
    full[rng.random(full.shape) < 0.3] = -np.inf
    full[0, 0, 0, :] = -np.inf  # a row that sees nothing: zeros and -Inf
    for name, mask in (("none", None), ("full", full), ("heads", full[:, :1]), ("rows", full[:1, :1])):
        for causal, off in ((False, 0), (True, K - Q)):
            gpu.say(f"attention B={B} H={H} HK={HK} Q={Q} K={K} D={D} DV={DV} mask={name} causal={causal}")
            out, lse = attention(q, k, v, scale, causal=causal, offset=off, mask=mask)
            wo, wl = O.attention(q, k, v, scale, causal=causal, causal_offset=off, mask=mask)
            close(out, wo, name); close(lse, wl, name + " lse")
    assert np.all(out[0, 0, 0] == 0) and lse[0, 0, 0] == -np.inf


@pytest.mark.parametrize("B,H,HK,Q,D", [(1, 32, 8, 1, 128), (2, 4, 2, 3, 16)])
def test_attention_without_keys(B, H, HK, Q, D):
    """K = 0 (NewAttentionShape allows it, backend/attention.go:36-62): zeros and a logsumexp of -Inf, with
    allocated key buffers and with none at all."""
    l = gpu.lib()
    rng = np.random.default_rng(9)
    qd = gpu.dev(rng.normal(size=(B, H, Q, D)).astype(np.float32))
    kd = torch.zeros(4, dtype=torch.float32, device="cuda:0")
    arr = lambda *a: (C.c_int64 * len(a))(*a)
    for kv in (kd.data_ptr(), None):
        for kv_dt in (capi.F32, capi.F16):
            out = torch.full((B, H, Q, D), float("nan"), dtype=torch.float32, device="cuda:0")
            lse = torch.full((B, H, Q), float("nan"), dtype=torch.float32, device="cuda:0")
            gpu.say(f"attention without keys B={B} H={H} Q={Q} D={D} kv={'set' if kv else 'null'} dt={kv_dt}")
            capi.check(l.mi355x_attention(qd.data_ptr(), arr(H * Q * D, Q * D, D), kv, arr(0, 0, D) if kv else None, kv, arr(0, 0, D) if kv else None,
                                          kv_dt, None, None, out.data_ptr(), arr(H * Q * D, Q * D, D), lse.data_ptr(), B, H, HK, Q, 0, D, D,
                                          1 / np.sqrt(D), 1, 0, gpu.stream()))
            gpu.sync()
            assert not out.cpu().numpy().any() and np.all(lse.cpu().numpy() == -np.inf)


@pytest.mark.parametrize("name,kw", [
    ("sdpa_causal", {"causal": True}),
    ("sdpa_causal_offset", {"causal": True, "offset": 4}),
    ("sdpa_gqa", {"causal": True, "offset": 2}),
])
def test_attention_golden(cases, name, kw):
    c = cases[name]
    q, k, v = (t.data for t in c["in"][:3])
    gpu.say(name)
    out, lse = attention(q, k, v, 1 / np.sqrt(q.shape[-1]), **kw)
    close(out, c["out"].data, name)
    wo, wl = O.attention(q, k, v, 1 / np.sqrt(q.shape[-1]), causal=kw.get("causal", False), causal_offset=kw.get("offset", 0))
    close(lse, wl, name + " lse")


@pytest.mark.parametrize("B,H,HK,D,cap,n", [(1, 32, 8, 128, 2304, 2049), (8, 32, 8, 128, 2304, 2049), (2, 8, 2, 64, 64, 37), (1, 4, 1, 64, 300, 300),
                                            (1, 6, 1, 16, 40, 1), (3, 5, 5, 8, 33, 33)])
def test_decode_attention_f16_cache(B, H, HK, D, cap, n):
    """One query per head over a binary16 cache holding n of cap positions: the
    decode step's shape (32 heads on 8 key heads of 128, 2049 keys) and small
    and ragged ones, groups of 4, 6 and 1 query heads per key head."""
    rng = np.random.default_rng(B * 1000 + n)
    q = rng.normal(size=(B, H, 1, D)).astype(np.float32)
    kh = O.f32_to_f16(rng.normal(size=(B, HK, cap, D)).astype(np.float32)); vh = O.f32_to_f16(rng.normal(size=(B, HK, cap, D)).astype(np.float32))
    gpu.say(f"decode attention B={B} H={H} HK={HK} D={D} n={n}")
    out, lse = attention(q, kh, vh, 1 / np.sqrt(D), kv_dt=capi.F16, k_len=n)
    wo, wl = O.attention(q, kh, vh, 1 / np.sqrt(D), kv_dt=O.F16, k_len=n)
    close(out, wo); close(lse, wl)
    out2, _ = attention(q, kh, vh, 1 / np.sqrt(D), causal=True, offset=n - 1, kv_dt=capi.F16, want_lse=False)  # the same keys, hidden causally
    close(out2, wo)  # the keys are shared out over the workgroups by capacity here, so sums may round another way
    # the general kernels on the same call, and the single-launch kernel again (its tickets must have reset)
    l = gpu.lib()
    try:
        capi.check(l.mi355x_tune(b"attention.path", 1))
        out3, lse3 = attention(q, kh, vh, 1 / np.sqrt(D), kv_dt=capi.F16, k_len=n)
    finally:
        capi.check(l.mi355x_tune(b"attention.path", 0))
    close(out3, wo); close(lse3, wl)
    out4, lse4 = attention(q, kh, vh, 1 / np.sqrt(D), kv_dt=capi.F16, k_len=n)
    assert bits_equal(out4, out) and bits_equal(lse4, lse)


@pytest.mark.parametrize("kv_dt", [capi.F32, capi.F16])
def test_decode_attention_few_and_no_keys(kv_dt):
    """Fewer keys than workgroups share them out to, one key, and none (zeros
    and -Inf, as a row that sees no key gets), float32 and binary16 caches."""
    rng = np.random.default_rng(11)
    B, H, HK, D, cap = 2, 8, 2, 128, 512
    q = rng.normal(size=(B, H, 1, D)).astype(np.float32)
    k = rng.normal(size=(B, HK, cap, D)).astype(np.float32); v = rng.normal(size=(B, HK, cap, D)).astype(np.float32)
    if kv_dt == capi.F16:
        k, v = O.f32_to_f16(k), O.f32_to_f16(v)
    odt = O.F16 if kv_dt == capi.F16 else O.F32
    for n in (1, 5, 33, 511):
        gpu.say(f"decode attention, {n} of {cap} keys, dtype {kv_dt}")
        out, lse = attention(q, k, v, 0.25, causal=True, offset=n - 1, kv_dt=kv_dt)
        wo, wl = O.attention(q, k, v, 0.25, kv_dt=odt, k_len=n)
        close(out, wo); close(lse, wl)
    out, lse = attention(q, k, v, 0.25, causal=True, offset=-1, kv_dt=kv_dt)
    assert not out.any() and np.all(lse == -np.inf)


def test_prompt_attention_f32_cache_and_empty_rows():
    rng = np.random.default_rng(5)
    B, H, HK, Q, D = 1, 8, 2, 17, 64
    q = rng.normal(size=(B, H, Q, D)).astype(np.float32); k = rng.normal(size=(B, HK, Q + 3, D)).astype(np.float32); v = rng.normal(size=(B, HK, Q + 3, D)).astype(np.float32)
    gpu.say("prompt attention causal offset 3, then offset -2")
    out, lse = attention(q, k, v, 0.3, causal=True, offset=3)
    wo, wl = O.attention(q, k, v, 0.3, causal=True, causal_offset=3)
    close(out, wo); close(lse, wl)
    out, lse = attention(q, k, v, 0.3, causal=True, offset=-2)  # rows 0 and 1 see no key
    wo, wl = O.attention(q, k, v, 0.3, causal=True, causal_offset=-2)
    assert not out[:, :, :2].any() and np.all(lse[:, :, :2] == -np.inf)
    close(out, wo); close(lse[:, :, 2:], wl[:, :, 2:])


def last_kernel():
    buf = C.create_string_buffer(200)
    capi.check(gpu.lib().mi355x_last_kernel(buf, 200))
    return buf.value.decode()


@pytest.mark.parametrize("B,H,HK,Q,K,D,kv_dt,causal,off", [
    (1, 8, 2, 64, 64, 128, capi.F16, True, 0),      # the smallest call the kernel takes: half a workgroup's rows
    (2, 8, 2, 300, 337, 128, capi.F16, True, 37),   # ragged rows and keys, a past of 37 positions
    (1, 4, 4, 129, 129, 64, capi.F32, True, 0),     # one row into a second workgroup, 64 features, a float32 cache
    (2, 6, 3, 200, 90, 64, capi.F16, False, 0),     # every row sees every key; groups of 2
    (1, 4, 1, 256, 256, 128, capi.F32, True, -40),  # the first 40 rows see no key: zeros and -Inf
    (1, 2, 1, 100, 400, 128, capi.F16, True, 500),  # the offset beyond the keys: every row sees all 400
    (1, 32, 8, 512, 512, 128, capi.F16, True, 0),   # a 512-token prompt of the 8B shape
    (4, 32, 8, 512, 512, 128, capi.F16, True, 0),   # four of them: enough workgroups of four wavefronts (fewer rows take two)
    (2, 64, 8, 450, 100, 64, capi.F32, False, 0),   # four wavefronts again: float32 cache, 64 features, ragged, every key seen
])
def test_prompt_attention_on_the_matrix_cores(B, H, HK, Q, K, D, kv_dt, causal, off):
    """Calls of 64 and more query positions go to the kernel that walks tiles of keys with 32 rows a wavefront: against
    the oracle to the float32 tolerance of the other attention tests, and against the kernel that takes a query row a
    workgroup (the same call with the route switched off), which it follows up to the order of the sums."""
    l = gpu.lib()
    rng = np.random.default_rng(Q * 1000 + K)
    q = rng.normal(size=(B, H, Q, D)).astype(np.float32)
    k = rng.normal(size=(B, HK, K, D)).astype(np.float32); v = rng.normal(size=(B, HK, K, D)).astype(np.float32)
    odt = O.F32
    if kv_dt == capi.F16:
        k, v, odt = O.f32_to_f16(k), O.f32_to_f16(v), O.F16
    scale = 1 / np.sqrt(D)
    gpu.say(f"prompt attention B={B} H={H} HK={HK} Q={Q} K={K} D={D} dt={kv_dt} causal={causal} offset={off}")
    out, lse = attention(q, k, v, scale, causal=causal, offset=off, kv_dt=kv_dt)
    assert last_kernel() == "attn_prompt_kernel"
    wo, wl = O.attention(q, k, v, scale, causal=causal, causal_offset=off, kv_dt=odt)
    close(out, wo); close(lse, wl)
    try:
        capi.check(l.mi355x_tune(b"attention.prompt", 0))
        out2, lse2 = attention(q, k, v, scale, causal=causal, offset=off, kv_dt=kv_dt)
        assert last_kernel() != "attn_prompt_kernel"
    finally:
        capi.check(l.mi355x_tune(b"attention.prompt", 1))
    close(out, out2); close(lse, lse2)
    if causal and off < 0:
        assert not out[:, :, :-off].any() and np.all(lse[:, :, :-off] == -np.inf)


@pytest.mark.parametrize("kv_dt,D", [(capi.F16, 128), (capi.F32, 64)])
def test_prompt_attention_with_nan_and_infinity_among_the_values(kv_dt, D):
    """A NaN or an infinity in the values of a key reaches the rows that see the key and no row before it (the reference
    reads a row's visible keys only, backend/cpu/attention.go:437-535), although the kernel multiplies whole tiles of
    keys: such a tile goes key by key. Also behind the last key, where a tile's rows repeat it."""
    l = gpu.lib()
    rng = np.random.default_rng(D)
    B, H, HK, Q, K = 2, 4, 2, 200, 215
    off = K - Q
    q = rng.normal(size=(B, H, Q, D)).astype(np.float32)
    k = rng.normal(size=(B, HK, K, D)).astype(np.float32); v = rng.normal(size=(B, HK, K, D)).astype(np.float32)
    v[0, 0, 70, 5] = np.nan      # seen from row 55 on, in the middle of a tile and of a wavefront's rows
    v[0, 1, 131, 9] = np.inf     # from row 116 on
    v[1, 0, 214, 3] = -np.inf    # the last key: the last row only
    v[1, 1, 32, :] = np.nan      # a tile's first key
    odt = O.F32
    if kv_dt == capi.F16:
        k, v, odt = O.f32_to_f16(k), O.f32_to_f16(v), O.F16
    scale = 1 / np.sqrt(D)
    def same(got, want, what):
        bad = ~np.isfinite(want)
        assert np.array_equal(np.isnan(got), np.isnan(want)), what
        assert np.array_equal(got[bad & ~np.isnan(want)], want[bad & ~np.isnan(want)]), what
        g, w = got[~bad].astype(np.float64), want[~bad]
        assert np.all(np.abs(g - w) <= ATOL + RTOL * np.abs(w)), what
    for causal in (True, False):
        gpu.say(f"prompt attention, NaN and infinities in the values, dt={kv_dt} D={D} causal={causal}")
        out, lse = attention(q, k, v, scale, causal=causal, offset=off, kv_dt=kv_dt)
        assert last_kernel() == "attn_prompt_kernel"
        wo, wl = O.attention(q, k, v, scale, causal=causal, causal_offset=off, kv_dt=odt)
        same(out, wo, "against the oracle"); close(lse, wl)
        if causal:  # heads 0, 1 on key head 0 and 2, 3 on key head 1
            assert np.isfinite(out[0, :2, :55]).all() and np.isnan(out[0, :2, 55:, 5]).all() and np.isfinite(out[0, :2, 55:, 6]).all()
            assert np.isfinite(out[0, 2:, :116]).all() and not np.isfinite(out[0, 2:, 116:, 9]).any()
            assert np.isfinite(out[1, :2, :199]).all() and (out[1, :2, 199, 3] == -np.inf).all()
            assert np.isfinite(out[1, 2:, :17]).all() and np.isnan(out[1, 2:, 17:]).all()
        try:
            capi.check(l.mi355x_tune(b"attention.prompt", 0))
            out2, lse2 = attention(q, k, v, scale, causal=causal, offset=off, kv_dt=kv_dt)
        finally:
            capi.check(l.mi355x_tune(b"attention.prompt", 1))
        same(out, out2, "against the kernel that takes a query row a workgroup"); close(lse, lse2)


def test_prompt_attention_leaves_other_calls_where_they_were():
    """Fewer than 64 query positions, values of another width than the keys, a mask, and rows of keys that do not start
    on 16 bytes stay on the other kernels."""
    rng = np.random.default_rng(77)
    def call(Q, D, DV, mask=False):
        q = rng.normal(size=(1, 2, Q, D)).astype(np.float32)
        k = rng.normal(size=(1, 2, 70, D)).astype(np.float32); v = rng.normal(size=(1, 2, 70, DV)).astype(np.float32)
        m = rng.normal(size=(1, 2, Q, 70)).astype(np.float32) if mask else None
        gpu.say(f"attention Q={Q} D={D} DV={DV} mask={mask}")
        out, lse = attention(q, k, v, 0.2, mask=m)
        wo, wl = O.attention(q, k, v, 0.2, mask=m)
        close(out, wo); close(lse, wl)
        return last_kernel()
    assert call(64, 64, 64) == "attn_prompt_kernel"
    assert call(63, 64, 64) != "attn_prompt_kernel"
    assert call(64, 64, 128) != "attn_prompt_kernel"
    assert call(64, 64, 64, mask=True) != "attn_prompt_kernel"
    assert call(64, 32, 32) != "attn_prompt_kernel"


def test_swiglu_add_argmax():
    l = gpu.lib()
    rng = np.random.default_rng(6)
    n = 14336
    g = (rng.normal(size=(2, n)) * 4).astype(np.float32); u = rng.normal(size=(2, n)).astype(np.float32)
    g[0, :5] = [-200, 200, 0, -88.5, 1e-30]
    gd, ud = gpu.dev(g), gpu.dev(u)
    out = torch.empty((2, n), dtype=torch.float32, device="cuda:0")
    gpu.say("swiglu")
    capi.check(l.mi355x_swiglu(gd.data_ptr(), ud.data_ptr(), out.data_ptr(), 2, n, n, gpu.stream())); gpu.sync()
    want = O.silu_mul(g, u)
    got = out.cpu().numpy()
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()  # exp2 differs in the last bits between libraries
    assert got[0, 0] == 0
    # halves of one fused [2, 2n] product
    both = np.concatenate([g, u], axis=1)
    bd = gpu.dev(both)
    capi.check(l.mi355x_swiglu(bd.data_ptr(), bd.data_ptr() + 4 * n, out.data_ptr(), 2, n, 2 * n, gpu.stream())); gpu.sync()
    assert bits_equal(out.cpu().numpy(), got)
    gpu.say("add")
    capi.check(l.mi355x_add(gd.data_ptr(), ud.data_ptr(), out.data_ptr(), 2 * n, gpu.stream())); gpu.sync()
    assert bits_equal(out.cpu().numpy(), g + u)
    gpu.say("argmax")
    logits = rng.normal(size=(4, 128256)).astype(np.float32)
    logits[1, 777] = logits[1, 90000] = 50.0          # a tie: the first index wins
    logits[2, 0] = np.nan                              # NaN at 0 is never beaten
    logits[3, 5] = np.nan; logits[3, 100000] = 60.0    # a NaN elsewhere never wins
    ld = gpu.dev(logits); idx = torch.full((4,), -1, dtype=torch.int32, device="cuda:0")
    capi.check(l.mi355x_argmax(ld.data_ptr(), 4, 128256, idx.data_ptr(), gpu.stream())); gpu.sync()
    assert idx.cpu().tolist() == [O.argmax(r) for r in logits] == [int(np.argmax(logits[0])), 777, 0, 100000]
    # ragged lengths over several workgroups a row, twice (the tickets reset themselves)
    for n2 in (8192, 10001, 300007):
        lg = rng.normal(size=(3, n2)).astype(np.float32)
        lg[1, n2 - 1] = 99.0; lg[2, 4095] = lg[2, 4096] = 77.0
        l2 = gpu.dev(lg)
        for _ in range(2):
            idx.fill_(-1)
            capi.check(l.mi355x_argmax(l2.data_ptr(), 3, n2, idx.data_ptr(), gpu.stream())); gpu.sync()
            assert idx.cpu().tolist()[:3] == [int(np.argmax(lg[0])), n2 - 1, 4095]
    tiny = gpu.dev(np.array([[-np.inf, -np.inf], [np.nan, np.nan]], np.float32))
    capi.check(l.mi355x_argmax(tiny.data_ptr(), 2, 2, idx.data_ptr(), gpu.stream())); gpu.sync()
    assert idx.cpu().tolist()[:2] == [0, 0]
