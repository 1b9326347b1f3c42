"""Pins the oracle's RMSNorm, RoPE and attention against the reference's
golden attention.mim (nn/transformer_test.go:56-93,131-147; tolerance
atol 1e-5, rtol 1e-4 at :139) and against brute force."""
import os

import numpy as np
import pytest

import oracle as O
from mimir_amd.mimfile import golden_cases

ATOL, RTOL = 1e-5, 1e-4


@pytest.fixture(scope="module")
def cases(golden_dir):
    return golden_cases(os.path.join(golden_dir, "attention.mim"))


def close(got, want):
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= ATOL + RTOL * np.abs(want)), float(np.abs(got - want).max())


def test_rms_norm(cases):
    c = cases["rms_norm"]  # nn.NewRMSNorm(8, Eps(1e-6))
    close(O.rmsnorm(c["in"][0].data, c["in"][1].data, 1e-6), c["out"].data)
    c = cases["rms_norm_default_eps"]  # eps = 2^-23
    close(O.rmsnorm(c["in"][0].data, c["in"][1].data, 2.0 ** -23), c["out"].data)


def test_rms_norm_brute_force():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 4096)).astype(np.float32); w = rng.normal(1, 0.02, 4096).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-5) * w
    got = O.rmsnorm(x, w, 1e-5)
    assert np.abs(got - want).max() <= 1e-5


@pytest.mark.parametrize("name,dim,inter,off,scaling,params", [
    ("rope_neox", 8, False, 3, O.ROPE_NONE, ()),
    ("rope_interleaved", 8, True, 3, O.ROPE_NONE, ()),
    ("rope_partial_scaled", 8, False, 2, O.ROPE_LLAMA3, (8, 1, 4, 64)),
])
def test_rope_golden(cases, name, dim, inter, off, scaling, params):
    c = cases[name]
    x = c["in"][0].data
    cos, sin = O.rope_angles(dim, 10000.0, off, x.shape[-2], scaling, params)
    close(O.rope_apply(x, cos, sin, dim, inter), c["out"].data)


def test_rope_is_a_rotation_and_composes():
    """Invariants the mathematics fixes: pair norms are kept, position 0 is the
    identity, and turning by p then q equals turning by p+q."""
    rng = np.random.default_rng(1)
    x = rng.normal(size=(2, 1, 128)).astype(np.float32)
    c0, s0 = O.rope_angles(128, 500000.0, 0, 1)
    assert np.array_equal(O.rope_apply(x, c0, s0, 128, True), x)
    c5, s5 = O.rope_angles(128, 500000.0, 5, 1); c7, s7 = O.rope_angles(128, 500000.0, 7, 1)
    c12, s12 = O.rope_angles(128, 500000.0, 12, 1)
    y = O.rope_apply(O.rope_apply(x, c5, s5, 128, True), c7, s7, 128, True)
    assert np.abs(y - O.rope_apply(x, c12, s12, 128, True)).max() < 1e-5
    pairs = lambda t: (t.reshape(2, 64, 2).astype(np.float64) ** 2).sum(-1)
    assert np.abs(pairs(y) - pairs(x)).max() < 1e-5
    # linear scaling by 2 at position 2p equals no scaling at position p
    a = O.rope_angles(16, 10000.0, 6, 1, O.ROPE_LINEAR, (2.0,)); b = O.rope_angles(16, 10000.0, 3, 1)
    assert np.allclose(a[0], b[0], atol=1e-7) and np.allclose(a[1], b[1], atol=1e-7)
    # frequency factors divide each pair's frequency
    ff = np.full(8, 4.0, np.float32)
    a = O.rope_angles(16, 10000.0, 8, 1, freq_factors=ff); b = O.rope_angles(16, 10000.0, 2, 1)
    assert np.allclose(a[0], b[0], atol=1e-7) and np.allclose(a[1], b[1], atol=1e-7)


@pytest.mark.parametrize("name,kw", [
    ("sdpa", {}),
    ("sdpa_causal", {"causal": True}),
    ("sdpa_causal_offset", {"causal": True, "causal_offset": 4}),
    ("sdpa_gqa", {"causal": True, "causal_offset": 2}),
    ("sdpa_scale", {"scale": 0.3}),
    ("sdpa_mask", {"mask": 3}),
])
def test_sdpa_golden(cases, name, kw):
    c = cases[name]
    q, k, v = (t.data for t in c["in"][:3])
    kw = dict(kw)
    scale = kw.pop("scale", 1 / np.sqrt(q.shape[-1]))
    if "mask" in kw:
        kw["mask"] = c["in"][kw["mask"]].data
    out, _ = O.attention(q, k, v, scale, **kw)
    close(out, c["out"].data)


def _brute(q, k, v, scale, causal, off, klen):
    B, H, Q, D = q.shape; HK = k.shape[1]
    out = np.zeros((B, H, Q, v.shape[-1])); lse = np.zeros((B, H, Q))
    for b in range(B):
        for h in range(H):
            kk = k[b, h // (H // HK), :klen].astype(np.float64); vv = v[b, h // (H // HK), :klen].astype(np.float64)
            s = q[b, h].astype(np.float64) @ kk.T * scale
            if causal:
                i, j = np.indices(s.shape)
                s = np.where(j > i + off, -np.inf, s)
            m = s.max(-1, keepdims=True)
            p = np.exp(s - m)
            out[b, h] = p @ vv / p.sum(-1, keepdims=True)
            lse[b, h] = (m + np.log(p.sum(-1, keepdims=True)))[:, 0]
    return out, lse


def test_decode_attention_f16_cache_brute_force():
    """One query per head over a binary16 cache of capacity 64 holding 37
    positions, 8 query heads on 2 key heads: the decode shape in miniature."""
    rng = np.random.default_rng(2)
    B, H, HK, D, cap, n = 2, 8, 2, 128, 64, 37
    q = rng.normal(size=(B, H, 1, D)).astype(np.float32)
    kf = rng.normal(size=(B, HK, cap, D)).astype(np.float32); vf = rng.normal(size=(B, HK, cap, D)).astype(np.float32)
    kh, vh = O.f32_to_f16(kf), O.f32_to_f16(vf)
    out, lse = O.attention(q, kh, vh, 1 / np.sqrt(D), kv_dt=O.F16, k_len=n)
    wo, wl = _brute(q, O.f16_to_f32(kh), O.f16_to_f32(vh), 1 / np.sqrt(D), False, 0, n)
    assert np.abs(out - wo).max() < 2e-6 and np.abs(lse - wl).max() < 1e-5
    # causal with offset n-1 over the whole capacity hides the same keys
    out2, _ = O.attention(q, kh, vh, 1 / np.sqrt(D), causal=True, causal_offset=n - 1, kv_dt=O.F16)
    assert np.array_equal(out, out2)


def test_attention_row_that_sees_no_key():
    q = np.ones((1, 1, 2, 4), np.float32); k = np.ones((1, 1, 3, 4), np.float32); v = np.ones((1, 1, 3, 4), np.float32)
    out, lse = O.attention(q, k, v, 1.0, causal=True, causal_offset=-1)  # row 0 sees nothing
    assert not out[0, 0, 0].any() and lse[0, 0, 0] == -np.inf
    assert np.allclose(out[0, 0, 1], 1)


def test_silu_and_argmax():
    g = np.linspace(-20, 20, 101).astype(np.float32); u = np.linspace(1, 2, 101).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.abs(O.silu_mul(g, u) - want).max() < 2e-6
    assert O.silu_mul(np.array([-200.0], np.float32), np.array([1.0], np.float32))[0] == 0  # 0, not NaN
    assert O.argmax([1, 3, 3, 2]) == 1            # first index wins ties (generate.go:46-51)
    assert O.argmax([np.nan, 1, 2]) == 0          # v > NaN is false
