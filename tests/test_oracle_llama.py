"""Pins the oracle's Llama forward against the logits the reference's own
tests hold: examples/llama/testdata/{spm,bpe}.logits.mim
(examples/llama/llama_test.go:160-222) and io/mim/testdata/llama/expected.json
(io/mim/mim_test.go:184-262), with those tests' tolerances."""
import base64
import json
import os

import numpy as np
import pytest

import oracle as O
from mimir_amd.mimfile import MimFile
from oracle.llama import Model


def compare_logits(got, want, vocab, tol):
    """compareLogits (examples/llama/llama_test.go:120-144)."""
    got = np.asarray(got, np.float64).reshape(-1, vocab); want = np.asarray(want, np.float64).reshape(-1, vocab)
    scale = np.abs(want).max()
    worst = np.abs(got - want).max(1)
    assert np.all(worst <= tol * scale), f"differs by {worst.max():.4g}, {100 * worst.max() / scale:.2g}% of {scale:.3g}"
    for p in range(want.shape[0]):
        a, b = O.argmax(got[p]), O.argmax(want[p])
        assert a == b or abs(want[p, a] - want[p, b]) <= tol * scale, f"position {p} picks {a}, want {b}"
    return worst.max() / scale


@pytest.mark.parametrize("name,deq,tol", [("spm", True, 1e-4), ("bpe", True, 1e-4), ("spm", False, 0.02), ("bpe", False, 0.04)])
def test_logits_match_the_reference_fixtures(golden_dir, name, deq, tol):
    m = Model.from_mim(MimFile(os.path.join(golden_dir, f"{name}.mim")), dequantized=deq)
    ref = MimFile(os.path.join(golden_dir, f"{name}.logits.mim"))
    tokens, want = ref["tokens"].data.tolist(), ref["logits"].data
    v = m.config.vocab
    batched = m.logits(tokens, m.new_caches(len(tokens)), all=True)
    compare_logits(batched, want, v, tol)
    caches = m.new_caches(len(tokens))
    stepped = np.stack([m.logits([t], caches) for t in tokens])
    compare_logits(stepped, want, v, tol)
    compare_logits(stepped, batched, v, 1e-4)


@pytest.fixture(scope="module")
def expected(golden_dir):
    e = json.load(open(os.path.join(golden_dir, "expected.json")))
    dec = lambda s: np.frombuffer(base64.b64decode(s), "<f4")
    return {"vocab": e["vocab"], "prompt": e["prompt_ids"], "prompt_logits": dec(e["prompt_logits"]), "greedy": e["greedy"],
            "greedy_logits": [dec(s) for s in e["greedy_logits"]], "llama_cpp": e["llama_cpp_max_diff"]}


@pytest.mark.parametrize("name,deq,cache,tol,abs_tol", [
    ("exact", True, O.F32, 2e-5, None),        # weights decoded, float32 products, float32 cache
    ("f16-cache", True, O.F16, 1e-3, None),    # the only reference-held vector for a binary16 cache
    ("a8", False, O.F16, None, 1.5),           # int8 activations: within 1.5x of llama.cpp's own distance
])
def test_quantized_llama_known_answers(golden_dir, expected, name, deq, cache, tol, abs_tol):
    e = expected
    m = Model.from_mim(MimFile(os.path.join(golden_dir, "tiny-q4km-exact.mim")), dequantized=deq)
    v = e["vocab"]

    def near(got, want):
        scale = np.abs(want).max()
        lim = abs_tol * e["llama_cpp"] if abs_tol else tol * scale
        assert np.abs(np.asarray(got, np.float64) - want).max() <= lim

    caches = m.new_caches(64, cache)
    all_ = m.logits(e["prompt"], caches, all=True)
    near(all_.reshape(-1), e["prompt_logits"])
    logits = all_[-1]
    for i, want_tok in enumerate(e["greedy"]):
        near(logits, e["greedy_logits"][i])
        if abs_tol is None:
            assert O.argmax(logits) == want_tok, f"step {i}"
        logits = m.logits([want_tok], caches)


def test_generate_is_the_argmax_of_a_full_pass(golden_dir):
    """examples/llama/llama_test.go:226-260: greedy generation equals the
    argmax of one pass over the whole sequence."""
    m = Model.from_mim(MimFile(os.path.join(golden_dir, "spm.mim")))
    prompt = [1, 17, 42, 99]
    out, margins = m.generate(prompt, 6)
    seq = prompt + out
    full = m.logits(seq[:-1], m.new_caches(len(seq)), all=True)
    for i, t in enumerate(out):
        row = full[len(prompt) - 1 + i]
        assert O.argmax(row) == t, f"token {i}: a full pass picks {O.argmax(row)}, cached steps picked {t}, margin there {margins[i]:.4g}"


# ---- qwen2: biases on the queries, keys and values, rotation over halves -------------------------
# The reference's only expectation for this model is the graph inside qwen2-exact.mim
# (llm/llm_test.go:36-39,131-160 compares Model with that graph), and the graph section's
# encoding lives in the mimir-model module, which the reference does not vendor. So this path
# has no reference-held vector; it is held by what the mathematics fixes instead.

QWEN_PROMPT = [1, 79, 110, 99, 101, 363, 264, 315, 307, 280]  # llm/llm_test.go:41


def _float64_forward(m: Model, tokens):
    """A second formulation of the same function: every position at once in float64, an explicit causal
    mask, softmax by its definition, the rotation written from RoPE's formula for the halves layout
    (feature i pairs with i + rope_dim/2), the bias added where Linear adds it. Shares no code with
    Model.logits beyond the weights' decoding."""
    c = m.config
    deq = lambda w: np.asarray(w.dequantized().data, np.float64).reshape(w.n, w.k)
    x = deq(m.embed)[np.asarray(tokens)]
    s = len(tokens)
    half = c.rope_dim // 2
    ang = np.arange(s)[:, None] * (c.rope_base ** (-2.0 * np.arange(half) / c.rope_dim))[None, :] / c.rope_scale
    cos, sin = np.cos(ang), np.sin(ang)

    def norm(v, w):
        return v / np.sqrt((v * v).mean(-1, keepdims=True) + c.eps) * w

    def rope(t):  # [s, heads, dim]
        a, b = t[..., :half].copy(), t[..., half:c.rope_dim].copy()
        out = t.copy()
        out[..., :half] = a * cos[:, None, :] - b * sin[:, None, :]
        out[..., half:c.rope_dim] = a * sin[:, None, :] + b * cos[:, None, :]
        return out

    for blk in m.blocks:
        h = norm(x, blk.attn_norm)
        q = (h @ deq(blk.q).T + blk.q_bias).reshape(s, c.heads, c.head_dim)
        k = (h @ deq(blk.k).T + blk.k_bias).reshape(s, c.kv_heads, c.head_dim)
        v = (h @ deq(blk.v).T + blk.v_bias).reshape(s, c.kv_heads, c.head_dim)
        q, k = rope(q), rope(k)
        g = c.heads // c.kv_heads
        att = np.empty((s, c.heads, c.head_dim))
        mask = np.where(np.arange(s)[None, :] <= np.arange(s)[:, None], 0.0, -np.inf)
        for hh in range(c.heads):
            sc = q[:, hh] @ k[:, hh // g].T / np.sqrt(c.head_dim) + mask
            p = np.exp(sc - sc.max(-1, keepdims=True))
            att[:, hh] = (p / p.sum(-1, keepdims=True)) @ v[:, hh // g]
        x = x + att.reshape(s, -1) @ deq(blk.o).T
        h = norm(x, blk.ffn_norm)
        gate, up = h @ deq(blk.gate).T, h @ deq(blk.up).T
        x = x + (gate / (1 + np.exp(-gate)) * up) @ deq(blk.down).T
    return norm(x, m.norm) @ deq(m.output).T


def test_qwen2_biases_and_halves_rotation(golden_dir):
    f = MimFile(os.path.join(golden_dir, "qwen2-exact.mim"))
    m = Model.from_mim(f, dequantized=True)
    assert m.config.arch == "qwen2" and not m.config.interleaved
    assert all(b.q_bias is not None and b.k_bias is not None and b.v_bias is not None for b in m.blocks)
    assert max(float(np.abs(b.q_bias).max()) for b in m.blocks) > 0  # the file's biases are not zeros: dropping them would show
    want = _float64_forward(m, QWEN_PROMPT)
    got = m.logits(QWEN_PROMPT, m.new_caches(64), all=True)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-5 * scale
    # a dropped bias, one added behind the rotation, or the pairs layout in place of the halves: each is far outside that bound
    for wrong in ("no_bias", "pairs"):
        m2 = Model.from_mim(f, dequantized=True)
        if wrong == "no_bias":
            for b in m2.blocks:
                b.k_bias = np.zeros_like(b.k_bias)
        else:
            m2.config.arch = "llama"
        bad = m2.logits(QWEN_PROMPT, m2.new_caches(64), all=True)
        assert np.abs(bad - want).max() > 1e-3 * scale, wrong
    # one token at a time through the caches (llm/llm_test.go:146-160), and int8 activations stay near
    caches = m.new_caches(64)
    stepped = np.stack([m.logits([t], caches) for t in QWEN_PROMPT])
    assert np.abs(stepped - got).max() <= 1e-4 * scale
    a8 = Model.from_mim(f).logits(QWEN_PROMPT, Model.from_mim(f).new_caches(64), all=True)
    assert np.abs(a8 - want).max() <= 0.05 * scale


def test_q4_0_container_code_is_the_callers(tmp_path):
    """The reference's fixtures hold no Q4_0 tensor and its accounting no code for one: MimFile refuses an
    unknown code, and reads it as 18-byte blocks of 32 when the caller names it as Q4_0's."""
    from mimir_amd.mimfile import MimError
    from oracle.llama import Config, synthetic
    from tests.helpers import synthetic_llama_mim
    c = Config(embed=128, hidden=256, layers=1, heads=2, kv_heads=1, head_dim=64, rope_dim=64, vocab=96, context=16)
    om = synthetic(c, seed=3)
    path = str(tmp_path / "q4_0.mim")
    synthetic_llama_mim(path, om, q4_0_code=65)
    with pytest.raises(MimError):
        MimFile(path)
    with pytest.raises(MimError):
        MimFile(path, q4_0_code=64)  # Q8_0's
    f = MimFile(path, q4_0_code=65)
    t = f["blk.0.attn_q.weight"]
    assert t.dtype_name == "q4_0" and t.quantized and t.shape == (128, 128) and t.data.nbytes == 128 * 128 // 32 * 18
    assert f["token_embd.weight"].dtype_name == "q8_0"
    m = Model.from_mim(f)
    toks = [5, 17, 80, 3]
    assert np.array_equal(m.logits(toks, m.new_caches(16)), om.logits(toks, om.new_caches(16)))
