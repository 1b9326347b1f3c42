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
        assert O.argmax(row) == t or margins[i] < 1e-3
