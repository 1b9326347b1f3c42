"""The benchmark configurations that name a decoder: one random-init layer at
the 8B model's shape stepping once against a binary16 cache prefilled with
2048 positions of N(0, 1) values, batch 1 and 8; and the whole
32-layer model decoding 64 greedy tokens, which must be the oracle's."""
import numpy as np
import pytest

import oracle as O
from mimir_amd import capi
from mimir_amd.llama import Llama
from oracle import llama as OL
from tests import gpu
from tests.test_gpu_llama import _oracle_config, _upload_synthetic

pytestmark = pytest.mark.gpu


def _config(layers, vocab, context, batch, cache):
    c = capi.LlamaConfig()
    c.embed, c.hidden, c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.vocab = 4096, 14336, layers, 32, 8, 128, 128, vocab
    c.context, c.interleaved, c.cache_dtype, c.batch = context, 1, cache, batch
    c.rope_base, c.rope_scale, c.eps = 500000.0, 1.0, 1e-5
    return c


@pytest.mark.parametrize("batch", [1, 8])
def test_one_layer_step_against_a_prefilled_cache(batch):
    """hidden 4096, 32 query heads on 8 key heads of 128, SwiGLU 14336, eps 1e-5,
    theta 500000, Q4_0 linears; position 2048. The output projection is Q4_0
    over a small vocabulary so that the comparison sees the layer: float32
    sums in two orders, and the step's own key and value rounded to binary16 on
    both sides (a last-bit difference before a rounding boundary moves the
    stored value by a binary16 step), held to 5e-4 of the largest logit (asked:
    1e-3; most sequences land near 1e-5)."""
    gpu.lib()
    past = 2048
    c = _config(1, 512, 2304, batch, capi.F16)
    om = OL.synthetic(_oracle_config(c), seed=0, output_dt=O.Q4_0)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(4)
    rng = np.random.default_rng(4)
    keys = O.f32_to_f16(rng.normal(size=(batch, c.kv_heads, past, c.head_dim)).astype(np.float32))
    values = O.f32_to_f16(rng.normal(size=(batch, c.kv_heads, past, c.head_dim)).astype(np.float32))
    gpu.say(f"one layer, one step at position {past}, batch {batch}")
    m.set_cache(0, keys, values)
    assert m.cache_len == past
    tokens = rng.integers(0, c.vocab, (batch, 1))
    got = m.logits(tokens)
    assert m.cache_len == past + 1
    for b in range(batch):
        caches = om.new_caches(c.context, O.F16)
        caches[0].keys[:, :past] = keys[b]; caches[0].values[:, :past] = values[b]; caches[0].n = past
        want = om.logits(tokens[b].tolist(), caches)
        err = np.abs(got[b] - want).max() / np.abs(want).max()
        assert err <= 5e-4, (b, float(err))
    # the same step through the fused launches and their graph: the tokens it chooses are the logits' largest
    m.set_cache(0, keys, values)
    toks, _ = m.generate(tokens, 3)
    assert toks[:, 0].tolist() == [int(np.argmax(got[b])) for b in range(batch)]


@pytest.fixture(scope="module")
def whole_model():
    """The oracle's copy of the whole random-init model of the last configuration (32 layers at full width,
    embeddings and output Q8_0 over the 128256-token vocabulary, Q4_0 linears; seed 0 with per-tensor seeds)."""
    return OL.synthetic(_oracle_config(_config(32, 128256, 200, 1, capi.F16)), seed=0)


def _logits_close(got, want, what):
    """The reference's bound for a model with quantized weights (2 % of the largest logit,
    examples/llama/llama_test.go:177) on every logit, and the median far inside it: the Q8_0 head rounds
    its input to int8 on both sides, a step function of the hidden state's last bits."""
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert err.max() <= 0.02 * scale and np.median(err) <= 1e-5 * scale, (what, float(err.max() / scale), float(np.median(err) / scale))


def test_whole_model_64_greedy_tokens(whole_model):
    """A 128-token prompt (the configuration's 512 is what bench.py checks in its default run) and 64 greedy
    tokens through the fused launches replayed as a graph: every one must be the oracle's, with no allowance
    for close logits (a mismatch prints the oracle's margin at that step). The logits themselves are compared
    at the end of the prompt and at the step that chooses token 63, through Model.Logits."""
    gpu.lib()
    om = whole_model
    c = _config(32, 128256, 200, 1, capi.F16)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(128)
    prompt = np.random.default_rng(0).integers(0, c.vocab, (1, 128))
    gpu.say("whole model, 128-token prompt, 64 greedy tokens")
    toks, _ = m.generate(prompt, 64)
    got = toks[0].tolist()
    caches = om.new_caches(c.context, O.F16)
    logits = om.logits(prompt[0].tolist(), caches)
    prompt_logits = logits
    want, margins = [], []
    for i in range(64):
        if i % 16 == 0:
            gpu.say(f"oracle step {i}")
        want.append(O.argmax(logits))
        top2 = np.partition(logits, -2)[-2:]
        margins.append(float(top2[1] - top2[0]))
        if i + 1 < 64:
            logits = om.logits([want[-1]], caches)
    first = next((i for i in range(64) if got[i] != want[i]), None)
    assert first is None, f"token {first}: device {got[first]}, oracle {want[first]}, oracle's margin there {margins[first]:.4g} (smallest of the run {min(margins):.4g})"
    # the logits: end of the prompt, then the oracle's tokens fed one by one up to the step that chooses token 63
    m.reset()
    gpu.say("whole model: logits at the end of the prompt and at step 63")
    _logits_close(m.logits(prompt)[0], prompt_logits, "end of the prompt")
    for t in want[:63]:
        last = m.logits(np.array([[t]]))[0]
    _logits_close(last, logits, "step 63")


def test_whole_model_batch_8_greedy_tokens(whole_model):
    """The same model decoding eight sequences in lockstep (the step that reads every weight once for all of
    them): a 48-token prompt each and 64 greedy tokens. Two of the sequences are held to the oracle's for all
    64 tokens, the other six for their first 16 (the oracle decodes a token a second)."""
    gpu.lib()
    om = whole_model
    c = _config(32, 128256, 112, 8, capi.F16)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(48)
    prompts = np.random.default_rng(1).integers(0, c.vocab, (8, 48))
    gpu.say("whole model, batch 8, 48-token prompts, 64 greedy tokens")
    toks, _ = m.generate(prompts, 64)
    for b in range(8):
        n = 64 if b in (0, 5) else 16
        gpu.say(f"oracle sequence {b}, {n} tokens")
        want, margins = om.generate(prompts[b].tolist(), n, capacity=c.context, cache_dtype=O.F16)
        got = toks[b].tolist()
        first = next((i for i in range(n) if got[i] != want[i]), None)
        assert first is None, f"sequence {b} token {first}: device {got[first]}, oracle {want[first]}, oracle's margin there {margins[first]:.4g}"


@pytest.mark.parametrize("batch", [1, 3])
def test_model_whose_greedy_tokens_vary_with_small_margins(batch):
    """The random-init model above repeats one token: uniform nibbles 0..15 average -0.5, so every linear adds a
    common-mode term that swamps what depends on the input. Here the Q4_0 linears are drawn without a mean (nibbles
    1..15): four layers at full width, a Q4_0 output projection over 32000 tokens (no int8 rounding of its input,
    so close calls are decided by float32 arithmetic alone). The oracle's 64 greedy tokens for this prompt are all
    different, the two best logits are within 1 of each other at more than twenty steps and within 0.17 (0.6 % of
    the largest logit) at the closest: the device must choose the same token every time, one sequence alone and in
    a batch."""
    gpu.lib()
    c = _config(4, 32000, 128, batch, capi.F16)
    om = OL.synthetic(_oracle_config(c), seed=0, centered=True, output_dt=O.Q4_0)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(32)
    prompt = np.random.default_rng(1).integers(0, c.vocab, 32)
    gpu.say(f"varied model, batch {batch}: oracle")
    want, margins = om.generate(prompt.tolist(), 64, capacity=c.context, cache_dtype=O.F16)
    assert len(set(want)) >= 20 and min(margins) < 1.0 and sum(mg < 1.0 for mg in margins) >= 10, (len(set(want)), sorted(margins)[:12])
    gpu.say(f"varied model, batch {batch}: device")
    toks, _ = m.generate(np.tile(prompt, (batch, 1)), 64)
    for b in range(batch):
        got = toks[b].tolist()
        first = next((i for i in range(64) if got[i] != want[i]), None)
        assert first is None, f"sequence {b} token {first}: device {got[first]}, oracle {want[first]}, oracle's margin there {margins[first]:.4g} (smallest {min(margins):.4g})"
