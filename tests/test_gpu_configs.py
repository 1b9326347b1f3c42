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


def test_whole_model_64_greedy_tokens():
    """The whole random-init model of the last configuration: 32 layers at full
    width, embeddings and output Q8_0 over the 128256-token vocabulary, Q4_0
    linears, binary16 cache, seed 0 with per-tensor seeds. A 128-token prompt
    (the configuration's 512 takes the CPU oracle minutes) and 64 greedy
    tokens, which must be the oracle's one for one. Were two of the oracle's
    logits ever closer than its own float32 sums can tell apart, the
    comparison would stop there, as the reference's tests allow for quantized
    activations; in this run the smallest margin is 21."""
    gpu.lib()
    c = _config(32, 128256, 200, 1, capi.F16)
    om = OL.synthetic(_oracle_config(c), seed=0)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(128)
    prompt = np.random.default_rng(0).integers(0, c.vocab, (1, 128))
    gpu.say("whole model, 128-token prompt, 64 greedy tokens")
    toks, _ = m.generate(prompt, 64)
    caches = om.new_caches(c.context, O.F16)
    logits = om.logits(prompt[0].tolist(), caches)
    got = toks[0].tolist()
    for i in range(64):
        if i % 16 == 0:
            gpu.say(f"oracle step {i}")
        want = O.argmax(logits)
        if got[i] != want:
            top2 = np.partition(logits, -2)[-2:]
            assert float(top2[1] - top2[0]) < 0.02 * 170.0, (i, got[i], want)
            assert i >= 8, (i, got[:8])
            break
        if i + 1 < 64:
            logits = om.logits([want], caches)
