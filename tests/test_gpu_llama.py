"""The device decoder against the reference's golden logits and against the
oracle's Llama forward, on a real MI355X: the tiny fixture models (Q8_0, F16,
BF16, F32, Q4_K and Q6_K weights), and a random-init Q4_0 / Q8_0 model at
reduced size with 8B-like proportions."""
import base64
import json
import os

import numpy as np
import pytest

import oracle as O
from mimir_amd import capi
from mimir_amd.llama import Llama, load_mim
from mimir_amd.mimfile import MimFile
from oracle import llama as OL
from tests import gpu
from tests.test_oracle_llama import compare_logits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,tol", [("spm", 0.02), ("bpe", 0.04)])
def test_fixture_models_match_golden_logits_and_oracle(golden_dir, name, tol):
    gpu.lib()
    path = os.path.join(golden_dir, f"{name}.mim")
    ref = MimFile(os.path.join(golden_dir, f"{name}.logits.mim"))
    tokens, want = ref["tokens"].data.tolist(), ref["logits"].data
    gpu.say(f"llama fixture {name}: batched pass")
    m = load_mim(path, max_tokens=len(tokens), context=len(tokens))
    v = m.config.vocab
    batched = m.logits(tokens, all=True)[0]
    compare_logits(batched, want, v, tol)  # examples/llama/llama_test.go:177: quantized weights, 2% / 4%
    # the oracle computes the same int8-activation products: far closer than that
    om = OL.Model.from_mim(MimFile(path))
    ow = om.logits(tokens, om.new_caches(len(tokens)), all=True)
    compare_logits(batched, ow, v, 1e-4)
    gpu.say(f"llama fixture {name}: one token at a time")
    m.reset()
    stepped = np.stack([m.logits([t])[0] for t in tokens])
    compare_logits(stepped, batched, v, 1e-4)  # llama_test.go:216
    assert m.cache_len == len(tokens)


def test_tiny_q4km_known_answers_with_f16_cache(golden_dir):
    """io/mim/mim_test.go:184-262: prompt logits, 8 greedy tokens and each
    step's logits, with a binary16 cache; int8 activations ("a8": within 1.5x
    of llama.cpp's own distance from the float64 oracle)."""
    e = json.load(open(os.path.join(golden_dir, "expected.json")))
    dec = lambda s: np.frombuffer(base64.b64decode(s), "<f4")
    gpu.lib()
    gpu.say("tiny-q4km a8")
    m = load_mim(os.path.join(golden_dir, "tiny-q4km-exact.mim"), max_tokens=16, context=64, cache_dtype=capi.F16)
    lim = 1.5 * e["llama_cpp_max_diff"]
    all_ = m.logits(e["prompt_ids"], all=True)[0]
    assert np.abs(all_.reshape(-1) - dec(e["prompt_logits"])).max() <= lim
    logits = all_[-1]
    om = OL.Model.from_mim(MimFile(os.path.join(golden_dir, "tiny-q4km-exact.mim")))
    caches = om.new_caches(64, O.F16)
    ologits = om.logits(e["prompt_ids"], caches, all=True)[-1]
    for i, tok in enumerate(e["greedy"]):
        assert np.abs(logits - dec(e["greedy_logits"][i])).max() <= lim
        assert np.abs(logits - ologits).max() <= 1e-4 * np.abs(ologits).max()  # the same arithmetic as the CPU path
        logits = m.logits([tok])[0]
        ologits = om.logits([tok], caches)
    # greedy generation picks what the oracle picks
    m.reset()
    got, _ = m.generate(e["prompt_ids"], 8)
    want, margins = om.generate(e["prompt_ids"], 8, capacity=64, cache_dtype=O.F16)
    for i, (a, b) in enumerate(zip(got[0].tolist(), want)):
        assert a == b, f"token {i}: device {a}, oracle {b}, the oracle's margin there {margins[i]:.4g}"


@pytest.mark.parametrize("cache", [capi.F32, capi.F16])
def test_qwen2_biases_on_queries_keys_and_values(golden_dir, cache):
    """The reference's qwen2 fixture (llm/llm_test.go:36-39): biases on q, k and v added behind the products and
    before the rotation (llm/model.go:251-258, nn/layers.go:49-55), rotation over halves. Every position of the
    prompt at once, then token by token through the caches, then greedy tokens: against the oracle's model, which
    multiplies with int8 activations as the device does."""
    path = os.path.join(golden_dir, "qwen2-exact.mim")
    prompt = [1, 79, 110, 99, 101, 363, 264, 315, 307, 280]
    gpu.lib()
    gpu.say(f"qwen2, cache dtype {cache}")
    m = load_mim(path, max_tokens=16, context=64, cache_dtype=cache)
    om = OL.Model.from_mim(MimFile(path))
    ocache = O.F32 if cache == capi.F32 else O.F16
    want = om.logits(prompt, om.new_caches(64, ocache), all=True)
    got = m.logits(prompt, all=True)[0]
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-4 * scale
    m.reset()
    caches = om.new_caches(64, ocache)
    for t in prompt:
        assert np.abs(m.logits([t])[0] - om.logits([t], caches)).max() <= 1e-4 * scale
    owant, margins = om.generate(prompt, 12, capacity=64, cache_dtype=ocache)
    # the decoding step three ways: launched operator by operator with the position from the host (2), its device-resident
    # form, where one launch adds the biases, rotates and writes the caches (1), and that form replayed from a graph (0, twice)
    lib = gpu.lib()
    try:
        for mode in (2, 1, 0, 0):
            gpu.say(f"qwen2, cache dtype {cache}: step mode {mode}")
            capi.check(lib.mi355x_tune(b"llama.step", mode))
            m.reset()
            toks, _ = m.generate(prompt, 12)
            assert toks[0].tolist() == owant, (mode, toks[0].tolist(), owant, min(margins))
    finally:
        capi.check(lib.mi355x_tune(b"llama.step", 0))


def test_some_but_not_all_biases_is_an_error(golden_dir):
    gpu.lib()
    path = os.path.join(golden_dir, "qwen2-exact.mim")
    f = MimFile(path)
    from mimir_amd.llama import config_from_metadata, _MIM_TO_ABI
    m = Llama(config_from_metadata(f.metadata, f["token_embd.weight"].shape[0], context=16))
    for name, t in f.tensors.items():
        if name.endswith(".weight"):
            m.set_tensor(name, _MIM_TO_ABI[t.dtype_name], t.data, int(np.prod(t.shape)))
    m.set_tensor("blk.0.attn_q.bias", capi.F32, f["blk.0.attn_q.bias"].data, int(np.prod(f["blk.0.attn_q.bias"].shape)))
    with pytest.raises(capi.Mi355xError) as ei:
        m.finalize(8)
    assert ei.value.status == capi.ERR_SHAPE


def test_q4_0_tensors_from_a_file_under_the_callers_code(tmp_path):
    """A .mim file whose Q4_0 tensors carry a container code that the caller names (the reference's fixtures
    hold none): load_mim uploads them as Q4_0 and the model decodes as the oracle's copy of it does."""
    from oracle.llama import Config, synthetic
    from tests.helpers import synthetic_llama_mim
    gpu.lib()
    oc = Config(embed=512, hidden=1024, layers=2, heads=4, kv_heads=2, head_dim=128, rope_dim=128, vocab=320, context=32, rope_base=500000.0)
    om = synthetic(oc, seed=5)
    path = str(tmp_path / "q4_0.mim")
    synthetic_llama_mim(path, om, q4_0_code=65)
    gpu.say("a .mim file with Q4_0 tensors")
    m = load_mim(path, max_tokens=8, q4_0_code=65, cache_dtype=capi.F16)
    prompt = [3, 200, 41, 7, 19]
    want = om.logits(prompt, om.new_caches(32, O.F16))
    got = m.logits(prompt)[0]
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    m.reset()
    toks, _ = m.generate(prompt, 8)
    owant, margins = om.generate(prompt, 8, capacity=32, cache_dtype=O.F16)
    assert toks[0].tolist() == owant, (toks[0].tolist(), owant, min(margins))


def test_errors_before_anything_is_queued(golden_dir):
    gpu.lib()
    m = load_mim(os.path.join(golden_dir, "spm.mim"), max_tokens=8, context=8)
    with pytest.raises(capi.Mi355xError) as ei:
        m.logits([1, 2, 400])  # llm/model.go:396-400
    assert ei.value.status == capi.ERR_INDEX
    with pytest.raises(capi.Mi355xError) as ei:
        m.logits(list(range(9)))
    assert ei.value.status == capi.ERR_SHAPE
    m.logits([1, 2, 3, 4, 5, 6, 7])
    with pytest.raises(capi.Mi355xError) as ei:  # a full cache (nn/transformer.go:408-411)
        m.logits([1, 2])
    assert ei.value.status == capi.ERR_SHAPE
    assert m.cache_len == 7


def _small_q4_config(batch, cache):
    c = capi.LlamaConfig()
    c.embed, c.hidden, c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.vocab = 512, 1792, 3, 4, 1, 128, 128, 1003
    c.context, c.interleaved, c.cache_dtype, c.batch = 96, 1, cache, batch
    c.rope_base, c.rope_scale, c.eps = 500000.0, 1.0, 1e-5
    return c


def _upload_synthetic(m: Llama, om: OL.Model):
    dt = {O.Q4_0: capi.Q4_0, O.Q8_0: capi.Q8_0, O.Q4_K: capi.Q4_K, O.Q6_K: capi.Q6_K}
    m.set_tensor("token_embd.weight", dt[om.embed.dtype], om.embed.data, om.embed.n * om.embed.k)
    m.set_tensor("output.weight", dt[om.output.dtype], om.output.data, om.output.n * om.output.k)
    m.set_tensor("output_norm.weight", capi.F32, om.norm, om.norm.size)
    for i, b in enumerate(om.blocks):
        p = f"blk.{i}."
        m.set_tensor(p + "attn_norm.weight", capi.F32, b.attn_norm, b.attn_norm.size)
        m.set_tensor(p + "ffn_norm.weight", capi.F32, b.ffn_norm, b.ffn_norm.size)
        for leaf, w in (("attn_q", b.q), ("attn_k", b.k), ("attn_v", b.v), ("attn_output", b.o), ("ffn_gate", b.gate), ("ffn_up", b.up), ("ffn_down", b.down)):
            m.set_tensor(p + leaf + ".weight", dt[w.dtype], w.data, w.n * w.k)


def _oracle_config(c):
    return OL.Config(arch="llama", embed=c.embed, hidden=c.hidden, layers=c.layers, heads=c.heads, kv_heads=c.kv_heads, head_dim=c.head_dim,
                     rope_dim=c.rope_dim, rope_base=c.rope_base, rope_scale=1.0, eps=c.eps, vocab=c.vocab, context=c.context)


def test_random_init_model_without_rounding_steps_is_close_everywhere():
    """Q4_0 linears, a Q4_0 output projection and a float32 cache: nothing on
    the way rounds to int8 or binary16, so the device and the CPU reference
    differ by float32 rounding alone: about 2e-7 of the largest logit at almost
    every position, which is also how far the float32 reference itself is from
    a float64 forward. One position of this prompt is ill-conditioned (the
    reference is 3e-5 from float64 there); it stays within 1e-3."""
    gpu.lib()
    c = _small_q4_config(1, capi.F32)
    om = OL.synthetic(_oracle_config(c), seed=0, output_dt=O.Q4_0)
    gpu.say("random-init q4_0 model, q4_0 output, f32 cache")
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(40)
    prompt = np.random.default_rng(0).integers(0, c.vocab, (1, 33))
    got = m.logits(prompt, all=True)[0]
    want = om.logits(prompt[0].tolist(), om.new_caches(c.context, O.F32), all=True)
    err = np.abs(got - want).max(1) / np.abs(want).max()
    assert err.max() <= 1e-3 and np.quantile(err, 0.9) <= 2e-6, err


@pytest.mark.parametrize("batch", [1, 3])
def test_random_init_q4_0_model_matches_oracle_and_greedy_tokens(batch):
    """A random-init decoder in the 8B model's proportions (heads of 128, four
    query heads a key head, SwiGLU 3.5x, theta 500000, Q4_0 linears, Q8_0
    embeddings and output), binary16 cache. The Q8_0 output projection rounds
    its input to int8 on both sides (backend/cpu/qmatmul.go:208-254), a step
    function: where a value sits on a rounding boundary, the last bit of the
    hidden state decides a quant, so single logits move by about 1e-3 of the
    largest. The bound is the reference's own for quantized weights, 2%
    (examples/llama/llama_test.go:177), with most positions far inside it; the
    greedy tokens are the same except where the reference's own top two logits
    are that close."""
    gpu.lib()
    c = _small_q4_config(batch, capi.F16)
    om = OL.synthetic(_oracle_config(c), seed=0)
    gpu.say(f"random-init q4_0 model batch={batch}")
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(40)
    rng = np.random.default_rng(0)
    prompts = rng.integers(0, c.vocab, (batch, 33))
    got = m.logits(prompts, all=True)
    for b in range(batch):
        want = om.logits(prompts[b].tolist(), om.new_caches(c.context, O.F16), all=True)
        scale = np.abs(want).max()
        err = np.abs(got[b] - want).max(1) / scale
        assert err.max() <= 0.02 and np.median(np.abs(got[b] - want)) <= 1e-5 * scale, (float(err.max()), err)
    m.reset()
    toks, _ = m.generate(prompts, 24)
    for b in range(batch):
        want, margins = om.generate(prompts[b].tolist(), 24, capacity=c.context, cache_dtype=O.F16)
        scale = 170.0
        for i, (a, w) in enumerate(zip(toks[b].tolist(), want)):
            assert a == w, f"token {i}: device {a}, oracle {w}, oracle's margin there {margins[i]:.4g}"


@pytest.mark.parametrize("batch,cache", [(1, capi.F32), (2, capi.F16)])
def test_fused_and_graph_replayed_steps_choose_the_per_operator_tokens(batch, cache):
    """The decoding step exists three times: per operator (what the logits tests
    above pin against the oracle), fused launches (norm with conversion, q|k|v
    in one product, rotation with the cache write, SwiGLU and residual
    epilogues), and those launches replayed as a graph that reads position and
    tokens from device memory. All three must choose the same tokens, replay
    after replay, and again on a second call that starts from another cache
    length with the graph the first call built."""
    lib = gpu.lib()
    c = _small_q4_config(batch, cache)
    om = OL.synthetic(_oracle_config(c), seed=1, output_dt=O.Q4_0)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(40)
    rng = np.random.default_rng(5)
    runs = {}
    try:
        for mode in (2, 1, 0, 0):
            gpu.say(f"generate, step mode {mode}, batch {batch}")
            capi.check(lib.mi355x_tune(b"llama.step", mode))
            m.reset()
            prompts = np.random.default_rng(5).integers(0, c.vocab, (batch, 9))
            first, _ = m.generate(prompts, 30)
            assert m.cache_len == 9 + 29
            # a second call continues the same caches from where the first stopped
            more, _ = m.generate(first[:, -1:], 12)
            assert m.cache_len == 9 + 29 + 1 + 11
            runs.setdefault(mode, []).append(np.concatenate([first, more], 1))
    finally:
        capi.check(lib.mi355x_tune(b"llama.step", 0))
    # the per-operator steps against the oracle, then the others against them
    want, margins = om.generate(prompts[0].tolist(), 30, capacity=c.context, cache_dtype=O.F32 if cache == capi.F32 else O.F16)
    got = runs[2][0][0, :30].tolist()
    for i, (a, w) in enumerate(zip(got, want)):
        assert a == w, f"token {i}: device {a}, oracle {w}, oracle's margin there {margins[i]:.4g}"
    # attention splits the keys differently when the position comes from the
    # device (a fixed plan for the whole context), so a sum may round another
    # way; tokens differ only if two logits tie to that precision
    same = [np.array_equal(runs[2][0], r) for r in (runs[1][0], runs[0][0], runs[0][1])]
    assert np.array_equal(runs[0][0], runs[0][1])
    assert np.array_equal(runs[1][0], runs[0][0])
    assert all(same), (runs[2][0], runs[0][0])


@pytest.mark.parametrize("embed,batch", [(4160, 1), (8192, 1), (8192, 2)])
def test_rows_longer_than_one_step_through_the_fused_rotation(embed, batch):
    """A llama-layout model whose rows of x are longer than 4096: the q|k|v product with the rotation and the cache
    writes as its tail then runs on the whole-chip kernel with every row cut into chunks over wavefronts (4160: two
    unequal chunks), the chunks' sums meeting in LDS before the rotation, and the norm in front of it as a launch of
    its own. Logits against the oracle, then the three step modes and the finer-grained launch ("q4_0.stream" = 1)
    must choose the oracle's tokens."""
    lib = gpu.lib()
    c = capi.LlamaConfig()
    c.embed, c.hidden, c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.vocab = embed, 1792, 2, 4, 1, 128, 128, 1003
    c.context, c.interleaved, c.cache_dtype, c.batch = 64, 1, capi.F16, batch
    c.rope_base, c.rope_scale, c.eps = 500000.0, 1.0, 1e-5
    om = OL.synthetic(_oracle_config(c), seed=3, output_dt=O.Q4_0, centered=True)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(16)
    prompts = np.random.default_rng(6).integers(0, c.vocab, (batch, 9))
    gpu.say(f"long rows: embed {embed}, batch {batch}: logits")
    got = m.logits(prompts, all=True)
    for b in range(batch):
        want = om.logits(prompts[b].tolist(), om.new_caches(c.context, O.F16), all=True)
        assert np.abs(got[b] - want).max() <= 1e-3 * np.abs(want).max()
    wants = [om.generate(prompts[b].tolist(), 24, capacity=c.context, cache_dtype=O.F16) for b in range(batch)]
    try:
        for mode, stream in ((2, 0), (1, 0), (0, 0), (0, 1)):
            gpu.say(f"long rows: embed {embed}, batch {batch}: step mode {mode}, q4_0.stream {stream}")
            capi.check(lib.mi355x_tune(b"llama.step", mode))
            capi.check(lib.mi355x_tune(b"q4_0.stream", stream))
            m.reset()
            toks, _ = m.generate(prompts, 24)
            for b in range(batch):
                want, margins = wants[b]
                gotb = toks[b].tolist()
                first = next((i for i in range(24) if gotb[i] != want[i]), None)
                assert first is None, f"mode {mode} stream {stream} sequence {b} token {first}: device {gotb[first]}, oracle {want[first]}, margin {margins[first]:.4g}"
    finally:
        capi.check(lib.mi355x_tune(b"llama.step", 0))
        capi.check(lib.mi355x_tune(b"q4_0.stream", 0))


@pytest.mark.parametrize("batch", [2, 5, 8, 11, 16])
def test_batch_step_that_reads_weights_once_chooses_the_same_tokens(batch):
    """Two to sixty-four sequences decode with products that read each weight once per eight of them (int8 matrix
    cores, the output and down projections cut into two shares of K that the next norm adds; the rotation
    with the cache writes and SiLU * up with its conversion ride on the products, or run as launches of
    their own). Their integers are those of the one-sequence kernels, only float32 sums are ordered differently, so the tokens
    must be those of the one-sequence kernels run per sequence (llama.rows = 1), of the per-operator path,
    and, up to near-ties, the oracle's."""
    lib = gpu.lib()
    c = _small_q4_config(batch, capi.F16)
    om = OL.synthetic(_oracle_config(c), seed=2, output_dt=O.Q4_0)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(40)
    prompts = np.random.default_rng(17).integers(0, c.vocab, (batch, 11))
    runs = {}
    try:
        for name, key, v in (("rows graph", b"llama.rows", 0), ("rows launches", b"llama.step", 1), ("rows without riders", b"llama.rows", 2),
                             ("per sequence", b"llama.rows", 1), ("per operator", b"llama.step", 2)):
            capi.check(lib.mi355x_tune(b"llama.rows", 0))
            capi.check(lib.mi355x_tune(b"llama.step", 0))
            capi.check(lib.mi355x_tune(key, v))
            gpu.say(f"generate batch {batch}: {name}")
            m.reset()
            first, _ = m.generate(prompts, 30)
            more, _ = m.generate(first[:, -1:], 10)  # the graph of the first call, from another cache length
            runs[name] = np.concatenate([first, more], 1)
    finally:
        capi.check(lib.mi355x_tune(b"llama.rows", 0))
        capi.check(lib.mi355x_tune(b"llama.step", 0))
    for name in ("rows launches", "rows without riders", "per sequence", "per operator"):
        assert np.array_equal(runs["rows graph"], runs[name]), (name, runs["rows graph"], runs[name])
    for b in range(batch):
        want, margins = om.generate(prompts[b].tolist(), 30, capacity=c.context, cache_dtype=O.F16)
        for i, (a, w) in enumerate(zip(runs["rows graph"][b, :30].tolist(), want)):
            assert a == w, f"token {i}: device {a}, oracle {w}, oracle's margin there {margins[i]:.4g}"


def test_fused_steps_without_their_riders_choose_the_per_operator_tokens():
    """The fused step lets the rotation, the norms and the conversion of SwiGLU's results ride on the products
    only where their shapes allow: interleaved pairs, rows of x one step of a wavefront long. A model with
    half-split pairs (qwen2's layout) and 4160 features takes the separate launches instead, and must choose the
    same tokens as the per-operator path."""
    lib = gpu.lib()
    c = capi.LlamaConfig()
    c.embed, c.hidden, c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.vocab = 4160, 320, 2, 2, 1, 64, 64, 301
    c.context, c.interleaved, c.cache_dtype, c.batch = 48, 0, capi.F16, 2
    c.rope_base, c.rope_scale, c.eps = 10000.0, 1.0, 1e-5
    oc = OL.Config(arch="qwen2", embed=c.embed, hidden=c.hidden, layers=c.layers, heads=c.heads, kv_heads=c.kv_heads, head_dim=c.head_dim,
                   rope_dim=c.rope_dim, rope_base=c.rope_base, rope_scale=1.0, eps=c.eps, vocab=c.vocab, context=c.context)
    om = OL.synthetic(oc, seed=3, output_dt=O.Q4_0)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(16)
    prompts = np.random.default_rng(9).integers(0, c.vocab, (2, 7))
    runs = {}
    try:
        for mode in (2, 1, 0):
            gpu.say(f"generate without riders, step mode {mode}")
            capi.check(lib.mi355x_tune(b"llama.step", mode))
            m.reset()
            runs[mode], _ = m.generate(prompts, 20)
    finally:
        capi.check(lib.mi355x_tune(b"llama.step", 0))
    want, margins = om.generate(prompts[0].tolist(), 20, capacity=c.context, cache_dtype=O.F16)
    for i, (a, w) in enumerate(zip(runs[2][0].tolist(), want)):
        assert a == w, f"token {i}: device {a}, oracle {w}, oracle's margin there {margins[i]:.4g}"
    assert np.array_equal(runs[1], runs[2]) and np.array_equal(runs[0], runs[2])


@pytest.mark.parametrize("linear_dt,batch,heads,head_dim", [(O.Q4_K, 1, 4, 64), (O.Q6_K, 2, 4, 64), (O.Q8_0, 1, 4, 64), (O.Q4_K, 5, 4, 64),
                                                            (O.Q4_K, 11, 4, 64), (O.Q6_K, 9, 4, 64), (O.Q4_K, 1, 4, 128), (O.Q6_K, 3, 8, 64),
                                                            (O.Q4_K, 9, 16, 128)])
def test_k_quant_and_q8_0_models_decode_from_a_graph(linear_dt, batch, heads, head_dim):
    """Models whose linears are not Q4_0 take the generic decoding step: q|k|v and gate|up as one product
    each over weights kept together, norm and SwiGLU with the int8 conversion in the same launch (K-quants),
    residuals in the products' epilogues, the position on the device, the whole step replayed as a graph. It
    must choose the tokens of the per-operator path (position from the host) and of the oracle. Where the query
    heads of a key-value head are whole super-blocks of 256 (the last three shapes), attention leaves its result
    in the int8 form the K-quant output projection reads."""
    lib = gpu.lib()
    c = capi.LlamaConfig()
    c.embed, c.hidden, c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.vocab = 512, 1024, 2, heads, 2, head_dim, head_dim, 301
    c.context, c.interleaved, c.cache_dtype, c.batch = 64, 1, capi.F16, batch
    c.rope_base, c.rope_scale, c.eps = 10000.0, 1.0, 1e-5
    om = OL.synthetic(_oracle_config(c), seed=7, linear_dt=linear_dt)
    m = Llama(c)
    _upload_synthetic(m, om)
    m.finalize(16)
    prompts = np.random.default_rng(11).integers(0, c.vocab, (batch, 6))
    runs = {}
    try:
        for mode in (2, 1, 0, 0):
            gpu.say(f"generate dtype {linear_dt}, step mode {mode}, batch {batch}")
            capi.check(lib.mi355x_tune(b"llama.step", mode))
            m.reset()
            first, _ = m.generate(prompts, 20)
            more, _ = m.generate(first[:, -1:], 9)  # a second call continues the caches (and replays the graph)
            runs.setdefault(mode, []).append(np.concatenate([first, more], 1))
    finally:
        capi.check(lib.mi355x_tune(b"llama.step", 0))
    want, margins = om.generate(prompts[0].tolist(), 20, capacity=c.context, cache_dtype=O.F16)
    for i, (a, w) in enumerate(zip(runs[2][0][0, :20].tolist(), want)):
        assert a == w, f"token {i}: device {a}, oracle {w}, oracle's margin there {margins[i]:.4g}"
    assert np.array_equal(runs[1][0], runs[2][0]) and np.array_equal(runs[0][0], runs[2][0]) and np.array_equal(runs[0][1], runs[2][0])
