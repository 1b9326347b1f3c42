"""The reference's Llama forward, restated over the oracle's C primitives.

TEST INFRASTRUCTURE (see oracle/mimir_oracle.c). Follows llm/model.go:391-455
(Logits, the general path), nn/layers.go:49-55,103-116 (Linear, Embedding),
nn/transformer.go:50-61,146-257,348-423 (RMSNorm, RotaryEmbedding, KVCache) and
examples/llama/generate.go:44-53,162-202 (greedy generation).

A Linear by a block-quantized weight multiplies as the reference's CPU does:
int8 activations for Q8_0/Q4_K/Q6_K (tensor/quant.go:35-56 ->
backend/cpu/qmatmul.go), the float32 product of the decoded weights for Q4_0
(io/mim/dtype.go:118-123); `dequantized=True` decodes every weight to float32
first, which is what the reference's own "dequantized"/"exact" test variants
do (examples/llama/llama_test.go:177, io/mim/mim_test.go:207-210).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

import oracle as O

# dtype names of mimir_amd.mimfile -> oracle dtype codes
_MIM_TO_ORACLE = {"q8_0": O.Q8_0, "q4_K": O.Q4_K, "q6_K": O.Q6_K, "q4_0": O.Q4_0}


@dataclass
class Config:
    arch: str = "llama"
    embed: int = 0
    hidden: int = 0
    layers: int = 0
    heads: int = 0
    kv_heads: int = 0
    head_dim: int = 0
    rope_dim: int = 0
    rope_base: float = 10000.0
    rope_scale: float = 1.0
    eps: float = 1e-5
    vocab: int = 0
    context: int = 2048

    @property
    def interleaved(self) -> bool:  # llm/model.go:321
        return self.arch == "llama"


@dataclass
class Weight:
    """A [n, k] matrix: raw ggml bytes with an oracle dtype, or float32 values."""
    dtype: int
    n: int
    k: int
    data: np.ndarray

    def dequantized(self) -> "Weight":
        if self.dtype == O.F32:
            return self
        return Weight(O.F32, self.n, self.k, O.dequantize(self.dtype, self.data).reshape(self.n, self.k))


@dataclass
class Block:
    attn_norm: np.ndarray = None
    ffn_norm: np.ndarray = None
    q: Weight = None
    k: Weight = None
    v: Weight = None
    o: Weight = None
    gate: Weight = None
    up: Weight = None
    down: Weight = None
    q_bias: np.ndarray | None = None  # qwen2's (llm/model.go:251-258), float32 [n]
    k_bias: np.ndarray | None = None
    v_bias: np.ndarray | None = None


@dataclass
class KVCache:
    """Keys and values of one block, [kv_heads, capacity, head_dim], float32 or
    binary16 bits (nn/transformer.go:348-423)."""
    keys: np.ndarray
    values: np.ndarray
    dtype: int
    n: int = 0


@dataclass
class Model:
    config: Config
    embed: Weight = None
    blocks: list = field(default_factory=list)
    norm: np.ndarray = None
    output: Weight = None
    freq_factors: np.ndarray | None = None
    threads: int = 0

    # ---- construction --------------------------------------------------
    @staticmethod
    def from_mim(f, dequantized: bool = False) -> "Model":
        md = f.metadata
        arch = md.get("general.architecture")
        if arch not in ("llama", "qwen2"):
            raise ValueError(f"architecture {arch!r}")

        def mi(key, default=None):
            v = md.get(f"{arch}.{key}", default)
            if v is None:
                raise KeyError(f"{arch}.{key}")
            return v

        c = Config(arch=arch, embed=int(mi("embedding_length")), hidden=int(mi("feed_forward_length")),
                   layers=int(mi("block_count")), heads=int(mi("attention.head_count")),
                   rope_base=float(mi("rope.freq_base", 10000.0)), eps=float(mi("attention.layer_norm_rms_epsilon", 1e-5)),
                   context=int(mi("context_length", 2048)))
        c.kv_heads = int(mi("attention.head_count_kv", c.heads))
        c.head_dim = int(mi("attention.key_length", c.embed // max(c.heads, 1)))
        c.rope_dim = int(mi("rope.dimension_count", c.head_dim))
        scaling = md.get(f"{arch}.rope.scaling.type", "none")
        if scaling == "none":
            c.rope_scale = float(mi("rope.scale_linear", 1.0))
        elif scaling == "linear":
            c.rope_scale = float(mi("rope.scaling.factor", 1.0))
        else:
            raise ValueError(f"rope scaling {scaling!r}")

        def weight(name):
            t = f[name]
            n, k = t.shape
            if t.quantized:
                w = Weight(_MIM_TO_ORACLE[t.dtype_name], n, k, t.data)
            elif t.dtype_name == "f32":
                w = Weight(O.F32, n, k, np.ascontiguousarray(t.data, np.float32))
            elif t.dtype_name == "f16":
                w = Weight(O.F32, n, k, O.f16_to_f32(t.data.view(np.uint16)).reshape(n, k))
            elif t.dtype_name == "bf16":
                w = Weight(O.F32, n, k, O.bf16_to_f32(t.data).reshape(n, k))
            else:
                raise ValueError(f"{name}: dtype {t.dtype_name}")
            return w.dequantized() if dequantized else w

        m = Model(c)
        m.embed = weight("token_embd.weight")
        c.vocab = m.embed.n
        m.norm = f["output_norm.weight"].data.astype(np.float32)
        m.output = weight("output.weight") if "output.weight" in f else m.embed  # tied (llm/model.go:283-288)
        for i in range(c.layers):
            p = f"blk.{i}."
            bias = (lambda leaf: f[p + leaf + ".bias"].data.astype(np.float32)) if arch == "qwen2" else (lambda leaf: None)
            m.blocks.append(Block(
                q_bias=bias("attn_q"), k_bias=bias("attn_k"), v_bias=bias("attn_v"),
                attn_norm=f[p + "attn_norm.weight"].data.astype(np.float32),
                ffn_norm=f[p + "ffn_norm.weight"].data.astype(np.float32),
                q=weight(p + "attn_q.weight"), k=weight(p + "attn_k.weight"), v=weight(p + "attn_v.weight"),
                o=weight(p + "attn_output.weight"), gate=weight(p + "ffn_gate.weight"), up=weight(p + "ffn_up.weight"),
                down=weight(p + "ffn_down.weight")))
        if "rope_freqs.weight" in f:
            m.freq_factors = f["rope_freqs.weight"].data.astype(np.float32)
        return m

    # ---- pieces ----------------------------------------------------------
    def new_caches(self, capacity: int, dtype: int = O.F32) -> list:
        c = self.config
        dt = np.float32 if dtype == O.F32 else np.uint16
        return [KVCache(np.zeros((c.kv_heads, capacity, c.head_dim), dt), np.zeros((c.kv_heads, capacity, c.head_dim), dt), dtype)
                for _ in range(c.layers)]

    def linear(self, x: np.ndarray, w: Weight, bias: np.ndarray | None = None) -> np.ndarray:
        """x [..., k] . w^T, then + bias in float32 if the layer has one (nn/layers.go:49-55 -> tensor/quant.go:35-56)."""
        if w.dtype == O.F32:
            y = O.sgemv(w.data, x, self.threads)
        else:
            y = O.qmatmul(w.dtype, w.data, x, w.n, w.k, simd=True, threads=self.threads)
        return y if bias is None else (y + bias.astype(np.float32)).astype(np.float32)

    def embed_tokens(self, tokens) -> np.ndarray:
        w = self.embed
        idx = np.asarray(tokens, np.int32)
        if w.dtype == O.F32:
            return w.data[idx].copy()
        return O.gather_rows(w.dtype, w.data, w.n, w.k, idx)

    def rope(self, x: np.ndarray, past: int) -> np.ndarray:
        """x [heads, S, head_dim] (nn/transformer.go:225-257 with llm/model.go:318-346)."""
        c = self.config
        s = x.shape[-2]
        scaling, params = (O.ROPE_LINEAR, (c.rope_scale,)) if c.rope_scale != 1 else (O.ROPE_NONE, ())
        cos, sin = O.rope_angles(c.rope_dim, c.rope_base, past, s, scaling, params, self.freq_factors)
        return O.rope_apply(x, cos, sin, c.rope_dim, c.interleaved)

    # ---- forward ---------------------------------------------------------
    def logits(self, tokens, caches, all: bool = False) -> np.ndarray:
        """llm/model.go:391-437. Appends to the caches; returns [vocab] or [S, vocab]."""
        c = self.config
        s = len(tokens)
        x = self.embed_tokens(tokens)  # [S, embed]
        for blk, cache in zip(self.blocks, caches):
            past = cache.n
            h = O.rmsnorm(x, blk.attn_norm, c.eps)
            q = self.linear(h, blk.q, blk.q_bias).reshape(s, c.heads, c.head_dim).transpose(1, 0, 2)
            k = self.linear(h, blk.k, blk.k_bias).reshape(s, c.kv_heads, c.head_dim).transpose(1, 0, 2)
            v = self.linear(h, blk.v, blk.v_bias).reshape(s, c.kv_heads, c.head_dim).transpose(1, 0, 2)
            q, k = self.rope(np.ascontiguousarray(q), past), self.rope(np.ascontiguousarray(k), past)
            if past + s > cache.keys.shape[1]:
                raise ValueError(f"append {s} positions to a cache holding {past} of {cache.keys.shape[1]}")
            if cache.dtype == O.F32:
                cache.keys[:, past:past + s] = k
                cache.values[:, past:past + s] = v
            else:  # cast to the cache's dtype (nn/transformer.go:412-414)
                cache.keys[:, past:past + s] = O.f32_to_f16(k)
                cache.values[:, past:past + s] = O.f32_to_f16(np.ascontiguousarray(v))
            cache.n = past + s
            a, _ = O.attention(q[None], cache.keys[None], cache.values[None], 1 / np.sqrt(c.head_dim), causal=True,
                               causal_offset=past, kv_dt=cache.dtype, k_len=cache.n)
            a = a[0].transpose(1, 0, 2).reshape(s, c.heads * c.head_dim)
            x = x + self.linear(np.ascontiguousarray(a), blk.o)
            h = O.rmsnorm(x, blk.ffn_norm, c.eps)
            x = x + self.linear(O.silu_mul(self.linear(h, blk.gate), self.linear(h, blk.up)), blk.down)
        if not all:
            x = x[-1:]
        out = self.linear(O.rmsnorm(x, self.norm, c.eps), self.output)
        return out if all else out[0]

    def generate(self, prompt, n_new: int, capacity: int | None = None, cache_dtype: int = O.F32):
        """Greedy decoding (examples/llama/generate.go:162-202 with Sample at
        :44-53): returns the new tokens and, per step, the margin between the
        two largest logits."""
        caches = self.new_caches(capacity or len(prompt) + n_new, cache_dtype)
        logits = self.logits(list(prompt), caches)
        out, margins = [], []
        for _ in range(n_new):
            t = O.argmax(logits)
            top2 = np.partition(logits, -2)[-2:]
            out.append(t)
            margins.append(float(top2[1] - top2[0]))
            if len(out) == n_new:
                break
            logits = self.logits([t], caches)
        return out, margins


# ---- synthetic models in the shapes the benchmark configurations name -----

def _q_blocks(rng, dt, n, k, centered=False):
    """Random blocks of dtype dt for an [n, k] weight: quants uniform over their range, binary16 scales
    |N(0, 0.02)| (divided by 32 for the K-quants, whose sub-block scales multiply them). centered (Q4_0): nibbles
    1..15 only, so that the weights -7..7 have no mean (uniform nibbles 0..15 average -0.5, which gives every
    linear a common-mode term that swamps what depends on the token)."""
    def half(count, scale):
        d = np.abs(rng.normal(0, scale, count)).astype(np.float32).astype(np.float16).view(np.uint16)
        return np.stack([d & 0xff, d >> 8], 1).astype(np.uint8)

    if dt in (O.Q4_K, O.Q6_K):
        nb = n * k // 256
        bb = 144 if dt == O.Q4_K else 210
        b = rng.integers(0, 256, (nb, bb), dtype=np.uint8)
        if dt == O.Q4_K:
            b[:, 0:2], b[:, 2:4] = half(nb, 0.02 / 32), half(nb, 0.02 / 32)
        else:
            b[:, 208:210] = half(nb, 0.02 / 32)
        return Weight(dt, n, k, b.reshape(-1))
    nb = n * k // 32
    bb = 18 if dt == O.Q4_0 else 34
    b = np.empty((nb, bb), np.uint8)
    b[:, 0:2] = half(nb, 0.02)
    if dt == O.Q4_0:
        if centered:
            nib = rng.integers(1, 16, (nb, 32), dtype=np.uint8)
            b[:, 2:] = nib[:, :16] | (nib[:, 16:] << 4)
        else:
            b[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    else:
        b[:, 2:] = rng.integers(-127, 128, (nb, 32)).astype(np.int8).view(np.uint8)
    return Weight(dt, n, k, b.reshape(-1))


def tensor_seed(seed: int, name: str) -> int:
    """A per-tensor seed derived from the tensor's name, so that any one tensor
    can be regenerated alone."""
    h = 1469598103934665603
    for ch in f"{seed}/{name}".encode():
        h = ((h ^ ch) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def synthetic(config: Config, seed: int = 0, linear_dt: int = O.Q4_0, table_dt: int = O.Q8_0, output_dt: int | None = None,
              centered: bool = False) -> Model:
    """A random-init Llama: linear weights of linear_dt, embeddings and the
    output projection of table_dt, norm weights N(1, 0.02); block scales
    |N(0, 0.02)| as binary16, quants uniform over their range (centered: Q4_0
    linears drawn without a mean, see _q_blocks)."""
    c = config
    m = Model(c)

    def rng(name):
        return np.random.default_rng(tensor_seed(seed, name))

    m.embed = _q_blocks(rng("token_embd.weight"), table_dt, c.vocab, c.embed)
    m.output = _q_blocks(rng("output.weight"), table_dt if output_dt is None else output_dt, c.vocab, c.embed)
    m.norm = rng("output_norm.weight").normal(1, 0.02, c.embed).astype(np.float32)
    qd, kvd = c.heads * c.head_dim, c.kv_heads * c.head_dim
    for i in range(c.layers):
        p = f"blk.{i}."
        m.blocks.append(Block(
            attn_norm=rng(p + "attn_norm.weight").normal(1, 0.02, c.embed).astype(np.float32),
            ffn_norm=rng(p + "ffn_norm.weight").normal(1, 0.02, c.embed).astype(np.float32),
            q=_q_blocks(rng(p + "attn_q.weight"), linear_dt, qd, c.embed, centered), k=_q_blocks(rng(p + "attn_k.weight"), linear_dt, kvd, c.embed, centered),
            v=_q_blocks(rng(p + "attn_v.weight"), linear_dt, kvd, c.embed, centered), o=_q_blocks(rng(p + "attn_output.weight"), linear_dt, c.embed, qd, centered),
            gate=_q_blocks(rng(p + "ffn_gate.weight"), linear_dt, c.hidden, c.embed, centered), up=_q_blocks(rng(p + "ffn_up.weight"), linear_dt, c.hidden, c.embed, centered),
            down=_q_blocks(rng(p + "ffn_down.weight"), linear_dt, c.embed, c.hidden, centered)))
    return m
