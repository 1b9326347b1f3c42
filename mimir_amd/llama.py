"""Loads a llama-architecture model into the device decoder of
libmimir_mi355x.so: the counterpart of the reference's llm.Load
(llm/model.go:216-311) over a .mim file, and of Model.Logits / greedy
generation. Weights are uploaded in the file's block dtypes (no decode to
float32); every compute call goes through the C ABI.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .mimfile import MimFile

# container dtype codes (mimfile) -> C-ABI dtype codes
# dtype names of mimir_amd.mimfile -> dtype codes of the C ABI
_MIM_TO_ABI = {"f32": capi.F32, "f16": capi.F16, "bf16": capi.BF16, "q8_0": capi.Q8_0, "q4_K": capi.Q4_K, "q6_K": capi.Q6_K, "q4_0": capi.Q4_0}


class Llama:
    """A handle on mi355x_llama_*."""

    def __init__(self, config: capi.LlamaConfig):
        self.lib = capi.load()
        self.config = config
        self._h = C.c_void_p()
        capi.check(self.lib.mi355x_llama_create(C.byref(config), C.byref(self._h)))

    def close(self):
        if self._h:
            self.lib.mi355x_llama_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_tensor(self, name: str, dtype: int, data: np.ndarray, n_elems: int):
        data = np.ascontiguousarray(data)
        capi.check(self.lib.mi355x_llama_set_tensor(self._h, name.encode(), dtype, data.ctypes.data, n_elems))

    def set_rope_factors(self, factors):
        f = np.ascontiguousarray(factors, np.float32)
        capi.check(self.lib.mi355x_llama_set_rope_factors(self._h, f.ctypes.data, f.size))

    def finalize(self, max_tokens: int):
        capi.check(self.lib.mi355x_llama_finalize(self._h, max_tokens))

    def reset(self):
        capi.check(self.lib.mi355x_llama_reset(self._h))

    def set_cache(self, layer: int, keys, values):
        """keys, values [batch, kv_heads, n, head_dim] in the cache's dtype
        (float32, or binary16 bits as uint16)."""
        k = np.ascontiguousarray(keys); v = np.ascontiguousarray(values)
        capi.check(self.lib.mi355x_llama_set_cache(self._h, layer, k.ctypes.data, v.ctypes.data, k.shape[2]))

    @property
    def cache_len(self) -> int:
        return self.lib.mi355x_llama_cache_len(self._h)

    def logits(self, tokens, all: bool = False) -> np.ndarray:
        """tokens [batch, n] (or [n] for batch 1) -> [batch, vocab] or [batch, n, vocab]."""
        c = self.config
        t = np.ascontiguousarray(tokens, np.int32).reshape(c.batch, -1)
        n = t.shape[1]
        out = np.empty((c.batch, n, c.vocab) if all else (c.batch, c.vocab), np.float32)
        capi.check(self.lib.mi355x_llama_logits(self._h, t.ctypes.data, n, int(all), out.ctypes.data))
        return out

    def generate(self, prompt, n_new: int):
        """Greedy tokens [batch, n_new] and (prompt seconds, decode seconds)."""
        c = self.config
        t = np.ascontiguousarray(prompt, np.int32).reshape(c.batch, -1)
        out = np.empty((c.batch, n_new), np.int32)
        secs = (C.c_double * 2)()
        capi.check(self.lib.mi355x_llama_generate(self._h, t.ctypes.data, t.shape[1], n_new, out.ctypes.data, secs))
        return out, (secs[0], secs[1])


def config_from_metadata(md: dict, vocab: int, context: int | None = None, batch: int = 1, cache_dtype: int = capi.F32) -> capi.LlamaConfig:
    """readConfig (llm/model.go:97-171)."""
    arch = md.get("general.architecture")
    if arch not in ("llama", "qwen2"):
        raise ValueError(f"architecture {arch!r}, want llama or qwen2")

    def get(key, default=None):
        v = md.get(f"{arch}.{key}", default)
        if v is None:
            raise KeyError(f"no {arch}.{key}")
        return v

    c = capi.LlamaConfig()
    c.embed = int(get("embedding_length")); c.hidden = int(get("feed_forward_length")); c.layers = int(get("block_count"))
    c.heads = int(get("attention.head_count")); c.kv_heads = int(get("attention.head_count_kv", c.heads))
    c.head_dim = int(get("attention.key_length", c.embed // max(c.heads, 1)))
    c.rope_dim = int(get("rope.dimension_count", c.head_dim))
    c.vocab = vocab
    c.context = int(context if context is not None else get("context_length", 2048))
    c.interleaved = int(arch == "llama")
    c.cache_dtype = cache_dtype
    c.batch = batch
    c.rope_base = float(get("rope.freq_base", 10000.0))
    c.eps = float(get("attention.layer_norm_rms_epsilon", 1e-5))
    scaling = md.get(f"{arch}.rope.scaling.type", "none")
    if scaling == "none":
        c.rope_scale = float(get("rope.scale_linear", 1.0))
    elif scaling == "linear":
        c.rope_scale = float(get("rope.scaling.factor", 1.0))
    else:
        raise ValueError(f"rope scaling {scaling!r}")
    return c


def load_mim(path: str, max_tokens: int = 64, q4_0_code: int | None = None, **kw) -> Llama:
    """llm.Load (llm/model.go:224-316): every tensor the reference reads, the biases that
    qwen2 gives its queries, keys and values among them (:251-258); a qwen2 file without
    them is an error, as it is there."""
    f = MimFile(path, q4_0_code=q4_0_code)  # the container's code for Q4_0 blocks, if the caller knows it
    emb = f["token_embd.weight"]
    c = config_from_metadata(f.metadata, emb.shape[0], **kw)
    m = Llama(c)
    biased = f.metadata.get("general.architecture") == "qwen2"
    for name, t in f.tensors.items():
        if name == "rope_freqs.weight":
            m.set_rope_factors(t.data)
        elif name.startswith("blk.") and name.rsplit(".", 2)[-2:] in (["attn_q", "bias"], ["attn_k", "bias"], ["attn_v", "bias"]):
            if not biased:
                continue  # the reference reads them for qwen2 only
            if t.dtype_name != "f32":
                raise ValueError(f"{name}: dtype {t.dtype_name}, want f32")
            m.set_tensor(name, capi.F32, np.ascontiguousarray(t.data, np.float32), int(np.prod(t.shape)))
        elif name.endswith(".weight") and (name.startswith("blk.") or name in ("token_embd.weight", "output_norm.weight", "output.weight")):
            if t.dtype_name not in _MIM_TO_ABI:
                raise ValueError(f"{name}: dtype {t.dtype_name}")
            m.set_tensor(name, _MIM_TO_ABI[t.dtype_name], t.data, int(np.prod(t.shape)))
    if biased:
        for i in range(c.layers):
            for leaf in ("attn_q", "attn_k", "attn_v"):
                if f"blk.{i}.{leaf}.bias" not in f:
                    raise KeyError(f"blk.{i}.{leaf}.bias: a qwen2 model has biases on its queries, keys and values")
    m.finalize(max_tokens)
    return m
