#!/usr/bin/env python3
"""Benchmark of the quantized decode product on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: the
Q4_0 decode GEMV y = x . W^T at the Llama-3-8B gate/up shape (W 14336 x 4096,
batch 1), inputs resident in HBM. Successive steps read different copies of W
(more of them than the last-level cache holds) so that every step streams its
weights from HBM, as a decode loop over a whole model does.

Prints one JSON line: whole-job throughput in algorithmic GB/s, the roofline
object of the kernel, and a CPU baseline (the oracle's restatement of the
reference's CPU path, timed on this host's cores on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
# HBM bytes of one launch of the GEMV kernel at the benchmark shape, from
# rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter
# reads for a copy kernel of known size (the summaries under profiles/ hold the
# runs): FETCH_SIZE 16278.986 KiB x 1024 x 1.99967 + WRITE_SIZE 56 KiB x 1024 x 1.0.
TRAFFIC_BYTES_PER_LAUNCH = 33398365
TRAFFIC_KERNEL = "qgemv_q4_0_stream_kernel<0, 2, 7>"  # the kernel those counter runs launched


def gemv_bytes(n: int, k: int, block_bytes: int = 18) -> int:
    """Algorithmic bytes of one batch-1 product: W once, x in, y out."""
    return n * (k // 32) * block_bytes + 4 * k + 4 * n


def bench_blocks_q4_0(rng, n_elems):
    nb = n_elems // 32
    b = np.empty((nb, 18), np.uint8)
    d = np.abs(rng.normal(0, 0.02, nb)).astype(np.float32).astype(np.float16).view(np.uint16)
    b[:, 0] = d & 0xff
    b[:, 1] = d >> 8
    b[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    return b.reshape(-1)


class Gemv:
    """One product y = x . W^T (Q4_0 unless kind says "q8_0") with n_bufs HBM-resident copies of W."""

    def __init__(self, lib, capi, torch, n, k, n_bufs, seed=0, kind="q4_0"):
        self.lib, self.capi, self.torch, self.n, self.k, self.n_bufs = lib, capi, torch, n, k, n_bufs
        self.kind, self.dt, self.block_bytes = kind, (capi.Q4_0 if kind == "q4_0" else capi.Q8_0), (18 if kind == "q4_0" else 34)
        rng = np.random.default_rng(seed)
        self.raw = bench_blocks_q4_0(rng, n * k) if kind == "q4_0" else q_blocks(rng, "q8_0", n * k)
        self.x = rng.normal(size=k).astype(np.float32)
        w0 = torch.from_numpy(self.raw).to("cuda:0")
        self.bufs = [w0] + [w0.clone() for _ in range(n_bufs - 1)]
        self.xd = torch.from_numpy(self.x).to("cuda:0")
        self.y = torch.empty(n, dtype=torch.float32, device="cuda:0")
        self.act = torch.empty(lib.mi355x_act_bytes(self.dt, k) + 64, dtype=torch.uint8, device="cuda:0")
        self.stream = torch.cuda.Stream()

    def bytes(self):
        return gemv_bytes(self.n, self.k, self.block_bytes)

    def step(self, i):
        """The boundary's product, float32 x in and float32 y out: one launch, whose workgroups
        convert x to the kernel's fixed-point form for themselves before they multiply."""
        self.capi.check(self.lib.mi355x_qgemv(self.dt, self.bufs[i % self.n_bufs].data_ptr(), self.xd.data_ptr(), self.y.data_ptr(),
                                              1, self.n, self.k, self.k, self.stream.cuda_stream))

    def kernel_name(self):
        """Which kernel the library's dispatch launched for the latest step of this thread."""
        import ctypes as C
        buf = C.create_string_buffer(200)
        self.capi.check(self.lib.mi355x_last_kernel(buf, 200))
        return buf.value.decode()

    kernel = step  # the step is its dominant kernel and nothing else

    def from_converted(self, i):
        """The same product over activations converted beforehand (what a decoding step's fused launches use)."""
        self.capi.check(self.lib.mi355x_qgemv_act(self.dt, self.bufs[i % self.n_bufs].data_ptr(), self.act.data_ptr(), self.y.data_ptr(),
                                                  1, self.n, self.k, self.stream.cuda_stream))

    def check(self):
        """Both routes against the oracle, before anything is timed."""
        import oracle as O
        want = O.qmatmul(O.Q4_0 if self.kind == "q4_0" else O.Q8_0, self.raw, self.x, self.n, self.k)
        self.capi.check(self.lib.mi355x_convert_act(self.dt, self.xd.data_ptr(), 1, self.k, self.k, self.act.data_ptr(), self.stream.cuda_stream))
        for name, fn in (("qgemv", self.step), ("qgemv_act", self.from_converted)):
            self.y.zero_()
            self.torch.cuda.synchronize()
            fn(0)
            self.stream.synchronize()
            err = np.abs(self.y.cpu().numpy() - want) / np.maximum(1, np.abs(want))
            if not np.all(err <= 1e-3):
                raise SystemExit(f"bench: {name} {self.n}x{self.k} differs from the oracle: worst {err.max():.3e}")

    def kernel_durations(self, steps, warmup):
        """Mean, min and max microseconds of the GEMV kernel itself over `steps`
        launches in a row: each launch carries its own pair of HIP events on the
        launching stream, which read the kernel's begin and end as the
        profiler's kernel trace does."""
        import ctypes as C
        with self.torch.cuda.stream(self.stream):
            for i in range(max(warmup, 3)):
                self.kernel(i)
            self.stream.synchronize()
            t_warm = time.perf_counter()
            while time.perf_counter() - t_warm < 0.25:  # untimed: the device's clocks up, as in time()
                for i in range(64):
                    self.kernel(i)
                self.stream.synchronize()
            # The host needs longer to launch a kernel with its pair of events than the kernel runs, and a kernel that
            # starts on an idle device takes longer than one that follows another. So every 256 timed launches queue
            # behind a graph of 512 untimed ones, not waited for: while it runs the host gets ahead, and the timed
            # launches follow each other as the launches of a graph do.
            ahead = self.torch.cuda.CUDAGraph()
            with self.torch.cuda.graph(ahead, stream=self.stream):
                for i in range(512):
                    self.kernel(i)
            self.capi.check(self.lib.mi355x_timed_begin(steps))
            for i in range(steps):
                if i % 256 == 0:
                    ahead.replay()
                self.kernel(i)
            ms = (C.c_float * steps)()
            n = C.c_int(0)
            self.capi.check(self.lib.mi355x_timed_end(ms, C.byref(n)))
        if n.value != steps:
            raise SystemExit(f"bench: {n.value} timed launches, want {steps}")
        us = np.array(ms[:steps], np.float64) * 1e3
        return float(us.mean()), float(us.min()), float(us.max())

    def time_independent(self, width, rounds=64):
        """Microseconds per product when `width` chains of them run side by side with no edges between the chains:
        each chain is a graph of `rounds` products on a stream of its own (its own copies of W, its own y), all
        launched together. What of a launch's ramp and tail another chain's launches can fill."""
        torch = self.torch
        sides = [torch.cuda.Stream() for _ in range(width)]
        ys = [torch.empty_like(self.y) for _ in range(width)]
        def call(i, w):
            self.capi.check(self.lib.mi355x_qgemv(self.dt, self.bufs[i % self.n_bufs].data_ptr(), self.xd.data_ptr(), ys[w].data_ptr(),
                                                  1, self.n, self.k, self.k, sides[w].cuda_stream))
        graphs = []
        for w in range(width):
            with torch.cuda.stream(sides[w]):
                call(w, w)
                sides[w].synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=sides[w]):
                    for r in range(rounds):
                        call(r * width + w, w)
                g.replay()
                sides[w].synchronize()
            graphs.append(g)
        main = self.stream
        reps = 4
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(main)
        for w in range(width):
            sides[w].wait_event(e0)
        for _ in range(reps):
            for w in range(width):
                with torch.cuda.stream(sides[w]):
                    graphs[w].replay()
        for w in range(width):
            done = torch.cuda.Event()
            done.record(sides[w])
            main.wait_event(done)
        e1.record(main)
        main.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * rounds * width)

    def time(self, fn, steps, warmup, graph=True):
        """Milliseconds per call of fn over exactly `steps` calls after `warmup`,
        between HIP events on the stream that carries the launches. With graph,
        the calls are captured into one graph (very many steps: n_bufs at a time,
        plus one graph for the remainder) and replayed, as the decoder replays its
        step, so the host's launch cost stays off the device's timeline. Also
        returns wall ms/call."""
        torch, s = self.torch, self.stream
        with torch.cuda.stream(s):
            for i in range(max(warmup, 3)):
                fn(i)
            s.synchronize()
            graphs = []
            if graph:
                # the timed region is one graph of exactly `steps` launches where that is a graph of reasonable size (one
                # graph launch to pay for), else a graph of n_bufs launches replayed plus one for the remainder
                counts = (steps, 0) if steps <= 4096 else (self.n_bufs, steps % self.n_bufs)
                for count in counts:
                    g = None
                    if count:
                        g = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(g, stream=s):
                            for i in range(count):
                                fn(i)
                    graphs.append(g)
                graphs[0].replay()
                s.synchronize()
            # untimed, beyond the warm-up steps asked for: a quarter of a second of the same work, so that the device's
            # clocks are where a decoding loop holds them (a timed region of a few hundred microseconds from idle otherwise
            # reads 10 % slow)
            t_warm = time.perf_counter()
            while time.perf_counter() - t_warm < 0.25:
                for _ in range(32):
                    if graph:
                        graphs[0].replay()
                    else:
                        fn(0)
                s.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record(s)
            if graph:
                for _ in range(1 if steps <= 4096 else steps // self.n_bufs):
                    graphs[0].replay()
                if graphs[1] is not None:
                    graphs[1].replay()
            else:
                for i in range(steps):
                    fn(i)
            e1.record(s)
            s.synchronize()
            wall = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall


def stream_ceiling(lib, capi, torch, nbytes, n_bufs, steps):
    """GB/s of a plain 128-bit streaming read of nbytes, rotating buffers."""
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda:0").random_(0, 255) for _ in range(n_bufs)]
    grid, threads = 2048, 512
    scratch = torch.empty(grid * threads // 64, dtype=torch.float32, device="cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    for i in range(20):
        capi.check(lib.mi355x_stream_read(bufs[i % n_bufs].data_ptr(), nbytes, scratch.data_ptr(), grid, threads, st))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        capi.check(lib.mi355x_stream_read(bufs[i % n_bufs].data_ptr(), nbytes, scratch.data_ptr(), grid, threads, st))
    e1.record()
    torch.cuda.synchronize()
    return nbytes / (e0.elapsed_time(e1) / steps * 1e-3) / 1e9


def tensor_seed(seed: int, name: str) -> int:
    h = 1469598103934665603
    for ch in f"{seed}/{name}".encode():
        h = ((h ^ ch) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def q_blocks(rng, kind, n_elems):
    """Blocks as the configurations draw them: quants uniform over their range,
    one binary16 scale |N(0, 0.02)| per block of 32."""
    nb = n_elems // 32
    bb = 18 if kind == "q4_0" else 34
    b = np.empty((nb, bb), np.uint8)
    d = np.abs(rng.normal(0, 0.02, nb)).astype(np.float32).astype(np.float16).view(np.uint16)
    b[:, 0], b[:, 1] = d & 0xff, d >> 8
    if kind == "q4_0":
        b[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    else:
        b[:, 2:] = rng.integers(-127, 128, (nb, 32)).astype(np.int8).view(np.uint8)
    return b.reshape(-1)


def build_llama(capi, layers=32, batch=1, context=1024, max_tokens=512, seed=0, embed=4096, hidden=14336, heads=32, kv_heads=8,
                head_dim=128, vocab=128256, linear="q4_0"):
    """A random-init Llama-3-8B-shaped decoder on the device: Q4_0 linears (or
    Q4_K, Q6_K with `linear`), Q8_0 embeddings and output, norm weights
    N(1, 0.02), binary16 KV cache. Each tensor's generator is seeded from its name."""
    from mimir_amd.llama import Llama
    c = capi.LlamaConfig()
    c.embed, c.hidden, c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.vocab = embed, hidden, layers, heads, kv_heads, head_dim, head_dim, vocab
    c.context, c.interleaved, c.cache_dtype, c.batch = context, 1, capi.F16, batch
    c.rope_base, c.rope_scale, c.eps = 500000.0, 1.0, 1e-5
    m = Llama(c)
    rng = lambda name: np.random.default_rng(tensor_seed(seed, name))
    m.set_tensor("token_embd.weight", capi.Q8_0, q_blocks(rng("token_embd.weight"), "q8_0", vocab * embed), vocab * embed)
    m.set_tensor("output.weight", capi.Q8_0, q_blocks(rng("output.weight"), "q8_0", vocab * embed), vocab * embed)
    m.set_tensor("output_norm.weight", capi.F32, rng("output_norm.weight").normal(1, 0.02, embed).astype(np.float32), embed)
    qd, kvd = heads * head_dim, kv_heads * head_dim
    for i in range(layers):
        p = f"blk.{i}."
        for leaf in ("attn_norm", "ffn_norm"):
            m.set_tensor(p + leaf + ".weight", capi.F32, rng(p + leaf + ".weight").normal(1, 0.02, embed).astype(np.float32), embed)
        for leaf, n, k in (("attn_q", qd, embed), ("attn_k", kvd, embed), ("attn_v", kvd, embed), ("attn_output", embed, qd),
                           ("ffn_gate", hidden, embed), ("ffn_up", hidden, embed), ("ffn_down", embed, hidden)):
            if linear == "q4_0":
                m.set_tensor(p + leaf + ".weight", capi.Q4_0, q_blocks(rng(p + leaf + ".weight"), "q4_0", n * k), n * k)
            else:
                dt, bb = (capi.Q4_K, 144) if linear == "q4_K" else (capi.Q6_K, 210)
                m.set_tensor(p + leaf + ".weight", dt, bench_blocks_kquant(rng(p + leaf + ".weight"), bb, n * k), n * k)
    m.finalize(max_tokens)
    return m


def decode_bench(capi, layers=32, batch=1, prompt=512, new=256, check=0, linear="q4_0", want_tokens=None):
    """Whole-model greedy decoding: a prompt of uniform-random token ids, then
    `new` tokens a sequence. Returns tokens/s of the decoding steps. With
    check, the first `check` tokens of sequence 0 are compared with the CPU
    oracle's greedy decoding of the same model and prompt."""
    t0 = time.perf_counter()
    m = build_llama(capi, layers=layers, batch=batch, context=prompt + new, max_tokens=prompt, linear=linear)
    build_s = time.perf_counter() - t0
    toks = np.random.default_rng(0).integers(0, m.config.vocab, (batch, prompt))
    out, (t_prompt, t_decode) = m.generate(toks, new)
    per_tok_bytes = layers * 218103808 * {"q4_0": 0.5625, "q4_K": 0.5625, "q6_K": 0.8203125}[linear] + 128256 * 4096 * 1.0625
    verdict = {}
    if want_tokens:
        # sequence 0 of a batch has the prompt of the one-sequence run: its tokens against the oracle's of that run
        got = out[0, :len(want_tokens)].tolist()
        first = next((i for i, (a, b) in enumerate(zip(got, want_tokens)) if a != b), None)
        verdict = {"greedy_checked": len(want_tokens), "greedy_identical": sum(a == b for a, b in zip(got, want_tokens)), "first_mismatch": first,
                   "checked": "sequence 0 against the CPU oracle's tokens for the same prompt"}
    if check:
        import oracle as O
        from oracle import llama as OL
        c = m.config
        om = OL.synthetic(OL.Config(arch="llama", embed=c.embed, hidden=c.hidden, layers=c.layers, heads=c.heads, kv_heads=c.kv_heads,
                                    head_dim=c.head_dim, rope_dim=c.rope_dim, rope_base=c.rope_base, rope_scale=1.0, eps=c.eps,
                                    vocab=c.vocab, context=c.context), seed=0)
        # the oracle's greedy decoding, step by step so that a long check shows it is alive
        caches = om.new_caches(c.context, O.F16)
        print(f"bench.py: CPU oracle: prompt of {prompt} tokens", file=sys.stderr, flush=True)
        logits = om.logits(toks[0].tolist(), caches)
        want, margins = [], []
        for i in range(check):
            want.append(O.argmax(logits))
            top2 = np.partition(logits, -2)[-2:]
            margins.append(float(top2[1] - top2[0]))
            if i % 16 == 15:
                print(f"bench.py: CPU oracle: {i + 1} of {check} greedy tokens", file=sys.stderr, flush=True)
            if i + 1 < check:
                logits = om.logits([want[-1]], caches)
        got = out[0, :check].tolist()
        first = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), None)
        verdict = {"greedy_checked": check, "greedy_identical": sum(a == b for a, b in zip(got, want)), "first_mismatch": first,
                   "oracle_min_margin": round(min(margins), 4), "oracle_tokens": want}
    return {**verdict, "linear_dtype": linear, "layers": layers, "batch": batch, "prompt": prompt, "new": new, "prompt_s": round(t_prompt, 4), "decode_s": round(t_decode, 4),
            "decode_tok_per_s": round(batch * (new - 1) / t_decode, 1), "ms_per_step": round(t_decode / (new - 1) * 1e3, 4),
            "weight_GBps": round(per_tok_bytes / (t_decode / (new - 1)) / 1e9, 1), "build_s": round(build_s, 1),
            "first_tokens": out[0, :8].tolist(), "distinct_tokens": len(set(out[0].tolist()))}


def gemv_stamps(lib, capi, torch, n=14336, k=4096, bufs=16, launches=40):
    """Where a launch of the whole-chip Q4_0 GEMV spends its time: every workgroup's first thread reads the device's
    100 MHz clock at entry, once x is staged in LDS, after its first and its last row of W, and at exit
    (mi355x_gemv_stamps). Microseconds from the first workgroup's entry, medians over `launches` launches, each
    synchronized on its own; cold: W rotated over `bufs` copies, hot: one copy, which the caches then hold."""
    rng = np.random.default_rng(0)
    w0 = torch.from_numpy(bench_blocks_q4_0(rng, n * k)).to("cuda:0")
    ws = [w0] + [w0.clone() for _ in range(bufs - 1)]
    x = torch.randn(k, device="cuda:0")
    y = torch.empty(n, device="cuda:0")
    stamps = torch.zeros(5 * 1024, dtype=torch.int64, device="cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    call = lambda i: capi.check(lib.mi355x_qgemv(capi.Q4_0, ws[i % bufs].data_ptr(), x.data_ptr(), y.data_ptr(), 1, n, k, k, st))
    for i in range(50):
        call(i)
    torch.cuda.synchronize()
    capi.check(lib.mi355x_gemv_stamps(stamps.data_ptr()))
    out = {}
    try:
        for name in ("cold", "hot"):
            rows = []
            for i in range(launches):
                stamps.zero_()
                torch.cuda.synchronize()
                call(0 if name == "hot" else i + 3)
                torch.cuda.synchronize()
                s = stamps.cpu().numpy().reshape(-1, 5)
                s = s[s[:, 0] != 0]
                rel = (s - s[:, 0].min()) / 100.0
                rows.append([rel[:, 0].max(), np.median(rel[:, 1]), rel[:, 1].max(), np.median(rel[:, 2]), rel[:, 2].max(),
                             np.median(rel[:, 3]), rel[:, 3].max(), rel[:, 4].max(), len(s)])
            r = np.median(np.array(rows), axis=0)
            out[name] = {"workgroups": int(r[8]), "last_entry_us": round(float(r[0]), 2),
                         "x_staged_us": {"median": round(float(r[1]), 2), "last": round(float(r[2]), 2)},
                         "first_row_done_us": {"median": round(float(r[3]), 2), "last": round(float(r[4]), 2)},
                         "last_row_done_us": {"median": round(float(r[5]), 2), "last": round(float(r[6]), 2)},
                         "last_exit_us": round(float(r[7]), 2)}
    finally:
        capi.check(lib.mi355x_gemv_stamps(None))
    return out


def layer_step_bench(capi, cached=2048, new=33):
    """One decoder layer's decoding step against caches holding `cached` positions (batch 1 and 8): the whole
    model's step timed with two and with six layers, the difference divided by four, so that embedding, head and
    argmax drop out. The caches are filled by a prompt of `cached` tokens."""
    out = {}
    for batch in (1, 8):
        ms = {}
        for layers in (2, 6):
            m = build_llama(capi, layers=layers, batch=batch, context=cached + new, max_tokens=cached)
            toks = np.random.default_rng(0).integers(0, m.config.vocab, (batch, cached))
            _, (_, t_decode) = m.generate(toks, new)
            ms[layers] = t_decode / (new - 1) * 1e3
            del m
        us = (ms[6] - ms[2]) / 4 * 1e3
        # what a layer's step must read: its seven Q4_0 matrices once, and every sequence's cached keys and values (binary16)
        layer_bytes = 218103808 * 18 // 32 + batch * cached * 8 * 128 * 2 * 2
        out[f"batch{batch}"] = {"us_per_layer": round(us, 2), "bytes_per_layer": layer_bytes, "GBps": round(layer_bytes / (us * 1e-6) / 1e9, 1),
                                "frac": round(layer_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                "ms_per_step_2_layers": round(ms[2], 4), "ms_per_step_6_layers": round(ms[6], 4)}
    out["cached_positions"] = cached
    return out


def bench_blocks_kquant(rng, dtype_bytes, n_elems):
    """Random Q4_K (144-byte) or Q6_K (210-byte) super-blocks: every field uniform, the binary16 scales |N(0, 0.02)|."""
    raw = rng.integers(0, 256, size=(n_elems // 256, dtype_bytes), dtype=np.uint8)
    scales = np.abs(rng.normal(0, 0.02, size=(raw.shape[0], 2))).astype(np.float16).view(np.uint8).reshape(-1, 4)
    if dtype_bytes == 144:
        raw[:, 0:4] = scales
    else:
        raw[:, 208:210] = scales[:, 0:2]
    return raw.reshape(-1)


def rows_bench(lib, capi, torch, m=8, shapes=((14336, 4096), (4096, 14336), (4096, 4096), (6144, 4096), (28672, 4096)), iters=200, only=None):
    """The product of a few rows of x (a decoding step of a batch), mi355x_qgemv as a whole (conversion
    of x and product, two launches) over rotating copies of W. Q4_0: the kernel that reads W once for eight rows
    on the int8 matrix cores, its variant that loads each lane's block where it lies, and the one-row kernel
    run per row. Q4_K, Q6_K: the kernel that reads W once for eight rows, the tiled matrix-core kernel and the
    one-row kernels run per row. `only` (a variant's name): a few launches of that variant and nothing else, for
    counter runs."""
    rng = np.random.default_rng(0)
    st = torch.cuda.Stream()
    out = {}
    # name, dtype, bytes of a block of W and weights in it, the tune keys that select the variant
    variants = (("rows_kernel", capi.Q4_0, 18, 32, ((b"q4_0.rows_path", 0),)),
                ("rows_kernel_no_lds_pass", capi.Q4_0, 18, 32, ((b"q4_0.rows_path", 2),)),
                ("one_row_kernel_per_row", capi.Q4_0, 18, 32, ((b"q4_0.rows_path", 1),)),
                ("q4_K_rows_kernel", capi.Q4_K, 144, 256, ()),
                ("q4_K_tiled_kernel", capi.Q4_K, 144, 256, ((b"kquant.path", 3),)),
                ("q4_K_one_row_kernel_per_row", capi.Q4_K, 144, 256, ((b"kquant.path", 2), (b"kquant.mfma_rows", 1))),
                ("q6_K_rows_kernel", capi.Q6_K, 210, 256, ()),
                ("q6_K_tiled_kernel", capi.Q6_K, 210, 256, ((b"kquant.path", 3),)),
                ("q6_K_one_row_kernel_per_row", capi.Q6_K, 210, 256, ((b"kquant.path", 2), (b"kquant.mfma_rows", 1))))
    reset = ((b"q4_0.rows_path", 0), (b"kquant.path", 0), (b"kquant.mfma_rows", 0))
    try:
        for n, k in shapes:
            res = {}
            for dt in (capi.Q4_0, capi.Q4_K, capi.Q6_K):
                mine = [v for v in variants if v[1] == dt and (not only or v[0] == only)]
                if not mine:
                    continue
                bb, per = mine[0][2], mine[0][3]
                raw = bench_blocks_q4_0(rng, n * k) if dt == capi.Q4_0 else bench_blocks_kquant(rng, bb, n * k)
                nbuf = max(2, min(32, int(300e6 // raw.size)))
                w0 = torch.from_numpy(raw).to("cuda:0")
                bufs = [w0] + [w0.clone() for _ in range(nbuf - 1)]
                x = torch.randn(m, k, device="cuda:0")
                y = torch.empty(m, n, device="cuda:0")
                torch.cuda.synchronize()
                for name, _, _, _, keys in mine:
                    for key, v in reset + keys:
                        capi.check(lib.mi355x_tune(key, v))
                    with torch.cuda.stream(st):
                        call = lambda i: capi.check(lib.mi355x_qgemv(dt, bufs[i % nbuf].data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, k, st.cuda_stream))
                        for i in range(4 if only else 10):
                            call(i)
                        st.synchronize()
                        if only:
                            continue
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record(st)
                        for i in range(iters):
                            call(i)
                        e1.record(st)
                        st.synchronize()
                    us = e0.elapsed_time(e1) / iters * 1e3
                    res[name] = {"us": round(us, 2), "W_GBps": round(raw.size / (us * 1e-6) / 1e9, 1)}
                del bufs, w0, x, y
            out[f"M{m}_N{n}_K{k}"] = res
    finally:
        for key, v in reset:
            capi.check(lib.mi355x_tune(key, v))
    return out


def gemm_bench(lib, capi, torch, shapes=((512, 4096), (512, 14336), (2048, 4096), (2048, 14336)), k=4096, iters=50, kquants=True):
    """The prompt-sized products with bfloat16 activations and results, mi355x_qgemm_bf16 as a whole
    (for Q4_K and Q6_K that includes the casts and the int8 rounding of x): TFLOP/s (2 M N K) between
    HIP events on its stream, against the dense peak of the matrix instruction used (bfloat16 2.5 PFLOP/s
    for Q4_0, int8 5.0 POP/s for the K-quants; each weight takes two multiplications in both)."""
    out = {}
    rng = np.random.default_rng(0)
    st = torch.cuda.Stream()
    # "q4_0_binary16_weights": the same call with "qgemm.f16" = 1 (every weight rounded once to binary16, one
    # multiplication a weight; results within 1e-3, not exact)
    kinds = (("q4_0", capi.Q4_0, 2500.0, "frac_of_bf16_peak"), ("q4_0_binary16_weights", capi.Q4_0, 2500.0, "frac_of_f16_peak"),
             ("q4_K", capi.Q4_K, 5000.0, "frac_of_int8_peak"), ("q6_K", capi.Q6_K, 5000.0, "frac_of_int8_peak"))
    # float32 activations by Q4_0 (what the decoder's prompt pass multiplies): mi355x_qgemv, whose 24-bit
    # fixed-point x takes three int8 multiplications a weight, or, where the library's cost model says so, two
    # binary16 ones (the same integers as pairs of 12-bit digits, the same bits); priced against the int8 peak
    res = {}
    for m, n in shapes:
        w = torch.from_numpy(bench_blocks_q4_0(rng, n * k)).to("cuda:0")
        x = torch.randn(m, k, device="cuda:0")
        y = torch.empty(m, n, dtype=torch.float32, device="cuda:0")
        torch.cuda.synchronize()
        with torch.cuda.stream(st):
            call = lambda: capi.check(lib.mi355x_qgemv(capi.Q4_0, w.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, k, st.cuda_stream))
            for _ in range(5):
                call()
            st.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(st)
            for _ in range(iters):
                call()
            e1.record(st)
            st.synchronize()
        us = e0.elapsed_time(e1) / iters * 1e3
        tf = 2.0 * m * n * k / (us * 1e-6) / 1e12
        res[f"M{m}_N{n}_K{k}"] = {"us": round(us, 2), "TFLOPs": round(tf, 1), "frac_of_int8_peak": round(tf / 5000.0, 4)}
        del w, x, y
    out["q4_0_f32_x"] = res
    for name, dt, peak, frac_key in kinds:
        if dt != capi.Q4_0 and not kquants:
            continue
        res = {}
        capi.check(lib.mi355x_tune(b"qgemm.f16", 1 if name == "q4_0_binary16_weights" else 0))
        for m, n in shapes:
            if dt == capi.Q4_0:
                raw = bench_blocks_q4_0(rng, n * k)
            else:
                raw = bench_blocks_kquant(rng, 144 if dt == capi.Q4_K else 210, n * k)
            w = torch.from_numpy(raw).to("cuda:0")
            x = torch.randn(m, k, device="cuda:0").to(torch.bfloat16)
            y = torch.empty(m, n, dtype=torch.bfloat16, device="cuda:0")
            torch.cuda.synchronize()
            with torch.cuda.stream(st):
                call = lambda: capi.check(lib.mi355x_qgemm_bf16(dt, w.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, k, capi.BF16, st.cuda_stream))
                for _ in range(5):
                    call()
                st.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(st)
                for _ in range(iters):
                    call()
                e1.record(st)
                st.synchronize()
            us = e0.elapsed_time(e1) / iters * 1e3
            tf = 2.0 * m * n * k / (us * 1e-6) / 1e12
            res[f"M{m}_N{n}_K{k}"] = {"us": round(us, 2), "TFLOPs": round(tf, 1), frac_key: round(tf / peak, 4)}
            del w, x, y
        out[name] = res
    capi.check(lib.mi355x_tune(b"qgemm.f16", 0))
    return out


def shapes_bench(lib, capi, torch, launches=1024):
    """The one-row products of the other configurations, each as the boundary takes it (float32 x in, one
    mi355x_qgemv call, graph-replayed over rotating copies of W that together exceed the last-level cache):
    the Q8_0 4096 x 4096 product and the Q4_0 down, q/o and k/v shapes. Checked against the oracle before timing."""
    out = {}
    for name, kind, n, k in (("q8_0_4096x4096", "q8_0", 4096, 4096), ("q4_0_down_14336->4096", "q4_0", 4096, 14336),
                             ("q4_0_qo_4096->4096", "q4_0", 4096, 4096), ("q4_0_kv_4096->1024", "q4_0", 1024, 4096)):
        bb = 18 if kind == "q4_0" else 34
        nb = int(min(256, max(16, 600e6 // gemv_bytes(n, k, bb) + 1)))
        g = Gemv(lib, capi, torch, n, k, nb, kind=kind)
        g.check()
        ms, _ = g.time(g.step, max(launches, 2 * nb) // nb * nb, 2 * nb)
        gbps = g.bytes() / (ms * 1e-3) / 1e9
        out[name] = {"N": n, "K": k, "us_per_step": round(ms * 1e3, 3), "bytes": g.bytes(), "GBps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBS, 4),
                     "copies_of_W": nb}
        if kind == "q4_0":
            g.step(0)
            out[name]["kernel"] = g.kernel_name()
        del g
    return out


def cpu_baseline_q8_0(n=4096, k=4096, seconds=5.0):
    """The reference's CPU route for a Q8_0 linear, restated by the oracle: x rounded to int8 per block of 32
    (quantizeRow, backend/cpu/qmatmul.go:208-254), then the AVX2 integer dot products
    (tools/asmgen/qamd64/main.go:173-226) over rows of W shared among all host cores (qmatmul.go:285-302)."""
    import oracle as O
    rng = np.random.default_rng(0)
    raw = q_blocks(rng, "q8_0", n * k)
    x = rng.normal(size=k).astype(np.float32)
    threads = O.lib().mo_num_threads()
    simd = bool(O.lib().mo_has_simd())
    O.qmatmul(O.Q8_0, raw, x, n, k, simd=simd)  # warm
    iters, t0 = 0, time.perf_counter()
    while True:
        O.qmatmul(O.Q8_0, raw, x, n, k, simd=simd)
        iters += 1
        dt = time.perf_counter() - t0
        if dt >= seconds and iters >= 5:
            break
    per = dt / iters
    return {"value": round(gemv_bytes(n, k, 34) / per / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port", "avx2": simd,
            "sample": f"{iters} Q8_0 products {n}x{k} (quantizeRow of x, then int8 dot products, {per * 1e6:.1f} us each), {dt:.1f} s wall"}


def cpu_baseline(n, k, seconds=2.0):
    """The reference's CPU route for a Q4_0 linear, restated by the oracle:
    weights decoded to float32 once (untimed), then the float32 GEMV over all
    host cores. Throughput is quoted in the same algorithmic bytes as the GPU's."""
    import oracle as O
    rng = np.random.default_rng(0)
    raw = bench_blocks_q4_0(rng, n * k)
    x = rng.normal(size=k).astype(np.float32)
    wf = O.dequantize(O.Q4_0, raw).reshape(n, k)
    threads = O.lib().mo_num_threads()
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), model)
    except OSError:
        pass
    O.sgemv(wf, x)  # warm
    iters, t0 = 0, time.perf_counter()
    while True:
        O.sgemv(wf, x)
        iters += 1
        dt = time.perf_counter() - t0
        if dt >= seconds and iters >= 5:
            break
    per = dt / iters
    return {
        "value": round(gemv_bytes(n, k) / per / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"{iters} float32 GEMVs {n}x{k} over weights decoded once from Q4_0 ({wf.nbytes / 1e6:.0f} MB read per GEMV, "
                  f"{per * 1e3:.2f} ms each; {wf.nbytes / per / 1e9:.1f} GB/s of float32 reads), {dt:.1f} s wall, on {model}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--bufs", type=int, default=16, help="copies of W to rotate over (16 x 33 MB > the 256 MB last-level cache)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--all-shapes", action="store_true", help="also time the other decode shapes and the streaming-read ceiling")
    ap.add_argument("--counters", type=int, default=0, metavar="N",
                    help="only launch the GEMV kernel and a 256 MiB copy N times each (for rocprofv3 --pmc runs)")
    ap.add_argument("--gemv-stamps", action="store_true", help="only: per-workgroup clock readings of the GEMV's launches (dispatch, x staging, rows, exit)")
    ap.add_argument("--gemm", action="store_true", help="time the prompt-sized products of Q4_K and Q6_K too (the Q4_0 ones are in every run)")
    ap.add_argument("--no-gemm", action="store_true", help="skip the prompt-sized products")
    ap.add_argument("--gemm-shapes", default=None, metavar="MxN[,MxN...]", help="the prompt-sized products of these shapes only (K = 4096), e.g. 2048x14336")
    ap.add_argument("--gemm-iters", type=int, default=50, help="timed calls per prompt-sized product")
    ap.add_argument("--no-shapes", action="store_true", help="skip the one-row products of the other shapes (Q8_0 4096x4096; Q4_0 down, q/o, k/v)")
    ap.add_argument("--rows", action="store_true", help="also time the Q4_0, Q4_K and Q6_K products of eight rows of x (a batch's decoding step) at the model's shapes")
    ap.add_argument("--rows-counters", metavar="VARIANT", default=None,
                    help="only launch that variant of the eight-row product a few times at 14336x4096 (for rocprofv3 --pmc runs): "
                         "rows_kernel, rows_kernel_no_lds_pass, one_row_kernel_per_row (Q4_0), q4_K_rows_kernel, q6_K_rows_kernel, ...")
    ap.add_argument("--layer-step", action="store_true", help="(default; kept for older command lines)")
    ap.add_argument("--no-layer-step", action="store_true", help="skip one decoder layer's decoding step against 2048 cached positions (batch 1, 8)")
    ap.add_argument("--eager", action="store_true", help="launch the timed steps one by one instead of replaying a HIP graph")
    ap.add_argument("--no-decode", action="store_true", help="skip decoding with the whole random-init 8B-shaped model")
    ap.add_argument("--decode", action="store_true", help="(default; kept for older command lines)")
    ap.add_argument("--decode-check", type=int, default=64, metavar="N",
                    help="compare the first N greedy tokens of the 512-token prompt with the CPU oracle's (0: skip; about a minute of CPU time for 64)")
    ap.add_argument("--no-decode-batch8", action="store_true", help="skip the second decoding run, with eight sequences")
    ap.add_argument("--decode-layers", type=int, default=32)
    ap.add_argument("--decode-batch", type=int, default=1)
    ap.add_argument("--decode-linear", choices=("q4_0", "q4_K", "q6_K"), default="q4_0",
                    help="block dtype of the decoder's linear weights (the oracle check is for q4_0)")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="a launch-plan override for mi355x_tune before anything runs (may be repeated), e.g. q4_0.stream=1")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on one GPU; --gpus must be 1 (no collectives or sharding are built)")

    import torch
    from mimir_amd import capi
    lib = capi.load()  # raises if the HIP library is not built: there is no fallback
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible")
    capi.check(lib.mi355x_init(0))
    for kv in args.tune:
        key, _, val = kv.partition("=")
        capi.check(lib.mi355x_tune(key.encode(), int(val)))

    if args.rows_counters:
        rows_bench(lib, capi, torch, shapes=((14336, 4096),), only=args.rows_counters)
        per_weight = {"q4_K": 144 / 256, "q6_K": 210 / 256}.get(args.rows_counters[:4], 18 / 32)
        print(json.dumps({"rows_counters": args.rows_counters, "launches": 4, "W_bytes": int(14336 * 4096 * per_weight)}))
        return
    n, k = 14336, 4096
    if args.gemv_stamps:
        print(json.dumps({"gemv_stamps": gemv_stamps(lib, capi, torch, n, k, args.bufs)}))
        return
    g = Gemv(lib, capi, torch, n, k, args.bufs)
    g.check()
    if args.counters:
        # for a counter run of the profiler: a few launches of the GEMV kernel and,
        # to scale the counters by, of a copy of known size (256 MiB read, 256 MiB
        # written), each from buffers the cache does not hold
        src = [torch.empty(1 << 28, dtype=torch.uint8, device="cuda:0").random_(0, 255) for _ in range(2)]
        dst = torch.empty(1 << 28, dtype=torch.uint8, device="cuda:0")
        with torch.cuda.stream(g.stream):
            for i in range(args.counters):
                g.kernel(i)
                dst.copy_(src[i % 2])
            g.stream.synchronize()
        print(json.dumps({"counters": args.counters, "gemv_bytes": gemv_bytes(n, k), "copy_read_bytes": 1 << 28, "copy_write_bytes": 1 << 28}))
        return
    # a step: the product as the boundary takes it (float32 activations in, float32 out), one launch,
    # graph-replayed; the roofline: that launch's kernel, each launch between its own pair of events
    step_ms, step_wall_ms = g.time(g.step, args.steps, args.warmup, graph=not args.eager)
    seq_ms, _ = g.time(g.from_converted, args.steps, args.warmup, graph=True)
    hot_ms, _ = g.time(lambda i: g.step(0), args.steps, args.warmup, graph=True)  # one copy of W: the last-level cache serves it
    kern_us, kern_min, kern_max = g.kernel_durations(args.steps, args.warmup)
    bytes_ = gemv_bytes(n, k)
    g.step(0)
    kernel = g.kernel_name()  # what the library's dispatch launched for this shape
    g.stream.synchronize()
    value = bytes_ / (step_ms * 1e-3) / 1e9
    achieved = bytes_ / (kern_us * 1e-6) / 1e9
    out = {
        "metric": "Q4_0 GEMV HBM GB/s (% of peak); decode tok/s, 8B-shape, batch 1",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i4 x 24-bit fixed point, f32 scales and output", "data": "synthetic",
        "config": {"workload": "Q4_0 decode GEMV 4096->14336 (Llama-3-8B gate/up), batch 1, W rotated over "
                               f"{args.bufs} HBM-resident copies; a step = one mi355x_qgemv call (float32 x in, its conversion to "
                               "fixed point inside the GEMV launch, float32 y out), "
                               + ("launched one by one" if args.eager else "replayed from a HIP graph"),
                   "N": n, "K": k, "M": 1, "wall_ms_per_step": round(step_wall_ms, 6)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH if kernel == TRAFFIC_KERNEL else None,
                     "kernel": kernel, "bytes_per_launch": bytes_, "us_per_launch": round(kern_us, 3),
                     "us_min": round(kern_min, 3), "us_max": round(kern_max, 3),
                     # the product over activations converted beforehand (as a decoding step's launches take them),
                     # back to back in a graph, the wait between dependent kernels included
                     "us_per_launch_from_converted_in_sequence": round(seq_ms * 1e3, 3),
                     # the step over a single copy of W, which the 256 MB last-level cache then holds: not an HBM figure
                     "us_per_step_cache_resident": round(hot_ms * 1e3, 3)},
    }
    # what a plain 128-bit streaming read of the same bytes, over as many rotating buffers, reaches on this device
    out["roofline"]["stream_read_same_bytes_GBps"] = round(stream_ceiling(lib, capi, torch, 33030144, args.bufs, args.steps), 1)
    # the same product as one, two and four chains side by side on streams of their own, no edges between the chains
    out["roofline"]["us_per_launch_in_parallel_chains"] = {str(w): round(g.time_independent(w), 3) for w in (1, 2, 4)}
    extra = {}
    if args.all_shapes:
        for name, (nn, kk) in {"down_14336->4096": (4096, 14336), "qo_4096->4096": (4096, 4096), "kv_4096->1024": (1024, 4096)}.items():
            nb = min(256, max(args.bufs, int(600e6 // gemv_bytes(nn, kk)) + 1))
            gg = Gemv(lib, capi, torch, nn, kk, nb)
            gg.check()
            e, _ = gg.time(gg.kernel, args.steps, args.warmup)
            extra[name] = {"us_per_launch": round(e * 1e3, 3), "GBps": round(gemv_bytes(nn, kk) / (e * 1e-3) / 1e9, 1)}
            del gg
        extra["gate_up_eager_step_us"] = round(g.time(g.step, args.steps, args.warmup, graph=False)[0] * 1e3, 3)
        extra["stream_read_33MB_GBps"] = out["roofline"]["stream_read_same_bytes_GBps"]
        extra["stream_read_1GB_GBps"] = round(stream_ceiling(lib, capi, torch, 1 << 30, 2, 50), 1)
        out["extra"] = extra
    del g
    if not args.no_shapes:
        out["gemv_shapes"] = shapes_bench(lib, capi, torch)
    if not args.no_gemm:
        if args.gemm_shapes:
            shapes = tuple(tuple(int(v) for v in sh.split("x")) for sh in args.gemm_shapes.split(","))
            out["prefill_gemm"] = gemm_bench(lib, capi, torch, shapes=shapes, kquants=args.gemm, iters=args.gemm_iters)
        else:
            out["prefill_gemm"] = gemm_bench(lib, capi, torch, kquants=args.gemm, iters=args.gemm_iters)
    if args.rows:
        out["batch_rows_gemv"] = rows_bench(lib, capi, torch)
    if not args.no_layer_step:
        out["layer_step"] = layer_step_bench(capi)
    if not args.no_decode:
        out["decode"] = decode_bench(capi, layers=args.decode_layers, batch=args.decode_batch, check=args.decode_check if args.decode_linear == "q4_0" else 0,
                                     linear=args.decode_linear)
        if args.decode_batch == 1 and args.decode_linear == "q4_0" and args.decode_layers == 32 and not args.no_decode_batch8:
            # the same model with eight sequences: every weight read once a step for all of them
            out["decode_batch8"] = decode_bench(capi, layers=32, batch=8, want_tokens=out["decode"].get("oracle_tokens"))
        out["decode"].pop("oracle_tokens", None)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(n, k, seconds=10.0)
        out["cpu_baseline_q8_0"] = cpu_baseline_q8_0(seconds=5.0)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
