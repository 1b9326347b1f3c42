"""Shared helpers of the tests: seeded synthetic blocks in the shapes the
benchmark configurations name, the independent dequantizer used to pin the
oracle, and the comparison rule of the reference's kernel conformance check
(backend/internal/kerneltest/kerneltest.go:77-125)."""
import numpy as np

import oracle as O


def random_scale_bits(rng, n):
    """Finite binary16 scales below 1/2 in magnitude, one in eight subnormal or
    zero, as internal/quanttest/quanttest.go:57-66 draws them."""
    sign = rng.integers(0, 2, n).astype(np.uint16) << 15
    exp = (1 + rng.integers(0, 13, n)).astype(np.uint16)
    exp[rng.integers(0, 8, n) == 0] = 0
    return sign | (exp << 10) | rng.integers(0, 1024, n).astype(np.uint16)


def random_blocks(rng, dt, n_elems):
    """Random blocks of dt: every byte uniform, scales finite
    (internal/quanttest/quanttest.go:33-55; Q4_0 likewise)."""
    bs, bb = O.block_size(dt), O.block_bytes(dt)
    nb = n_elems // bs
    b = rng.integers(0, 256, (nb, bb), dtype=np.uint8)

    def put(col, bits):
        b[:, col] = bits & 0xff
        b[:, col + 1] = bits >> 8

    if dt in (O.Q8_0, O.Q4_0):
        put(0, random_scale_bits(rng, nb))
    elif dt == O.Q4_K:
        put(0, random_scale_bits(rng, nb)); put(2, random_scale_bits(rng, nb))
    elif dt == O.Q6_K:
        put(208, random_scale_bits(rng, nb))
    return b.reshape(-1)


def bench_blocks(rng, dt, n_elems):
    """Weights as the benchmark configurations draw them: quants uniform over
    their range ([-127,127] for Q8_0, nibbles [0,15] for Q4_0) and one
    binary16 scale |N(0, 0.02)| per block."""
    bs, bb = O.block_size(dt), O.block_bytes(dt)
    nb = n_elems // bs
    b = np.empty((nb, bb), np.uint8)
    d = np.abs(rng.normal(0, 0.02, nb)).astype(np.float32).astype(np.float16).view(np.uint16)
    b[:, 0] = d & 0xff
    b[:, 1] = d >> 8
    if dt == O.Q8_0:
        b[:, 2:] = rng.integers(-127, 128, (nb, 32)).astype(np.int8).view(np.uint8)
    elif dt == O.Q4_0:
        b[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    else:
        raise ValueError(dt)
    return b.reshape(-1)


def exact_rows(rng, dt, m, k):
    """Rows the CPU path rounds to int8 without error: integers over 128 with
    one +-127/128 per activation block (backend/internal/kerneltest/quant.go:45-64)."""
    bs = 32 if dt in (O.Q8_0, O.Q4_0) else 256
    x = (rng.integers(0, 255, m * k) - 127).astype(np.float32) / 128
    for b in range(0, m * k, bs):
        x[b + rng.integers(0, bs)] = (2 * rng.integers(0, 2) - 1) * 127 / 128
    return x.reshape(m, k)


# ---- an independent dequantizer (numpy, float32 step by step) -------------
# Transcribed from ggml's published dequantize_row_* loops the way
# internal/quanttest/quanttest.go:90-165 does, not from the oracle.

def half_bits_to_f32(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


def ref_dequant(dt, data):
    data = np.asarray(data, np.uint8)
    bb = O.block_bytes(dt)
    blk = data.reshape(-1, bb)
    nb = blk.shape[0]
    f = np.float32
    if dt == O.Q8_0:
        d = half_bits_to_f32(blk[:, 0].astype(np.uint16) | blk[:, 1].astype(np.uint16) << 8)
        return (blk[:, 2:].view(np.int8).astype(f) * d[:, None]).reshape(-1)
    if dt == O.Q4_0:
        d = half_bits_to_f32(blk[:, 0].astype(np.uint16) | blk[:, 1].astype(np.uint16) << 8)
        lo = (blk[:, 2:] & 0xf).astype(np.int32) - 8
        hi = (blk[:, 2:] >> 4).astype(np.int32) - 8
        return (np.concatenate([lo, hi], axis=1).astype(f) * d[:, None]).reshape(-1)
    if dt == O.Q4_K:
        out = np.empty((nb, 256), f)
        d = half_bits_to_f32(blk[:, 0].astype(np.uint16) | blk[:, 1].astype(np.uint16) << 8)
        dmin = half_bits_to_f32(blk[:, 2].astype(np.uint16) | blk[:, 3].astype(np.uint16) << 8)
        s = blk[:, 4:16]
        q = blk[:, 16:]

        def scale_min(j):
            if j < 4:
                return s[:, j] & 63, s[:, j + 4] & 63
            return (s[:, j + 4] & 0xf) | ((s[:, j - 4] >> 6) << 4), (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)

        for j in range(4):
            sc, m = scale_min(2 * j)
            d1 = (d * sc.astype(f)).astype(f); m1 = (dmin * m.astype(f)).astype(f)
            sc, m = scale_min(2 * j + 1)
            d2 = (d * sc.astype(f)).astype(f); m2 = (dmin * m.astype(f)).astype(f)
            ql = q[:, 32 * j:32 * j + 32]
            out[:, 64 * j:64 * j + 32] = (d1[:, None] * (ql & 0xf).astype(f)).astype(f) - m1[:, None]
            out[:, 64 * j + 32:64 * j + 64] = (d2[:, None] * (ql >> 4).astype(f)).astype(f) - m2[:, None]
        return out.reshape(-1)
    if dt == O.Q6_K:
        out = np.empty((nb, 256), f)
        d = half_bits_to_f32(blk[:, 208].astype(np.uint16) | blk[:, 209].astype(np.uint16) << 8)
        for n in range(2):
            ql = blk[:, 64 * n:64 * n + 64]; qh = blk[:, 128 + 32 * n:128 + 32 * n + 32]
            sc = blk[:, 192 + 8 * n:192 + 8 * n + 8].view(np.int8)
            for l in range(32):
                i = l // 16
                q1 = ((ql[:, l] & 0xf) | (((qh[:, l] >> 0) & 3) << 4)).astype(np.int32) - 32
                q2 = ((ql[:, l + 32] & 0xf) | (((qh[:, l] >> 2) & 3) << 4)).astype(np.int32) - 32
                q3 = ((ql[:, l] >> 4) | (((qh[:, l] >> 4) & 3) << 4)).astype(np.int32) - 32
                q4 = ((ql[:, l + 32] >> 4) | (((qh[:, l] >> 6) & 3) << 4)).astype(np.int32) - 32
                out[:, 128 * n + l] = (d * sc[:, i].astype(f)).astype(f) * q1.astype(f)
                out[:, 128 * n + l + 32] = (d * sc[:, i + 2].astype(f)).astype(f) * q2.astype(f)
                out[:, 128 * n + l + 64] = (d * sc[:, i + 4].astype(f)).astype(f) * q3.astype(f)
                out[:, 128 * n + l + 96] = (d * sc[:, i + 6].astype(f)).astype(f) * q4.astype(f)
        return out.reshape(-1)
    raise ValueError(dt)


def bits_equal(a, b):
    """Bit equality of two float32 arrays, NaN matching NaN."""
    a = np.asarray(a, np.float32); b = np.asarray(b, np.float32)
    same = a.view(np.uint32) == b.view(np.uint32)
    return bool(np.all(same | (np.isnan(a) & np.isnan(b))))


def check_close(got, want, tol, what=""):
    """The reference's conformance rule: |got - want| <= tol * max(1, |want|),
    NaN matching NaN, infinities matching exactly."""
    got = np.asarray(got, np.float64).reshape(-1); want = np.asarray(want, np.float64).reshape(-1)
    assert got.shape == want.shape, (got.shape, want.shape)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan), f"{what}: NaN pattern differs"
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf]), f"{what}: infinities differ"
    ok = ~(nan | inf)
    err = np.abs(got[ok] - want[ok]); lim = tol * np.maximum(1, np.abs(want[ok]))
    bad = err > lim
    assert not bad.any(), f"{what}: {bad.sum()} of {ok.sum()} beyond tol {tol}; worst {err.max():.3e} at {int(np.argmax(err))}"


def rel_l2(got, want):
    got = np.asarray(got, np.float64).reshape(-1); want = np.asarray(want, np.float64).reshape(-1)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def write_mim(path, tensors, metadata):
    """A .mim container in the layout mimir_amd.mimfile reads (a preamble, an index of two sections and the
    tensor rows with their name pool, a "MIMM" metadata section, a weights section): tensors is a list of
    (name, container dtype code, logical shape, bytes); metadata maps keys to int, float or str."""
    import struct
    pool, rows, blob = b"", b"", b""
    for name, code, shape, data in tensors:
        nm = name.encode()
        while len(blob) % 64:
            blob += b"\0"
        dims = list(shape) + [0] * (8 - len(shape))
        rows += struct.pack("<IIIB3x", len(pool), len(nm), code, len(shape)) + struct.pack("<8Q", *dims) + struct.pack("<QQ", len(blob), len(data))
        pool += nm
        blob += bytes(data)
    mpool, ments = b"", b""
    for key, val in metadata.items():
        kb = key.encode()
        koff = len(mpool)
        mpool += kb
        if isinstance(val, bool):
            typ, v8, nbytes = 4, bytes([int(val)]) + b"\0" * 7, 0
        elif isinstance(val, int):
            typ, v8, nbytes = 1, struct.pack("<q", val), 0
        elif isinstance(val, float):
            typ, v8, nbytes = 3, struct.pack("<d", val), 0
        else:
            sb = str(val).encode()
            typ, v8, nbytes = 5, struct.pack("<Q", len(mpool)), len(sb)
            mpool += sb
        ments += struct.pack("<IIB3xI", koff, len(kb), typ, nbytes) + v8 + b"\0" * 8
    meta = b"MIMM" + struct.pack("<IQ", len(metadata), len(mpool)) + ments + mpool
    index_off = 64
    index_len = 16 + 2 * 64 + len(rows) + len(pool)
    meta_off = (index_off + index_len + 63) // 64 * 64
    data_off = (meta_off + len(meta) + 63) // 64 * 64
    file_len = data_off + len(blob)
    sect = lambda kind, off, length: struct.pack("<IIQQ", kind, 0, off, length) + b"\0" * 40
    index = struct.pack("<IIQ", 2, len(tensors), len(pool)) + sect(1, data_off, len(blob)) + sect(2, meta_off, len(meta)) + rows + pool
    head = b"MIM\0" + struct.pack("<HHIIQQQQQ", 0, 1, 0x0A0B0C0D, 64, index_off, index_len, data_off, len(blob), file_len)
    out = head + b"\0" * (64 - len(head)) + index
    out += b"\0" * (meta_off - len(out)) + meta
    out += b"\0" * (data_off - len(out)) + blob
    with open(path, "wb") as f:
        f.write(out)


def synthetic_llama_mim(path, om, q4_0_code, arch="llama"):
    """The oracle's synthetic model `om` (oracle.llama.synthetic) as a .mim file whose Q4_0 tensors carry
    the container code q4_0_code."""
    codes = {O.Q4_0: q4_0_code, O.Q8_0: 64, O.Q4_K: 66, O.Q6_K: 67}
    c = om.config
    tensors = []
    wt = lambda name, w: tensors.append((name, codes[w.dtype], (w.n, w.k), np.asarray(w.data, np.uint8).tobytes()))
    f32 = lambda name, v: tensors.append((name, 1, (len(v),), np.asarray(v, "<f4").tobytes()))
    wt("token_embd.weight", om.embed)
    wt("output.weight", om.output)
    f32("output_norm.weight", om.norm)
    for i, b in enumerate(om.blocks):
        p = f"blk.{i}."
        f32(p + "attn_norm.weight", b.attn_norm); f32(p + "ffn_norm.weight", b.ffn_norm)
        for leaf, w in (("attn_q", b.q), ("attn_k", b.k), ("attn_v", b.v), ("attn_output", b.o), ("ffn_gate", b.gate), ("ffn_up", b.up), ("ffn_down", b.down)):
            wt(p + leaf + ".weight", w)
    md = {"general.architecture": arch, f"{arch}.embedding_length": c.embed, f"{arch}.feed_forward_length": c.hidden,
          f"{arch}.block_count": c.layers, f"{arch}.attention.head_count": c.heads, f"{arch}.attention.head_count_kv": c.kv_heads,
          f"{arch}.attention.key_length": c.head_dim, f"{arch}.rope.dimension_count": c.rope_dim, f"{arch}.rope.freq_base": float(c.rope_base),
          f"{arch}.attention.layer_norm_rms_epsilon": float(c.eps), f"{arch}.context_length": c.context}
    write_mim(path, tensors, md)
