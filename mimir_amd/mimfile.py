"""Reader for Mimir Model (.mim) containers: tensors and metadata only.

The layout is the one the reference's fixture writer emits
(tools/golden/gen.py:937-997) and its loaders consume
(internal/goldentest/goldentest.go:96-169, llm/model.go:77-141): a 64-byte
little-endian preamble, an index of sections and tensor rows with a name
pool, a metadata section ("MIMM") and a weights section that tensor offsets
are relative to. Graph sections are skipped: the decode path needs weights
and hyperparameters alone (llm/llm_test.go:132-154).

Block-quantized tensors are returned as their raw ggml bytes (uint8), with
the logical element shape alongside, which is what a device upload wants.

Q4_0 has no container code here: the reference's block accounting
(backend/quant.go:24-48) and every fixture it holds know Q8_0, Q4_K and Q6_K
only, and the code a converter would write for Q4_0 is defined in the
mimir-model module, which the reference does not vendor. A caller who knows it
passes it as `q4_0_code`; tensors of that code are then kept as 18-byte blocks
of 32 (ggml's block_q4_0) under the dtype name "q4_0".
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np

# dtype codes of the container (observed in the reference's fixtures).
F32, F16, BF16, U8, I32, I64 = 1, 2, 3, 6, 9, 11
Q8_0, Q4_K, Q6_K = 64, 66, 67

_PLAIN = {
    F32: np.dtype("<f4"),
    F16: np.dtype("<f2"),
    BF16: np.dtype("<u2"),  # bits; numpy has no bfloat16
    U8: np.dtype("u1"),
    I32: np.dtype("<i4"),
    I64: np.dtype("<i8"),
}
# (elements per block, bytes per block), as backend/quant.go:24-48.
_BLOCKS = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}
DTYPE_NAMES = {F32: "f32", F16: "f16", BF16: "bf16", U8: "u8", I32: "i32", I64: "i64",
               Q8_0: "q8_0", Q4_K: "q4_K", Q6_K: "q6_K"}


Q4_0_BLOCK = (32, 18)


class MimError(ValueError):
    pass


@dataclass
class MimTensor:
    name: str
    dtype: int          # container dtype code
    shape: tuple        # logical element shape
    data: np.ndarray    # plain dtypes: array of `shape`; block dtypes: uint8 [nbytes]
    dtype_name: str = ""  # "f32", "q8_0", ...; "q4_0" for the code the file was opened with
    quantized: bool = False


class MimFile:
    """The tensors and metadata of one .mim file, read eagerly."""

    def __init__(self, path: str, q4_0_code: int | None = None):
        with open(path, "rb") as f:
            raw = f.read()
        self.path = path
        if q4_0_code is not None and (q4_0_code in _PLAIN or q4_0_code in _BLOCKS):
            raise MimError(f"{path}: container code {q4_0_code} is {DTYPE_NAMES[q4_0_code]}, not free for q4_0")
        self._blocks = dict(_BLOCKS)
        self._names = dict(DTYPE_NAMES)
        if q4_0_code is not None:
            self._blocks[q4_0_code] = Q4_0_BLOCK
            self._names[q4_0_code] = "q4_0"
        self.tensors: dict[str, MimTensor] = {}
        self.metadata: dict[str, object] = {}
        self._parse(raw)

    def names(self):
        return list(self.tensors)

    def __getitem__(self, name: str) -> MimTensor:
        return self.tensors[name]

    def __contains__(self, name: str) -> bool:
        return name in self.tensors

    # ---- parsing -----------------------------------------------------
    def _parse(self, raw: bytes) -> None:
        if len(raw) < 64 or raw[:4] != b"MIM\0":
            raise MimError(f"{self.path}: not a .mim file")
        major, minor, order, _align, index_off, index_len, data_off, data_len, file_len = struct.unpack_from(
            "<HHIIQQQQQ", raw, 4)
        if order != 0x0A0B0C0D:
            raise MimError(f"{self.path}: byte-order mark {order:#x}")
        if major != 0:
            raise MimError(f"{self.path}: container version {major}.{minor}")
        if file_len != len(raw) or index_off + index_len > len(raw) or data_off + data_len > len(raw):
            raise MimError(f"{self.path}: truncated ({len(raw)} bytes, header says {file_len})")
        n_sections, n_tensors, pool_len = struct.unpack_from("<IIQ", raw, index_off)
        at = index_off + 16
        sections = []
        for _ in range(n_sections):
            kind, _flags, off, length = struct.unpack_from("<IIQQ", raw, at)
            sections.append((kind, off, length))
            at += 64
        rows_at = at
        pool_at = rows_at + 96 * n_tensors
        if pool_at + pool_len > len(raw):
            raise MimError(f"{self.path}: index past end of file")
        weights = next(((o, l) for k, o, l in sections if k == 1), None)
        for i in range(n_tensors):
            r = rows_at + 96 * i
            name_off, name_len, dtype, ndim = struct.unpack_from("<IIIB", raw, r)
            dims = struct.unpack_from("<8Q", raw, r + 16)
            offset, nbytes = struct.unpack_from("<QQ", raw, r + 80)
            name = raw[pool_at + name_off: pool_at + name_off + name_len].decode()
            shape = tuple(int(d) for d in dims[:ndim])
            if weights is None or offset + nbytes > weights[1]:
                raise MimError(f"{self.path}: tensor {name} outside the weights section")
            blob = raw[weights[0] + offset: weights[0] + offset + nbytes]
            self.tensors[name] = self._tensor(name, dtype, shape, blob)
        for kind, off, length in sections:
            if kind == 2:
                self._metadata(raw[off: off + length])

    def _tensor(self, name, dtype, shape, blob) -> MimTensor:
        n = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if dtype in _PLAIN:
            dt = _PLAIN[dtype]
            if len(blob) != n * dt.itemsize:
                raise MimError(f"{self.path}: {name}: {len(blob)} bytes for {shape} {dt}")
            return MimTensor(name, dtype, shape, np.frombuffer(blob, dt).reshape(shape).copy(), self._names[dtype], False)
        if dtype in self._blocks:
            bs, bb = self._blocks[dtype]
            if not shape or shape[-1] % bs or len(blob) != n // bs * bb:
                raise MimError(f"{self.path}: {name}: {len(blob)} bytes for {shape} blocks of {bs}")
            return MimTensor(name, dtype, shape, np.frombuffer(blob, np.uint8).copy(), self._names[dtype], True)
        raise MimError(f"{self.path}: {name}: unknown dtype code {dtype}")

    def _metadata(self, sec: bytes) -> None:
        if sec[:4] != b"MIMM":
            raise MimError(f"{self.path}: metadata section magic {sec[:4]!r}")
        count, pool_len = struct.unpack_from("<IQ", sec, 4)
        pool_at = 16 + 32 * count
        pool = sec[pool_at: pool_at + pool_len]
        for i in range(count):
            e = 16 + 32 * i
            key_off, key_len, typ, nbytes = struct.unpack_from("<IIB3xI", sec, e)
            key = pool[key_off: key_off + key_len].decode()
            val = sec[e + 16: e + 24]
            if typ == 1:
                self.metadata[key] = struct.unpack("<q", val)[0]
            elif typ == 2:
                self.metadata[key] = struct.unpack("<Q", val)[0]
            elif typ == 3:
                self.metadata[key] = struct.unpack("<d", val)[0]
            elif typ == 4:
                self.metadata[key] = bool(val[0])
            elif typ == 5:
                off = struct.unpack("<Q", val)[0]
                self.metadata[key] = pool[off: off + nbytes].decode(errors="replace")
            else:  # arrays and anything newer: keep the raw bytes
                off = struct.unpack("<Q", val)[0]
                self.metadata[key] = bytes(pool[off: off + nbytes])


def golden_cases(path: str) -> dict[str, dict]:
    """Groups the tensors of a golden fixture by case: '<case>/in<i>', '<case>/out',
    '<case>/gout', '<case>/grad<i>' (tools/golden/gen.py:9-14)."""
    f = MimFile(path)
    cases: dict[str, dict] = {}
    for name, t in f.tensors.items():
        case, _, leaf = name.rpartition("/")
        c = cases.setdefault(case, {"in": {}, "grad": {}})
        if leaf.startswith("in"):
            c["in"][int(leaf[2:])] = t
        elif leaf.startswith("grad"):
            c["grad"][int(leaf[4:])] = t
        else:
            c[leaf] = t
    for c in cases.values():
        c["in"] = [c["in"][i] for i in sorted(c["in"])]
    return cases
