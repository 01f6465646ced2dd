"""Reader and writer for the `BSMXFIX1` golden-vector container.

TEST INFRASTRUCTURE: only tests (and the script that extracts the committed
golden subset) use this module; nothing on the product path imports it.

The container is the one the reference's recorded-MLX fixtures use
(reference: crates/nuvec-core/tests/common/fixture.rs:1-121): little-endian

    magic "BSMXFIX1" | meta:str | count:u32 | case*
    case   := name:str op:str n_in:u8 tensor* n_out:u8 tensor*
    tensor := dtype:u8 ndim:u8 dims:u64* nbytes:u64 data
    str    := len:u16 utf8

Parameters are spelled into `op` as `op|k=v|...`.  dtype codes index
`DTYPES` below (fixture.rs:15-30).
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field

import numpy as np

MAGIC = b"BSMXFIX1"
DTYPES = ["bool", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64",
          "f16", "bf16", "f32", "f64", "c64"]
# numpy has no bfloat16: bf16 tensors are carried as their uint16 bit patterns.
NP = {"bool": np.bool_, "u8": np.uint8, "u16": np.uint16, "u32": np.uint32,
      "u64": np.uint64, "i8": np.int8, "i16": np.int16, "i32": np.int32,
      "i64": np.int64, "f16": np.float16, "bf16": np.uint16, "f32": np.float32,
      "f64": np.float64, "c64": np.complex64}


@dataclass
class Tensor:
    dtype: str
    shape: tuple
    data: bytes

    def array(self) -> np.ndarray:
        """The tensor as a numpy array (bf16 as uint16 bit patterns)."""
        return np.frombuffer(self.data, dtype=NP[self.dtype]).reshape(self.shape)

    @property
    def code(self) -> int:
        return DTYPES.index(self.dtype)


@dataclass
class Case:
    name: str
    op: str
    params: dict = field(default_factory=dict)
    inputs: list = field(default_factory=list)
    outputs: list = field(default_factory=list)

    def spelled(self) -> str:
        return "|".join([self.op] + [f"{k}={v}" for k, v in self.params.items()])

    def nbytes(self) -> int:
        return sum(len(t.data) for t in self.inputs + self.outputs)


class _Reader:
    def __init__(self, buf):
        self.buf, self.pos = memoryview(buf), 0

    def take(self, n):
        out = self.buf[self.pos:self.pos + n]
        if len(out) != n:
            raise ValueError("truncated fixture file")
        self.pos += n
        return out

    def num(self, fmt):
        return struct.unpack("<" + fmt, self.take(struct.calcsize(fmt)))[0]

    def str(self):
        return bytes(self.take(self.num("H"))).decode("utf-8")

    def tensor(self):
        dtype = DTYPES[self.num("B")]
        ndim = self.num("B")
        shape = tuple(self.num("Q") for _ in range(ndim))
        return Tensor(dtype, shape, bytes(self.take(self.num("Q"))))


def parse(buf) -> tuple[str, list[Case]]:
    """Parses a fixture file into its metadata line and its cases."""
    if bytes(buf[:8]) != MAGIC:
        raise ValueError("not a BSMXFIX1 file")
    r = _Reader(buf)
    r.pos = 8
    meta = r.str()
    cases = []
    for _ in range(r.num("I")):
        name, spelled = r.str(), r.str()
        op, *kvs = spelled.split("|")
        params = dict(kv.split("=", 1) for kv in kvs)
        inputs = [r.tensor() for _ in range(r.num("B"))]
        outputs = [r.tensor() for _ in range(r.num("B"))]
        cases.append(Case(name, op, params, inputs, outputs))
    if r.pos != len(r.buf):
        raise ValueError("trailing bytes in fixture file")
    return meta, cases


def load(path) -> tuple[str, list[Case]]:
    with open(path, "rb") as f:
        return parse(f.read())


def dump(path, meta: str, cases: list[Case]) -> None:
    """Writes `cases` in the same container, so one reader serves both."""
    def s(text):
        raw = text.encode("utf-8")
        return struct.pack("<H", len(raw)) + raw

    out = [MAGIC, s(meta), struct.pack("<I", len(cases))]
    for c in cases:
        out += [s(c.name), s(c.spelled())]
        for group in (c.inputs, c.outputs):
            out.append(struct.pack("<B", len(group)))
            for t in group:
                out.append(struct.pack("<BB", t.code, len(t.shape)))
                out += [struct.pack("<Q", d) for d in t.shape]
                out += [struct.pack("<Q", len(t.data)), t.data]
    with open(path, "wb") as f:
        f.write(b"".join(out))
