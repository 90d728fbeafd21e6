"""GGUF container files: the on-disk side of the quantized Dense path.

A GGUF file holds the weight matrices in exactly the byte layout the kernels read: a tensor of
GGML type t with dimensions ne = [K, N] (innermost first) is N rows of ``row_bytes(t, K)`` bytes,
i.e. the ``Uint8 [N, bytesPerRow]`` tensor that nn.QuantizedDense takes
(ml/nn/quantized_dense.go:31-34) and that the reference uploads with tensors.FromRaw
(core/tensors/ondevice.go:696-737).  The reference's own loader lives outside its repository
(go-huggingface, README.md:188), so there is no reference interface to mirror here: the reader
follows the public GGUF specification (versions 2 and 3, little-endian).

File layout: magic "GGUF", u32 version, u64 tensor count, u64 key/value count; the key/value
pairs; the tensor infos (name, u32 rank, u64 dims innermost first, u32 GGML type, u64 offset into
the data section); padding to ``general.alignment`` (default 32); the data section.

Nothing here touches the GPU except ``GGUFFile.to_device``.
"""
from __future__ import annotations

import mmap
import os
import struct
from dataclasses import dataclass

import numpy as np

MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32

# value types of the key/value section
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<?", U64: "<Q", I64: "<q", F64: "<d"}

# GGML type id -> (name, values per block, bytes per block); public ggml numbering
GGML_TYPES = {
    0: ("F32", 1, 4), 1: ("F16", 1, 2), 2: ("Q4_0", 32, 18), 3: ("Q4_1", 32, 20), 6: ("Q5_0", 32, 22), 7: ("Q5_1", 32, 24),
    8: ("Q8_0", 32, 34), 9: ("Q8_1", 32, 36), 10: ("Q2_K", 256, 84), 11: ("Q3_K", 256, 110), 12: ("Q4_K", 256, 144),
    13: ("Q5_K", 256, 176), 14: ("Q6_K", 256, 210), 15: ("Q8_K", 256, 292), 16: ("IQ2_XXS", 256, 66), 17: ("IQ2_XS", 256, 74),
    18: ("IQ3_XXS", 256, 98), 19: ("IQ1_S", 256, 50), 20: ("IQ4_NL", 32, 18), 21: ("IQ3_S", 256, 110), 22: ("IQ2_S", 256, 82),
    23: ("IQ4_XS", 256, 136), 24: ("I8", 1, 1), 25: ("I16", 1, 2), 26: ("I32", 1, 4), 27: ("I64", 1, 8), 28: ("F64", 1, 8),
    29: ("IQ1_M", 256, 56), 30: ("BF16", 1, 2),
}
_PLAIN = {0: np.dtype("<f4"), 1: np.dtype("<f2"), 24: np.dtype("i1"), 25: np.dtype("<i2"), 26: np.dtype("<i4"), 27: np.dtype("<i8"),
          28: np.dtype("<f8"), 30: np.dtype("<u2")}  # BF16 comes back as raw 16-bit patterns


class GGUFError(ValueError):
    """The file is not a GGUF file this reader understands, or is internally inconsistent."""


@dataclass(frozen=True)
class TensorInfo:
    name: str
    ne: tuple          # dimensions as stored: innermost (contiguous) first
    ggml_type: int
    offset: int        # from the start of the data section
    nbytes: int

    @property
    def shape(self) -> tuple:
        """Dimensions outermost first, the order of a row-major array."""
        return tuple(reversed(self.ne))

    @property
    def type_name(self) -> str:
        return GGML_TYPES[self.ggml_type][0]


def tensor_nbytes(ggml_type: int, ne) -> int:
    if ggml_type not in GGML_TYPES:
        raise GGUFError(f"unknown GGML type id {ggml_type}")
    _, vpb, bpb = GGML_TYPES[ggml_type]
    if not ne:
        return bpb if vpb == 1 else 0
    if ne[0] % vpb:
        raise GGUFError(f"innermost dimension {ne[0]} is not a whole number of {vpb}-value blocks")
    n = ne[0] // vpb * bpb
    for d in ne[1:]:
        n *= d
    return n


class _Cursor:
    def __init__(self, buf, pos=0):
        self.buf, self.pos = buf, pos

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise GGUFError("file ends inside its header")
        (v,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise GGUFError("file ends inside a string")
        b = bytes(self.buf[self.pos:self.pos + n])
        self.pos += n
        return b.decode("utf-8", "replace")

    def value(self, vtype, depth=0):
        if vtype in _SCALAR:
            return self.take(_SCALAR[vtype])
        if vtype == STRING:
            return self.string()
        if vtype == ARRAY:
            if depth > 4:
                raise GGUFError("arrays nested too deeply")
            et, n = self.take("<I"), self.take("<Q")
            if et in _SCALAR and et != BOOL:  # bulk numeric arrays (token scores, ...) in one go
                dt = np.dtype(_SCALAR[et])
                if self.pos + n * dt.itemsize > len(self.buf):
                    raise GGUFError("file ends inside an array")
                a = np.frombuffer(self.buf, dt, n, self.pos).copy()
                self.pos += n * dt.itemsize
                return a
            return [self.value(et, depth + 1) for _ in range(n)]
        raise GGUFError(f"unknown metadata value type {vtype}")


class GGUFFile:
    """A memory-mapped GGUF file: ``metadata`` (dict), ``tensors`` (name -> TensorInfo, in file order)
    and zero-copy views of the tensor data."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 24:
            self._f.close()
            raise GGUFError("file too short for a GGUF header")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    def _parse(self):
        mm = self._mm
        if mm[:4] != MAGIC:
            raise GGUFError("not a GGUF file (bad magic)")
        c = _Cursor(mm, 4)
        self.version = c.take("<I")
        if self.version not in (2, 3):
            raise GGUFError(f"GGUF version {self.version} is not supported (2 and 3 are; a byte-swapped value means a big-endian file)")
        n_tensors, n_kv = c.take("<Q"), c.take("<Q")
        if n_tensors > 1 << 24 or n_kv > 1 << 24:
            raise GGUFError("implausible tensor or metadata count")
        self.metadata = {}
        for _ in range(n_kv):
            key = c.string()
            self.metadata[key] = c.value(c.take("<I"))
        self.alignment = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise GGUFError(f"alignment {self.alignment} is not a power of two")
        self.tensors = {}
        for _ in range(n_tensors):
            name = c.string()
            rank = c.take("<I")
            if rank > 8:
                raise GGUFError(f"tensor {name!r}: rank {rank}")
            ne = tuple(c.take("<Q") for _ in range(rank))
            t, off = c.take("<I"), c.take("<Q")
            if name in self.tensors:
                raise GGUFError(f"duplicate tensor name {name!r}")
            if off % self.alignment:
                raise GGUFError(f"tensor {name!r}: offset {off} is not {self.alignment}-byte aligned")
            self.tensors[name] = TensorInfo(name, ne, t, off, tensor_nbytes(t, ne))
        self.data_start = (c.pos + self.alignment - 1) // self.alignment * self.alignment
        for ti in self.tensors.values():
            if self.data_start + ti.offset + ti.nbytes > len(mm):
                raise GGUFError(f"tensor {ti.name!r} extends past the end of the file")

    def close(self):
        mm, self._mm = getattr(self, "_mm", None), None
        if mm is not None:
            try:
                mm.close()
            except BufferError:  # views handed out are still alive; the map goes with them
                pass
        if not self._f.closed:
            self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def raw(self, name: str) -> np.ndarray:
        """The tensor's bytes as a flat uint8 view of the file."""
        ti = self.tensors[name]
        return np.frombuffer(self._mm, np.uint8, ti.nbytes, self.data_start + ti.offset)

    def rows(self, name: str) -> np.ndarray:
        """``[N, bytesPerRow]`` uint8 view of a block-quantized (or plain) tensor: one row per index of
        the outer dimensions, blocks along the innermost one -- the weight operand of nn.QuantizedDense."""
        ti = self.tensors[name]
        if not ti.ne:
            raise GGUFError(f"tensor {name!r} is a scalar")
        _, vpb, bpb = GGML_TYPES[ti.ggml_type]
        rb = ti.ne[0] // vpb * bpb
        return self.raw(name).reshape(-1, rb) if rb else self.raw(name).reshape(0, 0)

    def array(self, name: str) -> np.ndarray:
        """A tensor of a plain element type (F32, F16, BF16 as uint16 patterns, integers) in its shape."""
        ti = self.tensors[name]
        if ti.ggml_type not in _PLAIN:
            raise GGUFError(f"tensor {name!r} is block-quantized ({ti.type_name}); use rows()")
        return self.raw(name).view(_PLAIN[ti.ggml_type]).reshape(ti.shape)

    def to_device(self, name: str, device="cuda"):
        """The tensor on the GPU, as tensors.FromRaw would upload it: uint8 ``[N, bytesPerRow]`` for a
        block-quantized tensor, its own element type and shape for F32 / F16 / integer tensors."""
        import torch
        ti = self.tensors[name]
        a = self.array(name) if ti.ggml_type in _PLAIN and ti.ggml_type != 30 else self.rows(name)
        return torch.from_numpy(np.array(a, copy=True)).to(device)


def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(v) -> bytes:
    """(type, payload) for a Python value: bool, int (I64, or U64 when too large), float (F32), str,
    numpy scalars and arrays by their dtype, lists of strings."""
    np_types = {np.dtype("u1"): U8, np.dtype("i1"): I8, np.dtype("<u2"): U16, np.dtype("<i2"): I16, np.dtype("<u4"): U32,
                np.dtype("<i4"): I32, np.dtype("<f4"): F32, np.dtype("<u8"): U64, np.dtype("<i8"): I64, np.dtype("<f8"): F64}
    if isinstance(v, (bool, np.bool_)):
        return struct.pack("<I?", BOOL, bool(v))
    if isinstance(v, np.generic):
        return struct.pack("<I", np_types[v.dtype]) + v.tobytes()
    if isinstance(v, int):
        return struct.pack("<Iq", I64, v) if v < 1 << 63 else struct.pack("<IQ", U64, v)
    if isinstance(v, float):
        return struct.pack("<If", F32, v)
    if isinstance(v, str):
        return struct.pack("<I", STRING) + _pack_string(v)
    if isinstance(v, np.ndarray):
        return struct.pack("<IIQ", ARRAY, np_types[v.dtype], v.size) + np.ascontiguousarray(v).tobytes()
    if isinstance(v, (list, tuple)) and all(isinstance(e, str) for e in v):
        return struct.pack("<IIQ", ARRAY, STRING, len(v)) + b"".join(_pack_string(e) for e in v)
    raise TypeError(f"cannot store {type(v).__name__} as GGUF metadata")


def write_gguf(path: str, metadata: dict, tensors, alignment: int = DEFAULT_ALIGNMENT, version: int = 3) -> None:
    """Writes a GGUF file.  ``tensors`` is a sequence of ``(name, ggml_type, ne, data)`` with ``ne`` the
    dimensions innermost first and ``data`` anything exposing the tensor's bytes (a uint8
    ``[N, bytesPerRow]`` array for block-quantized types)."""
    metadata = dict(metadata)
    if alignment != DEFAULT_ALIGNMENT:
        metadata["general.alignment"] = np.uint32(alignment)
    head = bytearray(MAGIC + struct.pack("<IQQ", version, len(tensors), len(metadata)))
    for k, v in metadata.items():
        head += _pack_string(k) + _pack_value(v)
    blobs, off = [], 0
    for name, t, ne, data in tensors:
        b = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        if b.size != tensor_nbytes(t, tuple(ne)):
            raise GGUFError(f"tensor {name!r}: {b.size} bytes given, {tensor_nbytes(t, tuple(ne))} expected for {ne} of type {t}")
        head += _pack_string(name) + struct.pack("<I", len(ne)) + b"".join(struct.pack("<Q", d) for d in ne) + struct.pack("<IQ", t, off)
        blobs.append((off, b))
        off = (off + b.size + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (-len(head) % alignment))
        base = f.tell()
        for o, b in blobs:
            f.write(b"\0" * (base + o - f.tell()))
            f.write(b.tobytes())
