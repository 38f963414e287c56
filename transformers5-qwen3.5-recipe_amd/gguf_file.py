"""GGUF container files -> packed tensors for the matmul path.

Stands in for the part of gguf-py the reference's tests use to feed real checkpoints to the kernels
(``gguf.GGUFReader(path)``, ``reader.tensors`` with ``.name``, ``.tensor_type``, ``.shape``, ``.data``;
test_fast_lora.py:37-46, test_fast_moe_lora.py real-model slices): the file is memory-mapped, nothing is copied
until a tensor is asked for, and a quantized tensor's ``data`` is its raw blocks viewed as uint8
``[..., rows, row_bytes]`` - exactly the payload layout of ``GGUFQuantizedTensor``.

The format (GGUF version 2 and 3, little-endian), restated from its public specification:

    header   : u32 magic "GGUF", u32 version, u64 tensor_count, u64 metadata_kv_count
    metadata : key (string), u32 value type, value; string = u64 length + bytes (UTF-8);
               types 0..12 = u8 i8 u16 i16 u32 i32 f32 bool string array u64 i64 f64;
               array = u32 element type, u64 count, elements
    tensors  : name (string), u32 n_dims, u64 ne[n_dims] (ne[0] = the contiguous dimension),
               u32 ggml type, u64 offset into the data section
    data     : starts at the next multiple of ``general.alignment`` (default 32) after the tensor table

``write_gguf`` writes the same layout (synthetic checkpoints for tests and tools).
"""

from __future__ import annotations

import mmap
import struct
from dataclasses import dataclass
from pathlib import Path

import numpy as np
import torch

from .gguf import GGML_QUANT_SIZES, GGUFQuantizedTensor

GGUF_MAGIC = 0x46554747  # "GGUF" read as a little-endian u32
DEFAULT_ALIGNMENT = 32

# GGML type id -> (elements per block, bytes per block) for the plain types; the block formats with kernels
# come from GGML_QUANT_SIZES
F32, F16, BF16, I8, I16, I32, I64, F64 = 0, 1, 30, 24, 25, 26, 27, 28
_PLAIN = {F32: np.dtype("<f4"), F16: np.dtype("<f2"), BF16: np.dtype("<u2"), I8: np.dtype("i1"), I16: np.dtype("<i2"),
          I32: np.dtype("<i4"), I64: np.dtype("<i8"), F64: np.dtype("<f8")}
# block formats this library has no kernels for: sizes only, so that a file holding them can still be walked
_OTHER_BLOCKS = {2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 9: (32, 36), 15: (256, 292), 17: (256, 74), 18: (256, 98),
                 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (256, 136), 29: (256, 56)}

_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_STRING, _ARRAY = 8, 9


def block_geometry(tensor_type: int) -> tuple[int, int]:
    """(elements per block, bytes per block) of a GGML type id."""
    if tensor_type in _PLAIN:
        return 1, _PLAIN[tensor_type].itemsize
    if tensor_type in GGML_QUANT_SIZES:
        return GGML_QUANT_SIZES[tensor_type]
    if tensor_type in _OTHER_BLOCKS:
        return _OTHER_BLOCKS[tensor_type]
    raise ValueError(f"unknown GGML type id {tensor_type}")


@dataclass(frozen=True)
class ReaderTensor:
    name: str
    tensor_type: int             # GGML type id
    shape: tuple[int, ...]       # GGUF order: shape[0] is the contiguous dimension
    n_elements: int
    n_bytes: int
    data_offset: int             # absolute offset in the file
    data: np.ndarray             # view of the mapped file: typed for plain types, uint8 [..., rows, row_bytes] for block types

    @property
    def logical_shape(self) -> tuple[int, ...]:
        """Row-major shape, outermost first (``[experts, rows, K]`` for expert stacks)."""
        return tuple(reversed(self.shape))


class _Cursor:
    def __init__(self, buf, size: int):
        self.buf, self.size, self.pos = buf, size, 0

    def take(self, fmt: str):
        n = struct.calcsize(fmt)
        if self.pos + n > self.size:
            raise ValueError("GGUF file is truncated")
        (v,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += n
        return v

    def string(self, len_fmt: str) -> str:
        n = self.take(len_fmt)
        if self.pos + n > self.size:
            raise ValueError("GGUF file is truncated (string runs past the end)")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="replace")
        self.pos += n
        return s

    def value(self, vtype: int, len_fmt: str, depth: int = 0):
        if vtype in _SCALARS:
            return self.take(_SCALARS[vtype])
        if vtype == _STRING:
            return self.string(len_fmt)
        if vtype == _ARRAY:
            if depth > 4:
                raise ValueError("GGUF metadata arrays are nested too deeply")
            etype = self.take("<I")
            count = self.take(len_fmt)
            if etype in _SCALARS:  # one bulk read
                dt = np.dtype(_SCALARS[etype])
                nbytes = dt.itemsize * count
                if self.pos + nbytes > self.size:
                    raise ValueError("GGUF file is truncated (array runs past the end)")
                arr = np.frombuffer(self.buf, dtype=dt, count=count, offset=self.pos).tolist()
                self.pos += nbytes
                return arr
            return [self.value(etype, len_fmt, depth + 1) for _ in range(count)]
        raise ValueError(f"unknown GGUF metadata value type {vtype}")


class GGUFReader:
    """Memory-maps a GGUF file; ``fields`` holds the metadata (key -> Python value), ``tensors`` the tensor table."""

    def __init__(self, path):
        self.path = Path(path)
        self._file = open(self.path, "rb")
        try:
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError as exc:  # empty file
            self._file.close()
            raise ValueError(f"{self.path}: not a GGUF file (empty)") from exc
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    def _parse(self) -> None:
        size = len(self._map)
        cur = _Cursor(self._map, size)
        if size < 8 or cur.take("<I") != GGUF_MAGIC:
            raise ValueError(f"{self.path}: not a GGUF file (bad magic)")
        self.version = cur.take("<I")
        if self.version not in (2, 3):
            raise ValueError(f"{self.path}: GGUF version {self.version} is not supported (2 and 3 are)")
        len_fmt = "<Q"
        n_tensors, n_kv = cur.take(len_fmt), cur.take(len_fmt)
        self.fields: dict[str, object] = {}
        for _ in range(n_kv):
            key = cur.string(len_fmt)
            self.fields[key] = cur.value(cur.take("<I"), len_fmt)
        self.alignment = int(self.fields.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise ValueError(f"{self.path}: general.alignment {self.alignment} is not a power of two")
        infos = []
        for _ in range(n_tensors):
            name = cur.string(len_fmt)
            n_dims = cur.take("<I")
            if n_dims > 8:
                    raise ValueError(f"{self.path}: tensor {name!r} has {n_dims} dimensions")
            shape = tuple(cur.take("<Q") for _ in range(n_dims))
            infos.append((name, shape, cur.take("<I"), cur.take("<Q")))
        self.data_offset = (cur.pos + self.alignment - 1) // self.alignment * self.alignment
        self.tensors: list[ReaderTensor] = []
        whole = np.frombuffer(self._map, dtype=np.uint8)
        for name, shape, ttype, rel in infos:
            elems, nbytes = block_geometry(ttype)
            n_elements = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if shape and shape[0] % elems:
                    raise ValueError(f"{self.path}: tensor {name!r}: {shape[0]} contiguous elements are not whole blocks of {elems}")
            n_bytes = n_elements // elems * nbytes
            start = self.data_offset + rel
            if rel % self.alignment or start + n_bytes > size:
                    raise ValueError(f"{self.path}: tensor {name!r} is misaligned or runs past the end of the file")
            raw = whole[start:start + n_bytes]
            outer = tuple(reversed(shape[1:]))
            if ttype in _PLAIN:
                data = raw.view(_PLAIN[ttype]).reshape(outer + (shape[0],) if shape else ())
            else:
                data = raw.reshape(outer + (shape[0] // elems * nbytes,))
            self.tensors.append(ReaderTensor(name, ttype, shape, n_elements, n_bytes, start, data))
        self._by_name = {t.name: t for t in self.tensors}

    def get_tensor(self, name: str) -> ReaderTensor:
        try:
            return self._by_name[name]
        except KeyError:
            raise KeyError(f"{self.path}: no tensor named {name!r}") from None

    def packed(self, name: str, device="cuda", rows: slice | None = None) -> GGUFQuantizedTensor:
        """The named block-quantized tensor (optionally a slice of its outermost dimension) as a ``GGUFQuantizedTensor`` on
        ``device``: one host copy of the selected bytes, then one transfer."""
        t = self.get_tensor(name)
        if t.tensor_type not in GGML_QUANT_SIZES:
            raise ValueError(f"tensor {name!r} has GGML type {t.tensor_type}, which has no native kernels (supported: {sorted(GGML_QUANT_SIZES)})")
        data = t.data if rows is None else t.data[rows]
        logical = tuple(data.shape[:-1]) + (t.shape[0],)
        payload = torch.from_numpy(np.array(data, dtype=np.uint8, copy=True, order="C")).to(device)
        return GGUFQuantizedTensor(payload, t.tensor_type, logical)

    def plain(self, name: str, device="cuda") -> torch.Tensor:
        """The named F32 / F16 / BF16 / integer tensor as a torch tensor on ``device``."""
        t = self.get_tensor(name)
        if t.tensor_type not in _PLAIN:
            raise ValueError(f"tensor {name!r} is block-quantized (GGML type {t.tensor_type}); use packed()")
        host = np.array(t.data, copy=True, order="C")
        if t.tensor_type == BF16:
            return torch.from_numpy(host.view(np.int16)).view(torch.bfloat16).to(device)
        return torch.from_numpy(host).to(device)

    def close(self) -> None:
        self.tensors = []
        self._by_name = {}
        try:
            self._map.close()
        except (BufferError, ValueError):
            pass  # views handed out earlier still reference the mapping; it goes with the last of them
        self._file.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _encode_value(v) -> tuple[int, bytes]:
    if isinstance(v, np.generic):  # numpy scalars name their width (np.float64 is also a Python float)
        code = {np.uint8: 0, np.int8: 1, np.uint16: 2, np.int16: 3, np.uint32: 4, np.int32: 5, np.float32: 6, np.bool_: 7,
                np.uint64: 10, np.int64: 11, np.float64: 12}[type(v)]
        return code, struct.pack(_SCALARS[code], v.item())
    if isinstance(v, bool):
        return 7, struct.pack("<?", v)
    if isinstance(v, int):  # the narrowest of i32, i64, u64 that holds it
        if -2 ** 31 <= v < 2 ** 31:
            return 5, struct.pack("<i", v)
        if -2 ** 63 <= v < 2 ** 63:
            return 11, struct.pack("<q", v)
        return 10, struct.pack("<Q", v)
    if isinstance(v, float):
        return 6, struct.pack("<f", v)
    if isinstance(v, str):
        b = v.encode("utf-8")
        return _STRING, struct.pack("<Q", len(b)) + b
    if isinstance(v, (list, tuple)):
        if not v:
            return _ARRAY, struct.pack("<IQ", 5, 0)
        parts = [_encode_value(e) for e in v]
        etype = parts[0][0]
        if any(p[0] != etype for p in parts):
            raise ValueError("GGUF arrays hold one element type")
        return _ARRAY, struct.pack("<IQ", etype, len(parts)) + b"".join(p[1] for p in parts)
    raise TypeError(f"cannot store a {type(v).__name__} as GGUF metadata")


def write_gguf(path, metadata: dict, tensors: list[tuple[str, int, tuple[int, ...], np.ndarray]], alignment: int = DEFAULT_ALIGNMENT) -> None:
    """Writes a version-3 file.  ``tensors``: (name, GGML type id, logical shape outermost-first, data) with data either the
    typed array of a plain type or the uint8 payload ``[..., rows, row_bytes]`` of a block type."""
    meta = dict(metadata)
    if alignment != DEFAULT_ALIGNMENT:
        meta["general.alignment"] = np.uint32(alignment)
    out = bytearray(struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(meta)))
    for key, v in meta.items():
        kb = key.encode("utf-8")
        code, body = _encode_value(v)
        out += struct.pack("<Q", len(kb)) + kb + struct.pack("<I", code) + body
    blobs, rel = [], 0
    for name, ttype, logical, data in tensors:
        elems, nbytes = block_geometry(ttype)
        logical = tuple(int(d) for d in logical)
        n_elements = int(np.prod(logical, dtype=np.int64)) if logical else 1
        blob = np.ascontiguousarray(data).tobytes()
        if (logical and logical[-1] % elems) or len(blob) != n_elements // elems * nbytes:
            raise ValueError(f"tensor {name!r}: {len(blob)} bytes do not hold shape {logical} of GGML type {ttype}")
        nb = name.encode("utf-8")
        out += struct.pack("<Q", len(nb)) + nb + struct.pack("<I", len(logical))
        out += b"".join(struct.pack("<Q", d) for d in reversed(logical))
        out += struct.pack("<IQ", ttype, rel)
        blobs.append((rel, blob))
        rel = (rel + len(blob) + alignment - 1) // alignment * alignment
    start = (len(out) + alignment - 1) // alignment * alignment
    out += b"\0" * (start - len(out))
    for rel_off, blob in blobs:
        out += b"\0" * (start + rel_off - len(out))
        out += blob
    Path(path).write_bytes(bytes(out))
