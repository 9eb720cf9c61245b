"""Memory-mapped reader for GGUF files (format versions 2 and 3).

The reference opens checkpoints with ``gguf.GGUFReader`` (mini_llm/external/qwen3next_gguf.py:
100-113); that package is not part of this environment, so this module restates the published
container format (ggml's ``docs/gguf.md``): a little-endian header, typed key/value metadata,
tensor descriptors, then the tensor payloads at ``general.alignment`` (default 32) boundaries.

It exposes the surface the index code relies on and nothing more:

* ``reader.fields[name].contents(0)``  metadata values (arrays: element ``index``),
* ``reader.tensors``                   objects with ``name``, ``shape`` in GGML order (innermost
                                       dimension first), ``tensor_type.name`` and ``data``,
                                       a NumPy view on the memory map (nothing is copied).

Payload views: F32 / F16 / F64 / integer tensors come typed and shaped (row-major, i.e. the
reversed GGML shape); everything else, BF16 included, is a flat ``uint8`` view of the blocks.
The reader must outlive every array taken from it.
"""
import mmap
import os
import struct
from types import SimpleNamespace

import numpy as np

GGUF_MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32

# ggml_type id -> (name, elements per block, bytes per block)
GGML_TYPES = {
    0: ("F32", 1, 4), 1: ("F16", 1, 2), 2: ("Q4_0", 32, 18), 3: ("Q4_1", 32, 20),
    6: ("Q5_0", 32, 22), 7: ("Q5_1", 32, 24), 8: ("Q8_0", 32, 34), 9: ("Q8_1", 32, 36),
    10: ("Q2_K", 256, 84), 11: ("Q3_K", 256, 110), 12: ("Q4_K", 256, 144), 13: ("Q5_K", 256, 176),
    14: ("Q6_K", 256, 210), 15: ("Q8_K", 256, 292), 16: ("IQ2_XXS", 256, 66), 17: ("IQ2_XS", 256, 74),
    18: ("IQ3_XXS", 256, 98), 19: ("IQ1_S", 256, 50), 20: ("IQ4_NL", 32, 18), 21: ("IQ3_S", 256, 110),
    22: ("IQ2_S", 256, 82), 23: ("IQ4_XS", 256, 136), 24: ("I8", 1, 1), 25: ("I16", 1, 2),
    26: ("I32", 1, 4), 27: ("I64", 1, 8), 28: ("F64", 1, 8), 29: ("IQ1_M", 256, 56), 30: ("BF16", 1, 2),
}
GGML_TYPE_IDS = {name: tid for tid, (name, _, _) in GGML_TYPES.items()}
_TYPED = {"F32": "<f4", "F16": "<f2", "F64": "<f8", "I8": "i1", "I16": "<i2", "I32": "<i4", "I64": "<i8"}

# metadata value types
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_STRING, _ARRAY = 8, 9


class GGUFField:
    """One metadata entry; ``contents(i)`` is the value (arrays: element ``i``)."""

    def __init__(self, name, value_type, value):
        self.name, self.value_type, self.value = name, value_type, value

    def contents(self, index=None):
        if isinstance(self.value, list) and index is not None:
            return self.value[index]
        return self.value


class _Cursor:
    def __init__(self, buf):
        self.buf, self.at = buf, 0

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.at + size > len(self.buf):
            raise ValueError("GGUF: truncated file")
        (value,) = struct.unpack_from(fmt, self.buf, self.at)
        self.at += size
        return value

    def string(self):
        length = self.take("<Q")
        if self.at + length > len(self.buf):
            raise ValueError("GGUF: string runs past the end of the file")
        raw = bytes(self.buf[self.at:self.at + length])
        self.at += length
        return raw.decode("utf-8", errors="replace")

    def value(self, value_type):
        if value_type in _SCALARS:
            return self.take(_SCALARS[value_type])
        if value_type == _STRING:
            return self.string()
        if value_type == _ARRAY:
            item_type, count = self.take("<I"), self.take("<Q")
            if item_type == _ARRAY:
                raise ValueError("GGUF: nested metadata arrays are not part of the format")
            return [self.value(item_type) for _ in range(count)]
        raise ValueError(f"GGUF: unknown metadata value type {value_type}")


class GGUFFile:
    """Parsed header of one GGUF file plus zero-copy views of its tensors."""

    def __init__(self, path):
        self.path = os.fspath(path)
        self._file = open(self.path, "rb")
        try:
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError as exc:  # empty file
            self._file.close()
            raise ValueError(f"GGUF: {self.path} is empty") from exc
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    def _parse(self):
        cur = _Cursor(self._map)
        if bytes(self._map[:4]) != GGUF_MAGIC:
            raise ValueError(f"{self.path}: not a GGUF file")
        cur.at = 4
        self.version = cur.take("<I")
        if self.version not in (2, 3):
            raise ValueError(f"{self.path}: GGUF version {self.version} is not supported (2 and 3 are)")
        n_tensors, n_fields = cur.take("<Q"), cur.take("<Q")
        self.fields = {}
        for _ in range(n_fields):
            name = cur.string()
            value_type = cur.take("<I")
            self.fields[name] = GGUFField(name, value_type, cur.value(value_type))
        align_field = self.fields.get("general.alignment")
        self.alignment = int(align_field.contents()) if align_field is not None else DEFAULT_ALIGNMENT
        if self.alignment <= 0 or self.alignment % 8:
            raise ValueError(f"{self.path}: invalid general.alignment {self.alignment}")
        infos = []
        for _ in range(n_tensors):
            name = cur.string()
            n_dims = cur.take("<I")
            if n_dims > 8:
                raise ValueError(f"{self.path}: tensor {name!r} has {n_dims} dimensions")
            dims = tuple(cur.take("<Q") for _ in range(n_dims))
            infos.append((name, dims, cur.take("<I"), cur.take("<Q")))
        self.data_offset = (cur.at + self.alignment - 1) // self.alignment * self.alignment
        whole = np.frombuffer(self._map, dtype=np.uint8)
        self.tensors = []
        for name, dims, type_id, offset in infos:
            kind, elems, nbytes = GGML_TYPES.get(type_id, (f"TYPE_{type_id}", 0, 0))
            count = 1
            for d in dims:
                count *= d
            if offset % self.alignment:
                raise ValueError(f"{self.path}: tensor {name!r} is not aligned to {self.alignment} bytes")
            data = None
            if elems:
                if dims and dims[0] % elems:
                    raise ValueError(f"{self.path}: tensor {name!r}: innermost dimension {dims[0]} is not a multiple of the {kind} block")
                size = count // elems * nbytes
                start = self.data_offset + offset
                if start + size > whole.size:
                    raise ValueError(f"{self.path}: tensor {name!r} runs past the end of the file")
                data = whole[start:start + size]
                if kind in _TYPED:
                    data = data.view(_TYPED[kind]).reshape(tuple(reversed(dims)))
            self.tensors.append(SimpleNamespace(name=name, shape=dims, tensor_type=SimpleNamespace(name=kind, value=type_id),
                                                data=data, data_offset=self.data_offset + offset))

    def close(self):
        # NumPy views keep the map alive; closing it under them would raise BufferError
        try:
            self._map.close()
        except (BufferError, AttributeError):
            pass
        self._file.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
