"""Test helper: writes small GGUF (version 3) files for the reader / index tests.

Layout per the published container format: header, key/value metadata, tensor descriptors, then
payloads at ``alignment`` boundaries (offsets relative to the aligned start of the data section).
"""
import struct

import numpy as np

from mylocal_llm_amd.gguf_file import GGML_TYPE_IDS

_U32, _F32, _STR, _ARR, _U64 = 4, 6, 8, 9, 10


def _string(text):
    raw = text.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


def _value(value):
    if isinstance(value, str):
        return struct.pack("<I", _STR) + _string(value)
    if isinstance(value, bool):
        return struct.pack("<I", 7) + struct.pack("<?", value)
    if isinstance(value, int):
        return struct.pack("<I", _U32) + struct.pack("<I", value)
    if isinstance(value, float):
        return struct.pack("<I", _F32) + struct.pack("<f", value)
    if isinstance(value, (list, tuple)):
        if all(isinstance(v, str) for v in value):
            return struct.pack("<IIQ", _ARR, _STR, len(value)) + b"".join(_string(v) for v in value)
        return struct.pack("<IIQ", _ARR, _U32, len(value)) + b"".join(struct.pack("<I", v) for v in value)
    raise TypeError(type(value))


def write_gguf(path, metadata, tensors, alignment=32):
    """tensors: list of (name, canonical row-major shape, ggml type name, payload bytes/array)."""
    if alignment != 32:
        metadata = dict(metadata, **{"general.alignment": alignment})
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(metadata))
    for key, value in metadata.items():
        head += _string(key) + _value(value)
    offset, payloads = 0, []
    for name, shape, kind, data in tensors:
        raw = np.ascontiguousarray(data).reshape(-1).view(np.uint8).tobytes()
        dims = tuple(reversed(shape))
        head += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", GGML_TYPE_IDS[kind], offset)
        payloads.append((offset, raw))
        offset = (offset + len(raw) + alignment - 1) // alignment * alignment
    start = (len(head) + alignment - 1) // alignment * alignment
    blob = bytearray(head + b"\0" * (start - len(head)) + b"\0" * offset)
    for at, raw in payloads:
        blob[start + at:start + at + len(raw)] = raw
    with open(path, "wb") as fh:
        fh.write(bytes(blob))
    return start
