"""Unquantised GGUF tensors (F32 / F16 / BF16) as host arrays.

Behaviour of mini_llm/external/gguf_tensor.py:10-51: F32 and F16 come back as the reader's own
typed view once its shape agrees with the header; BF16 comes as raw bytes or 16-bit words and is
widened to fp32 with integer shifts only, so signed zeros and every NaN payload survive.  Packed
(quantised) tensors never pass through here.
"""
from numbers import Integral
from types import SimpleNamespace

import numpy as np


def canonical_shape(tensor):
    """Row-major shape of a GGUF tensor; the file lists dimensions innermost first."""
    return tuple(int(extent) for extent in tensor.shape)[::-1]


def _typed_view(tensor, shape):
    values = np.asarray(tensor.data)
    if values.shape == shape:
        return values
    raise ValueError(f"GGUF {tensor.name}: tensor data {values.shape} != metadata {shape}")


def _bf16_words(tensor, payload):
    """The payload as one flat array of little-endian 16-bit words."""
    if payload.dtype == np.uint8:
        return np.ascontiguousarray(payload).reshape(-1).view("<u2")
    if payload.dtype.kind == "u" and payload.dtype.itemsize == 2:
        return payload.reshape(-1)
    raise ValueError(f"GGUF {tensor.name}: BF16 payload must be uint8 bytes or uint16 words, not {payload.dtype}")


def _widen_bf16(tensor, shape):
    if min(shape, default=1) <= 0:
        raise ValueError(f"GGUF {tensor.name}: invalid BF16 shape {shape}")
    payload = np.asarray(tensor.data)
    need = 2 * int(np.prod(shape, dtype=np.int64))
    if payload.nbytes != need:
        raise ValueError(f"GGUF {tensor.name}: BF16 payload has {payload.nbytes} bytes; expected {need} for shape {shape}")
    wide = _bf16_words(tensor, payload).astype(np.uint32)
    wide <<= 16
    return wide.view(np.float32).reshape(shape)


_DECODERS = {"F32": _typed_view, "F16": _typed_view, "BF16": _widen_bf16}
DENSE_KINDS = frozenset(_DECODERS)


def decode_gguf_dense(tensor):
    """Values of ``tensor`` in canonical row-major shape."""
    kind = tensor.tensor_type.name
    decoder = _DECODERS.get(kind)
    if decoder is None:
        raise NotImplementedError(f"{tensor.name}: unsupported dense GGUF type {kind}")
    return decoder(tensor, canonical_shape(tensor))


def _bf16_row_payload(tensor, shape, row):
    """The bytes (or words) of one row of a BF16 matrix, still undecoded."""
    payload = np.asarray(tensor.data)
    rows, width = shape
    if not payload.flags.c_contiguous or payload.nbytes != 2 * rows * width:
        raise ValueError(f"{tensor.name}: invalid contiguous BF16 matrix payload")
    if payload.dtype == np.uint8:
        flat = payload.reshape(-1)
        return flat[2 * width * row:2 * width * (row + 1)]
    if payload.dtype.kind == "u" and payload.dtype.itemsize == 2:
        return payload.reshape(shape)[row]
    raise ValueError(f"{tensor.name}: BF16 row payload must be uint8 or uint16")


def decode_gguf_row(tensor, row):
    """One row of a canonical [rows, width] tensor without expanding the rest of it
    (mini_llm/external/gguf_tensor.py:54-89): a packed tensor decodes the blocks of that row only,
    BF16 is sliced as bytes before it is widened, F32 / F16 rows are views of the reader's array."""
    from .quantized_weight import BLOCK_FORMATS, PackedGGUFWeight
    shape = canonical_shape(tensor)
    if len(shape) != 2 or min(shape) <= 0:
        raise ValueError(f"{tensor.name}: row access requires a positive matrix shape")
    if isinstance(row, bool) or not isinstance(row, Integral):
        raise TypeError("row must be an integer")
    if row < 0 or row >= shape[0]:
        raise IndexError(row)
    kind = tensor.tensor_type.name
    if kind == "BF16":
        one = SimpleNamespace(name=tensor.name, shape=(shape[1],), tensor_type=tensor.tensor_type,
                              data=_bf16_row_payload(tensor, shape, int(row)))
        return decode_gguf_dense(one)
    if kind in BLOCK_FORMATS:
        return PackedGGUFWeight(tensor.data, shape, kind).select_outer(int(row)).dequantize_reference()
    if kind in DENSE_KINDS:
        return decode_gguf_dense(tensor)[row]
    raise NotImplementedError(f"{tensor.name}: unsupported row type {kind}")
