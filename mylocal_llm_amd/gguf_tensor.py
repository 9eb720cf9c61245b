"""Unquantised GGUF tensors (F32 / F16 / BF16) as host arrays.

Behaviour of mini_llm/external/gguf_tensor.py:10-51: F32 and F16 come back as the reader's own
typed view once its shape agrees with the header; BF16 comes as raw bytes or 16-bit words and is
widened to fp32 with integer shifts only, so signed zeros and every NaN payload survive.  Packed
(quantised) tensors never pass through here.
"""
from numbers import Integral

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


def _row_of_typed(tensor, shape, row):
    return _typed_view(tensor, shape)[row]


def _row_of_bf16(tensor, shape, row):
    """Row ``row`` of a BF16 matrix: its 2 * width bytes (or width words) are cut out of the payload
    first and only they are widened."""
    payload = np.asarray(tensor.data)
    width = shape[1]
    if payload.nbytes != 2 * shape[0] * width or not payload.flags.c_contiguous:
        raise ValueError(f"{tensor.name}: invalid contiguous BF16 matrix payload")
    per_row = {1: 2 * width, 2: width}.get(payload.dtype.itemsize if payload.dtype.kind == "u" else 0)
    if per_row is None:
        raise ValueError(f"{tensor.name}: BF16 row payload must be uint8 or uint16")
    cut = payload.reshape(-1)[per_row * row:per_row * (row + 1)]
    wide = _bf16_words(tensor, cut).astype(np.uint32)
    wide <<= 16
    return wide.view(np.float32)


def _row_of_packed(tensor, shape, row):
    from .quantized_weight import PackedGGUFWeight
    return PackedGGUFWeight(tensor.data, shape, tensor.tensor_type.name).select_outer(row).dequantize_reference()


_ROW_READERS = {"F32": _row_of_typed, "F16": _row_of_typed, "BF16": _row_of_bf16}


def decode_gguf_row(tensor, row):
    """One row of a canonical [rows, width] tensor without expanding the rest of it
    (mini_llm/external/gguf_tensor.py:54-89): a packed tensor decodes the blocks of that row only,
    BF16 is sliced as bytes before it is widened, F32 / F16 rows are views of the reader's array."""
    from .quantized_weight import BLOCK_FORMATS
    shape = canonical_shape(tensor)
    if len(shape) != 2 or min(shape) <= 0:
        raise ValueError(f"{tensor.name}: row access requires a positive matrix shape")
    if isinstance(row, bool) or not isinstance(row, Integral):
        raise TypeError("row must be an integer")
    if row not in range(shape[0]):
        raise IndexError(row)
    kind = tensor.tensor_type.name
    reader = _ROW_READERS.get(kind) or (_row_of_packed if kind in BLOCK_FORMATS else None)
    if reader is None:
        raise NotImplementedError(f"{tensor.name}: unsupported row type {kind}")
    return reader(tensor, shape, int(row))
