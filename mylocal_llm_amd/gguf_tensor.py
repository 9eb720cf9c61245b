"""Unquantised GGUF tensors (F32 / F16 / BF16) as host arrays.

Behaviour of mini_llm/external/gguf_tensor.py:10-51: F32 and F16 come back as the reader's own
typed view once its shape agrees with the header; BF16 comes as raw bytes or 16-bit words and is
widened to fp32 with integer shifts only, so signed zeros and every NaN payload survive.  Packed
(quantised) tensors never pass through here.
"""
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
