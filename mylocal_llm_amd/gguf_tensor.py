"""Decoding of individual unquantised GGUF tensors (F32 / F16 / BF16) on the host.

Follows mini_llm/external/gguf_tensor.py:10-51: F32 / F16 keep the reader's typed view after a
strict shape check; BF16 arrives as bytes (or 16-bit words) and is expanded by integer shifts, so
signed zeros and every NaN payload survive.  Quantised tensors never pass through here.
"""
import math

import numpy as np


def decode_gguf_dense(tensor):
    """Values of ``tensor`` in canonical row-major shape (the reversed GGML shape)."""
    kind = tensor.tensor_type.name
    if kind not in {"F32", "F16", "BF16"}:
        raise NotImplementedError(f"{tensor.name}: unsupported dense GGUF type {kind}")
    shape = tuple(int(d) for d in reversed(tensor.shape))
    values = np.asarray(tensor.data)
    if kind != "BF16":
        if values.shape != shape:
            raise ValueError(f"GGUF {tensor.name}: tensor data {values.shape} != metadata {shape}")
        return values
    if any(d <= 0 for d in shape):
        raise ValueError(f"GGUF {tensor.name}: invalid BF16 shape {shape}")
    expected = math.prod(shape) * 2
    if values.nbytes != expected:
        raise ValueError(f"GGUF {tensor.name}: BF16 payload has {values.nbytes} bytes; expected {expected} for shape {shape}")
    if values.dtype == np.dtype("uint8"):
        words = np.ascontiguousarray(values).reshape(-1).view("<u2")
    elif values.dtype.kind == "u" and values.dtype.itemsize == 2:
        words = values.reshape(-1)
    else:
        raise ValueError(f"GGUF {tensor.name}: BF16 payload must be uint8 bytes or uint16 words, not {values.dtype}")
    return (words.astype(np.uint32) << 16).view(np.float32).reshape(shape)
