"""Host-side packed GGUF weight container.

Mirrors ``PackedGGUFWeight`` of the reference (mini_llm/ops/quantized_weight.py:44-99):
validation of shape / block alignment / byte count, a flat uint8 *view* of the caller's
buffer (an mmap stays the owner), and zero-copy ``select_outer``.  Constructing it never
materialises a floating-point matrix.  The ``*_reference`` methods of the reference's container
(mini_llm/ops/quantized_weight.py:101-250, NumPy decoders there) keep their names, arguments and
errors and are host functions here too: they run the scalar C++ decoder / linear of the
library's host twins (``qmoe_dequantize_cpu`` / ``qmoe_linear_cpu``), whose decoded values are
those of the device decoder bit for bit.  None of them touches the GPU.
"""
from dataclasses import dataclass
import math

import numpy as np

# (elements per block, bytes per block); mini_llm/ops/quantized_weight.py:24-37 for the
# GGUF entries.  "BF16" (1 element / 2 bytes) is this package's extension so that BF16
# tensors go through the same linear operator (the reference decodes them densely,
# mini_llm/external/gguf_tensor.py:30-51).
BLOCK_FORMATS = {
    "Q8_0": (32, 34),
    "Q4_0": (32, 18),
    "Q4_K": (256, 144),
    "Q3_K": (256, 110),
    "Q5_K": (256, 176),
    "Q6_K": (256, 210),
    "BF16": (1, 2),
}


@dataclass(frozen=True)
class PackedGGUFWeight:
    """Validated packed tensor in canonical row-major shape; ``data`` aliases the owner."""

    data: np.ndarray
    shape: tuple
    quant_type: str

    def __post_init__(self):
        if self.quant_type not in BLOCK_FORMATS:
            raise ValueError(f"Unsupported packed GGUF type: {self.quant_type}")
        shape = tuple(int(d) for d in self.shape)
        if not shape or any(d <= 0 for d in shape):
            raise ValueError("Packed GGUF shape must have positive dimensions")
        elems, nbytes = BLOCK_FORMATS[self.quant_type]
        if shape[-1] % elems:
            raise ValueError(f"GGUF {self.quant_type}: innermost dimension must be a multiple of {elems}")
        raw = np.asarray(self.data)
        if not raw.flags.c_contiguous:
            raise ValueError("GGUF packed data must be contiguous")
        raw = raw.view(np.uint8).reshape(-1)
        expected = math.prod(shape) // elems * nbytes
        if raw.size != expected:
            raise ValueError(f"GGUF {self.quant_type}: expected {expected} bytes, got {raw.size}")
        object.__setattr__(self, "shape", shape)
        object.__setattr__(self, "data", raw)

    @property
    def nbytes(self):
        return int(self.data.nbytes)

    @property
    def block_elements(self):
        return BLOCK_FORMATS[self.quant_type][0]

    def select_outer(self, index):
        """Zero-copy slice along the leading dimension (one expert of [E, N, K])."""
        if len(self.shape) < 2:
            raise ValueError("select_outer requires at least two dimensions")
        if not 0 <= int(index) < self.shape[0]:
            raise IndexError(index)
        elems, nbytes = BLOCK_FORMATS[self.quant_type]
        chunk = math.prod(self.shape[1:]) // elems * nbytes
        begin = int(index) * chunk
        return PackedGGUFWeight(self.data[begin:begin + chunk], self.shape[1:], self.quant_type)

    def select_rows(self, start, stop):
        """Zero-copy row range of a matrix (e.g. the gate or up half of a fused gate_up)."""
        if len(self.shape) != 2:
            raise ValueError("select_rows requires a matrix; select_outer first")
        if not 0 <= start < stop <= self.shape[0]:
            raise IndexError((start, stop))
        row_bytes = self.nbytes // self.shape[0]
        return PackedGGUFWeight(self.data[start * row_bytes:stop * row_bytes],
                                (stop - start, self.shape[1]), self.quant_type)

    # ---- the reference's host helpers, on the library's host twins -----------------------------
    @staticmethod
    def _reference_tile_rows(tile_rows):
        if isinstance(tile_rows, (bool, np.bool_)) or not isinstance(tile_rows, (int, np.integer)) or tile_rows <= 0:
            raise ValueError("tile_rows must be a positive integer")
        return int(tile_rows)

    def _decode_rows(self, raw, rows):
        """fp32 [rows, columns] of ``rows`` packed rows lying contiguously in ``raw``."""
        import ctypes
        from . import _lib
        raw = np.ascontiguousarray(np.asarray(raw).reshape(-1).view(np.uint8))
        out = np.empty((rows, self.shape[-1]), dtype=np.float32)
        if rows:
            rc = _lib.load().qmoe_dequantize_cpu(ctypes.c_void_p(raw.ctypes.data), _lib.FORMAT_ID[self.quant_type], rows,
                                                 self.shape[-1], ctypes.c_void_p(out.ctypes.data))
            _lib.check(rc, "Host dequantize")
        return out

    def dequantize_reference(self):
        """fp32 ndarray of ``shape``, bit-identical to quantized_weight.py:151-250."""
        return self._decode_rows(self.data, math.prod(self.shape[:-1])).reshape(self.shape)

    def dequantize_rows_reference(self, indices, *, tile_rows=32):
        """Selected rows of a matrix, order and duplicates preserved (quantized_weight.py:101-125);
        only the requested rows are decoded, ``tile_rows`` of them at a time."""
        if len(self.shape) != 2:
            raise ValueError("selected rows require a matrix; select_outer first")
        tile_rows = self._reference_tile_rows(tile_rows)
        indices = np.asarray(indices)
        if indices.ndim != 1 or indices.dtype.kind not in "iu":
            raise ValueError("indices must be a one-dimensional integer array")
        if np.any(indices >= self.shape[0]) or np.any(indices < 0):
            raise IndexError("packed row index out of range")
        result = np.empty((len(indices), self.shape[1]), dtype=np.float32)
        raw = self.data.reshape(self.shape[0], self.nbytes // self.shape[0])
        for start in range(0, len(indices), tile_rows):
            selected = indices[start:start + tile_rows]
            result[start:start + len(selected)] = self._decode_rows(raw[selected], len(selected))
        return result

    def matvec_reference(self, vector, *, tile_rows=32):
        """fp32 ``W @ vector`` (quantized_weight.py:133-149) through the host linear; ``tile_rows`` is
        validated as in the reference (the host linear walks row by row and needs no tiling)."""
        if len(self.shape) != 2:
            raise ValueError("matvec requires a matrix; select_outer first")
        self._reference_tile_rows(tile_rows)
        vector = np.asarray(vector, dtype=np.float32)
        if vector.shape != (self.shape[1],):
            raise ValueError("vector shape must equal (matrix columns,)")
        from .native_packed_cpu import packed_cpu_linear
        return packed_cpu_linear(vector[None], self)[0]
