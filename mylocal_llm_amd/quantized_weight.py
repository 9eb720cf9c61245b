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
import ctypes
import operator
from dataclasses import dataclass
from functools import reduce

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


def _count(dims):
    return reduce(operator.mul, dims, 1)


def _packed_bytes(quant_type, dims):
    """Bytes that ``dims`` elements take in ``quant_type`` (the innermost dimension is whole blocks)."""
    per_block, block_size = BLOCK_FORMATS[quant_type]
    return _count(dims) // per_block * block_size


def _positive_int(value, message):
    """``value`` as an int if it is a true integer above zero (a bool is not), else ValueError."""
    is_integer = isinstance(value, (int, np.integer)) and not isinstance(value, (bool, np.bool_))
    if not is_integer or value <= 0:
        raise ValueError(message)
    return int(value)


@dataclass(frozen=True)
class PackedGGUFWeight:
    """Validated packed tensor in canonical row-major shape; ``data`` aliases the owner."""

    data: np.ndarray
    shape: tuple
    quant_type: str

    def __post_init__(self):
        fmt = self.quant_type
        geometry = BLOCK_FORMATS.get(fmt)
        if geometry is None:
            raise ValueError(f"Unsupported packed GGUF type: {fmt}")
        dims = tuple(map(int, self.shape))
        if len(dims) == 0 or min(dims) <= 0:
            raise ValueError("Packed GGUF shape must have positive dimensions")
        if dims[-1] % geometry[0] != 0:
            raise ValueError(f"GGUF {fmt}: innermost dimension must be a multiple of {geometry[0]}")
        payload = np.asarray(self.data)
        if not payload.flags.c_contiguous:
            raise ValueError("GGUF packed data must be contiguous")
        flat = payload.view(np.uint8).reshape(-1)   # a view: the caller's buffer (an mmap) stays the owner
        want = _packed_bytes(fmt, dims)
        if flat.size != want:
            raise ValueError(f"GGUF {fmt}: expected {want} bytes, got {flat.size}")
        for name, value in (("shape", dims), ("data", flat)):
            object.__setattr__(self, name, value)

    @property
    def nbytes(self):
        return int(self.data.nbytes)

    @property
    def block_elements(self):
        return BLOCK_FORMATS[self.quant_type][0]

    @property
    def _row_bytes(self):
        return _packed_bytes(self.quant_type, self.shape[-1:])

    def _view(self, first_byte, dims):
        """Zero-copy sub-tensor of shape ``dims`` that starts ``first_byte`` bytes into the payload."""
        size = _packed_bytes(self.quant_type, dims)
        return PackedGGUFWeight(self.data[first_byte:first_byte + size], tuple(dims), self.quant_type)

    def select_outer(self, index):
        """Zero-copy slice along the leading dimension (one expert of [E, N, K])."""
        if len(self.shape) < 2:
            raise ValueError("select_outer requires at least two dimensions")
        which = int(index)
        if which < 0 or which >= self.shape[0]:
            raise IndexError(index)
        inner = self.shape[1:]
        return self._view(which * _packed_bytes(self.quant_type, inner), inner)

    def select_rows(self, start, stop):
        """Zero-copy row range of a matrix (e.g. the gate or up half of a fused gate_up)."""
        if len(self.shape) != 2:
            raise ValueError("select_rows requires a matrix; select_outer first")
        if not 0 <= start < stop <= self.shape[0]:
            raise IndexError((start, stop))
        return self._view(start * self._row_bytes, (stop - start, self.shape[1]))

    # ---- the reference's host helpers, on the library's host twins -----------------------------
    def _decode_rows(self, raw, rows):
        """fp32 [rows, columns] of ``rows`` packed rows lying contiguously in ``raw``."""
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
        return self._decode_rows(self.data, _count(self.shape[:-1])).reshape(self.shape)

    def dequantize_rows_reference(self, indices, *, tile_rows=32):
        """Selected rows of a matrix, order and duplicates preserved (quantized_weight.py:101-125);
        only the requested rows are decoded, ``tile_rows`` of them at a time."""
        if len(self.shape) != 2:
            raise ValueError("selected rows require a matrix; select_outer first")
        step = _positive_int(tile_rows, "tile_rows must be a positive integer")
        wanted = np.asarray(indices)
        if wanted.ndim != 1 or wanted.dtype.kind not in "iu":
            raise ValueError("indices must be a one-dimensional integer array")
        n_rows, n_cols = self.shape
        if wanted.size and (int(wanted.min()) < 0 or int(wanted.max()) >= n_rows):
            raise IndexError("packed row index out of range")
        by_row = self.data.reshape(n_rows, self._row_bytes)
        pieces = [self._decode_rows(by_row[wanted[at:at + step]], len(wanted[at:at + step]))
                  for at in range(0, wanted.size, step)]
        if not pieces:
            return np.empty((0, n_cols), dtype=np.float32)
        return np.concatenate(pieces, axis=0)

    def matvec_reference(self, vector, *, tile_rows=32):
        """fp32 ``W @ vector`` (quantized_weight.py:133-149) through the host linear; ``tile_rows`` is
        validated as in the reference (the host linear walks row by row and needs no tiling)."""
        if len(self.shape) != 2:
            raise ValueError("matvec requires a matrix; select_outer first")
        _positive_int(tile_rows, "tile_rows must be a positive integer")
        vector = np.asarray(vector, dtype=np.float32)
        if vector.shape != (self.shape[1],):
            raise ValueError("vector shape must equal (matrix columns,)")
        from .native_packed_cpu import packed_cpu_linear
        return packed_cpu_linear(vector[None], self)[0]
