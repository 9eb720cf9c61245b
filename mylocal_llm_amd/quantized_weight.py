"""Host-side packed GGUF weight container.

Mirrors ``PackedGGUFWeight`` of the reference (mini_llm/ops/quantized_weight.py:44-99):
validation of shape / block alignment / byte count, a flat uint8 *view* of the caller's
buffer (an mmap stays the owner), and zero-copy ``select_outer``.  Constructing it never
materialises a floating-point matrix.  Decoding happens on the device only
(``DevicePackedGGUFWeight.dequantize``); this package has no host decoder.
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
