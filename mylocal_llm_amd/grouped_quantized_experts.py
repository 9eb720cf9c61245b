"""Single-token grouped packed experts on the device.

Same entry points as the reference's mini_llm/ops/grouped_quantized_experts.py
(``grouped_quantized_experts_forward`` :159-217, ``supports_grouped_quantized_experts``
:141-150): E expert handles in the order they are to be summed, fp32 x [1, D], fp32 routes
[E] (any stride), optional host ``routing_slots``.  Graph: fp32 gate/up GEMVs -> stored fp32
SwiGLU -> fp32 down GEMV -> stored fp32 product with the route -> sequential fp32 adds from
zero in handle order (no FMA, no tree).
"""
import ctypes

import numpy as np
import torch

from . import _lib
from .quantized_linear import (
    DevicePackedGGUFWeight, PackedExpertFFNInference, _FORMAT_ID, _ptr, _stream,
)
from .quantized_weight import BLOCK_FORMATS


def _is_index(value, bound):
    return isinstance(value, (int, np.integer)) and not isinstance(value, bool) and 0 <= value < bound


def _device_f32(t):
    return isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32


def _storage_ok(w):
    """The packed bytes of one projection are a contiguous uint8 tensor of exactly the size its shape asks for."""
    per_block, block_size = BLOCK_FORMATS[w.quant_type]
    rows, cols = w.shape
    return (w.data.dtype == torch.uint8 and w.data.is_contiguous() and cols % per_block == 0
            and w.data.numel() == rows * cols // per_block * block_size)


def _operand_checks(x, experts, routes, block_k, slots):
    """(passes, reason) pairs about the call's own operands, cheapest first; evaluated lazily."""
    yield block_k in (256, 512, 1024), "block_k must be 256, 512 or 1024"
    yield _device_f32(x), "x must be a CUDA FP32 tensor"
    yield (x.ndim == 2 and x.shape[0] == 1 and x.shape[1] > 0 and x.is_contiguous()), \
        "x must be contiguous [1, D] with positive D"
    yield (isinstance(experts, (list, tuple)) and 0 < len(experts) < 65536), \
        "experts must be a nonempty list/tuple of at most 65535 handles"
    count = len(experts)
    if slots is not None:
        yield (isinstance(slots, (tuple, list)) and len(slots) == count and all(_is_index(s, count) for s in slots)), \
            "routing_slots must be host integer indices into the [E] routing weights"
    yield (_device_f32(routes) and tuple(routes.shape) == (count,)), \
        "routing_weights must be a CUDA FP32 [E] tensor (slices allowed)"
    yield routes.device == x.device, "all operands must be on the same device"


def _handle_checks(x, handle, first):
    """(passes, reason) pairs about one expert handle; ``first`` is the handle all others must match."""
    yield isinstance(handle, PackedExpertFFNInference), "experts must contain PackedExpertFFNInference handles"
    triple = (handle.gate, handle.up, handle.down)
    yield all(isinstance(w, DevicePackedGGUFWeight) for w in triple), \
        "all projections must be DevicePackedGGUFWeight (no host fallback)"
    d = x.shape[1]
    gate_shape = tuple(handle.gate.shape)
    yield (len(gate_shape) == 2 and min(gate_shape) > 0 and gate_shape[1] == d
           and tuple(handle.up.shape) == gate_shape and tuple(handle.down.shape) == gate_shape[::-1]), \
        "expert shapes must be gate/up [F, D], down [D, F] matching x"
    if handle is not first:
        same = all((tuple(w.shape), w.quant_type) == (tuple(v.shape), v.quant_type)
                   for w, v in zip(triple, (first.gate, first.up, first.down)))
        yield same, "all experts must share per-projection shapes and quantization formats"
    for w in triple:
        yield _storage_ok(w), "invalid packed projection storage or block alignment"
        yield w.data.device == x.device, "all operands must be on the same device"


def _unsupported_reason(x, experts, routing_weights, block_k, routing_slots=None):
    """None if the call is one the grouped path takes, else the reason (the conditions of
    mini_llm/ops/grouped_quantized_experts.py:82-138 that apply to device tensors)."""
    for passes, reason in _operand_checks(x, experts, routing_weights, block_k, routing_slots):
        if not passes:
            return reason
    for handle in experts:
        for passes, reason in _handle_checks(x, handle, experts[0]):
            if not passes:
                return reason
    return None


def supports_grouped_quantized_experts(x, experts, routing_weights, *, block_k=512,
                                       routing_slots=None) -> bool:
    """Metadata-only support check; no allocation, transfers, or GPU kernels."""
    return _unsupported_reason(x, experts, routing_weights, block_k, routing_slots) is None


# Host lists of up to this many experts travel in the kernel arguments (qmoe_grouped_decode_listed).
_LISTED_MAX = 16
# One scratch tensor per (device, stream) grown on demand: a decode loop calls with the same sizes
# every token, so a call allocates nothing but its fresh output.  Work on one stream is ordered, so
# consecutive calls may share the scratch; calls on different streams get different tensors.
_SCRATCH = {}


def _scratch(device, floats):
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    held = _SCRATCH.get(key)
    if held is None or held.numel() < floats:
        held = torch.empty(floats, dtype=torch.float32, device=device)
        _SCRATCH[key] = held
    return held


def grouped_quantized_experts_forward(x, experts, routing_weights, *, block_k=512,
                                      routing_slots=None):
    """Return a fresh FP32 [1, D] weighted expert sum on torch's current stream.

    Up to 16 handles (a decode step's top-k) are handed over as a host list: pointers and route
    positions go into the kernel arguments and the scratch is reused across calls, so the call
    uploads nothing and allocates only its output.  Longer lists build a device pointer table as the
    reference does (mini_llm/ops/grouped_quantized_experts.py:180-186)."""
    reason = _unsupported_reason(x, experts, routing_weights, block_k, routing_slots)
    if reason is not None:
        raise ValueError(f"Unsupported grouped quantized experts: {reason}")
    e, d, f = len(experts), x.shape[1], experts[0].gate.shape[0]
    lib = _lib.load()
    first = experts[0]
    formats = tuple(_FORMAT_ID[w.quant_type] for w in (first.gate, first.up, first.down))
    out = torch.empty((1, d), dtype=torch.float32, device=x.device)
    stride = routing_weights.stride(0)
    pointers = [w.data.data_ptr() for h in experts for w in (h.gate, h.up, h.down)]
    with torch.cuda.device(x.device):
        if e <= _LISTED_MAX:
            table = (ctypes.c_void_p * (3 * e))(*pointers)
            slots = (ctypes.c_int32 * e)(*(int(s) for s in routing_slots)) if routing_slots is not None else None
            workspace = _scratch(x.device, e * (f + d + 8))
            rc = lib.qmoe_grouped_decode_listed(
                _ptr(x), ctypes.cast(table, ctypes.c_void_p), e, *formats, d, f, _ptr(routing_weights), stride,
                ctypes.cast(slots, ctypes.c_void_p) if slots is not None else ctypes.c_void_p(0),
                _ptr(out), _ptr(workspace), _stream())
        else:
            table = torch.from_numpy(np.asarray(pointers, dtype=np.uint64).view(np.int64)).to(x.device, non_blocking=False)
            slots = None
            if routing_slots is not None:
                slots = torch.tensor([int(s) for s in routing_slots], dtype=torch.int32).to(x.device)
            workspace = torch.empty(e * (f + d), dtype=torch.float32, device=x.device)
            rc = lib.qmoe_grouped_decode(
                _ptr(x), _ptr(table), e, *formats, d, f, _ptr(routing_weights), stride,
                _ptr(slots) if slots is not None else ctypes.c_void_p(0),
                _ptr(out), _ptr(workspace), _stream())
    _lib.check(rc, "Grouped packed experts")
    return out
