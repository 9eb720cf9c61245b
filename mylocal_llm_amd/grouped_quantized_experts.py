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


def _unsupported_reason(x, experts, routing_weights, block_k, routing_slots=None):
    if block_k not in (256, 512, 1024):
        return "block_k must be 256, 512 or 1024"
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float32:
        return "x must be a CUDA FP32 tensor"
    if x.ndim != 2 or x.shape[0] != 1 or x.shape[1] <= 0 or not x.is_contiguous():
        return "x must be contiguous [1, D] with positive D"
    if not isinstance(experts, (list, tuple)) or not 1 <= len(experts) <= 65535:
        return "experts must be a nonempty list/tuple of at most 65535 handles"
    if routing_slots is not None and (
            not isinstance(routing_slots, (tuple, list)) or len(routing_slots) != len(experts)
            or any(not isinstance(slot, (int, np.integer)) or isinstance(slot, bool)
                   or not 0 <= slot < len(experts) for slot in routing_slots)):
        return "routing_slots must be host integer indices into the [E] routing weights"
    if (not isinstance(routing_weights, torch.Tensor) or not routing_weights.is_cuda
            or routing_weights.dtype != torch.float32
            or tuple(routing_weights.shape) != (len(experts),)):
        return "routing_weights must be a CUDA FP32 [E] tensor (slices allowed)"
    if routing_weights.device != x.device:
        return "all operands must be on the same device"
    signature = None
    for expert in experts:
        if not isinstance(expert, PackedExpertFFNInference):
            return "experts must contain PackedExpertFFNInference handles"
        projections = (expert.gate, expert.up, expert.down)
        if not all(isinstance(w, DevicePackedGGUFWeight) for w in projections):
            return "all projections must be DevicePackedGGUFWeight (no host fallback)"
        gate, up, down = projections
        if (len(gate.shape) != 2 or min(gate.shape) <= 0
                or gate.shape != up.shape or gate.shape[1] != x.shape[1]
                or down.shape != (x.shape[1], gate.shape[0])):
            return "expert shapes must be gate/up [F, D], down [D, F] matching x"
        current = tuple((w.shape, w.quant_type) for w in projections)
        if signature is not None and current != signature:
            return "all experts must share per-projection shapes and quantization formats"
        signature = current
        for w in projections:
            qk, qb = BLOCK_FORMATS[w.quant_type]
            if (w.data.dtype != torch.uint8 or not w.data.is_contiguous() or w.shape[1] % qk
                    or w.data.numel() != w.shape[0] * w.shape[1] // qk * qb):
                return "invalid packed projection storage or block alignment"
            if w.data.device != x.device:
                return "all operands must be on the same device"
    return None


def supports_grouped_quantized_experts(x, experts, routing_weights, *, block_k=512,
                                       routing_slots=None) -> bool:
    """Metadata-only support check; no allocation, transfers, or GPU kernels."""
    return _unsupported_reason(x, experts, routing_weights, block_k, routing_slots) is None


def grouped_quantized_experts_forward(x, experts, routing_weights, *, block_k=512,
                                      routing_slots=None):
    """Return a fresh FP32 [1, D] weighted expert sum on torch's current stream."""
    reason = _unsupported_reason(x, experts, routing_weights, block_k, routing_slots)
    if reason is not None:
        raise ValueError(f"Unsupported grouped quantized experts: {reason}")
    e, d, f = len(experts), x.shape[1], experts[0].gate.shape[0]
    host = np.asarray([[w.data.data_ptr() for w in (h.gate, h.up, h.down)] for h in experts], dtype=np.uint64)
    table = torch.from_numpy(host.view(np.int64)).to(x.device, non_blocking=False)
    slots = None
    if routing_slots is not None:
        slots = torch.tensor([int(s) for s in routing_slots], dtype=torch.int32).to(x.device)
    workspace = torch.empty(e * (f + d), dtype=torch.float32, device=x.device)
    out = torch.empty((1, d), dtype=torch.float32, device=x.device)
    gate, up, down = experts[0].gate, experts[0].up, experts[0].down
    stride = routing_weights.stride(0)
    with torch.cuda.device(x.device):
        rc = _lib.load().qmoe_grouped_decode(
            _ptr(x), _ptr(table), e, _FORMAT_ID[gate.quant_type], _FORMAT_ID[up.quant_type],
            _FORMAT_ID[down.quant_type], d, f, _ptr(routing_weights), stride,
            _ptr(slots) if slots is not None else ctypes.c_void_p(0),
            _ptr(out), _ptr(workspace), _stream())
    _lib.check(rc, "Grouped packed experts")
    return out
