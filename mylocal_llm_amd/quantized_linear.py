"""Device packed-weight linear, fused SwiGLU and packed expert operators.

Same entry points and argument meaning as the reference's
mini_llm/ops/quantized_linear.py (``quantized_linear`` :272, ``quantized_swiglu`` :338,
``PackedExpertFFNInference`` :403, ``DevicePackedGGUFWeight`` / ``packed_to_device``
:45-86, ``supports_packed_gpu_type`` :36-42).  Device arrays are ``torch.Tensor`` on the
MI355X; every operator enqueues hand-written HIP kernels of libqmoe_hip.so on torch's
current stream through the C ABI.  NumPy activations with host ``PackedGGUFWeight`` matrices
take the host branch of the reference (:292-305), computed by the library's scalar C++ twins;
a device tensor never does: mixing a device activation with a host weight is an error, and the
device path raises when the library is missing.
"""
from dataclasses import dataclass
import ctypes
import math

import numpy as np
import torch

from . import _lib
from .quantized_weight import BLOCK_FORMATS, PackedGGUFWeight

_FORMAT_ID = {name: _lib.FORMAT_ID[name] for name in BLOCK_FORMATS}
SUPPORTED_GPU_PACKED_FORMATS = frozenset(_FORMAT_ID)
_TORCH_DTYPE_ID = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def supports_packed_gpu_type(quant_type):
    """Report kernel format support, independently of runtime availability."""
    return quant_type in SUPPORTED_GPU_PACKED_FORMATS


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(tensor):
    return ctypes.c_void_p(tensor.data_ptr())


@dataclass(frozen=True)
class DevicePackedGGUFWeight:
    """HBM-resident packed matrix [N, K]; same layout contract as PackedGGUFWeight."""

    data: object
    shape: tuple
    quant_type: str

    def __post_init__(self):
        if self.quant_type not in BLOCK_FORMATS:
            raise ValueError(f"Unsupported GGUF type {self.quant_type}")
        if not supports_packed_gpu_type(self.quant_type):
            raise NotImplementedError(f"No packed GPU kernel for {self.quant_type}")
        if not isinstance(self.data, torch.Tensor) or self.data.dtype != torch.uint8 or not self.data.is_cuda:
            raise TypeError("Device packed bytes must be a CUDA torch.uint8 tensor")
        if not self.data.is_contiguous():
            raise ValueError("Device packed bytes must be contiguous")
        shape = tuple(int(i) for i in self.shape)
        if len(shape) != 2 or min(shape) <= 0:
            raise ValueError("Device packed linear weights must be [N, K]")
        elems, block_bytes = BLOCK_FORMATS[self.quant_type]
        if shape[-1] % elems or int(self.data.numel()) != math.prod(shape) // elems * block_bytes:
            raise ValueError("Invalid packed byte length or K block alignment")
        object.__setattr__(self, "shape", shape)

    @property
    def nbytes(self):
        return int(self.data.numel())

    def dequantize(self):
        """Dense fp32 [N, K] on the device; bit-identical to the reference's host decoder."""
        n, k = self.shape
        out = torch.empty((n, k), dtype=torch.float32, device=self.data.device)
        with torch.cuda.device(self.data.device):
            rc = _lib.load().qmoe_dequantize(_ptr(self.data), _FORMAT_ID[self.quant_type], n, k, _ptr(out), _stream())
        _lib.check(rc, "Packed dequantize")
        return out


def _upload_bytes(array, device):
    """uint8 bytes (possibly a read-only view of a memory-mapped file) as a tensor on ``device``."""
    import warnings
    array = np.ascontiguousarray(array)
    with warnings.catch_warnings():
        # the host tensor is only the source of the copy and is never written through
        warnings.filterwarnings("ignore", message="The given NumPy array is not writable")
        return torch.from_numpy(array).to(device)


def packed_to_device(weight, device=None):
    """Upload the *packed bytes* of one matrix/expert to HBM once (no expansion)."""
    if not isinstance(weight, PackedGGUFWeight) or len(weight.shape) != 2:
        raise TypeError("Expected a two-dimensional PackedGGUFWeight")
    if not supports_packed_gpu_type(weight.quant_type):
        raise NotImplementedError(f"No packed GPU kernel for {weight.quant_type}")
    if not torch.cuda.is_available():
        raise RuntimeError("Packed GPU weights require a HIP device")
    _lib.load()
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    return DevicePackedGGUFWeight(_upload_bytes(weight.data, device), weight.shape, weight.quant_type)


def _check_activation(x, what):
    if not isinstance(x, torch.Tensor) or not x.is_cuda:
        raise TypeError(f"{what} must be a CUDA torch.Tensor (or a NumPy array with host-packed weights)")
    if x.dtype not in _TORCH_DTYPE_ID:
        raise TypeError("GPU input must be FP16, BF16, or FP32")


def _host_linear(x, weight, backend):
    """NumPy activations: host-packed weight only (quantized_linear.py:292-305)."""
    from . import native_packed_cpu
    if x.ndim not in (2, 3):
        raise ValueError("Expected x as [M, K] or [B, T, K]")
    if x.shape[-1] != weight.shape[-1]:
        raise ValueError("Input K does not match packed weight K")
    if len(weight.shape) != 2:
        raise ValueError("Packed linear weights must be [N, K]")
    if not isinstance(weight, PackedGGUFWeight):
        raise TypeError("NumPy input requires a host PackedGGUFWeight; device weights take CUDA tensors")
    if x.dtype not in (np.float16, np.float32, np.float64):
        raise TypeError("Reference CPU inference requires FP16/FP32/FP64 input")
    native_packed_cpu.check_backend(backend)
    return native_packed_cpu.packed_cpu_linear(x, weight, backend=backend)


def quantized_linear(x, weight, *, block_k=512, cpu_packed_backend="reference"):
    """Compute ``x @ weight.T`` for a packed GGUF [out_features, in_features] matrix.

    x is a contiguous CUDA tensor [M, K] or [B, T, K] (fp16 / bf16 / fp32); the result has
    shape ``x.shape[:-1] + (N,)`` and x's dtype, accumulated in fp32 and rounded once.
    ``block_k`` is validated as in the reference and otherwise unused.  A NumPy ``x`` (fp16 /
    fp32 / fp64) with a host ``PackedGGUFWeight`` is computed on the CPU in fp32 by the library's
    scalar C++ (every ``cpu_packed_backend`` name selects that same code).
    """
    if isinstance(x, np.ndarray):
        return _host_linear(x, weight, cpu_packed_backend)
    _check_activation(x, "Packed linear input")
    if x.ndim not in (2, 3):
        raise ValueError("Expected x as [M, K] or [B, T, K]")
    if x.shape[-1] != weight.shape[-1]:
        raise ValueError("Input K does not match packed weight K")
    if len(weight.shape) != 2:
        raise ValueError("Packed linear weights must be [N, K]")
    if isinstance(weight, PackedGGUFWeight):
        raise TypeError("Packed host weight requires a NumPy input; upload it with packed_to_device for device tensors")
    if not isinstance(weight, DevicePackedGGUFWeight):
        raise TypeError("Expected PackedGGUFWeight or DevicePackedGGUFWeight")
    if not x.is_contiguous():
        raise ValueError("GPU input must be a contiguous tensor")
    if x.device != weight.data.device:
        raise ValueError("all operands must be on the same device")
    if block_k not in (256, 512, 1024):
        raise ValueError("block_k must be 256, 512 or 1024")
    n, k = weight.shape
    m = x.numel() // k
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if m:
        with torch.cuda.device(x.device):
            rc = _lib.load().qmoe_linear(_ptr(weight.data), _FORMAT_ID[weight.quant_type], n, k,
                                         _ptr(x), _TORCH_DTYPE_ID[x.dtype], m,
                                         _ptr(out), _TORCH_DTYPE_ID[x.dtype], _stream())
        _lib.check(rc, "Packed linear")
    return out.reshape(tuple(x.shape[:-1]) + (n,))


def quantized_linear_batch(problems):
    """Several independent ``quantized_linear`` calls enqueued through one ABI call.

    ``problems`` is a sequence of (x, weight) pairs; returns the list of outputs.
    """
    outs, descs = [], (_lib.LinearProblem * len(problems))()
    for i, (x, weight) in enumerate(problems):
        _check_activation(x, "Packed linear input")
        if not isinstance(weight, DevicePackedGGUFWeight):
            raise TypeError("Expected DevicePackedGGUFWeight")
        if x.ndim not in (2, 3) or not x.is_contiguous():
            raise ValueError("Expected contiguous x as [M, K] or [B, T, K]")
        n, k = weight.shape
        if x.shape[-1] != k:
            raise ValueError("Input K does not match packed weight K")
        m = x.numel() // k
        if m < 1:
            raise ValueError("Batched linear needs at least one token per problem")
        if x.device != problems[0][0].device or weight.data.device != x.device:
            raise ValueError("All activations and weights of a batch must live on one device")
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
        outs.append(out.reshape(tuple(x.shape[:-1]) + (n,)))
        d = descs[i]
        d.w, d.x, d.y = weight.data.data_ptr(), x.data_ptr(), out.data_ptr()
        d.fmt, d.n, d.k, d.tokens = _FORMAT_ID[weight.quant_type], n, k, m
        d.x_dtype = d.y_dtype = _TORCH_DTYPE_ID[x.dtype]
    if problems:
        with torch.cuda.device(problems[0][0].device):
            rc = _lib.load().qmoe_linear_batch(descs, len(problems), _stream())
        _lib.check(rc, "Packed linear batch")
    return outs


def quantized_swiglu(x, gate, up, *, block_k=512):
    """Compute ``SiLU(x @ gate.T) * (x @ up.T)`` in one launch; gate/up formats may differ."""
    if not isinstance(gate, (PackedGGUFWeight, DevicePackedGGUFWeight)) or not isinstance(
            up, (PackedGGUFWeight, DevicePackedGGUFWeight)):
        raise TypeError("gate and up must be packed GGUF weights")
    if type(gate) is not type(up):
        raise TypeError("gate and up must both be host-packed or both device-packed")
    if len(gate.shape) != 2 or up.shape != gate.shape:
        raise ValueError("gate/up must share two-dimensional [F,K] shape")
    if not isinstance(x, np.ndarray):
        _check_activation(x, "Quantized SwiGLU input")
    if x.ndim not in (2, 3):
        raise ValueError("Expected x as [M,K] or [B,T,K]")
    f, k = gate.shape
    if x.shape[-1] != k:
        raise ValueError("Input K does not match gate/up K")
    if isinstance(gate, PackedGGUFWeight):
        if not isinstance(x, np.ndarray):
            raise TypeError("Host packed gate/up require NumPy activations")
        from . import native_packed_cpu
        return native_packed_cpu.packed_cpu_swiglu(x, gate, up)
    if isinstance(x, np.ndarray):
        raise TypeError("Device packed gate/up require CUDA tensors")
    if not x.is_contiguous():
        raise ValueError("GPU activations must be a contiguous tensor")
    if block_k not in (256, 512, 1024):
        raise ValueError("block_k must be 256, 512 or 1024")
    m = x.numel() // k
    out = torch.empty((m, f), dtype=x.dtype, device=x.device)
    if m:
        with torch.cuda.device(x.device):
            rc = _lib.load().qmoe_swiglu(_ptr(gate.data), _FORMAT_ID[gate.quant_type],
                                         _ptr(up.data), _FORMAT_ID[up.quant_type], f, k,
                                         _ptr(x), _TORCH_DTYPE_ID[x.dtype], m,
                                         _ptr(out), _TORCH_DTYPE_ID[x.dtype], _stream())
        _lib.check(rc, "Packed SwiGLU")
    return out.reshape(tuple(x.shape[:-1]) + (f,))


class PackedExpertFFNInference:
    """Three packed GGUF projections of one SwiGLU expert (gate, up [F, D]; down [D, F])."""

    def __init__(self, gate, up, down, *, fuse_gate_up=True):
        self.gate, self.up, self.down = gate, up, down
        self.fuse_gate_up = bool(fuse_gate_up)
        if gate.shape != up.shape:
            raise ValueError("Gate and up projections must have identical dimensions")
        if down.shape != (gate.shape[1], gate.shape[0]):
            raise ValueError("Down projection dimensions must be transposed")

    def forward(self, x):
        if self.fuse_gate_up:
            h = quantized_swiglu(x, self.gate, self.up)
        else:
            g = quantized_linear(x, self.gate)
            u = quantized_linear(x, self.up)
            if isinstance(g, np.ndarray):
                g32 = g.astype(np.float32)
                h = ((g32 / (1.0 + np.exp(-g32))).astype(g.dtype) * u)
            else:
                h = (g * torch.sigmoid(g.float()).to(g.dtype)) * u
        if isinstance(h, np.ndarray):
            return quantized_linear(np.ascontiguousarray(h), self.down)
        return quantized_linear(h.contiguous(), self.down)
