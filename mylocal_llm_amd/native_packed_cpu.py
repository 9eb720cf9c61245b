"""Host-side packed operators: NumPy activations, host-packed weights, scalar C++ in the library.

The surface of the reference's native CPU backend (``packed_cpu_linear`` / ``packed_cpu_expert``,
mini_llm/ops/native_packed_cpu.py:102-163) over this package's own host twins
(``qmoe_linear_cpu`` / ``qmoe_expert_cpu`` in libqmoe_hip.so).  The reference compiles its C++ on
first use and may fall back to a NumPy decoder; here the twins are part of the prebuilt library, so
every backend name computes the same way and nothing is ever dequantised to a dense matrix.
The calls release the GIL.  None of this runs on, or stands in for, the GPU path: device tensors
never reach these functions.
"""
import ctypes

import numpy as np

from . import _lib
from .quantized_weight import PackedGGUFWeight

BACKENDS = ("reference", "auto", "native")
_HOST_FLOATS = (np.float16, np.float32, np.float64)


def check_backend(name):
    if name not in BACKENDS:
        raise ValueError("cpu_packed_backend must be 'reference', 'auto' or 'native'")


def _address(array):
    return ctypes.c_void_p(array.ctypes.data)


def _weight_args(weight):
    """(address, format id) of a host-packed matrix; keeps a contiguous view alive for the call."""
    data = np.ascontiguousarray(np.asarray(weight.data).reshape(-1).view(np.uint8))
    return data, (_address(data), _lib.FORMAT_ID[weight.quant_type])


def _as_rows(x, columns, what):
    x = np.asarray(x)
    if x.dtype not in _HOST_FLOATS:
        raise TypeError(f"{what} must be FP16, FP32 or FP64")
    return x, np.ascontiguousarray(x.reshape(-1, columns), dtype=np.float32)


def _finish(out32, x, columns):
    return out32.astype(x.dtype, copy=False).reshape(tuple(x.shape[:-1]) + (columns,))


def packed_cpu_linear(x, weight, *, backend="native"):
    """``x @ weight.T`` for NumPy ``x`` [M, K] / [B, T, K] and a host ``PackedGGUFWeight`` [N, K];
    fp32 arithmetic, result in x's dtype."""
    if not isinstance(weight, PackedGGUFWeight) or len(weight.shape) != 2:
        raise TypeError("Expected a packed [N,K] GGUF matrix")
    check_backend(backend)
    n, k = weight.shape
    if np.ndim(x) not in (2, 3) or np.shape(x)[-1] != k:
        raise ValueError("Expected [M,K] or [B,T,K] activations matching weight")
    x, rows = _as_rows(x, k, "CPU activation")
    out = np.empty((rows.shape[0], n), np.float32)
    if rows.shape[0]:
        keep, (address, fmt) = _weight_args(weight)
        rc = _lib.load().qmoe_linear_cpu(address, fmt, n, k, _address(rows), rows.shape[0], _address(out))
        _lib.check(rc, "Native packed GEMV")
    return _finish(out, x, n)


def packed_cpu_swiglu(x, gate, up):
    """``silu(x @ gate.T) * (x @ up.T)`` on the host; gate and up [F, K] may differ in format."""
    f, k = gate.shape
    x, rows = _as_rows(x, k, "CPU activation")
    out = np.empty((rows.shape[0], f), np.float32)
    if rows.shape[0]:
        keep_g, (g_address, g_fmt) = _weight_args(gate)
        keep_u, (u_address, u_fmt) = _weight_args(up)
        rc = _lib.load().qmoe_swiglu_cpu(g_address, g_fmt, u_address, u_fmt, f, k, _address(rows), rows.shape[0], _address(out))
        _lib.check(rc, "Native packed SwiGLU")
    return _finish(out, x, f)


def packed_cpu_expert(x, weights, *, backend="native"):
    """One whole SwiGLU expert on the host: ``down(silu(x @ gate.T) * (x @ up.T))`` for x [M, D]."""
    if len(weights) != 3 or not all(isinstance(w, PackedGGUFWeight) for w in weights):
        raise TypeError("Expected three PackedGGUFWeight projections")
    gate, up, down = weights
    if gate.shape != up.shape or down.shape != (gate.shape[1], gate.shape[0]):
        raise ValueError("Invalid packed expert projection shapes")
    check_backend(backend)
    f, d = gate.shape
    if np.ndim(x) != 2 or np.shape(x)[1] != d:
        raise ValueError("Expert activations must be [M,d_model]")
    x, rows = _as_rows(x, d, "Expert activations")
    out = np.empty((rows.shape[0], d), np.float32)
    if rows.shape[0]:
        keep = [_weight_args(w) for w in weights]
        flat = [item for _, pair in keep for item in pair]
        rc = _lib.load().qmoe_expert_cpu(*flat, d, f, _address(rows), rows.shape[0], _address(out))
        _lib.check(rc, "Native packed expert")
    return out.astype(x.dtype, copy=False)


def router_topk_cpu(logits, k, *, floor=1.0, renormalize=False):
    """Softmax over all experts, exact top-k, optional renormalisation, for NumPy logits [..., E]:
    (weights fp32, ids int64), both shaped ``logits.shape[:-1] + (k,)``."""
    logits = np.asarray(logits)
    if logits.ndim < 1 or not 1 <= int(k) <= logits.shape[-1]:
        raise ValueError("expert router expects 1 <= k <= n_experts")
    n, k = logits.shape[-1], int(k)
    rows = np.ascontiguousarray(logits.reshape(-1, n), dtype=np.float32)
    weights = np.empty((rows.shape[0], k), np.float32)
    ids = np.empty((rows.shape[0], k), np.int64)
    if rows.shape[0]:
        rc = _lib.load().qmoe_router_topk_cpu(_address(rows), rows.shape[0], n, k, float(floor), int(bool(renormalize)),
                                              _address(weights), _address(ids))
        _lib.check(rc, "Host router top-k")
    shape = tuple(logits.shape[:-1]) + (k,)
    return weights.reshape(shape), ids.reshape(shape)
