"""ctypes binding of libqmoe_hip.so (the C ABI declared in include/qmoe.h).

The library is built in-tree by ``mylocal_llm_amd._build`` (``__graft_entry__.build()``).
There is no CPU fallback: if the shared library is missing or does not load, every
operator of this package raises instead of computing anything.
"""
import ctypes
import os
import threading

from . import _build

_P = ctypes.c_void_p
_I = ctypes.c_int
_I64 = ctypes.c_int64
_F = ctypes.c_float
_SZ = ctypes.c_size_t

FORMAT_ID = {"Q8_0": 0, "Q4_0": 1, "Q4_K": 2, "Q3_K": 3, "Q5_K": 4, "Q6_K": 5, "BF16": 100}
DTYPE_ID = {"float32": 0, "float16": 1, "bfloat16": 2}


class LinearProblem(ctypes.Structure):
    _fields_ = [("w", _P), ("x", _P), ("y", _P), ("fmt", _I), ("n", _I), ("k", _I), ("tokens", _I),
                ("x_dtype", _I), ("y_dtype", _I)]


class ExpertBank(ctypes.Structure):
    _fields_ = [("gate", _P), ("up", _P), ("down", _P),
                ("gate_stride", _I64), ("up_stride", _I64), ("down_stride", _I64),
                ("gate_fmt", _I), ("up_fmt", _I), ("down_fmt", _I),
                ("n_experts", _I), ("d_model", _I), ("d_ff", _I)]


class MoeArgs(ctypes.Structure):
    _fields_ = [("hidden", _P), ("hidden_dtype", _I), ("tokens", _I), ("top_k", _I),
                ("logits", _P), ("floor_value", _F), ("renormalize", _I),
                ("in_weights", _P), ("in_ids", _P),
                ("bank", ExpertBank),
                ("shared_gate_w", _P), ("shared_up_w", _P), ("shared_down_w", _P),
                ("shared_gate_fmt", _I), ("shared_up_fmt", _I), ("shared_down_fmt", _I),
                ("d_ff_shared", _I), ("shared_gate", _P),
                ("out", _P), ("out_dtype", _I), ("out_weights", _P), ("out_ids", _P), ("residual", _P), ("status_out", _P)]


ABI_VERSION = 5   # QMOE_ABI_VERSION of include/qmoe.h this binding was written against

_SIGNATURES = {
    "qmoe_abi_version": ([], _I),
    "qmoe_last_error": ([], ctypes.c_char_p),
    "qmoe_init": ([], _I),
    "qmoe_check_status": ([_P], _I),
    "qmoe_set_wait_limit": ([ctypes.c_longlong], None),
    "qmoe_format_info": ([_I, ctypes.POINTER(_I), ctypes.POINTER(_I)], _I),
    "qmoe_dequantize": ([_P, _I, _I64, _I64, _P, _P], _I),
    "qmoe_linear": ([_P, _I, _I, _I, _P, _I, _I, _P, _I, _P], _I),
    "qmoe_linear_batch": ([ctypes.POINTER(LinearProblem), _I, _P], _I),
    "qmoe_swiglu": ([_P, _I, _P, _I, _I, _I, _P, _I, _I, _P, _I, _P], _I),
    "qmoe_expert": ([_P, _I, _P, _I, _P, _I, _I, _I, _P, _I, _I, _P, _I, _P, _P], _I),
    "qmoe_router_topk": ([_P, _I, _I, _I, _F, _I, _P, _P, _P], _I),
    "qmoe_grouped_decode": ([_P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _P, _P], _I),
    "qmoe_grouped_decode_listed": ([_P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _P, _P], _I),
    "qmoe_moe_workspace_bytes": ([_I, _I, _I, _I, _I, _I], _SZ),
    "qmoe_moe_forward": ([ctypes.POINTER(MoeArgs), _P, _SZ, _P], _I),
    "qmoe_norm_router": ([_P, _I, _I, _P, _F, _P, _P, _I, _P, _P, _P], _I),
    "qmoe_router_logits": ([_P, _I, _I, _P, _P, _I, _P, _P], _I),
    "qmoe_routing_plan": ([_P, _P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P], _I),
    "qmoe_read_probe": ([_P, _SZ, ctypes.c_uint32, _P, _P], _I),
    "qmoe_dequantize_cpu": ([_P, _I, _I64, _I64, _P], _I),
    "qmoe_linear_cpu": ([_P, _I, _I, _I, _P, _I, _P], _I),
    "qmoe_swiglu_cpu": ([_P, _I, _P, _I, _I, _I, _P, _I, _P], _I),
    "qmoe_expert_cpu": ([_P, _I, _P, _I, _P, _I, _I, _I, _P, _I, _P], _I),
    "qmoe_router_topk_cpu": ([_P, _I, _I, _I, _F, _I, _P, _P], _I),
    "qmoe_moe_static_scratch_bytes": ([], _SZ),
    "qmoe_moe_forward_static": ([ctypes.POINTER(MoeArgs), _P], _I),
}
EXPORTS = tuple(_SIGNATURES)

_LOCK = threading.Lock()
_LIB = None


def library_path():
    """The library this process binds: QMOE_LIBRARY names another build of it (the measurement
    variant with time stamps, say), otherwise the one built in-tree."""
    return os.environ.get("QMOE_LIBRARY") or _build.LIB_PATH


def load():
    """Return the loaded library; raise RuntimeError if it is not there."""
    global _LIB
    with _LOCK:
        if _LIB is None:
            path = library_path()
            if not os.path.exists(path):
                raise RuntimeError(
                    f"{path} is missing: build it with `python -m mylocal_llm_amd._build` "
                    "(or __graft_entry__.build()); this package has no CPU fallback")
            lib = ctypes.CDLL(path)
            for name, (argtypes, restype) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.argtypes = argtypes
                fn.restype = restype
            if lib.qmoe_abi_version() != ABI_VERSION:
                raise RuntimeError(f"{path}: unexpected ABI version {lib.qmoe_abi_version()}")
            _LIB = lib
        return _LIB


def check(rc, what):
    """Raise the reference's error shape (RuntimeError with the code) on nonzero status."""
    if rc:
        message = load().qmoe_last_error().decode(errors="replace")
        if rc == 2:
            raise NotImplementedError(f"{what} failed with error code {rc}: {message}")
        raise RuntimeError(f"{what} failed with error code {rc}: {message}")
