"""ctypes access to the C oracle and to the reference's own native library.

TEST INFRASTRUCTURE ONLY.  ``load_oracle()`` loads ``oracle/liboracle.so`` (built
from ``oracle/oracle.c``); ``load_ref()`` loads ``oracle/_ref/libref_packed_cpu.so``,
which ``oracle/Makefile`` builds from the reference's
``mini_llm/ops/native_packed_cpu.cpp`` where that checkout is present, and
returns ``None`` where it was never built.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
FORMAT_ID = {"Q8_0": 0, "Q4_0": 1, "Q4_K": 2, "Q3_K": 3, "Q5_K": 4, "Q6_K": 5, "BF16": 100}
_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
_ORACLE = None
_REF = False


def build():
    """Compile the oracle (and oracle/_ref when the reference checkout is there)."""
    subprocess.run(["make", "-s", "-C", _HERE, "all"], check=True)


def load_oracle():
    global _ORACLE
    if _ORACLE is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        lib.oracle_dequantize.argtypes = [_P, _I, _L, _L, _P]
        lib.oracle_linear.argtypes = [_P, _I, _I, _I, _P, _I, _P]
        lib.oracle_swiglu.argtypes = [_P, _I, _P, _I, _I, _I, _P, _I, _P]
        lib.oracle_expert.argtypes = [_P, _I, _P, _I, _P, _I, _I, _I, _P, _I, _P]
        lib.oracle_router_topk.argtypes = [_P, _I, _I, _I, _F, _I, _P, _P]
        for name in ("oracle_dequantize", "oracle_linear", "oracle_swiglu", "oracle_expert",
                     "oracle_router_topk"):
            getattr(lib, name).restype = _I
        _ORACLE = lib
    return _ORACLE


def load_ref():
    """The reference's native packed CPU library, or None if it was not built."""
    global _REF
    if _REF is False:
        path = os.path.join(_HERE, "_ref", "libref_packed_cpu.so")
        if os.path.exists(path):
            lib = ctypes.CDLL(path)
            lib.mylocal_packed_gemv.argtypes = [_P, _I, _I, _I, _P, _I, _P]
            lib.mylocal_packed_gemv.restype = _I
            lib.mylocal_packed_expert.argtypes = [_P, _I, _P, _I, _P, _I, _I, _I, _P, _I, _P]
            lib.mylocal_packed_expert.restype = _I
            _REF = lib
        else:
            _REF = None
    return _REF


def _bytes(a):
    return np.ascontiguousarray(np.asarray(a).view(np.uint8).reshape(-1))


def c_dequantize(data, shape, fmt):
    raw = _bytes(data)
    n = int(np.prod(shape[:-1]))
    out = np.empty((n, shape[-1]), np.float32)
    rc = load_oracle().oracle_dequantize(raw.ctypes.data, FORMAT_ID[fmt], n, shape[-1], out.ctypes.data)
    if rc:
        raise RuntimeError(f"oracle_dequantize failed with {rc}")
    return out.reshape(shape)


def c_linear(x, data, shape, fmt):
    raw = _bytes(data)
    x32 = np.ascontiguousarray(np.asarray(x, np.float32).reshape(-1, shape[1]))
    y = np.empty((x32.shape[0], shape[0]), np.float32)
    rc = load_oracle().oracle_linear(raw.ctypes.data, FORMAT_ID[fmt], shape[0], shape[1],
                                     x32.ctypes.data, x32.shape[0], y.ctypes.data)
    if rc:
        raise RuntimeError(f"oracle_linear failed with {rc}")
    return y


def c_expert(x, gate, up, down):
    """gate/up/down are (data, shape, fmt)."""
    g, u, d = (_bytes(w[0]) for w in (gate, up, down))
    x32 = np.ascontiguousarray(np.asarray(x, np.float32))
    out = np.empty((x32.shape[0], gate[1][1]), np.float32)
    rc = load_oracle().oracle_expert(g.ctypes.data, FORMAT_ID[gate[2]], u.ctypes.data, FORMAT_ID[up[2]],
                                     d.ctypes.data, FORMAT_ID[down[2]], gate[1][1], gate[1][0],
                                     x32.ctypes.data, x32.shape[0], out.ctypes.data)
    if rc:
        raise RuntimeError(f"oracle_expert failed with {rc}")
    return out


def c_router_topk(logits, k, floor=2.0 ** -14, renorm=True):
    z = np.ascontiguousarray(np.asarray(logits, np.float32))
    n = z.shape[-1]
    t = z.size // n
    w = np.empty((t, k), np.float32)
    ids = np.empty((t, k), np.int64)
    rc = load_oracle().oracle_router_topk(z.ctypes.data, t, n, k, floor, int(renorm),
                                          w.ctypes.data, ids.ctypes.data)
    if rc:
        raise RuntimeError(f"oracle_router_topk failed with {rc}")
    return w.reshape(z.shape[:-1] + (k,)), ids.reshape(z.shape[:-1] + (k,))


def ref_gemv(x, data, shape, fmt):
    """x @ W.T through the reference's own mylocal_packed_gemv (None if not built)."""
    lib = load_ref()
    if lib is None or fmt == "BF16":
        return None
    raw = _bytes(data)
    x32 = np.ascontiguousarray(np.asarray(x, np.float32).reshape(-1, shape[1]))
    y = np.empty((x32.shape[0], shape[0]), np.float32)
    rc = lib.mylocal_packed_gemv(raw.ctypes.data, FORMAT_ID[fmt], shape[0], shape[1],
                                 x32.ctypes.data, x32.shape[0], y.ctypes.data)
    if rc:
        raise RuntimeError(f"mylocal_packed_gemv failed with {rc}")
    return y


def ref_expert(x, gate, up, down):
    lib = load_ref()
    if lib is None:
        return None
    g, u, d = (_bytes(w[0]) for w in (gate, up, down))
    x32 = np.ascontiguousarray(np.asarray(x, np.float32))
    out = np.empty((x32.shape[0], gate[1][1]), np.float32)
    rc = lib.mylocal_packed_expert(g.ctypes.data, FORMAT_ID[gate[2]], u.ctypes.data, FORMAT_ID[up[2]],
                                   d.ctypes.data, FORMAT_ID[down[2]], gate[1][1], gate[1][0],
                                   x32.ctypes.data, x32.shape[0], out.ctypes.data)
    if rc:
        raise RuntimeError(f"mylocal_packed_expert failed with {rc}")
    return out
