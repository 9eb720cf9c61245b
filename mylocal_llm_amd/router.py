"""Expert router on the device: full softmax, exact top-k, optional renormalisation.

Same entry points as the reference: ``expert_topk_forward`` (mini_llm/ops/router.py:21-43),
``RouterInference`` (mini_llm/ops/router_inference.py:10-61) and ``try_normalized_topk``
(mini_llm/ops/router_decode.py:247-273).  Selection order is descending logit, lower expert
id on exact ties, NaN last (router_decode.py:19-26); ids are int64.
"""
import math

import numpy as np
import torch

from . import _lib
from .quantized_linear import _ptr, _stream

_MAX_EXPERTS = 4096
_MAX_K = 32


def _topk(logits2d, k, floor, renormalize):
    t, n = logits2d.shape
    weights = torch.empty((t, k), dtype=torch.float32, device=logits2d.device)
    ids = torch.empty((t, k), dtype=torch.int64, device=logits2d.device)
    if t:
        with torch.cuda.device(logits2d.device):
            rc = _lib.load().qmoe_router_topk(_ptr(logits2d), t, n, k, float(floor), int(renormalize),
                                              _ptr(weights), _ptr(ids), _stream())
        _lib.check(rc, "Router top-k")
    return weights, ids


def expert_topk_forward(logits, k, output_dtype=None, return_cache=True):
    """Full-expert softmax followed by top-k selection, without renormalisation.  NumPy logits are
    routed on the host by the library's scalar C++ twin, CUDA tensors by the device kernel."""
    if isinstance(logits, np.ndarray):
        from .native_packed_cpu import router_topk_cpu
        weights, ids = router_topk_cpu(logits, k)
        if output_dtype is not None and np.dtype(output_dtype) in (np.float16,):
            weights = weights.astype(output_dtype)
        return weights, ids, None
    if not isinstance(logits, torch.Tensor) or not logits.is_cuda:
        raise TypeError("router logits must be a CUDA torch.Tensor or a NumPy array")
    if logits.ndim < 1 or not (1 <= int(k) <= int(logits.shape[-1])):
        raise ValueError("expert router expects 1 <= k <= n_experts")
    n = logits.shape[-1]
    if n > _MAX_EXPERTS or int(k) > _MAX_K:
        raise NotImplementedError("router kernel covers at most 4096 experts and k <= 32")
    work = logits.to(torch.float32).contiguous().reshape(-1, n)
    weights, ids = _topk(work, int(k), 1.0, False)
    shape = tuple(logits.shape[:-1]) + (int(k),)
    weights = weights.reshape(shape)
    if output_dtype is not None and output_dtype in (torch.float16, torch.bfloat16):
        weights = weights.to(output_dtype)
    return weights, ids.reshape(shape), None


def try_normalized_topk(logits, k, normalization_floor):
    """Weights/ids for fp32 logits, or None for metadata the kernel does not cover."""
    tiny, big = float(np.finfo(np.float32).tiny), float(np.finfo(np.float32).max)
    if (not isinstance(logits, torch.Tensor) or not logits.is_cuda
            or logits.dtype != torch.float32 or not logits.is_contiguous()
            or logits.ndim < 1 or not 1 <= logits.shape[-1] <= _MAX_EXPERTS
            or not 1 <= k <= min(_MAX_K, logits.shape[-1])
            or not tiny <= normalization_floor <= big):
        return None
    n = logits.shape[-1]
    weights, ids = _topk(logits.reshape(-1, n), int(k), normalization_floor, True)
    shape = tuple(logits.shape[:-1]) + (int(k),)
    return weights.reshape(shape), ids.reshape(shape)


class RouterInference:
    """Full-softmax-then-top-k router; optional inference-only renormalisation."""

    def __init__(self, d_model, n_experts, k, dtype="float32", *,
                 renormalize_selected=False, normalization_floor=1e-30):
        self.d_model = d_model
        self.n_experts = n_experts
        if not (1 <= int(k) <= int(n_experts)):
            raise ValueError("expert router expects 1 <= k <= n_experts")
        self.k = int(k)
        if not isinstance(renormalize_selected, bool):
            raise TypeError("renormalize_selected must be bool")
        if not math.isfinite(normalization_floor) or normalization_floor <= 0:
            raise ValueError("normalization_floor must be finite and positive")
        self.renormalize_selected = renormalize_selected
        self.normalization_floor = float(normalization_floor)
        self.W_router = None      # [d_model, n_experts], the reference's orientation
        self.b_router = None
        self._rows = None         # (identity of W_router, its [n_experts, d_model] copy for the kernel)

    def route_logits(self, logits):
        """Selection and weights from precomputed logits [B, T, E] (or [T, E])."""
        if self.renormalize_selected:
            floor = max(self.normalization_floor, float(np.finfo(np.float32).tiny))
            decoded = try_normalized_topk(logits.to(torch.float32).contiguous(), self.k, floor)
            if decoded is None:
                raise NotImplementedError("router kernel covers at most 4096 experts and k <= 32")
            return decoded
        weights, ids, _ = expert_topk_forward(logits, self.k, return_cache=False)
        return weights, ids

    def rows_and_bias(self):
        """The router matrix as the kernels read it ([n_experts, d_model] fp32, cached until W_router
        is replaced or written to) and the bias as fp32 (or None)."""
        w = self.W_router
        stamp = (w.data_ptr(), w._version, tuple(w.shape), w.device)
        if self._rows is None or self._rows[0] != stamp:
            self._rows = (stamp, w.to(torch.float32).t().contiguous())
        bias = None if self.b_router is None else self.b_router.to(torch.float32).contiguous()
        return self._rows[1], bias

    def logits(self, x2):
        """fp32 logits [T, n_experts] of rows ``x2`` [T, d_model]."""
        from .moe import router_logits
        rows, bias = self.rows_and_bias()
        return router_logits(x2.to(torch.float32).contiguous(), rows, bias)

    def forward(self, x):
        batch_size, seq_len, _ = x.shape
        logits = self.logits(x.reshape(batch_size * seq_len, self.d_model))
        logits = logits.reshape(batch_size, seq_len, self.n_experts)
        weights, ids = self.route_logits(logits)
        return weights.to(x.dtype), ids
