"""Packed-expert MoE step on the device.

``ExpertsInference`` and ``Qwen3NextMoEInference`` keep the call signatures of the
reference (mini_llm/ops/experts_inference.py:123-171, mini_llm/external/qwen3next_moe.py:129)
but hold an HBM-resident expert *bank* instead of an executor with a cache: all experts of a
layer live in three packed tensors [E, F, D], [E, F, D], [E, D, F]
(mini_llm/external/qwen3next_gguf.py:153-169).  One ABI call runs the router (optional), the
device-side token->expert plan, the grouped expert kernels, the shared expert and the ordered
combine; expert ids never travel to the host.
"""
import ctypes
import math
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib
from .quantized_linear import (
    DevicePackedGGUFWeight, _FORMAT_ID, _TORCH_DTYPE_ID, _ptr, _stream, _upload_bytes, packed_to_device,
)
from .quantized_weight import BLOCK_FORMATS, PackedGGUFWeight
from .router import RouterInference

_NULL = ctypes.c_void_p(0)
# The plan kernel keeps an [experts x tokens] bitmap in LDS; larger batches are split here.
_PLAN_LDS_BYTES = 60 * 1024


class DevicePackedExpertBank:
    """E SwiGLU experts resident in HBM as packed [E,F,D] gate, [E,F,D] up, [E,D,F] down.

    ``gate_up`` may instead be one fused tensor [E, 2F, D] (gate rows then up rows).
    Each argument is a (uint8 CUDA tensor, shape, quant_type) triple or a host
    ``PackedGGUFWeight`` with a three-dimensional shape, which is uploaded once.
    """

    def __init__(self, gate=None, up=None, down=None, *, gate_up=None, device=None):
        if gate_up is not None:
            if gate is not None or up is not None:
                raise ValueError("pass either gate_up or gate and up")
            data, shape, fmt = self._resolve(gate_up, device)
            if shape[1] % 2:
                raise ValueError("fused gate_up must have an even number of rows")
            e, f2, d = shape
            self.gate_data = self.up_data = data
            self.gate_fmt = self.up_fmt = fmt
            row = self._row_bytes(fmt, d)
            self.gate_stride = self.up_stride = f2 * row
            self._up_offset = (f2 // 2) * row
            gshape = ushape = (e, f2 // 2, d)
        else:
            self.gate_data, gshape, self.gate_fmt = self._resolve(gate, device)
            self.up_data, ushape, self.up_fmt = self._resolve(up, device)
            self.gate_stride = gshape[1] * self._row_bytes(self.gate_fmt, gshape[2])
            self.up_stride = ushape[1] * self._row_bytes(self.up_fmt, ushape[2])
            self._up_offset = 0
        self.down_data, dshape, self.down_fmt = self._resolve(down, device)
        if gshape != ushape:
            raise ValueError("gate/up banks must share [E, F, D]")
        e, f, d = gshape
        if dshape != (e, d, f):
            raise ValueError("down bank must be [E, D, F]")
        self.n_experts, self.d_ff, self.d_model = e, f, d
        self.down_stride = d * self._row_bytes(self.down_fmt, f)
        self.device = self.down_data.device

    @staticmethod
    def _row_bytes(fmt, k):
        elems, nbytes = BLOCK_FORMATS[fmt]
        return k // elems * nbytes

    @staticmethod
    def _resolve(item, device):
        if isinstance(item, PackedGGUFWeight):
            if len(item.shape) != 3:
                raise ValueError("expert banks are three-dimensional [E, N, K]")
            if not torch.cuda.is_available():
                raise RuntimeError("Packed GPU weights require a HIP device")
            dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
            return _upload_bytes(item.data, dev), item.shape, item.quant_type
        data, shape, fmt = item
        shape = tuple(int(s) for s in shape)
        if fmt not in BLOCK_FORMATS:
            raise ValueError(f"Unsupported GGUF type {fmt}")
        if not isinstance(data, torch.Tensor) or data.dtype != torch.uint8 or not data.is_cuda or not data.is_contiguous():
            raise TypeError("bank bytes must be a contiguous CUDA torch.uint8 tensor")
        elems, nbytes = BLOCK_FORMATS[fmt]
        if len(shape) != 3 or min(shape) <= 0 or shape[-1] % elems or data.numel() != math.prod(shape) // elems * nbytes:
            raise ValueError("Invalid packed bank shape, byte length or K block alignment")
        return data, shape, fmt

    @property
    def nbytes(self):
        total = self.gate_data.numel() + self.down_data.numel()
        if self.up_data is not self.gate_data:
            total += self.up_data.numel()
        return int(total)

    @property
    def expert_nbytes(self):
        return self.nbytes // self.n_experts

    def expert(self, index):
        """Views of one expert as three DevicePackedGGUFWeight matrices."""
        if not 0 <= int(index) < self.n_experts:
            raise IndexError(index)
        i = int(index)
        grow = self._row_bytes(self.gate_fmt, self.d_model) * self.d_ff
        urow = self._row_bytes(self.up_fmt, self.d_model) * self.d_ff
        g0 = i * self.gate_stride
        u0 = i * self.up_stride + self._up_offset
        d0 = i * self.down_stride
        return (DevicePackedGGUFWeight(self.gate_data[g0:g0 + grow], (self.d_ff, self.d_model), self.gate_fmt),
                DevicePackedGGUFWeight(self.up_data[u0:u0 + urow], (self.d_ff, self.d_model), self.up_fmt),
                DevicePackedGGUFWeight(self.down_data[d0:d0 + self.down_stride], (self.d_model, self.d_ff), self.down_fmt))

    def fill(self, c_bank):
        c_bank.gate = self.gate_data.data_ptr()
        c_bank.up = self.up_data.data_ptr() + self._up_offset
        c_bank.down = self.down_data.data_ptr()
        c_bank.gate_stride, c_bank.up_stride, c_bank.down_stride = self.gate_stride, self.up_stride, self.down_stride
        c_bank.gate_fmt = _FORMAT_ID[self.gate_fmt]
        c_bank.up_fmt = _FORMAT_ID[self.up_fmt]
        c_bank.down_fmt = _FORMAT_ID[self.down_fmt]
        c_bank.n_experts, c_bank.d_model, c_bank.d_ff = self.n_experts, self.d_model, self.d_ff


def _max_tokens_per_call(n_experts):
    words = max(1, _PLAN_LDS_BYTES // 4 // n_experts - 1)
    return words * 32


def norm_router(x, gamma, eps, router_weight, router_bias=None):
    """RMSNorm of fp32 ``x`` [T, D] followed by the router's logits, in one launch.

    Returns ``(normalized [T, D], logits [T, E])``: ``normalized = (x * inv_rms) * gamma`` as
    RMSNormInference.forward computes it (mini_llm/ops/rmsnorm_inference.py:109-118) and
    ``logits = normalized @ router_weight.T (+ bias)`` (mini_llm/ops/router_inference.py:40-46);
    ``router_weight`` is fp32 [E, D], the orientation of the checkpoint's ``ffn_gate_inp``.
    """
    for name, tensor in (("x", x), ("gamma", gamma), ("router_weight", router_weight)):
        if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda or tensor.dtype != torch.float32 or not tensor.is_contiguous():
            raise TypeError(f"{name} must be a contiguous CUDA float32 tensor")
    if x.ndim != 2 or gamma.shape != (x.shape[1],) or router_weight.ndim != 2 or router_weight.shape[1] != x.shape[1]:
        raise ValueError("x [T, D], gamma [D] and router_weight [E, D] do not fit together")
    t, d = x.shape
    e = router_weight.shape[0]
    if router_bias is not None and (router_bias.dtype != torch.float32 or tuple(router_bias.shape) != (e,) or not router_bias.is_cuda):
        raise ValueError("router_bias must be CUDA float32 [E]")
    normalized = torch.empty_like(x)
    logits = torch.empty((t, e), dtype=torch.float32, device=x.device)
    if t:
        with torch.cuda.device(x.device):
            rc = _lib.load().qmoe_norm_router(_ptr(x), t, d, _ptr(gamma), float(eps), _ptr(router_weight),
                                              _ptr(router_bias) if router_bias is not None else _NULL, e,
                                              _ptr(normalized), _ptr(logits), _stream())
        _lib.check(rc, "RMSNorm + router logits")
    return normalized, logits


def router_logits(x, router_weight, router_bias=None):
    """``x @ router_weight.T (+ bias)`` for fp32 ``x`` [T, D] and ``router_weight`` [E, D], on the
    library's router kernel (RouterInference.forward, mini_llm/ops/router_inference.py:40-46)."""
    for name, tensor in (("x", x), ("router_weight", router_weight)):
        if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda or tensor.dtype != torch.float32 or not tensor.is_contiguous():
            raise TypeError(f"{name} must be a contiguous CUDA float32 tensor")
    if x.ndim != 2 or router_weight.ndim != 2 or router_weight.shape[1] != x.shape[1] or router_weight.device != x.device:
        raise ValueError("x [T, D] and router_weight [E, D] do not fit together")
    t, d = x.shape
    e = router_weight.shape[0]
    if router_bias is not None and (router_bias.dtype != torch.float32 or tuple(router_bias.shape) != (e,) or router_bias.device != x.device):
        raise ValueError("router_bias must be CUDA float32 [E]")
    if d % 4 or x.data_ptr() % 16 or router_weight.data_ptr() % 16:
        # outside what the kernel reads with 16-byte loads: the plain fp32 product, as the reference computes it
        out = x @ router_weight.t()
        return out if router_bias is None else out + router_bias
    logits = torch.empty((t, e), dtype=torch.float32, device=x.device)
    if t:
        with torch.cuda.device(x.device):
            rc = _lib.load().qmoe_router_logits(_ptr(x), t, d, _ptr(router_weight),
                                                _ptr(router_bias) if router_bias is not None else _NULL, e,
                                                _ptr(logits), _stream())
        _lib.check(rc, "router logits")
    return logits


def moe_step(hidden, bank, top_k, *, logits=None, weights=None, ids=None, shared=None,
             shared_gate=None, floor=2.0 ** -14, renormalize=True, out_dtype=None,
             return_routing=False, residual=None, check_routing=False):
    """One MoE step over hidden [T, D]: routed experts (+ shared expert) -> [T, D].

    Routing comes from fp32 ``logits`` [T, E] (softmax/top-k on the device) or from
    precomputed ``weights`` fp32 / ``ids`` int64 [T, k].  ``shared`` is an optional
    (gate, up, down) triple of DevicePackedGGUFWeight; ``shared_gate`` an optional fp32 [D]
    admission vector (sigmoid gate).  Accumulation is fp32; the output is rounded once to
    ``out_dtype`` (default: hidden's dtype).  ``residual`` (optional fp32 [T, D]) is added to the
    block's output in the same kernels: ``residual + (routed + shared * sigmoid)``.

    Precomputed ``ids`` outside ``[0, n_experts)``, or an expert repeated within one token, contribute
    nothing (of a repeated expert the first slot counts).  With ``check_routing`` the step's status
    word is read back afterwards (one synchronisation) and such ids raise ``ValueError``, where the
    reference hands them to its general dispatcher (mini_llm/ops/device_expert_plan.py:183-186).
    """
    if not isinstance(hidden, torch.Tensor) or not hidden.is_cuda or hidden.dtype not in _TORCH_DTYPE_ID:
        raise TypeError("MoE hidden must be a CUDA FP16/BF16/FP32 tensor")
    if hidden.ndim != 2 or hidden.shape[1] != bank.d_model or not hidden.is_contiguous():
        raise ValueError("hidden must be contiguous [tokens, d_model]")
    t = hidden.shape[0]
    out_dtype = hidden.dtype if out_dtype is None else out_dtype
    out = torch.empty((t, bank.d_model), dtype=out_dtype, device=hidden.device)
    if logits is not None:
        if logits.dtype != torch.float32 or tuple(logits.shape) != (t, bank.n_experts) or not logits.is_contiguous():
            raise ValueError("router logits must be contiguous FP32 [tokens, n_experts]")
    else:
        if weights is None or ids is None:
            raise ValueError("need router logits or weights and ids")
        if (weights.dtype != torch.float32 or ids.dtype != torch.int64
                or tuple(weights.shape) != (t, top_k) or tuple(ids.shape) != (t, top_k)
                or not weights.is_contiguous() or not ids.is_contiguous()):
            raise ValueError("routing weights / ids must be contiguous FP32 / int64 [tokens, k]")
    if residual is not None and (not isinstance(residual, torch.Tensor) or residual.dtype != torch.float32 or not residual.is_cuda
                                 or tuple(residual.shape) != (t, bank.d_model) or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous CUDA FP32 [tokens, d_model]")
    out_w = torch.empty((t, top_k), dtype=torch.float32, device=hidden.device) if return_routing else None
    out_i = torch.empty((t, top_k), dtype=torch.int64, device=hidden.device) if return_routing else None
    if t == 0:
        return (out, out_w, out_i) if return_routing else out
    lib = _lib.load()
    f_shared = shared[0].shape[0] if shared is not None else 0
    step = min(t, _max_tokens_per_call(bank.n_experts))
    nbytes = lib.qmoe_moe_workspace_bytes(step, top_k, bank.n_experts, bank.d_model, bank.d_ff, f_shared)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=hidden.device)
    status = torch.zeros(1, dtype=torch.int32, device=hidden.device) if check_routing else None
    with torch.cuda.device(hidden.device):
        for lo in range(0, t, step):
            hi = min(t, lo + step)
            args = _lib.MoeArgs()
            args.hidden, args.hidden_dtype = hidden[lo:hi].data_ptr(), _TORCH_DTYPE_ID[hidden.dtype]
            args.tokens, args.top_k = hi - lo, top_k
            args.floor_value, args.renormalize = float(floor), int(bool(renormalize))
            if logits is not None:
                args.logits = logits[lo:hi].data_ptr()
            else:
                args.in_weights, args.in_ids = weights[lo:hi].data_ptr(), ids[lo:hi].data_ptr()
            bank.fill(args.bank)
            if shared is not None:
                g, u, d = shared
                args.shared_gate_w, args.shared_up_w, args.shared_down_w = (
                    g.data.data_ptr(), u.data.data_ptr(), d.data.data_ptr())
                args.shared_gate_fmt = _FORMAT_ID[g.quant_type]
                args.shared_up_fmt = _FORMAT_ID[u.quant_type]
                args.shared_down_fmt = _FORMAT_ID[d.quant_type]
                args.d_ff_shared = f_shared
                if shared_gate is not None:
                    args.shared_gate = shared_gate.data_ptr()
            args.out, args.out_dtype = out[lo:hi].data_ptr(), _TORCH_DTYPE_ID[out_dtype]
            if residual is not None:
                args.residual = residual[lo:hi].data_ptr()
            if return_routing:
                args.out_weights, args.out_ids = out_w[lo:hi].data_ptr(), out_i[lo:hi].data_ptr()
            if status is not None:
                args.status_out = status.data_ptr()
            rc = lib.qmoe_moe_forward(ctypes.byref(args), _ptr(workspace), nbytes, _stream())
            _lib.check(rc, "Packed MoE step")
    if status is not None:
        bits = int(status.item())
        if bits:
            what = [name for bit, name in ((1, "expert ids outside the bank"), (2, "an expert repeated within a token")) if bits & bit]
            raise ValueError("Invalid routing: " + " and ".join(what))
    return (out, out_w, out_i) if return_routing else out


class ExpertsInference:
    """Sparse expert dispatch + ordered weighted combine.

    ``expert_executor`` is either a resident ``DevicePackedExpertBank`` (the layer's experts) or an
    executor with the hooks of the reference's (mini_llm/ops/experts_inference.py:188-197:
    ``try_forward_device_plan`` for one token; this package's executor also offers
    ``try_forward_batch`` for more), e.g. ``expert_executor.ResidentExpertExecutor``.
    """

    def __init__(self, d_model, d_ff, n_experts, dtype="float32", *, expert_executor=None, layer_id=0):
        self.d_model, self.d_ff, self.n_experts = d_model, d_ff, n_experts
        self.layer_id = int(layer_id)
        self.bank = self.expert_executor = None
        if isinstance(expert_executor, DevicePackedExpertBank):
            self.set_bank(expert_executor)
        elif expert_executor is not None:
            if (expert_executor.d_model, expert_executor.d_ff) != (d_model, d_ff):
                raise ValueError("Executor dimensions do not match MoE tensors")
            self.expert_executor = expert_executor

    def set_bank(self, bank):
        if (bank.d_model, bank.d_ff, bank.n_experts) != (self.d_model, self.d_ff, self.n_experts):
            raise ValueError("Executor dimensions do not match MoE tensors")
        self.bank = bank

    def forward(self, x, weights, expert_indices, *, on_cpu_submitted=None):
        """y[tok] = sum over its experts, ascending id, of w * expert(x[tok]); x is [B, T, D]."""
        batch_size, seq_len, d_model = x.shape
        k = weights.shape[-1]
        n = batch_size * seq_len
        flat = x.reshape(n, d_model).contiguous()
        if self.expert_executor is not None:
            ex = self.expert_executor
            y = None
            if n == 1 and getattr(ex, "try_forward_device_plan", None) is not None:
                args = (self.layer_id, flat, weights.reshape(-1), expert_indices.reshape(-1), self.n_experts)
                y = (ex.try_forward_device_plan(*args, on_cpu_submitted=on_cpu_submitted) if on_cpu_submitted is not None
                     else ex.try_forward_device_plan(*args))
                if y is not None:
                    return y.reshape(batch_size, seq_len, d_model)
            batch = getattr(ex, "try_forward_batch", None)
            if batch is None:
                raise RuntimeError("the expert executor offers neither try_forward_device_plan for this call nor try_forward_batch")
            with ex.dispatch_scope(self.layer_id, ()):
                y = batch(self.layer_id, flat, weights.reshape(n, k), expert_indices.reshape(n, k))
            if on_cpu_submitted is not None:
                on_cpu_submitted()
            return y.reshape(batch_size, seq_len, d_model)
        if self.bank is None:
            raise RuntimeError("ExpertsInference has no resident expert bank")
        y = moe_step(flat, self.bank, k,
                     weights=weights.reshape(n, k).to(torch.float32).contiguous(),
                     ids=expert_indices.reshape(n, k).to(torch.int64).contiguous())
        if on_cpu_submitted is not None:
            on_cpu_submitted()
        return y.reshape(batch_size, seq_len, d_model)


@dataclass(frozen=True)
class Qwen3NextMoESpec:
    """Sizes of one Qwen3-Next MoE block, validated against the checkpoint's headers
    (mini_llm/external/qwen3next_moe.py:21-90); no payload is touched."""
    d_model: int
    d_ff: int
    shared_d_ff: int
    n_experts: int
    top_k: int

    @classmethod
    def from_index(cls, index, layer_id):
        from .qwen3next_gguf import check_moe_block
        return cls(*check_moe_block(index, layer_id))


class Qwen3NextMoEInference:
    """Renormalised routed SwiGLU experts plus a sigmoid-gated shared SwiGLU expert."""

    def __init__(self, bank, top_k, router_weight, shared, shared_gate, *, normalization_floor=2.0 ** -14):
        """router_weight: fp32 [E, D] (GGUF ffn_gate_inp orientation); shared: (gate, up, down)
        DevicePackedGGUFWeight triple, or three dense fp32 [out, in] tensors (checkpoints that keep
        the shared expert in F32 / F16); shared_gate: fp32 [D]."""
        self.bank = bank
        self.top_k = int(top_k)
        self.router = RouterInference(bank.d_model, bank.n_experts, self.top_k,
                                      renormalize_selected=True, normalization_floor=normalization_floor)
        self._router_weight = router_weight.to(torch.float32).contiguous()  # [E, D], as stored
        self.router.W_router = self._router_weight.t().contiguous()
        self.router.b_router = torch.zeros(bank.n_experts, dtype=torch.float32, device=router_weight.device)
        self.shared_is_dense = all(isinstance(w, torch.Tensor) for w in shared)
        if not self.shared_is_dense and not all(isinstance(w, DevicePackedGGUFWeight) for w in shared):
            raise TypeError('shared expert: three DevicePackedGGUFWeight or three dense tensors')
        self.shared = tuple(w.to(torch.float32).contiguous() for w in shared) if self.shared_is_dense else shared
        self.shared_gate = shared_gate.to(torch.float32).contiguous()
        self.experts = ExpertsInference(bank.d_model, bank.d_ff, bank.n_experts, expert_executor=bank)

    @classmethod
    def from_index(cls, index, layer_id, *, expert_executor=None, device=None):
        """Build the block of ``layer_id`` from a ``Qwen3NextGGUFIndex``
        (mini_llm/external/qwen3next_moe.py:100-127).  ``expert_executor`` may be a resident
        ``DevicePackedExpertBank`` the caller already holds for this layer or an executor that
        holds it (``ResidentExpertExecutor``); otherwise the layer's routed tensors are uploaded."""
        spec = Qwen3NextMoESpec.from_index(index, layer_id)
        if not torch.cuda.is_available():
            raise RuntimeError('Packed GPU weights require a HIP device')
        dev = torch.device('cuda', torch.cuda.current_device()) if device is None else torch.device(device)
        if expert_executor is None:
            bank = index.expert_bank(layer_id, dev)
        elif isinstance(expert_executor, DevicePackedExpertBank):
            bank = expert_executor
        else:  # an executor holding this layer's bank (expert_executor.ResidentExpertExecutor)
            if getattr(expert_executor, 'compute_dtype', 'float32') != 'float32':
                raise ValueError('Qwen3-Next adapter requires float32 expert compute')
            bank = expert_executor.bank(layer_id)
        if (bank.d_model, bank.d_ff) != (spec.d_model, spec.d_ff) or bank.n_experts != spec.n_experts:
            raise ValueError('Executor dimensions do not match MoE tensors')
        stem = f'blk.{layer_id}.'

        def dense(name):
            return torch.from_numpy(np.ascontiguousarray(index.non_expert_weight(stem + name), dtype=np.float32)).to(dev)

        host = [index.projection(stem + name) for name in ('ffn_gate_shexp.weight', 'ffn_up_shexp.weight', 'ffn_down_shexp.weight')]
        if all(isinstance(w, PackedGGUFWeight) for w in host):
            shared = tuple(packed_to_device(w, dev) for w in host)
        else:  # any F32 / F16 projection: the shared expert runs as dense fp32 matmuls
            shared = tuple(torch.from_numpy(np.ascontiguousarray(
                w.dequantize_reference() if isinstance(w, PackedGGUFWeight) else w, dtype=np.float32)).to(dev) for w in host)
        result = cls(bank, spec.top_k, dense('ffn_gate_inp.weight'), shared, dense('ffn_gate_inp_shexp.weight'))
        result.index, result.layer_id, result.spec = index, layer_id, spec
        return result

    def forward_after_norm(self, residual, gamma, eps):
        """``residual + forward(rmsnorm(residual))``: the second half of a decoder layer
        (mini_llm/external/qwen3next_decoder.py:120) with the norm and the router's logits in one
        launch in front of the block and the residual add inside its last kernels."""
        if not isinstance(residual, torch.Tensor) or residual.dtype != torch.float32:
            raise TypeError('Qwen3-Next MoE requires backend float32 hidden')
        if residual.ndim != 3 or residual.shape[0] < 1 or residual.shape[-1] != self.bank.d_model:
            raise ValueError('hidden must have shape [positive batch,time,d_model]')
        if not residual.shape[1]:
            return residual.clone()
        rows, bias = self.router.rows_and_bias()   # (whatever the router holds now, bias included)
        if self.shared_is_dense:
            normalized, _ = norm_router(residual.reshape(-1, residual.shape[-1]).contiguous(), gamma, eps, rows, bias)
            return residual + self.forward(normalized.reshape(residual.shape))
        b, t, d = residual.shape
        flat = residual.reshape(b * t, d).contiguous()
        normalized, logits = norm_router(flat, gamma, eps, rows, bias)
        out = moe_step(normalized, self.bank, self.top_k, logits=logits, shared=self.shared, shared_gate=self.shared_gate,
                       floor=self.router.normalization_floor, residual=flat)
        return out.reshape(b, t, d)

    def forward(self, hidden):
        if not isinstance(hidden, torch.Tensor) or hidden.dtype != torch.float32:
            raise TypeError('Qwen3-Next MoE requires backend float32 hidden')
        if hidden.ndim != 3 or hidden.shape[0] < 1 or hidden.shape[-1] != self.bank.d_model:
            raise ValueError('hidden must have shape [positive batch,time,d_model]')
        if not hidden.shape[1]:
            return torch.empty_like(hidden)
        b, t, d = hidden.shape
        flat = hidden.reshape(b * t, d).contiguous()
        logits = self.router.logits(flat)
        if self.shared_is_dense:
            # routed part on the packed kernels; shared expert and its admission gate as fp32
            # matmuls (mini_llm/external/gguf_projection.py:40-88, qwen3next_moe.py:145-147)
            routed = moe_step(flat, self.bank, self.top_k, logits=logits, floor=self.router.normalization_floor)
            gate_w, up_w, down_w = self.shared
            g = flat @ gate_w.t()
            act = (g * (1.0 / (1.0 + torch.exp(-g)))) * (flat @ up_w.t())
            sig = torch.exp(-torch.logaddexp(torch.zeros((), device=flat.device), -(flat @ self.shared_gate)))
            out = routed + (act @ down_w.t()) * sig[:, None]
        else:
            out = moe_step(flat, self.bank, self.top_k, logits=logits, shared=self.shared,
                           shared_gate=self.shared_gate, floor=self.router.normalization_floor)
        return out.reshape(b, t, d)
