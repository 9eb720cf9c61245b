"""Token -> expert plan built on the device.

The surface of ``RoutingPlan`` (mini_llm/ops/routing_plan.py:15-138): the T*k assignments of a
router's top-k output grouped by expert id, ascending token inside an expert, with
``get_expert_assignments`` / ``active_expert_ids`` / ``get_assignment_count`` for dispatch loops.
The grouping itself is ``qmoe_routing_plan`` -- the same kernel that ``qmoe_moe_forward`` runs in
front of its expert kernels -- so what a caller inspects here is the plan the MoE step executes.
Like the reference, only the E+1 offsets travel to the host (once, when the plan is made).
"""
import torch

from . import _lib
from .quantized_linear import _ptr, _stream


class RoutingPlan:
    """Sorted assignment arrays (device tensors) plus host-side offsets and sizes."""

    def __init__(self, token_indices, slot_indices, expert_indices, weights, order, expert_offsets, n_experts, k, N):
        self.token_indices, self.slot_indices, self.expert_indices = token_indices, slot_indices, expert_indices
        self.weights, self.order = weights, order
        self.expert_offsets = tuple(int(v) for v in expert_offsets)
        self.expert_sizes = tuple(b - a for a, b in zip(self.expert_offsets, self.expert_offsets[1:]))
        self.n_experts, self.k, self.N = int(n_experts), int(k), int(N)
        self._active_experts = tuple(e for e, size in enumerate(self.expert_sizes) if size)

    @classmethod
    def from_router_outputs(cls, expert_indices, weights, k, n_experts=None):
        """``expert_indices`` int64 and ``weights`` fp32, both [B, T, k] CUDA tensors."""
        for name, tensor, dtype in (("expert_indices", expert_indices, torch.int64), ("weights", weights, torch.float32)):
            if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda or tensor.dtype != dtype:
                raise TypeError(f"{name} must be a CUDA {dtype} tensor")
        if expert_indices.ndim != 3 or expert_indices.shape[-1] != int(k) or weights.shape != expert_indices.shape:
            raise ValueError("expert_indices and weights must both be [batch, time, k]")
        if n_experts is None:   # the reference's compatibility fallback: one host synchronisation
            n_experts = int(expert_indices.max().item()) + 1
        k, n_experts = int(k), int(n_experts)
        tokens = expert_indices.shape[0] * expert_indices.shape[1]
        total = tokens * k
        device = expert_indices.device
        ids, w = expert_indices.contiguous(), weights.contiguous()
        ints = lambda n: torch.empty(n, dtype=torch.int32, device=device)
        offsets, active, n_active, status = ints(n_experts + 1), ints(n_experts), ints(1), ints(1)
        order, sorted_token, pos_of = ints(total), ints(total), ints(total)
        sorted_weight = torch.empty(total, dtype=torch.float32, device=device)
        with torch.cuda.device(device):
            rc = _lib.load().qmoe_routing_plan(_ptr(ids), _ptr(w), tokens, k, n_experts, _ptr(offsets), _ptr(active),
                                               _ptr(n_active), _ptr(order), _ptr(sorted_token), _ptr(sorted_weight),
                                               _ptr(pos_of), _ptr(status), _stream())
        _lib.check(rc, "Routing plan")
        host = torch.cat([offsets, status]).cpu().tolist()     # the one small transfer
        if host[-1]:
            raise ValueError("Invalid routing: expert ids outside the bank or an expert repeated within a token")
        order = order.to(torch.int64)
        plan = cls(sorted_token.to(torch.int64), order % k, ids.reshape(-1)[order], sorted_weight, order,
                   host[:-1], n_experts, k, tokens)
        plan.position_of_assignment = pos_of.reshape(tokens, k)
        return plan

    def active_expert_ids(self):
        return self._active_experts

    def get_expert_assignments(self, expert_idx):
        """(token ids, top-k slot ids, routing weights) of one expert."""
        start, end = self.expert_offsets[expert_idx], self.expert_offsets[expert_idx + 1]
        return self.token_indices[start:end], self.slot_indices[start:end], self.weights[start:end]

    def get_assignment_count(self, expert_idx):
        return self.expert_sizes[expert_idx]


def create_routing_plan(expert_indices, weights, k, n_experts):
    return RoutingPlan.from_router_outputs(expert_indices, weights, k, n_experts)
