"""Token -> expert plan built on the device.

The surface of ``RoutingPlan`` (mini_llm/ops/routing_plan.py:15-138): the T*k assignments of a
router's top-k output grouped by expert id, ascending token inside an expert, with
``get_expert_assignments`` / ``active_expert_ids`` / ``get_assignment_count`` for dispatch loops.
The grouping itself is ``qmoe_routing_plan`` -- the same kernel that ``qmoe_moe_forward`` runs in
front of its expert kernels -- so what a caller inspects here is the plan the MoE step executes.
Like the reference, only the E+1 offsets travel to the host (once, when the plan is made).
One kernel call covers ``max_tokens_per_plan_call`` tokens (928 at 512 experts); longer batches
are planned in token chunks and the chunk plans are joined on the device.
"""
import torch

from . import _lib
from .quantized_linear import _ptr, _stream

# The plan kernel is one workgroup with an [experts x tokens] bitmap in LDS (60 KiB): one call
# covers this many tokens, longer batches are planned in token chunks and merged.
_PLAN_LDS_BYTES = 60 * 1024


_CHUNK_TOKENS = 512   # tokens per call once a batch has to be cut (the size of a prefill step's plan)


def max_tokens_per_plan_call(n_experts):
    words = max(1, _PLAN_LDS_BYTES // 4 // int(n_experts) - 1)
    return words * 32


def _device_plan_call(ids, w, k, n_experts):
    """One qmoe_routing_plan call over ``ids`` / ``w`` [tokens, k] (contiguous device tensors).
    Returns int32 device tensors (offsets [E+1], order, sorted_token, pos_of [tokens*k], status [1])
    and the fp32 sorted weights; nothing is read back."""
    tokens = ids.shape[0]
    total = tokens * k
    device = ids.device
    ints = lambda n: torch.empty(n, dtype=torch.int32, device=device)
    offsets, active, n_active, status = ints(n_experts + 1), ints(n_experts), ints(1), ints(1)
    order, sorted_token, pos_of = ints(total), ints(total), ints(total)
    sorted_weight = torch.empty(total, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        rc = _lib.load().qmoe_routing_plan(_ptr(ids), _ptr(w), tokens, k, n_experts, _ptr(offsets), _ptr(active),
                                           _ptr(n_active), _ptr(order), _ptr(sorted_token), _ptr(sorted_weight),
                                           _ptr(pos_of), _ptr(status), _stream())
    _lib.check(rc, "Routing plan")
    return offsets, order, sorted_token, sorted_weight, pos_of, status


def _merge_chunk_plans(chunks, ids, k, n_experts):
    """Plans of consecutive token chunks joined into the plan of the whole batch.

    ``chunks`` is a list of ``(first_token, plan)`` with ``plan`` as ``_device_plan_call`` returns it;
    ``ids`` is the whole batch [tokens, k].  An expert's assignments are its assignments of chunk 0,
    then of chunk 1, ...: tokens stay ascending inside an expert, as one stable sort would leave
    them.  Index arithmetic on the plans' device arrays only; nothing is read back."""
    total = ids.shape[0] * k
    device = ids.device
    counts = torch.stack([(plan[0][1:] - plan[0][:-1]).to(torch.int64) for _, plan in chunks])      # [chunks, E]
    zero = torch.zeros(1, dtype=torch.int64, device=device)
    starts = torch.cat([zero, counts.sum(0).cumsum(0)])                                              # [E + 1]
    earlier = counts.cumsum(0) - counts            # an expert's assignments in the chunks before this one
    order = torch.empty(total, dtype=torch.int64, device=device)
    token = torch.empty(total, dtype=torch.int64, device=device)
    weight = torch.empty(total, dtype=torch.float32, device=device)
    pos_of = torch.empty(total, dtype=torch.int64, device=device)
    status = torch.zeros(1, dtype=torch.int32, device=device)
    flat = ids.reshape(-1)
    for index, (first_token, (off_c, order_c, token_c, weight_c, pos_c, status_c)) in enumerate(chunks):
        n = order_c.numel()
        lo = first_token * k
        # (invalid routing leaves the chunk's plan flagged and partly unwritten: every look-up below
        # is kept in range, the flag decides afterwards)
        order_c = order_c.to(torch.int64).clamp(0, n - 1)
        expert = flat[lo:lo + n][order_c].clamp(0, n_experts - 1)
        place = (starts[expert] + earlier[index][expert]
                 + (torch.arange(n, dtype=torch.int64, device=device) - off_c.to(torch.int64)[expert]))
        place = place.clamp(0, total - 1)
        order[place] = order_c + lo
        token[place] = token_c.to(torch.int64) + first_token
        weight[place] = weight_c
        pos_of[lo:lo + n] = place[pos_c.to(torch.int64).clamp(0, n - 1)]
        status |= status_c
    return starts, order, token, weight, pos_of, status


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
        return cls._build(expert_indices, weights, int(k), int(n_experts), _device_plan_call)

    @classmethod
    def _build(cls, expert_indices, weights, k, n_experts, plan_call):
        tokens = expert_indices.shape[0] * expert_indices.shape[1]
        ids, w = expert_indices.contiguous().reshape(tokens, k), weights.contiguous().reshape(tokens, k)
        limit = max_tokens_per_plan_call(n_experts)
        step = min(limit, _CHUNK_TOKENS)
        if tokens <= limit:
            offsets, order, sorted_token, sorted_weight, pos_of, status = plan_call(ids, w, k, n_experts)
            order, sorted_token = order.to(torch.int64), sorted_token.to(torch.int64)
        else:   # token chunks of the size one call covers, joined on the device
            chunks = [(lo, plan_call(ids[lo:lo + step], w[lo:lo + step], k, n_experts)) for lo in range(0, tokens, step)]
            offsets, order, sorted_token, sorted_weight, pos_of, status = _merge_chunk_plans(chunks, ids, k, n_experts)
        host = torch.cat([offsets.to(torch.int64), status.to(torch.int64)]).cpu().tolist()     # the one small transfer
        if host[-1]:
            raise ValueError("Invalid routing: expert ids outside the bank or an expert repeated within a token")
        plan = cls(sorted_token, order % k, ids.reshape(-1)[order], sorted_weight, order, host[:-1], n_experts, k, tokens)
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
