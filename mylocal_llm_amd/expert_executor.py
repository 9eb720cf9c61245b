"""An expert executor whose experts are all resident in HBM.

The reference's ``ExpertsInference`` (mini_llm/ops/experts_inference.py:160-312) talks to a
``HeterogeneousExpertExecutor`` (mini_llm/ops/expert_residency.py:797-819) through a small set of
hooks: ``try_forward_device_plan`` for one token (:1025-1030), ``dispatch_scope`` around a layer's
launches (:539-560), ``try_forward_grouped`` for the singleton decode plan (:1166-1193),
``try_forward_decode_batch`` for the same plan inside a dispatch scope (:1032-1068) and
``forward(layer, expert, x)`` for one expert.  That executor exists to juggle a device cache, host
copies and CPU workers for a model that does not fit the GPU.  On a part with 288 GB of HBM every
expert of every layer stays on the device, so this executor keeps one ``DevicePackedExpertBank``
per layer and answers the same hooks from it: nothing is ever evicted, no request is declined for
residency, there is no CPU side to overlap with.
"""
from collections import Counter
from contextlib import contextmanager

import torch

from .moe import DevicePackedExpertBank, moe_step
from .quantized_linear import PackedExpertFFNInference


class ResidentExpertExecutor:
    """All routed experts of the registered layers, resident; same hooks as the reference's executor."""

    compute_dtype = "float32"
    overlaps_cpu_gpu = False          # no CPU workers: submit / resolve are synchronous
    device_expert_plan = True
    routing_profiler = None

    def __init__(self, d_model, d_ff, *, model_id="model"):
        self.d_model, self.d_ff, self.model_id = int(d_model), int(d_ff), model_id
        self.banks = {}
        self.counters = Counter()
        self._dispatch_depth = 0
        self._closed = False

    # ---- residency -------------------------------------------------------------------------------
    def register_layer(self, layer_id, bank):
        if not isinstance(bank, DevicePackedExpertBank):
            raise TypeError("a layer's experts are registered as one DevicePackedExpertBank")
        if (bank.d_model, bank.d_ff) != (self.d_model, self.d_ff):
            raise ValueError("Executor dimensions do not match MoE tensors")
        self.banks[int(layer_id)] = bank

    @classmethod
    def from_index(cls, index, layers=None, *, device=None, model_id=None):
        """Upload the routed banks of ``layers`` (default: all) of a ``Qwen3NextGGUFIndex``."""
        result = cls(index.d_model, index.d_ff, model_id=model_id or index.source_path or "gguf")
        for layer_id in (range(index.layers) if layers is None else layers):
            result.register_layer(layer_id, index.expert_bank(layer_id, device))
        return result

    def bank(self, layer_id):
        try:
            return self.banks[int(layer_id)]
        except KeyError:
            raise KeyError(f"layer {layer_id} has no resident expert bank") from None

    @property
    def resident_bytes(self):
        return sum(b.nbytes for b in self.banks.values())

    @contextmanager
    def dispatch_scope(self, layer_id, expert_ids):
        """The reference protects the selected experts from eviction here; resident banks need none."""
        self.bank(layer_id)
        self._dispatch_depth += 1
        try:
            yield
        finally:
            self._dispatch_depth -= 1

    # ---- execution -------------------------------------------------------------------------------
    def forward(self, layer_id, expert_id, x):
        """One expert's SwiGLU FFN on rows ``x`` [N, D]."""
        gate, up, down = self.bank(layer_id).expert(expert_id)
        self.counters["gpu_experts"] += 1
        return PackedExpertFFNInference(gate, up, down).forward(x)

    def submit(self, layer_id, expert_id, x):
        return self.forward(layer_id, expert_id, x)

    @staticmethod
    def resolve(work):
        return work

    def try_forward_device_plan(self, layer_id, x, weights, indices, n_experts, *, on_cpu_submitted=None, gpu_branch=None):
        """One token: routing weights [k] and expert ids [k] stay on the device; the step is the
        decode launches of the MoE path.  Never declines for a registered layer."""
        bank = self.bank(layer_id)
        if n_experts != bank.n_experts or x.shape[0] != 1:
            return None
        k = weights.numel()
        out = moe_step(x.contiguous(), bank, k, weights=weights.reshape(1, k).to(torch.float32).contiguous(),
                       ids=indices.reshape(1, k).to(torch.int64).contiguous())
        self.counters["device_plan_dispatches"] += 1
        if on_cpu_submitted is not None:
            on_cpu_submitted()
        return out

    def try_forward_batch(self, layer_id, x, weights, indices):
        """Any number of tokens: x [N, D], weights / ids [N, k]; one MoE step (no counterpart in the
        reference, whose executor is asked expert by expert for N > 1)."""
        bank = self.bank(layer_id)
        k = weights.shape[-1]
        self.counters["batch_dispatches"] += 1
        return moe_step(x.contiguous(), bank, k, weights=weights.to(torch.float32).contiguous(),
                        ids=indices.to(torch.int64).contiguous())

    def try_forward_grouped(self, layer_id, expert_ids, x, routing_weights, slots):
        """Singleton decode plan: ascending ``expert_ids`` with their routing ``slots``."""
        from .grouped_quantized_experts import grouped_quantized_experts_forward, supports_grouped_quantized_experts
        if x.shape[0] != 1 or not len(expert_ids):
            return None
        bank = self.bank(layer_id)
        experts = [PackedExpertFFNInference(*bank.expert(e)) for e in expert_ids]
        if not supports_grouped_quantized_experts(x, experts, routing_weights, routing_slots=slots):
            return None
        self.counters["gpu_experts"] += len(experts)
        self.counters["grouped_gpu_dispatches"] += 1
        return grouped_quantized_experts_forward(x, experts, routing_weights, routing_slots=slots)

    def try_forward_decode_batch(self, layer_id, expert_ids, x, routing_weights, slots, *, on_cpu_submitted=None):
        """Singleton decode inside a dispatch scope: unique ascending ``expert_ids`` share one fp32
        activation (mini_llm/ops/expert_residency.py:1032-1068).  The reference shares that
        activation across CPU misses and takes the grouped device path when every expert is already
        admitted; here every expert always is, so the call is that grouped path.  Declines (None) what
        the reference declines: outside a dispatch scope, another shape or dtype, ids that are not
        unique and ascending."""
        if (not self._dispatch_depth or tuple(x.shape) != (1, self.d_model) or x.dtype != torch.float32
                or routing_weights.dtype != torch.float32):
            return None
        expert_ids = tuple(int(e) for e in expert_ids)
        if not expert_ids or expert_ids != tuple(sorted(set(expert_ids))):
            return None
        output = self.try_forward_grouped(layer_id, expert_ids, x, routing_weights, tuple(slots))
        if output is None:
            return None
        self.counters["admission_grouped_dispatches"] += 1
        if on_cpu_submitted is not None:
            on_cpu_submitted()
        return output

    def stats(self):
        return {"layers": len(self.banks), "resident_bytes": self.resident_bytes, **self.counters}

    def close(self):
        self.banks.clear()
        self._closed = True
