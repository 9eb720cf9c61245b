"""Routing plans of batches longer than one plan-kernel call covers (collected late on purpose:
the plan object is a side door of the MoE step, not part of it)."""
import numpy as np
import pytest
import torch

from mylocal_llm_amd import synthetic
from mylocal_llm_amd.routing_plan import create_routing_plan, max_tokens_per_plan_call
from oracle import reference_np as R
from gpu_util import announce

pytestmark = pytest.mark.gpu


def test_routing_plan_beyond_one_call_matches_the_oracle(cuda):
    """1500 tokens x 512 experts x top-10 (one call covers 928): planned in chunks of 512 tokens by
    the plan kernel and joined on the device; offsets, order, tokens, slots, weights and the inverse
    map against the oracle's stable sort of the whole batch (routing_plan.py:52-118)."""
    tokens, e, k = 1500, 512, 10
    announce("routing plan in chunks", tokens)
    assert tokens > max_tokens_per_plan_call(e)
    logits = synthetic.router_logits(tokens, e, 9, zipf=1.1)
    w, ids = R.router_topk(logits, k, floor=2.0 ** -14)
    plan = create_routing_plan(torch.from_numpy(ids.reshape(1, tokens, k)).to(cuda), torch.from_numpy(w.reshape(1, tokens, k)).to(cuda), k, e)
    token, slot, order, offsets = R.routing_plan(ids, e)
    assert plan.expert_offsets == tuple(int(v) for v in offsets)
    assert (plan.N, plan.k, plan.n_experts) == (tokens, k, e)
    np.testing.assert_array_equal(plan.order.cpu().numpy(), order)
    np.testing.assert_array_equal(plan.token_indices.cpu().numpy(), token)
    np.testing.assert_array_equal(plan.slot_indices.cpu().numpy(), slot)
    np.testing.assert_array_equal(plan.expert_indices.cpu().numpy(), ids.reshape(-1)[order])
    np.testing.assert_array_equal(plan.weights.cpu().numpy(), w.reshape(-1)[order])
    pos = plan.position_of_assignment.cpu().numpy().reshape(-1)
    np.testing.assert_array_equal(order[pos], np.arange(tokens * k))
    bad = ids.copy().reshape(1, tokens, k)
    bad[0, 1400, 3] = e
    with pytest.raises(ValueError, match="Invalid routing"):
        create_routing_plan(torch.from_numpy(bad).to(cuda), torch.from_numpy(w.reshape(1, tokens, k)).to(cuda), k, e)
