"""The resident expert executor behind the reference's executor hooks."""
import numpy as np
import pytest
import torch

from oracle import reference_np as R
from mylocal_llm_amd import synthetic
from mylocal_llm_amd.expert_executor import ResidentExpertExecutor
from mylocal_llm_amd.moe import DevicePackedExpertBank, ExpertsInference, Qwen3NextMoEInference
from mylocal_llm_amd.qwen3next_gguf import Qwen3NextGGUFIndex
from gpu_util import announce, rel_l2, triple
from test_gguf_index import moe_file
from test_gpu_moe import make_layer

pytestmark = pytest.mark.gpu


def routed_reference(hidden, weights, ids, gate, up, down):
    ef = lambda i, rows: R.expert_ffn(rows, triple(gate.select_outer(i)), triple(up.select_outer(i)), triple(down.select_outer(i)))
    return R.experts_forward(hidden, weights, ids, gate.shape[0], ef)


def test_hooks_answer_from_the_resident_bank(cuda):
    announce("resident executor hooks")
    e, d, f, k = 12, 256, 256, 3
    layers = {3: make_layer(e, d, f, 256, ("Q8_0", "Q8_0", "Q8_0"), 51), 7: make_layer(e, d, f, 256, ("Q6_K", "Q6_K", "Q6_K"), 52)}
    ex = ResidentExpertExecutor(d, f, model_id="test")
    for lid, (gate, up, down, _, _) in layers.items():
        ex.register_layer(lid, DevicePackedExpertBank(gate, up, down, device=cuda))
    assert ex.compute_dtype == "float32" and not ex.overlaps_cpu_gpu
    assert ex.resident_bytes == sum(g.nbytes + u.nbytes + dn.nbytes for g, u, dn, _, _ in layers.values())
    rng = np.random.default_rng(5)
    for lid, (gate, up, down, _, _) in layers.items():
        # one expert on some rows
        x = rng.standard_normal((3, d)).astype(np.float32)
        want = R.expert_ffn(x, triple(gate.select_outer(4)), triple(up.select_outer(4)), triple(down.select_outer(4)))
        got = ex.forward(lid, 4, torch.from_numpy(x).to(cuda))
        assert rel_l2(got.cpu().numpy(), want) <= 2e-5
        assert torch.equal(ex.resolve(ex.submit(lid, 4, torch.from_numpy(x).to(cuda))), got)
        # one token through the device plan hook and through the grouped singleton hook
        x1 = rng.standard_normal((1, d)).astype(np.float32)
        ids = np.array([[9, 2, 5]], np.int64)
        w = np.array([[0.5, 0.3, 0.2]], np.float32)
        want = routed_reference(x1, w, ids, gate, up, down)
        called = []
        xd, wd, idd = torch.from_numpy(x1).to(cuda), torch.from_numpy(w).to(cuda), torch.from_numpy(ids).to(cuda)
        got = ex.try_forward_device_plan(lid, xd, wd.reshape(-1), idd.reshape(-1), e, on_cpu_submitted=lambda: called.append(1))
        assert called == [1] and rel_l2(got.cpu().numpy(), want) <= 2e-5
        assert ex.try_forward_device_plan(lid, xd, wd.reshape(-1), idd.reshape(-1), e + 1) is None   # not this layer's expert count
        with ex.dispatch_scope(lid, (2, 5, 9)):
            grouped = ex.try_forward_grouped(lid, (2, 5, 9), xd, wd.reshape(-1), (1, 2, 0))    # slots of experts 2, 5, 9
        assert rel_l2(grouped.cpu().numpy(), want) <= 2e-5
        # the decode-batch hook: the same plan inside a dispatch scope, None for what the reference declines
        assert ex.try_forward_decode_batch(lid, (2, 5, 9), xd, wd.reshape(-1), (1, 2, 0)) is None          # no scope
        with ex.dispatch_scope(lid, (2, 5, 9)):
            seen = []
            batched = ex.try_forward_decode_batch(lid, (2, 5, 9), xd, wd.reshape(-1), (1, 2, 0), on_cpu_submitted=lambda: seen.append(1))
            assert seen == [1] and torch.equal(batched, grouped)
            assert ex.try_forward_decode_batch(lid, (5, 2, 9), xd, wd.reshape(-1), (2, 1, 0)) is None      # not ascending
            assert ex.try_forward_decode_batch(lid, (2, 2, 9), xd, wd.reshape(-1), (1, 1, 0)) is None      # not unique
            assert ex.try_forward_decode_batch(lid, (2, 5, 9), xd.half(), wd.reshape(-1), (1, 2, 0)) is None
            assert ex.try_forward_decode_batch(lid, (), xd, wd.reshape(-1), ()) is None
        # several tokens in one step
        xn = rng.standard_normal((6, d)).astype(np.float32)
        idn = np.stack([rng.permutation(e)[:k] for _ in range(6)]).astype(np.int64)
        wn = rng.dirichlet(np.ones(k), 6).astype(np.float32)
        got = ex.try_forward_batch(lid, torch.from_numpy(xn).to(cuda), torch.from_numpy(wn).to(cuda), torch.from_numpy(idn).to(cuda))
        assert rel_l2(got.cpu().numpy(), routed_reference(xn, wn, idn, gate, up, down)) <= 2e-5
    assert ex.stats()["layers"] == 2 and ex.stats()["device_plan_dispatches"] == 2
    with pytest.raises(KeyError, match="layer 5"):
        ex.forward(5, 0, xd)
    with pytest.raises(ValueError, match="dimensions"):
        ex.register_layer(9, DevicePackedExpertBank(*make_layer(4, 512, 256, 256, ("Q8_0",) * 3, 1)[:3], device=cuda))
    with pytest.raises(TypeError):
        ex.register_layer(9, object())
    ex.close()
    assert not ex.banks


@pytest.mark.parametrize("tokens", [1, 7])
def test_experts_inference_goes_through_the_executor(cuda, tokens):
    announce("experts inference over executor", tokens)
    e, d, f, k = 12, 256, 256, 3
    gate, up, down, _, _ = make_layer(e, d, f, 256, ("Q8_0", "Q8_0", "Q8_0"), 61)
    bank = DevicePackedExpertBank(gate, up, down, device=cuda)
    ex = ResidentExpertExecutor(d, f)
    ex.register_layer(2, bank)
    rng = np.random.default_rng(tokens)
    x = torch.from_numpy(rng.standard_normal((1, tokens, d)).astype(np.float32)).to(cuda)
    ids = torch.from_numpy(np.stack([rng.permutation(e)[:k] for _ in range(tokens)]).astype(np.int64).reshape(1, tokens, k)).to(cuda)
    w = torch.from_numpy(rng.dirichlet(np.ones(k), tokens).astype(np.float32).reshape(1, tokens, k)).to(cuda)
    seen = []
    over_executor = ExpertsInference(d, f, e, expert_executor=ex, layer_id=2).forward(x, w, ids, on_cpu_submitted=lambda: seen.append(1))
    over_bank = ExpertsInference(d, f, e, expert_executor=bank).forward(x, w, ids)
    assert seen == [1] and torch.equal(over_executor, over_bank)
    assert ex.counters["device_plan_dispatches" if tokens == 1 else "batch_dispatches"] == 1
    with pytest.raises(ValueError, match="dimensions"):
        ExpertsInference(d, f + 1, e, expert_executor=ex)


def test_block_over_an_executor_built_from_a_file(cuda, tmp_path):
    announce("executor from gguf")
    path = tmp_path / "m.gguf"
    gate, up, down, sh, router, sgate = moe_file(path, fused=True, e=8, d=512, f=256, fsh=512, k=3)
    idx = Qwen3NextGGUFIndex.open(path)
    ex = ResidentExpertExecutor.from_index(idx, device=cuda)
    assert sorted(ex.banks) == [0] and ex.resident_bytes == gate.nbytes + up.nbytes + down.nbytes
    moe = Qwen3NextMoEInference.from_index(idx, 0, expert_executor=ex, device=cuda)
    assert moe.bank is ex.bank(0)
    hidden = (np.random.default_rng(2).standard_normal((1, 4, 512)) * 0.5).astype(np.float32)
    direct = Qwen3NextMoEInference.from_index(idx, 0, device=cuda).forward(torch.from_numpy(hidden).to(cuda))
    assert torch.equal(moe.forward(torch.from_numpy(hidden).to(cuda)), direct)
