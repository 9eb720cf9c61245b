"""A GGUF file on disk -> device expert bank -> MoE block, against the oracle on the same bytes."""
import numpy as np
import pytest
import torch

from oracle import reference_np as R
from mylocal_llm_amd import synthetic
from mylocal_llm_amd.moe import DevicePackedExpertBank, Qwen3NextMoEInference
from mylocal_llm_amd.qwen3next_gguf import Qwen3NextGGUFIndex
from gpu_util import announce, rel_l2, triple
from test_gguf_index import moe_file

pytestmark = pytest.mark.gpu


def oracle_block(hidden, router, k, gate, up, down, shared, sgate):
    logits = hidden @ router.T
    ef = lambda i, rows: R.expert_ffn(rows, triple(gate.select_outer(i)), triple(up.select_outer(i)), triple(down.select_outer(i)))
    want, _, _ = R.moe_forward(hidden, logits, k, gate.shape[0], ef, tuple(triple(w) for w in shared), sgate)
    return want, logits


@pytest.mark.parametrize("fused,fmt,shared", [(True, "Q8_0", ("Q8_0", "Q8_0", "BF16")),
                                              (False, "Q4_K", ("Q5_K", "Q5_K", "Q6_K")),
                                              (True, "Q6_K", ("BF16", "BF16", "BF16"))])
def test_moe_block_from_gguf_file(cuda, tmp_path, fused, fmt, shared):
    announce("gguf moe block", fused, fmt, shared)
    path = tmp_path / "block.gguf"
    gate, up, down, sh, router, sgate = moe_file(path, fused=fused, fmt=fmt, shared=shared, e=8, d=512, f=256, fsh=512, k=3)
    idx = Qwen3NextGGUFIndex.open(path)
    moe = Qwen3NextMoEInference.from_index(idx, 0, device=cuda)
    assert isinstance(moe.bank, DevicePackedExpertBank) and moe.bank.n_experts == 8
    assert moe.bank.nbytes == gate.nbytes + up.nbytes + down.nbytes
    assert not moe.shared_is_dense
    hidden = (np.random.default_rng(5).standard_normal((2, 3, 512)) * (0.5 if fmt != "Q4_K" else 2.0 ** -4)).astype(np.float32)
    want, logits = oracle_block(hidden.reshape(6, 512), router, 3, gate, up, down, sh, sgate)
    assert not synthetic.has_topk_ties(logits, 3)
    got = moe.forward(torch.from_numpy(hidden).to(cuda)).reshape(6, 512).cpu().numpy()
    assert rel_l2(got, want) <= 3e-5
    # a bank the caller already holds is used as it is
    again = Qwen3NextMoEInference.from_index(idx, 0, expert_executor=moe.bank, device=cuda)
    assert again.bank is moe.bank


def test_dense_shared_expert_takes_fp32_matmuls(cuda, tmp_path):
    """F32 / F16 shared projections have no packed form: the routed part still runs on the packed
    kernels, the shared expert as dense fp32 matmuls."""
    announce("gguf moe block, dense shared expert")
    from gguf_writer import write_gguf
    e, d, f, fsh, k = 4, 256, 256, 256, 2
    gate = synthetic.packed_weight("Q8_0", (e, f, d), 1)
    up = synthetic.packed_weight("Q8_0", (e, f, d), 2)
    down = synthetic.packed_weight("Q8_0", (e, d, f), 3)
    rng = np.random.default_rng(9)
    router = rng.standard_normal((e, d), dtype=np.float32)
    sgate = rng.standard_normal(d, dtype=np.float32) * np.float32(0.1)
    sg, su = (rng.standard_normal((fsh, d), dtype=np.float32) * np.float32(0.05) for _ in range(2))
    sd = (rng.standard_normal((d, fsh)) * 0.05).astype(np.float16)
    path = tmp_path / "dense.gguf"
    write_gguf(path, {"general.architecture": "qwen3next", "qwen3next.block_count": 1, "qwen3next.embedding_length": d,
                      "qwen3next.expert_count": e, "qwen3next.expert_used_count": k,
                      "qwen3next.expert_shared_feed_forward_length": fsh},
               [("blk.0.ffn_down_exps.weight", down.shape, "Q8_0", down.data), ("blk.0.ffn_gate_exps.weight", gate.shape, "Q8_0", gate.data),
                ("blk.0.ffn_up_exps.weight", up.shape, "Q8_0", up.data), ("blk.0.ffn_gate_inp.weight", router.shape, "F32", router),
                ("blk.0.ffn_gate_inp_shexp.weight", sgate.shape, "F32", sgate), ("blk.0.ffn_gate_shexp.weight", sg.shape, "F32", sg),
                ("blk.0.ffn_up_shexp.weight", su.shape, "F32", su), ("blk.0.ffn_down_shexp.weight", sd.shape, "F16", sd)])
    moe = Qwen3NextMoEInference.from_index(Qwen3NextGGUFIndex.open(path), 0, device=cuda)
    assert moe.shared_is_dense
    hidden = rng.standard_normal((1, 5, d), dtype=np.float32) * np.float32(0.5)
    flat = hidden.reshape(5, d)
    logits = flat @ router.T
    w, ids = R.router_topk(logits, k, renormalize=True, floor=2.0 ** -14)
    ef = lambda i, rows: R.expert_ffn(rows, triple(gate.select_outer(i)), triple(up.select_outer(i)), triple(down.select_outer(i)))
    routed = R.experts_forward(flat, w, ids, e, ef)
    x64 = flat.astype(np.float64)
    g64 = x64 @ sg.astype(np.float64).T
    act = g64 / (1 + np.exp(-g64)) * (x64 @ su.astype(np.float64).T)
    want = routed + (act @ sd.astype(np.float64).T) * R.shared_gate_sigmoid(flat, sgate)[:, None]
    got = moe.forward(torch.from_numpy(hidden).to(cuda)).reshape(5, d).cpu().numpy()
    assert rel_l2(got, want.astype(np.float32)) <= 3e-5
