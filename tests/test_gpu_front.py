"""The steps either side of the MoE block: RMSNorm + router logits in front, residual add behind."""
import numpy as np
import pytest
import torch

from oracle import reference_np as R
from mylocal_llm_amd import synthetic
from mylocal_llm_amd.moe import DevicePackedExpertBank, Qwen3NextMoEInference, moe_step, norm_router
from gpu_util import announce, rel_l2, triple, upload
from test_gpu_moe import make_layer, oracle_step

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,d,e", [(1, 2048, 512), (4, 2048, 512), (9, 1024, 60), (40, 256, 16), (3, 36, 5)])
def test_norm_router_matches_oracle(cuda, tokens, d, e):
    announce("norm + router", tokens, d, e)
    rng = np.random.default_rng(tokens * 7 + d)
    x = (rng.standard_normal((tokens, d)) * 3).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    w = (rng.standard_normal((e, d)) * 0.2).astype(np.float32)
    b = rng.standard_normal(e).astype(np.float32)
    xd, gd, wd, bd = (torch.from_numpy(a).to(cuda) for a in (x, gamma, w, b))
    for eps in (1e-6, 1e-2):
        normalized, logits = norm_router(xd, gd, eps, wd, bd)
        want_n = R.rmsnorm(x, gamma, eps)
        # the sum of squares is taken in another order: inv_rms may differ in its last place or two
        np.testing.assert_allclose(normalized.cpu().numpy(), want_n, rtol=6e-7, atol=0)
        assert rel_l2(logits.cpu().numpy(), R.router_logits(want_n, w, b)) <= 2e-6
    normalized, logits = norm_router(xd, gd, 1e-6, wd)
    assert rel_l2(logits.cpu().numpy(), R.router_logits(R.rmsnorm(x, gamma, 1e-6), w)) <= 2e-6
    with pytest.raises(ValueError):
        norm_router(xd, gd[:-1].contiguous(), 1e-6, wd)
    with pytest.raises(TypeError):
        norm_router(xd.half(), gd, 1e-6, wd)


@pytest.mark.parametrize("tokens", [1, 4, 9, 40])
def test_residual_is_added_inside_the_step(cuda, tokens):
    """Every token-count regime (fused decode, routing kernel + list, token-tile GEMM)."""
    announce("moe residual", tokens)
    e, d, f, fsh, k = 16, 256, 256, 512, 4
    gate, up, down, shared, gate_vec = make_layer(e, d, f, fsh, ("Q8_0", "Q8_0", "Q8_0"), 41)
    bank = DevicePackedExpertBank(gate, up, down, device=cuda)
    dshared = tuple(upload(w, cuda) for w in shared)
    hidden = torch.from_numpy(synthetic.activations((tokens, d), 5)).to(cuda)
    logits = torch.from_numpy(synthetic.router_logits(tokens, e, 6)).to(cuda)
    residual = torch.from_numpy(np.random.default_rng(8).standard_normal((tokens, d)).astype(np.float32) * 50).to(cuda)
    sg = torch.from_numpy(gate_vec).to(cuda)
    plain = moe_step(hidden, bank, k, logits=logits, shared=dshared, shared_gate=sg)
    fused = moe_step(hidden, bank, k, logits=logits, shared=dshared, shared_gate=sg, residual=residual)
    assert torch.equal(fused, residual + plain)          # one fp32 add either way
    low = moe_step(hidden, bank, k, logits=logits, shared=dshared, shared_gate=sg, residual=residual, out_dtype=torch.bfloat16)
    assert torch.equal(low, (residual + plain).to(torch.bfloat16))
    with pytest.raises(ValueError, match="residual"):
        moe_step(hidden, bank, k, logits=logits, residual=residual[:, :-1])


@pytest.mark.parametrize("tokens", [1, 5, 33])
def test_second_half_of_a_decoder_layer(cuda, tokens):
    """residual + moe(rmsnorm(residual)) against the oracle's composition."""
    announce("layer half", tokens)
    e, d, f, fsh, k = 16, 256, 256, 512, 4
    gate, up, down, shared, gate_vec = make_layer(e, d, f, fsh, ("Q8_0", "Q8_0", "Q6_K"), 720)
    rng = np.random.default_rng(78)
    router_w = rng.normal(0, .3, (e, d)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    residual = rng.normal(0, 2, (1, tokens, d)).astype(np.float32)
    bank = DevicePackedExpertBank(gate, up, down, device=cuda)
    moe = Qwen3NextMoEInference(bank, k, torch.from_numpy(router_w).to(cuda), tuple(upload(w, cuda) for w in shared),
                                torch.from_numpy(gate_vec).to(cuda))
    flat = residual.reshape(tokens, d)
    normalized = R.rmsnorm(flat, gamma, 1e-6)
    logits = R.router_logits(normalized, router_w)
    assert not synthetic.has_topk_ties(logits, k)
    block, _, _ = oracle_step(normalized, logits, k, gate, up, down, shared, gate_vec)
    want = flat + block
    got = moe.forward_after_norm(torch.from_numpy(residual).to(cuda), torch.from_numpy(gamma).to(cuda), 1e-6)
    assert got.shape == residual.shape
    assert rel_l2(got.reshape(tokens, d).cpu().numpy(), want) <= 2e-5
    # the same through the unfused calls of the module
    hd = torch.from_numpy(residual).to(cuda)
    nd, _ = norm_router(hd.reshape(tokens, d), torch.from_numpy(gamma).to(cuda), 1e-6, moe._router_weight)
    unfused = hd + moe.forward(nd.reshape(1, tokens, d))
    assert rel_l2(got.cpu().numpy().reshape(tokens, d), unfused.cpu().numpy().reshape(tokens, d)) <= 2e-6
    assert moe.forward_after_norm(hd[:, :0], torch.from_numpy(gamma).to(cuda), 1e-6).shape == (1, 0, d)


def test_router_bias_set_later_is_used_and_odd_widths_route(cuda):
    """A bias written to the module's router after construction changes the routing of forward and
    forward_after_norm (both read the router's current weight and bias); logits of rows whose width
    is not a multiple of four come from the plain fp32 product instead of an error."""
    from mylocal_llm_amd.moe import router_logits
    from mylocal_llm_amd.router import RouterInference
    announce("router bias / odd width")
    e, d, f, fsh, k, tokens = 16, 256, 256, 512, 4, 3
    gate, up, down, shared, gate_vec = make_layer(e, d, f, fsh, ("Q8_0", "Q8_0", "Q8_0"), 910)
    rng = np.random.default_rng(91)
    router_w = rng.normal(0, .3, (e, d)).astype(np.float32)
    bias = np.zeros(e, np.float32)
    bias[[3, 11]] = 50.0                                   # these two experts now win every row
    hidden = rng.normal(0, 2, (1, tokens, d)).astype(np.float32)
    moe = Qwen3NextMoEInference(DevicePackedExpertBank(gate, up, down, device=cuda), k, torch.from_numpy(router_w).to(cuda),
                                tuple(upload(w, cuda) for w in shared), torch.from_numpy(gate_vec).to(cuda))
    hd = torch.from_numpy(hidden).to(cuda)
    before = moe.forward(hd)
    moe.router.b_router = torch.from_numpy(bias).to(cuda)
    after = moe.forward(hd)
    flat = hidden.reshape(tokens, d)
    logits = R.router_logits(flat, router_w, bias)
    assert not synthetic.has_topk_ties(logits, k)
    want, _, ids = oracle_step(flat, logits, k, gate, up, down, shared, gate_vec)
    assert {3, 11} <= set(ids[0].tolist())
    assert rel_l2(after.reshape(tokens, d).cpu().numpy(), want) <= 2e-5
    assert rel_l2(before.reshape(tokens, d).cpu().numpy(), want) > 1e-3
    # odd width: d_model = 6
    r = RouterInference(6, 5, 2)
    r.W_router = torch.from_numpy(rng.normal(0, 1, (6, 5)).astype(np.float32)).to(cuda)
    r.b_router = torch.from_numpy(rng.normal(0, 1, 5).astype(np.float32)).to(cuda)
    x = torch.from_numpy(rng.normal(0, 1, (2, 3, 6)).astype(np.float32)).to(cuda)
    w, ids = r.forward(x)
    want_logits = x.reshape(6, 6).cpu().numpy() @ r.W_router.cpu().numpy() + r.b_router.cpu().numpy()
    want_w, want_ids = R.router_topk(want_logits, 2, renormalize=False)
    np.testing.assert_array_equal(ids.reshape(6, 2).cpu().numpy(), want_ids)
    np.testing.assert_allclose(w.reshape(6, 2).cpu().numpy(), want_w, rtol=2e-6, atol=2e-7)
    assert router_logits(x.reshape(6, 6).contiguous(), r.W_router.t().contiguous()).shape == (6, 5)
