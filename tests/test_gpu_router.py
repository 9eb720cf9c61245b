"""GPU router: ids bit-exact, weights within the reference's own tolerance (2e-7)."""
import os

import numpy as np
import pytest
import torch

from oracle import reference_np as R
from mylocal_llm_amd import synthetic
from mylocal_llm_amd.router import RouterInference, expert_topk_forward, try_normalized_topk
from gpu_util import announce

pytestmark = pytest.mark.gpu
FV = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "format_vectors.npz"))


@pytest.mark.parametrize("n,k", [(1, 1), (3, 2), (32, 4), (512, 10), (4096, 32)])
@pytest.mark.parametrize("floor", [2 ** -14, .9, 2.0])
def test_exact_ids_and_probability_parity(cuda, n, k, floor):
    announce("router", n, k, floor)
    z = np.random.default_rng(n).normal(0, 5, (1, 1, n)).astype(np.float32)
    assert not synthetic.has_topk_ties(z, min(k, n - 1))
    logits = torch.from_numpy(z).to(cuda)
    before = logits.clone()
    want_w, want_ids = R.router_topk(z, k, floor=floor)
    got_w, got_ids = try_normalized_topk(logits, k, floor)
    np.testing.assert_array_equal(got_ids.cpu().numpy(), want_ids)
    np.testing.assert_allclose(got_w.cpu().numpy(), want_w, rtol=2e-7, atol=2e-7)
    assert torch.equal(logits, before)
    assert got_w.dtype == torch.float32 and got_ids.dtype == torch.int64 and got_ids.shape == (1, 1, k)


@pytest.mark.parametrize("i", range(7))
def test_ties_extremes_and_nonfinite(cuda, i):
    row, ids = FV[f"router_row{i}"], FV[f"router_row{i}_ids"]
    k = min(4, row.size)
    with np.errstate(all="ignore"):
        want_w, want_ids = R.router_topk(row[None], k, floor=2.0 ** -14)
    np.testing.assert_array_equal(want_ids[0], ids)
    got_w, got_ids = try_normalized_topk(torch.from_numpy(row[None]).to(cuda), k, 2.0 ** -14)
    np.testing.assert_array_equal(got_ids.cpu().numpy()[0], ids)
    np.testing.assert_allclose(got_w.cpu().numpy(), want_w, rtol=2e-7, atol=2e-7, equal_nan=True)


@pytest.mark.parametrize("tokens", [1, 4, 16, 512])
def test_many_rows_config_shapes(cuda, tokens):
    announce("router rows", tokens)
    z = synthetic.router_logits(tokens, 512, 11, zipf=1.1 if tokens == 512 else None)
    assert not synthetic.has_topk_ties(z, 10)
    want_w, want_ids = R.router_topk(z, 10, floor=2.0 ** -14)
    got_w, got_ids = try_normalized_topk(torch.from_numpy(z).to(cuda), 10, 2.0 ** -14)
    np.testing.assert_array_equal(got_ids.cpu().numpy(), want_ids)
    np.testing.assert_allclose(got_w.cpu().numpy(), want_w, rtol=2e-6, atol=2e-7)
    np.testing.assert_allclose(got_w.sum(-1).cpu().numpy(), 1.0, atol=1e-6)


@pytest.mark.parametrize("shape,k,floor", [((1, 512), 33, 1e-6), ((1, 4097), 10, 1e-6), ((1, 16), 3, 1e-50)])
def test_unsupported_returns_none(cuda, shape, k, floor):
    assert try_normalized_topk(torch.zeros(shape, device=cuda), k, floor) is None
    assert try_normalized_topk(torch.zeros((1, 8), device=cuda, dtype=torch.float64), 8, 1e-6) is None


def test_unnormalised_topk_and_router_module(cuda):
    z = np.random.default_rng(5).normal(0, 2, (2, 3, 64)).astype(np.float32)
    want_w, want_ids = R.router_topk(z, 5, renormalize=False)
    w, ids, cache = expert_topk_forward(torch.from_numpy(z).to(cuda), 5)
    assert cache is None
    np.testing.assert_array_equal(ids.cpu().numpy(), want_ids)
    np.testing.assert_allclose(w.cpu().numpy(), want_w, rtol=2e-6, atol=2e-7)
    rng = np.random.default_rng(10622)
    router = RouterInference(32, 64, 4, renormalize_selected=True, normalization_floor=2.0 ** -14)
    wr = rng.normal(0, .5, (32, 64)).astype(np.float32)
    router.W_router = torch.from_numpy(wr).to(cuda)
    router.b_router = torch.zeros(64, device=cuda)
    x = rng.normal(0, 1, (2, 3, 32)).astype(np.float32)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        weights, got_ids = router.forward(torch.from_numpy(x).to(cuda))
    stream.synchronize()
    logits = (torch.from_numpy(x).to(cuda).reshape(6, 32) @ router.W_router).cpu().numpy().reshape(2, 3, 64)
    ww, wi = R.router_topk(logits, 4, floor=2.0 ** -14)
    np.testing.assert_array_equal(got_ids.cpu().numpy(), wi)
    np.testing.assert_allclose(weights.cpu().numpy(), ww, rtol=2e-6, atol=2e-7)
    with pytest.raises(ValueError):
        RouterInference(4, 4, 5)
    with pytest.raises(TypeError):
        RouterInference(4, 4, 2, renormalize_selected=1)
