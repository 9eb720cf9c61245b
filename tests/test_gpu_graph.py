"""The library allocates, copies, clears and synchronises nothing itself, so its calls can be
recorded into a HIP graph: a recorded MoE step and a recorded streamed linear are replayed several
times, with eager work and synchronisations between the replays, and every replay is checked
against the eager result on the same inputs."""
import numpy as np
import pytest
import torch

from mylocal_llm_amd import synthetic
from mylocal_llm_amd.moe import DevicePackedExpertBank, moe_step
from mylocal_llm_amd.quantized_linear import quantized_linear
from gpu_util import announce, upload
from test_gpu_moe import make_layer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens", [1, 4, 9, 40])
def test_moe_step_replays_from_a_graph(cuda, tokens):
    announce("graph replay: moe step", tokens)
    e, d, f, fsh, k = 16, 256, 256, 512, 4
    gate, up, down, shared, gate_vec = make_layer(e, d, f, fsh, ("Q8_0", "Q8_0", "Q8_0"), 91)
    bank = DevicePackedExpertBank(gate, up, down, device=cuda)
    dshared = tuple(upload(w, cuda) for w in shared)
    sg = torch.from_numpy(gate_vec).to(cuda)
    hidden = torch.zeros((tokens, d), device=cuda)
    logits = torch.zeros((tokens, e), device=cuda)
    residual = torch.zeros((tokens, d), device=cuda)
    rng = np.random.default_rng(tokens)

    def refill():
        hidden.copy_(torch.from_numpy(rng.standard_normal((tokens, d)).astype(np.float32)))
        logits.copy_(torch.from_numpy(rng.standard_normal((tokens, e)).astype(np.float32)))
        residual.copy_(torch.from_numpy(rng.standard_normal((tokens, d)).astype(np.float32)))

    step = lambda: moe_step(hidden, bank, k, logits=logits, shared=dshared, shared_gate=sg, residual=residual)
    refill()
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = step()
    for _ in range(4):
        refill()
        eager = step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(recorded, eager)


def test_streamed_linear_replays_from_a_graph(cuda):
    announce("graph replay: linear")
    w = upload(synthetic.packed_weight("Q6_K", (512, 1024), 3), cuda)
    x = torch.zeros((1, 1024), device=cuda)
    x.copy_(torch.randn(1, 1024))
    quantized_linear(x, w)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = quantized_linear(x, w)
    for seed in range(3):
        x.copy_(torch.randn(1, 1024, generator=torch.Generator().manual_seed(seed)))
        eager = quantized_linear(x, w)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(recorded, eager)
