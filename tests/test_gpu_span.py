"""Single-token streaming kernel (rows through LDS rings): the lane layouts, activation types and
alignments the wider linear tests do not reach, and the bounded wait's give-up path."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import reference_np as R
from mylocal_llm_amd import _lib, synthetic
from mylocal_llm_amd.quantized_linear import DevicePackedGGUFWeight, quantized_linear, quantized_linear_batch, quantized_swiglu
from gpu_util import BF16_MAX_ABS, REL_L2, announce, rel_l2, triple, upload

pytestmark = pytest.mark.gpu
TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def close_enough(got, want, dtype):
    g = got.float().cpu().numpy()
    if dtype == "f32":
        assert rel_l2(g, want) <= 5e-6 <= REL_L2
    else:   # one rounding of the fp32 result to the 16-bit output type
        scale = max(1.0, float(np.abs(want).max()))
        assert np.abs(g - want).max() <= (BF16_MAX_ABS if dtype == "bf16" else 2e-3) * scale
        assert rel_l2(g, want) <= (5e-3 if dtype == "bf16" else 1e-3)


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K"])
@pytest.mark.parametrize("k", [768, 1536, 2304, 3072, 3840, 4096])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_one_token_idle_lanes_and_sixteen_bit_activations(cuda, fmt, k, dtype):
    """One token at row widths that leave lanes of a row group without a unit (768 .. 3840 columns),
    with fp16 / bf16 activations and outputs (staged through LDS stores instead of the DMA), a row
    count that ends inside a work item, alone, as a gate/up pair and in a batch with another width."""
    announce("span widths", fmt, k, dtype)
    n = 75
    tdt = TORCH_DT[dtype]
    hosts = [synthetic.packed_weight(fmt, (n, k), 60 + i) for i in range(2)]
    devs = [upload(w, cuda) for w in hosts]
    xd = torch.from_numpy(synthetic.activations((1, k), 61)).to(cuda).to(tdt)
    x = xd.float().cpu().numpy()
    got = quantized_linear(xd, devs[0])
    assert got.dtype == tdt and got.shape == (1, n)
    close_enough(got, R.linear(x, *triple(hosts[0])), dtype)
    pair = quantized_swiglu(xd, devs[0], devs[1])
    want_pair = R.swiglu(x, triple(hosts[0]), triple(hosts[1]))
    if dtype == "f32":
        assert rel_l2(pair.cpu().numpy(), want_pair) <= 1e-5
    else:
        close_enough(pair, want_pair, dtype)
    other = synthetic.packed_weight(fmt, (33, 2048), 64)
    xo = torch.from_numpy(synthetic.activations((1, 2048), 65)).to(cuda).to(tdt)
    outs = quantized_linear_batch([(xo, upload(other, cuda)), (xd, devs[1]), (xd, devs[0])])
    close_enough(outs[0], R.linear(xo.float().cpu().numpy(), *triple(other)), dtype)
    close_enough(outs[1], R.linear(x, *triple(hosts[1])), dtype)
    assert torch.equal(outs[2], got)


@pytest.mark.parametrize("offset", [2, 6, 14, 18])
def test_q6_k_rows_that_are_only_two_byte_aligned(cuda, offset):
    """A Q6_K matrix whose first byte lies an odd multiple of two bytes past a 16-byte boundary (an
    expert of a bank whose stride is not a multiple of four): its spans still travel by LDS-DMA."""
    announce("span q6_k alignment", offset)
    w = synthetic.packed_weight("Q6_K", (70, 2048), 71)
    raw = torch.zeros(w.nbytes + 64, dtype=torch.uint8, device=cuda)
    assert raw.data_ptr() % 16 == 0
    raw[offset:offset + w.nbytes] = torch.from_numpy(w.data).to(cuda)
    dev = DevicePackedGGUFWeight(raw[offset:offset + w.nbytes], w.shape, "Q6_K")
    assert dev.data.data_ptr() % 16 == offset % 16
    x = synthetic.activations((1, 2048), 72)
    got = quantized_linear(torch.from_numpy(x).to(cuda), dev).cpu().numpy()
    assert rel_l2(got, R.linear(x, *triple(w))) <= 2e-6


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K"])
def test_two_long_activation_rows_in_one_launch(cuda, fmt):
    """Two neighbouring problems whose activation rows (16384 and 8192 columns) fit LDS together only
    with a shallower ring, or not at all: the launch takes the shallower ring or the register-load
    kernel, and the results are the oracle's either way."""
    announce("span long rows", fmt)
    shapes = [(40, 16384), (24, 8192), (50, 1024)]
    hosts = [synthetic.packed_weight(fmt, s, 80 + i) for i, s in enumerate(shapes)]
    xs = [synthetic.activations((1, s[1]), 90 + i) for i, s in enumerate(shapes)]
    outs = quantized_linear_batch([(torch.from_numpy(x).to(cuda), upload(w, cuda)) for x, w in zip(xs, hosts)])
    for out, x, w in zip(outs, xs, hosts):
        assert rel_l2(out.cpu().numpy(), R.linear(x, *triple(w))) <= 3e-6


def test_expired_wait_is_reported_and_nothing_wrong_is_stored(cuda):
    """The kernel's waits for the other waves of a workgroup are bounded.  With the bound forced to
    expire at once every wave gives up: the launch still ends normally, stores nothing, and
    qmoe_check_status reports it (and clears the word); with the default bound the same call is right."""
    announce("span give-up")
    lib = _lib.load()
    assert lib.qmoe_init() == 0
    w = synthetic.packed_weight("Q8_0", (300, 2048), 91)
    dev = upload(w, cuda)
    x = synthetic.activations((1, 2048), 92)
    xd = torch.from_numpy(x).to(cuda)
    y = torch.full((1, 300), 7.0, dtype=torch.float32, device=cuda)
    null = ctypes.c_void_p(0)

    def run():
        return lib.qmoe_linear(ctypes.c_void_p(dev.data.data_ptr()), _lib.FORMAT_ID["Q8_0"], 300, 2048,
                               ctypes.c_void_p(xd.data_ptr()), 0, 1, ctypes.c_void_p(y.data_ptr()), 0, null)

    torch.cuda.synchronize()
    assert lib.qmoe_check_status(null) == 0
    lib.qmoe_set_wait_limit(-1)
    try:
        assert run() == 0
        torch.cuda.synchronize()          # the launch ends by itself
        assert lib.qmoe_check_status(null) == 3
        assert b"bounded wait" in lib.qmoe_last_error()
        assert bool((y == 7.0).all())     # no wave stored a result it could not vouch for
        assert lib.qmoe_check_status(null) == 0   # the word was cleared
    finally:
        lib.qmoe_set_wait_limit(0)
    assert run() == 0
    torch.cuda.synchronize()
    assert lib.qmoe_check_status(null) == 0
    assert rel_l2(y.cpu().numpy(), R.linear(x, *triple(w))) <= 2e-6
