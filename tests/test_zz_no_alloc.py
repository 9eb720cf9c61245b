"""The MoE step without a caller's workspace (qmoe_moe_forward_static) against qmoe_moe_forward."""
import ctypes

import numpy as np
import pytest
import torch

from mylocal_llm_amd import _lib, synthetic
from mylocal_llm_amd.moe import DevicePackedExpertBank
from gpu_util import announce, upload

pytestmark = pytest.mark.gpu


def _args(hidden, logits, bank, shared, gate_vec, out, top_k, hidden_dtype, out_dtype):
    a = _lib.MoeArgs()
    a.hidden, a.hidden_dtype, a.tokens, a.top_k = hidden.data_ptr(), hidden_dtype, hidden.shape[0], top_k
    a.logits, a.floor_value, a.renormalize = logits.data_ptr(), 2.0 ** -14, 1
    bank.fill(a.bank)
    g, u, d = shared
    a.shared_gate_w, a.shared_up_w, a.shared_down_w = g.data.data_ptr(), u.data.data_ptr(), d.data.data_ptr()
    fid = _lib.FORMAT_ID[g.quant_type]
    a.shared_gate_fmt = a.shared_up_fmt = a.shared_down_fmt = fid
    a.d_ff_shared, a.shared_gate = g.shape[0], gate_vec.data_ptr()
    a.out, a.out_dtype = out.data_ptr(), out_dtype
    return a


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K"])
def test_static_scratch_step_equals_workspace_step(cuda, fmt):
    """Two calls in a row through the C ABI, the second with fewer tokens (so the scratch still
    holds the first call's contents): each must give the bits of qmoe_moe_forward with a workspace
    of the caller's.  20 tokens take the token-batch kernels, 3 tokens the decode kernels."""
    lib = _lib.load()
    e, d, f, fsh, k = 32, 512, 256, 512, 4
    gate = synthetic.packed_weight(fmt, (e, f, d), 1)
    up = synthetic.packed_weight(fmt, (e, f, d), 2)
    down = synthetic.packed_weight(fmt, (e, d, f), 3)
    bank = DevicePackedExpertBank(gate, up, down, device=cuda)
    shared = tuple(upload(synthetic.packed_weight(fmt, s, 4 + i), cuda) for i, s in enumerate(((fsh, d), (fsh, d), (d, fsh))))
    gate_vec = torch.from_numpy(np.random.default_rng(7).normal(0, .05, d).astype(np.float32)).to(cuda)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.qmoe_moe_static_scratch_bytes() == 8 << 20
    for tokens in (20, 3):
        announce("static scratch", fmt, tokens)
        hidden = torch.from_numpy(synthetic.activations((tokens, d), 8 + tokens, "bf16")).to(cuda)
        logits = torch.from_numpy(synthetic.router_logits(tokens, e, 9 + tokens)).to(cuda)
        want = torch.empty((tokens, d), device=cuda, dtype=torch.float32)
        got = torch.full((tokens, d), float("nan"), device=cuda, dtype=torch.float32)
        nbytes = lib.qmoe_moe_workspace_bytes(tokens, k, e, d, f, fsh)
        assert 0 < nbytes <= lib.qmoe_moe_static_scratch_bytes()
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
        a = _args(hidden, logits, bank, shared, gate_vec, want, k, 0, 0)
        assert lib.qmoe_moe_forward(ctypes.byref(a), ctypes.c_void_p(workspace.data_ptr()), nbytes, stream) == 0
        b = _args(hidden, logits, bank, shared, gate_vec, got, k, 0, 0)
        # the device variables' addresses are resolved ahead of the call (qmoe_init), so the call itself
        # neither allocates nor looks anything up: device memory in use is the same before and after
        assert lib.qmoe_init() == 0
        torch.cuda.synchronize()
        held, free_before = torch.cuda.memory_allocated(cuda), torch.cuda.mem_get_info(cuda)[0]
        rc = lib.qmoe_moe_forward_static(ctypes.byref(b), stream)
        assert rc == 0, lib.qmoe_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(cuda) == held and torch.cuda.mem_get_info(cuda)[0] == free_before
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.cpu().numpy().view(np.uint32))


def test_static_scratch_rejects_steps_that_do_not_fit(cuda):
    lib = _lib.load()
    a = _lib.MoeArgs()
    a.tokens, a.top_k = 4096, 8
    a.bank.n_experts, a.bank.d_model, a.bank.d_ff = 64, 2048, 1024
    assert lib.qmoe_moe_workspace_bytes(4096, 8, 64, 2048, 1024, 0) > lib.qmoe_moe_static_scratch_bytes()
    rc = lib.qmoe_moe_forward_static(ctypes.byref(a), None)
    assert rc == 4 and b"scratch" in lib.qmoe_last_error()
