"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from mylocal_llm_amd.quantized_linear import DevicePackedGGUFWeight

# north_star tolerances: fp32-accumulated outputs within rel-L2 1e-3 of the NumPy reference,
# bf16 outputs within max-abs 2e-2; dequantised weights and top-k ids bit-exact.
REL_L2 = 1e-3
BF16_MAX_ABS = 2e-2


def rel_l2(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    denom = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (denom if denom else 1.0))


def upload(weight, device):
    data = torch.from_numpy(np.ascontiguousarray(weight.data)).to(device)
    return DevicePackedGGUFWeight(data, weight.shape, weight.quant_type)


def triple(w):
    return (w.data, w.shape, w.quant_type)


def announce(*what):
    print("[case]", *what, flush=True)
