"""GPU dequantisation through the C ABI: bit-exact against the oracle and the golden vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import reference_np as R
from mylocal_llm_amd import synthetic
from mylocal_llm_amd.quantized_weight import PackedGGUFWeight
from gpu_util import announce, upload

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FV = np.load(os.path.join(GOLDEN, "format_vectors.npz"))
RV = np.load(os.path.join(GOLDEN, "ref_native_vectors.npz"))
FORMATS = ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K", "BF16"]


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("case,fmt", [("q4_0_nibbles", "Q4_0"), ("q4_k_scales", "Q4_K"), ("q3_k_keep", "Q3_K"), ("q3_k_minus4", "Q3_K"),
                                      ("q5_k_group0", "Q5_K"), ("q5_k_group7", "Q5_K"),
                                      ("q6_k_all_codes", "Q6_K")])
def test_hand_packed_known_answers(cuda, case, fmt):
    announce("dequant golden", case)
    expected = FV[case + "_expected"]
    w = PackedGGUFWeight(FV[case + "_blocks"], (1, expected.size), fmt)
    got = upload(w, cuda).dequantize().cpu().numpy()
    np.testing.assert_array_equal(got.ravel(), expected)


@pytest.mark.parametrize("fmt", ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K"])
def test_reference_native_decoder_vectors(cuda, fmt):
    announce("dequant ref vectors", fmt)
    dense = RV[fmt + "_dense"]
    w = PackedGGUFWeight(RV[fmt + "_blocks"], dense.shape, fmt)
    np.testing.assert_array_equal(upload(w, cuda).dequantize().cpu().numpy(), dense)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("shape", [(1, 256), (7, 512), (33, 2048), (64, 4096 + 256)])
def test_bit_exact_against_oracle_random_bytes(cuda, fmt, shape):
    # uniformly random bytes: every code, scale, sign and NaN/inf scale pattern occurs
    announce("dequant random bytes", fmt, shape)
    raw = np.random.default_rng(hash((fmt, shape)) % 2 ** 32).integers(0, 256, R.packed_nbytes(shape, fmt), dtype=np.uint8)
    with np.errstate(all="ignore"):
        want = bits(R.dequantize(raw, shape, fmt))
    got = bits(upload(PackedGGUFWeight(raw, shape, fmt), cuda).dequantize().cpu().numpy())
    nan_w, nan_g = (want & 0x7FFFFFFF) > 0x7F800000, (got & 0x7FFFFFFF) > 0x7F800000
    np.testing.assert_array_equal(nan_g, nan_w)
    # bit patterns, so that signed zeros count
    np.testing.assert_array_equal(got[~nan_g], want[~nan_w])


@pytest.mark.parametrize("fmt,shape", [("Q8_0", (5, 32)), ("Q8_0", (3, 96)), ("Q4_0", (5, 32)), ("BF16", (3, 7)),
                                       ("BF16", (2, 1)), ("Q8_0", (4, 224))])
def test_rows_that_are_not_unit_aligned(cuda, fmt, shape):
    announce("dequant ragged", fmt, shape)
    w = synthetic.packed_weight(fmt, shape, 3)
    want = R.dequantize(w.data, shape, fmt)
    got = upload(w, cuda).dequantize().cpu().numpy()
    np.testing.assert_array_equal(bits(got), bits(want))


def test_bf16_every_bit_pattern(cuda):
    words = np.arange(65536, dtype="<u2")
    w = PackedGGUFWeight(words.view(np.uint8), (256, 256), "BF16")
    got = upload(w, cuda).dequantize().cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32).ravel(), words.astype(np.uint32) << 16)


def test_bf16_byte_fixture(cuda):
    w = PackedGGUFWeight(FV["bf16_bytes_blocks"], (2, 3), "BF16")
    got = upload(w, cuda).dequantize().cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32).ravel(), FV["bf16_bytes_expected_bits"])


def test_expert_view_of_a_bank_is_offset_aligned(cuda):
    # a select_outer view lands at a block-multiple offset that need not be 16-byte aligned
    bank = synthetic.packed_weight("Q6_K", (3, 5, 256), 8)
    dev = torch.from_numpy(bank.data.copy()).to(cuda)
    from mylocal_llm_amd.quantized_linear import DevicePackedGGUFWeight
    one = bank.select_outer(1)
    view = DevicePackedGGUFWeight(dev[one.nbytes:2 * one.nbytes], one.shape, "Q6_K")
    np.testing.assert_array_equal(bits(view.dequantize().cpu().numpy()), bits(R.dequantize(one.data, one.shape, "Q6_K")))


@pytest.mark.parametrize("fmt,shape", [("Q8_0", (4096, 4096)), ("Q6_K", (1024, 4096)), ("Q5_K", (1024, 4096)), ("Q4_K", (1024, 4096))])
def test_full_size_matrix_bit_exact(cuda, fmt, shape):
    announce("dequant full size", fmt, shape)
    w = synthetic.packed_weight(fmt, shape, 106)
    got = upload(w, cuda).dequantize().cpu().numpy()
    np.testing.assert_array_equal(bits(got), bits(R.dequantize(w.data, shape, fmt)))
