"""Host twins of the packed operators (scalar C++ inside the library, no GPU needed).

Checked against the reference's own native vectors (tests/golden/ref_native_vectors.npz, outputs
of the reference's C++ backend), against the restatement under oracle/ at the tolerance of the
reference's native-vs-NumPy test (rtol 3e-5, atol 2e-4 at unit scale), and for the thread
behaviour its test suite pins (tests/test_0106e_cpu_packed_and_gpu_swaps.py:78-88: four threads,
twelve calls each, bit-identical results).
"""
import ctypes
import os
import threading

import numpy as np
import pytest

from mylocal_llm_amd import _lib, synthetic
from mylocal_llm_amd.native_packed_cpu import packed_cpu_expert, packed_cpu_linear, router_topk_cpu
from mylocal_llm_amd.quantized_linear import PackedExpertFFNInference, quantized_linear, quantized_swiglu
from mylocal_llm_amd.quantized_weight import PackedGGUFWeight
from oracle import reference_np as R

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
RV = np.load(os.path.join(GOLDEN, "ref_native_vectors.npz"))
FV = np.load(os.path.join(GOLDEN, "format_vectors.npz"))
FORMATS = ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K", "BF16"]


def triple(w):
    return w.data, w.shape, w.quant_type


@pytest.mark.parametrize("fmt", [f for f in FORMATS if f != "BF16"])
def test_linear_matches_reference_native_gemv_vectors(fmt):
    blocks, x, y = RV[fmt + "_blocks"], RV[fmt + "_x"], RV[fmt + "_gemv"]
    w = PackedGGUFWeight(blocks.reshape(-1), (y.shape[1], x.shape[1]), fmt)
    scale = max(np.abs(y).max(), 1)
    np.testing.assert_allclose(quantized_linear(x, w), y, rtol=3e-5, atol=2e-4 * scale)
    np.testing.assert_allclose(packed_cpu_linear(x, w, backend="native"), y, rtol=3e-5, atol=2e-4 * scale)


def test_expert_matches_reference_native_expert_vector():
    d, f = RV["expert_x"].shape[1], RV["expert_gate"].shape[0] * 256 // RV["expert_x"].shape[1]
    gate = PackedGGUFWeight(RV["expert_gate"].reshape(-1), (f, d), "Q5_K")
    up = PackedGGUFWeight(RV["expert_up"].reshape(-1), (f, d), "Q5_K")
    down = PackedGGUFWeight(RV["expert_down"].reshape(-1), (d, f), "Q6_K")
    expect = RV["expert_out"]
    scale = np.abs(expect).max()
    np.testing.assert_allclose(packed_cpu_expert(RV["expert_x"], (gate, up, down)), expect, rtol=3e-5, atol=2e-4 * scale)
    for fuse in (True, False):
        got = PackedExpertFFNInference(gate, up, down, fuse_gate_up=fuse).forward(RV["expert_x"])
        np.testing.assert_allclose(got, expect, rtol=3e-5, atol=2e-4 * scale)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_linear_against_the_restatement(fmt, dtype):
    w = synthetic.packed_weight(fmt, (37, 768), 11)
    x = synthetic.activations((2, 3, 768), 12, np.float32).astype(dtype)
    got = quantized_linear(x, w)
    want = R.linear(x, *triple(w))
    assert got.dtype == dtype and got.shape == (2, 3, 37)
    scale = max(np.abs(want.astype(np.float64)).max(), 1)
    if dtype == np.float16:   # one rounding to fp16 of sums that agree to 3e-5
        np.testing.assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=2e-3 * scale)
    else:
        np.testing.assert_allclose(got, want, rtol=3e-5, atol=2e-4 * scale)


KNOWN = [("q4_0_nibbles", "Q4_0"), ("q4_k_scales", "Q4_K"), ("q3_k_keep", "Q3_K"), ("q3_k_minus4", "Q3_K"),
         ("q5_k_group0", "Q5_K"), ("q5_k_group7", "Q5_K"), ("q6_k_all_codes", "Q6_K")]


@pytest.mark.parametrize("case,fmt", KNOWN)
def test_hand_packed_known_answers(case, fmt):
    """A unit matrix as activations turns the linear into the decoder: one hand-packed block per
    case, every decoded weight bit-exact (1 * w plus exact zeros)."""
    blocks, expected = FV[case + "_blocks"], FV[case + "_expected"]
    k = expected.size
    got = quantized_linear(np.eye(k, dtype=np.float32), PackedGGUFWeight(blocks, (1, k), fmt))[:, 0]
    np.testing.assert_array_equal(got, expected)


@pytest.mark.parametrize("fmt", FORMATS)
def test_decoded_weights_are_those_of_the_reference_decoder(fmt):
    k = 512
    w = synthetic.packed_weight(fmt, (5, k), 21)
    dense = R.dequantize(*triple(w))
    assert np.all(np.isfinite(dense))
    np.testing.assert_array_equal(quantized_linear(np.eye(k, dtype=np.float32), w).T, dense)


@pytest.mark.parametrize("fmt", ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K", "BF16"])
def test_container_reference_helpers_are_host_functions(fmt):
    """PackedGGUFWeight.dequantize_reference / dequantize_rows_reference / matvec_reference keep the
    reference's names, arguments and errors (quantized_weight.py:101-250); the arithmetic is the
    library's host decoder and matches the oracle bit for bit (matvec: to fp32 rounding)."""
    w = synthetic.packed_weight(fmt, (3, 40, 512), 77)
    dense = R.dequantize(w.data, w.shape, fmt)
    np.testing.assert_array_equal(w.dequantize_reference().view(np.uint32), dense.view(np.uint32))
    one = w.select_outer(1)
    idx = np.array([39, 0, 7, 7, 12], np.int64)
    rows = one.dequantize_rows_reference(idx, tile_rows=2)
    np.testing.assert_array_equal(rows.view(np.uint32), dense[1][idx].view(np.uint32))
    x = synthetic.activations((512,), 78)
    y = one.matvec_reference(x, tile_rows=16)
    want = R.linear(x[None], one.data, one.shape, fmt)[0]
    assert y.shape == (40,) and y.dtype == np.float32
    assert np.linalg.norm(y - want) <= 2e-6 * np.linalg.norm(want)
    with pytest.raises(ValueError, match="matrix"):
        w.matvec_reference(x)
    with pytest.raises(ValueError, match="tile_rows"):
        one.matvec_reference(x, tile_rows=0)
    with pytest.raises(ValueError, match="vector shape"):
        one.matvec_reference(x[:-1])
    with pytest.raises(IndexError):
        one.dequantize_rows_reference(np.array([40]))
    with pytest.raises(ValueError, match="integer"):
        one.dequantize_rows_reference(np.array([0.5]))



def test_swiglu_mixed_formats_and_shapes():
    gate = synthetic.packed_weight("Q4_K", (48, 512), 3)
    up = synthetic.packed_weight("Q6_K", (48, 512), 4)
    x = synthetic.activations((5, 512), 5)
    want = R.swiglu(x, triple(gate), triple(up))
    got = quantized_swiglu(x, gate, up)
    np.testing.assert_allclose(got, want, rtol=3e-5, atol=2e-4 * max(np.abs(want).max(), 1))
    assert quantized_swiglu(x.astype(np.float16).reshape(1, 5, 512), gate, up).shape == (1, 5, 48)
    # large gates: the sigmoid neither overflows nor produces NaN
    big = np.full((1, 512), 200.0, np.float32)
    assert np.all(np.isfinite(quantized_swiglu(big, gate, up)) | np.isinf(quantized_swiglu(big, gate, up)))
    assert not np.any(np.isnan(quantized_swiglu(-big, gate, up)))


def test_empty_batch_and_errors():
    w = synthetic.packed_weight("Q8_0", (4, 64), 1)
    assert quantized_linear(np.zeros((0, 64), np.float32), w).shape == (0, 4)
    with pytest.raises(TypeError, match="FP16/FP32/FP64"):
        quantized_linear(np.zeros((2, 64), np.int32), w)
    with pytest.raises(ValueError, match="Input K"):
        quantized_linear(np.zeros((2, 32), np.float32), w)
    with pytest.raises(ValueError, match="Expected x"):
        quantized_linear(np.zeros(64, np.float32), w)
    with pytest.raises(ValueError, match="cpu_packed_backend"):
        quantized_linear(np.zeros((2, 64), np.float32), w, cpu_packed_backend="fast")
    with pytest.raises(TypeError, match="NumPy"):
        quantized_linear([[0.0] * 64], w)
    with pytest.raises(TypeError):
        packed_cpu_expert(np.zeros((1, 64), np.float32), (w, w))
    with pytest.raises(ValueError, match="projection shapes"):
        packed_cpu_expert(np.zeros((1, 64), np.float32), (w, w, w))


def test_abi_status_codes_of_the_twins():
    lib = _lib.load()
    null, fake = ctypes.c_void_p(0), ctypes.c_void_p(4096)   # never dereferenced: validation fails first
    assert lib.qmoe_linear_cpu(null, 0, 4, 32, fake, 1, fake) == 1
    assert lib.qmoe_linear_cpu(fake, 0, 4, 33, fake, 1, fake) == 1
    assert lib.qmoe_linear_cpu(fake, 0, 4, 32, fake, 0, fake) == 1
    assert lib.qmoe_linear_cpu(fake, 42, 4, 32, fake, 1, fake) == 2
    assert b"format 42" in lib.qmoe_last_error()
    assert lib.qmoe_swiglu_cpu(fake, 0, null, 0, 4, 32, fake, 1, fake) == 1
    assert lib.qmoe_expert_cpu(fake, 0, fake, 0, fake, 5, 32, 32, fake, 1, fake) == 1     # Q6_K down needs d_ff % 256 == 0
    assert lib.qmoe_router_topk_cpu(fake, 1, 4, 5, 1.0, 0, fake, fake) == 1
    assert lib.qmoe_router_topk_cpu(fake, 1, 4, 2, 0.0, 1, fake, fake) == 1


@pytest.mark.parametrize("i", range(7))
def test_router_tie_inf_nan_fixtures(i):
    row, ids = FV[f"router_row{i}"], FV[f"router_row{i}_ids"]
    k = min(4, row.size)
    w, got = router_topk_cpu(row[None], k, floor=2.0 ** -14, renormalize=True)
    np.testing.assert_array_equal(got[0], ids[:k])
    want_w, want_ids = R.router_topk(row[None], k, floor=2.0 ** -14)
    np.testing.assert_array_equal(got, want_ids)
    np.testing.assert_allclose(w, want_w, rtol=2e-6, atol=1e-30, equal_nan=True)


@pytest.mark.parametrize("renormalize", [False, True])
def test_router_random_rows(renormalize):
    logits = np.random.default_rng(7).standard_normal((3, 17, 96)).astype(np.float32) * 3
    w, ids = router_topk_cpu(logits, 8, floor=2.0 ** -14, renormalize=renormalize)
    want_w, want_ids = R.router_topk(logits, 8, renormalize=renormalize, floor=2.0 ** -14)
    assert w.shape == (3, 17, 8) and ids.dtype == np.int64
    np.testing.assert_array_equal(ids, want_ids)
    np.testing.assert_allclose(w, want_w, rtol=2e-6)


def test_expert_topk_forward_takes_numpy_logits():
    from mylocal_llm_amd.router import expert_topk_forward
    logits = np.random.default_rng(3).standard_normal((2, 5, 40)).astype(np.float32)
    w, ids, cache = expert_topk_forward(logits, 4)
    want_w, want_ids = R.router_topk(logits, 4, renormalize=False)
    assert cache is None
    np.testing.assert_array_equal(ids, want_ids)
    np.testing.assert_allclose(w, want_w, rtol=2e-6)
    with pytest.raises(ValueError, match="1 <= k"):
        expert_topk_forward(logits, 41)


def test_four_threads_twelve_calls_each_bit_identical():
    gate = synthetic.packed_weight("Q5_K", (64, 256), 1)
    up = synthetic.packed_weight("Q5_K", (64, 256), 2)
    down = synthetic.packed_weight("Q8_0", (256, 64), 3)
    w = synthetic.packed_weight("Q6_K", (96, 256), 4)
    x = synthetic.activations((3, 256), 5)
    want_linear = packed_cpu_linear(x, w)
    want_expert = packed_cpu_expert(x, (gate, up, down))
    failures = []

    def work():
        for _ in range(12):
            if not np.array_equal(packed_cpu_linear(x, w), want_linear):
                failures.append("linear")
            if not np.array_equal(packed_cpu_expert(x, (gate, up, down)), want_expert):
                failures.append("expert")

    threads = [threading.Thread(target=work) for _ in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures
