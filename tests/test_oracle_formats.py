"""Pins the CPU oracle's block decoders (oracle/reference_np.py, oracle/oracle.c) against the
reference's hand-packed known answers, its native C++ decoder's recorded outputs, the live
oracle/_ref build where present, and closed forms."""
import os

import numpy as np
import pytest

from oracle import native, reference_np as R
from mylocal_llm_amd import synthetic

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FV = np.load(os.path.join(GOLDEN, "format_vectors.npz"))
RV = np.load(os.path.join(GOLDEN, "ref_native_vectors.npz"))
PACKED = ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K"]


@pytest.mark.parametrize("case,fmt", [("q4_0_nibbles", "Q4_0"), ("q4_k_scales", "Q4_K"), ("q3_k_keep", "Q3_K"), ("q3_k_minus4", "Q3_K"),
                                      ("q5_k_group0", "Q5_K"), ("q5_k_group7", "Q5_K"),
                                      ("q6_k_all_codes", "Q6_K")])
@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_hand_packed_known_answers(case, fmt, impl):
    blocks, expected = FV[case + "_blocks"], FV[case + "_expected"]
    shape = (1, expected.size)
    fn = R.dequantize if impl == "numpy" else native.c_dequantize
    np.testing.assert_array_equal(fn(blocks, shape, fmt).ravel(), expected)


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_q8_0_closed_form_large_rows(impl):
    # q = row % 15 - 7 in every lane, d = 0.125 -> dense = 0.125 * q exactly
    rows = 4096
    q = np.broadcast_to((np.arange(rows) % 15 - 7).astype(np.int8)[:, None], (rows, 32)).copy()
    raw = np.concatenate((np.full((rows, 1), .125, "<f2").view(np.uint8), q.view(np.uint8)), axis=1).reshape(-1)
    fn = R.dequantize if impl == "numpy" else native.c_dequantize
    np.testing.assert_array_equal(fn(raw, (rows, 32), "Q8_0"), q.astype(np.float32) * np.float32(.125))


@pytest.mark.parametrize("fmt", PACKED)
def test_matches_reference_native_decoder_vectors(fmt):
    blocks, dense = RV[fmt + "_blocks"], RV[fmt + "_dense"]
    np.testing.assert_array_equal(R.dequantize(blocks, dense.shape, fmt), dense)
    np.testing.assert_array_equal(native.c_dequantize(blocks, dense.shape, fmt), dense)


@pytest.mark.parametrize("fmt", PACKED)
def test_matches_live_reference_build(fmt):
    if native.load_ref() is None:
        pytest.skip("oracle/_ref not built in this environment")
    w = synthetic.packed_weight(fmt, (5, 768 if fmt in ("Q8_0", "Q4_0") else 512), 31)
    k = w.shape[1]
    dense = native.ref_gemv(np.eye(k, dtype=np.float32), w.data, w.shape, fmt).T
    np.testing.assert_array_equal(R.dequantize(w.data, w.shape, fmt), dense)


@pytest.mark.parametrize("fmt", PACKED + ["BF16"])
def test_numpy_and_c_restatements_agree_bitwise(fmt):
    rng = np.random.default_rng(7)
    elems, nbytes = R.BLOCKS[fmt]
    shape = (3, 4 * max(elems, 64))
    raw = rng.integers(0, 256, R.packed_nbytes(shape, fmt), dtype=np.uint8)
    a = R.dequantize(raw, shape, fmt).view(np.uint32)
    b = native.c_dequantize(raw, shape, fmt).view(np.uint32)
    # random bytes include NaN/inf scales: compare bit patterns, treating every NaN alike
    nan_a, nan_b = (a & 0x7FFFFFFF) > 0x7F800000, (b & 0x7FFFFFFF) > 0x7F800000
    np.testing.assert_array_equal(nan_a, nan_b)
    np.testing.assert_array_equal(a[~nan_a], b[~nan_b])


def test_fp16_scale_subnormals_and_specials():
    halves = np.array([0x0001, 0x03FF, 0x0400, 0x8001, 0x7BFF, 0x7C00, 0xFC00, 0x0000, 0x8000], "<u2")
    blocks = np.zeros((halves.size, 34), np.uint8)
    blocks[:, 0:2] = halves.view(np.uint8).reshape(-1, 2)
    blocks[:, 2] = 1
    expect = halves.view("<f2").astype(np.float32)
    for fn in (R.dequantize, native.c_dequantize):
        got = fn(blocks, (halves.size, 32), "Q8_0")[:, 0]
        np.testing.assert_array_equal(got.view(np.uint32), expect.view(np.uint32))


def test_signed_zero_follows_float_operation_order():
    # Q6_K: (d*sc)*q with sc<0, q=0 is -0.0; an integer sc*q product would lose the sign.
    raw = np.zeros(210, np.uint8)
    raw[0:128] = 0x00
    raw[128:192] = 0xAA  # high bits 2 -> code 32 -> q = 0
    raw[192:208] = np.full(16, -3, np.int8).view(np.uint8)
    raw[208:210] = np.array([0.5], "<f2").view(np.uint8)
    for fn in (R.dequantize, native.c_dequantize):
        got = fn(raw, (1, 256), "Q6_K").view(np.uint32)
        assert np.all(got == 0x80000000)


@pytest.mark.parametrize("storage", ["bytes", "<u2", ">u2"])
def test_bf16_all_bit_patterns(storage):
    words = np.arange(65536, dtype=np.uint16)
    data = words.astype("<u2").view(np.uint8) if storage == "bytes" else words.astype(storage)
    got = R.bf16_expand(data)
    np.testing.assert_array_equal(got.view(np.uint32), words.astype(np.uint32) << 16)
    if storage == "bytes":
        np.testing.assert_array_equal(native.c_dequantize(data, (256, 256), "BF16").view(np.uint32).ravel(),
                                      words.astype(np.uint32) << 16)


def test_bf16_byte_fixture_and_rejections():
    got = R.bf16_expand(FV["bf16_bytes_blocks"])
    np.testing.assert_array_equal(got.view(np.uint32), FV["bf16_bytes_expected_bits"])
    with pytest.raises(ValueError):
        R.bf16_expand(np.zeros(4, np.float16))


def test_bf16_round_is_nearest_even_and_inverts_expand():
    words = np.arange(65536, dtype=np.uint16)
    vals = R.bf16_expand(words)
    finite = np.isfinite(vals)
    np.testing.assert_array_equal(R.bf16_round(vals)[finite], words[finite])
    # halfway cases: 1 + 2^-8 rounds to even (1.0), 1 + 3*2^-8 rounds up to 1 + 2^-6
    x = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8], np.float32)
    np.testing.assert_array_equal(R.bf16_round(x), np.array([0x3F80, 0x3F82], np.uint16))


def test_shape_and_length_errors():
    with pytest.raises(ValueError, match="innermost"):
        R.packed_nbytes((2, 100), "Q8_0")
    with pytest.raises(ValueError, match="expected"):
        R.dequantize(np.zeros(33, np.uint8), (1, 32), "Q8_0")


@pytest.mark.parametrize("fmt", PACKED)
def test_generators_respect_described_ranges(fmt):
    w = synthetic.packed_weight(fmt, (4, 1024), 5)
    dense = R.dequantize(w.data, w.shape, fmt)
    assert np.isfinite(dense).all()
    blk = w.data.reshape(-1, R.BLOCKS[fmt][1])
    if fmt == "Q8_0":
        q = blk[:, 2:].view(np.int8)
        assert q.min() >= -127 and abs(float(q.std()) - 40) < 3
        d = np.ascontiguousarray(blk[:, :2]).view("<f2").astype(np.float32)
        assert abs(float(d.mean()) - 5e-4) < 5e-5 and (d > 0).all()
    if fmt == "Q6_K":
        sc = blk[:, 192:208].view(np.int8)
        assert sc.min() >= -64 and sc.max() <= 63
