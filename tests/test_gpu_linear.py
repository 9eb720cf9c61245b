"""GPU linear / SwiGLU / expert parity through the C ABI against the CPU oracle."""
import os

import numpy as np
import pytest
import torch

from oracle import native, reference_np as R
from mylocal_llm_amd import synthetic
from mylocal_llm_amd.quantized_weight import PackedGGUFWeight
from mylocal_llm_amd.quantized_linear import (
    PackedExpertFFNInference, quantized_linear, quantized_linear_batch, quantized_swiglu,
)
from gpu_util import BF16_MAX_ABS, REL_L2, announce, rel_l2, triple, upload

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
RV = np.load(os.path.join(GOLDEN, "ref_native_vectors.npz"))
FORMATS = ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K", "BF16"]


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m", [1, 2, 4, 5, 16, 64])
def test_linear_matches_oracle(cuda, fmt, m):
    announce("linear", fmt, "M", m)
    w = synthetic.packed_weight(fmt, (96, 1024), 106)
    x = synthetic.activations((m, 1024), 103)
    want = R.linear(x, *triple(w))
    got = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    assert got.shape == (m, 96) and got.dtype == np.float32
    # more than one token runs on MFMA with weights and fp32 activations each split into two
    # bf16 terms (16 significant bits): still two orders of magnitude inside the 1e-3 bar
    tol = 2e-5 if m > 1 else 2e-6
    assert rel_l2(got, want) <= tol <= REL_L2
    np.testing.assert_allclose(got, native.c_linear(x, *triple(w)), rtol=10 * tol, atol=10 * tol * np.abs(want).max())


def test_config0_single_q8_0_matrix_batch1(cuda):
    # benchmark configuration 0: 2048 x 2048 Q8_0, fp32 [1, 2048]
    w = synthetic.packed_weight("Q8_0", (2048, 2048), 106)
    x = synthetic.activations((1, 2048), 103)
    want = R.linear(x, *triple(w))
    got = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    assert rel_l2(got, want) <= 2e-6
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("fmt", ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K"])
def test_linear_reference_native_vectors(cuda, fmt):
    blocks, x, y = RV[fmt + "_blocks"], RV[fmt + "_x"], RV[fmt + "_gemv"]
    w = PackedGGUFWeight(blocks, (y.shape[1], x.shape[1]), fmt)
    got = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    np.testing.assert_allclose(got, y, rtol=3e-5, atol=2e-4 * max(np.abs(y).max(), 1))


@pytest.mark.parametrize("rows", [65536, 151936])
@pytest.mark.parametrize("tokens", [1, 2])
def test_large_output_projection_exact(cuda, rows, tokens):
    # every partial sum is exactly representable, so any summation order must give equality
    announce("linear large N", rows, tokens)
    q = np.broadcast_to((np.arange(rows, dtype=np.int64) % 15 - 7).astype(np.int8)[:, None], (rows, 32)).copy()
    raw = np.concatenate((np.full((rows, 1), .125, "<f2").view(np.uint8), q.view(np.uint8)), axis=1).reshape(-1)
    w = PackedGGUFWeight(raw, (rows, 32), "Q8_0")
    hidden = np.stack([(np.arange(32, dtype=np.float32) + t) / 32 for t in range(tokens)])
    expected = hidden.sum(axis=1, keepdims=True) * (q[:, 0].astype(np.float32) * .125)[None]
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        got = quantized_linear(torch.from_numpy(hidden).to(cuda), upload(w, cuda))
    stream.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy(), expected)


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, BF16_MAX_ABS)])
@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K", "BF16"])
def test_linear_low_precision_activations(cuda, dtype, tol, fmt):
    announce("linear lowp", fmt, dtype)
    w = synthetic.packed_weight(fmt, (64, 512), 7)
    x = torch.from_numpy(synthetic.activations((3, 512), 5)).to(dtype)
    # oracle on the exactly representable upcast inputs; output rounded once to the dtype
    want = R.linear(x.float().numpy(), *triple(w))
    got = quantized_linear(x.to(cuda), upload(w, cuda))
    assert got.dtype == dtype
    want_rounded = torch.from_numpy(want).to(dtype).float().numpy()
    # one rounding to the output type: within an ulp of the rounded oracle value
    assert np.abs(got.float().cpu().numpy() - want_rounded).max() <= tol * max(1.0, float(np.abs(want).max()))
    assert rel_l2(got.float().cpu().numpy(), want) <= (5e-3 if dtype == torch.bfloat16 else 1e-3)


@pytest.mark.parametrize("shape", [(70, 320), (130, 1408), (64, 64), (200, 2112), (1, 4096)])
@pytest.mark.parametrize("tokens,dtype", [(3, "f32"), (17, "f32"), (40, "bf16"), (33, "f16")])
def test_q8_0_token_batches_ragged_rows(cuda, shape, tokens, dtype):
    """Q8_0 token batches take weight tiles of 64 or 128 rows x 256 columns through LDS: rows whose
    width ends inside a tile (320, 1408, 64, 2112 columns), row counts that end inside a tile, and
    a last row that ends the allocation, so nothing may be read behind it."""
    announce("linear q8_0 ragged", shape, tokens, dtype)
    w = synthetic.packed_weight("Q8_0", shape, 311)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    x = torch.from_numpy(synthetic.activations((tokens, shape[1]), 312)).to(tdt)
    want = R.linear(x.float().numpy(), *triple(w))
    got = quantized_linear(x.to(cuda), upload(w, cuda))
    assert got.dtype == tdt and got.shape == (tokens, shape[0])
    tol = {"f32": 2e-5, "f16": 1e-3, "bf16": 5e-3}[dtype]   # fp16 / bf16: the one rounding of the output
    assert rel_l2(got.float().cpu().numpy(), want) <= tol
    if dtype == "f32":
        assert tol <= REL_L2


@pytest.mark.parametrize("shape", [(1030, 1024), (257, 3072), (4096, 4096), (3, 2048), (4096, 14336), (130, 8192), (66, 16384), (97, 5120)])
@pytest.mark.parametrize("tokens,dtype", [(2, "f32"), (3, "bf16"), (4, "f32"), (4, "f16")])
def test_q8_0_two_to_four_tokens_streamed(cuda, shape, tokens, dtype):
    """Rows of 1024..16384 columns at 2..4 tokens take the streamed 4x4x4-MFMA kernel: every chunk
    count of the four-wave form (up to 4096 columns), the eight-wave form with one or two chunks a
    wave beyond, row counts that are not a multiple of four, every activation type; a batch of such
    problems equals the separate calls bit for bit."""
    announce("linear few tokens", shape, tokens, dtype)
    n, k = shape
    w = synthetic.packed_weight("Q8_0", (n, k), 411)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    xd = torch.from_numpy(synthetic.activations((tokens, k), 412, "bf16")).to(cuda).to(tdt)
    x = xd.float().cpu().numpy()
    want = R.linear(x, *triple(w))
    wd = upload(w, cuda)
    got = quantized_linear(xd, wd)
    assert got.dtype == tdt and got.shape == (tokens, n)
    g = got.float().cpu().numpy()
    if dtype == "f32":
        assert rel_l2(g, want) <= 2e-5 <= REL_L2
    else:
        assert np.abs(g - want).max() <= (BF16_MAX_ABS if dtype == "bf16" else 2e-3) * max(1.0, np.abs(want).max())
    w2 = synthetic.packed_weight("Q8_0", (64, k), 413)
    both = quantized_linear_batch([(xd, wd), (xd, upload(w2, cuda))])
    assert torch.equal(both[0], got)
    assert rel_l2(both[1].float().cpu().numpy(), R.linear(x, *triple(w2))) <= (2e-5 if dtype == "f32" else 5e-3)


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "BF16"])
@pytest.mark.parametrize("k", [18432, 32768])
@pytest.mark.parametrize("tokens", [1, 3, 20])
def test_rows_longer_than_the_streaming_kernel_takes(cuda, fmt, k, tokens):
    """Rows of more than 16384 columns (the down projections of 70B-class models): the token-tile
    GEMM has no row-length limit; one token goes there too (Q8_0) or to the general kernel."""
    announce("linear long rows", fmt, k, tokens)
    w = synthetic.packed_weight(fmt, (70, k), 411)
    x = synthetic.activations((tokens, k), 412)
    want = R.linear(x, *triple(w))
    got = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    assert rel_l2(got, want) <= 2e-5 <= REL_L2


def test_linear_three_dimensional_input_and_shape_errors(cuda):
    w = upload(synthetic.packed_weight("Q4_K", (7, 512), 1), cuda)
    x = torch.from_numpy(synthetic.activations((2, 3, 512), 2)).to(cuda)
    y = quantized_linear(x, w)
    assert y.shape == (2, 3, 7)
    np.testing.assert_array_equal(y.reshape(6, 7).cpu().numpy(), quantized_linear(x.reshape(6, 512), w).cpu().numpy())
    with pytest.raises(ValueError, match="Input K"):
        quantized_linear(torch.zeros((2, 128), device=cuda), w)
    with pytest.raises(ValueError, match="Expected x"):
        quantized_linear(torch.zeros((512,), device=cuda), w)
    with pytest.raises(ValueError, match="block_k"):
        quantized_linear(x, w, block_k=128)
    with pytest.raises(ValueError, match="contiguous"):
        quantized_linear(torch.zeros((2, 1024), device=cuda)[:, ::2], w)
    with pytest.raises(TypeError, match="FP16"):
        quantized_linear(torch.zeros((2, 512), device=cuda, dtype=torch.float64), w)
    assert quantized_linear(torch.zeros((0, 512), device=cuda), w).shape == (0, 7)
    # host and device operands do not mix: neither side is moved or dequantised behind the caller's back
    host = synthetic.packed_weight("Q4_K", (7, 512), 1)
    with pytest.raises(TypeError, match="NumPy input"):
        quantized_linear(x, host)
    with pytest.raises(TypeError, match="host PackedGGUFWeight"):
        quantized_linear(x.cpu().numpy(), w)
    with pytest.raises(TypeError, match="NumPy activations"):
        quantized_swiglu(x, host, host)
    with pytest.raises(TypeError, match="CUDA tensors"):
        quantized_swiglu(x.cpu().numpy(), w, w)
    # and the host twin agrees with the device kernel on the same operands
    np.testing.assert_allclose(quantized_linear(x.cpu().numpy(), host), y.cpu().numpy(), rtol=3e-5, atol=2e-4)


def test_linear_inputs_and_weights_are_not_mutated(cuda):
    w = synthetic.packed_weight("Q6_K", (16, 512), 1)
    dev = upload(w, cuda)
    x = torch.from_numpy(synthetic.activations((2, 512), 2)).to(cuda)
    before = x.clone()
    quantized_linear(x, dev)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(dev.data.cpu().numpy(), w.data)
    assert torch.equal(x, before)


@pytest.mark.parametrize("tokens", [1, 2, 40])
def test_linear_batch_equals_separate_calls(cuda, tokens):
    """One token: the batch shares the streaming launch and is bit-identical to separate calls.
    Token batches may take a different MFMA tiling in a batch than alone (same operand
    splitting, another summation order): equal to the oracle's tolerance, and against the oracle."""
    hosts = [synthetic.packed_weight(f, (n, 512), i) for i, (f, n) in enumerate([("Q8_0", 64), ("Q6_K", 32), ("Q5_K", 16), ("Q8_0", 200)])]
    ws = [upload(w, cuda) for w in hosts]
    xh = synthetic.activations((tokens, 512), 9)
    x = torch.from_numpy(xh).to(cuda)
    outs = quantized_linear_batch([(x, w) for w in ws])
    for out, w, host in zip(outs, ws, hosts):
        alone = quantized_linear(x, w)
        if tokens == 1:
            assert torch.equal(out, alone)
        else:
            assert rel_l2(out.cpu().numpy(), alone.cpu().numpy()) <= 2e-5
        assert rel_l2(out.cpu().numpy(), R.linear(xh, *triple(host))) <= 2e-5 <= REL_L2


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K", "BF16"])
@pytest.mark.parametrize("tokens,dtype", [(5, "f32"), (40, "f32"), (17, "f16"), (33, "bf16")])
def test_linear_batch_token_batches_long_rows(cuda, fmt, tokens, dtype):
    """Token batches through one batched launch: rows of 8192 and 14336 columns (split over the
    waves of a workgroup), a short matrix beside them, row counts that are not multiples of the
    row tiles, token counts that end in a partly filled tile, all activation types."""
    announce("linear batch long rows", fmt, tokens, dtype)
    shapes = [(160, 8192), (100, 1024), (72, 14336), (16, 4096)]
    hosts = [synthetic.packed_weight(fmt, shp, 700 + i) for i, shp in enumerate(shapes)]
    ws = [upload(w, cuda) for w in hosts]
    xs_host = [synthetic.activations((tokens, k), 800 + i) for i, (_, k) in enumerate(shapes)]
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    xs = [torch.from_numpy(x).to(cuda).to(tdt) for x in xs_host]
    outs = quantized_linear_batch(list(zip(xs, ws)))
    for out, x, host, (n, _) in zip(outs, xs, hosts, shapes):
        assert out.shape == (tokens, n) and out.dtype == tdt
        want = R.linear(x.float().cpu().numpy(), *triple(host))
        if dtype == "f32":
            assert rel_l2(out.cpu().numpy(), want) <= 2e-5 <= REL_L2
        else:
            scale = max(1.0, float(np.abs(want).max()))
            tol = 2e-3 if dtype == "f16" else BF16_MAX_ABS
            assert np.abs(out.float().cpu().numpy() - want).max() <= tol * scale


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K", "BF16"])
@pytest.mark.parametrize("k", [512, 1024, 2048, 6144, 8192, 14336])
def test_single_token_streaming_every_row_width(cuda, fmt, k):
    """One token through the streaming kernel at every lane layout: 8 / 16 / 32 lanes per row,
    two and four waves per row (6144 / 8192 and 14336 columns), alone and as a batch whose
    problems have different widths; plus the fused gate/up pair at the same widths."""
    announce("stream widths", fmt, k)
    n = 72
    hosts = [synthetic.packed_weight(fmt, (n, k), 40 + i) for i in range(2)]
    x = synthetic.activations((1, k), 41)
    xd = torch.from_numpy(x).to(cuda)
    devs = [upload(w, cuda) for w in hosts]
    for host, dev in zip(hosts, devs):
        got = quantized_linear(xd, dev).cpu().numpy()
        assert rel_l2(got, R.linear(x, *triple(host))) <= 2e-6 <= REL_L2
    other = synthetic.packed_weight(fmt, (40, 4096), 44)
    xo = synthetic.activations((1, 4096), 45)
    outs = quantized_linear_batch([(xd, devs[0]), (torch.from_numpy(xo).to(cuda), upload(other, cuda)), (xd, devs[1])])
    assert rel_l2(outs[0].cpu().numpy(), R.linear(x, *triple(hosts[0]))) <= 2e-6
    assert rel_l2(outs[1].cpu().numpy(), R.linear(xo, *triple(other))) <= 2e-6
    assert rel_l2(outs[2].cpu().numpy(), R.linear(x, *triple(hosts[1]))) <= 2e-6
    h = quantized_swiglu(xd, devs[0], devs[1]).cpu().numpy()
    assert rel_l2(h, R.swiglu(x, triple(hosts[0]), triple(hosts[1]))) <= 5e-6 <= REL_L2


@pytest.mark.parametrize("gf,uf", [("Q8_0", "Q8_0"), ("Q5_K", "Q4_K"), ("Q6_K", "Q6_K"), ("Q5_K", "Q5_K"), ("Q4_K", "Q4_K"), ("BF16", "Q8_0")])
@pytest.mark.parametrize("m", [1, 3, 16])
def test_swiglu_fused_matches_oracle_and_unfused(cuda, gf, uf, m):
    announce("swiglu", gf, uf, m)
    gate, up = synthetic.packed_weight(gf, (128, 512), 1), synthetic.packed_weight(uf, (128, 512), 2)
    # scale activations so that gate pre-activations are O(1)
    x = synthetic.activations((m, 512), 3) * np.float32(2.0)
    want = R.swiglu(x, triple(gate), triple(up))
    dg, du = upload(gate, cuda), upload(up, cuda)
    xd = torch.from_numpy(x).to(cuda)
    got = quantized_swiglu(xd, dg, du).cpu().numpy()
    # token batches of one format multiply on MFMA with 16-bit operand splits
    assert rel_l2(got, want) <= (5e-6 if m == 1 else 2e-5) <= REL_L2
    g, u = quantized_linear(xd, dg), quantized_linear(xd, du)
    unfused = ((g / (1 + torch.exp(-g))) * u).cpu().numpy()
    np.testing.assert_allclose(got, unfused, rtol=3e-4, atol=2e-4 * np.abs(want).max())
    with pytest.raises(ValueError, match="gate/up"):
        quantized_swiglu(xd, dg, upload(synthetic.packed_weight(uf, (64, 512), 2), cuda))
    with pytest.raises(ValueError, match="K"):
        quantized_swiglu(torch.zeros((1, 256), device=cuda), dg, du)
    with pytest.raises(TypeError, match="packed"):
        quantized_swiglu(xd, dg, object())


@pytest.mark.parametrize("fmts", [("Q8_0", "Q8_0", "Q8_0"), ("Q5_K", "Q5_K", "Q6_K"), ("Q6_K", "Q6_K", "Q6_K"), ("Q4_K", "Q4_K", "Q4_K")])
@pytest.mark.parametrize("fuse", [True, False])
def test_packed_expert_matches_oracle(cuda, fmts, fuse):
    announce("expert", fmts, fuse)
    d, f = 512, 256
    gate, up, down = (synthetic.packed_weight(fmts[0], (f, d), 1), synthetic.packed_weight(fmts[1], (f, d), 2),
                      synthetic.packed_weight(fmts[2], (d, f), 3))
    x = synthetic.activations((3, d), 4)
    want = R.expert_ffn(x, triple(gate), triple(up), triple(down))
    expert = PackedExpertFFNInference(upload(gate, cuda), upload(up, cuda), upload(down, cuda), fuse_gate_up=fuse)
    got = expert.forward(torch.from_numpy(x).to(cuda)).cpu().numpy()
    assert rel_l2(got, want) <= 5e-5 <= REL_L2  # three tokens: MFMA path, 16-bit operand splits
    with pytest.raises(ValueError, match="transposed"):
        PackedExpertFFNInference(expert.gate, expert.up, expert.gate)


def test_expert_reference_native_vector(cuda):
    d = RV["expert_x"].shape[1]
    f = RV["expert_gate"].shape[0] * 256 // d
    gate = PackedGGUFWeight(RV["expert_gate"], (f, d), "Q5_K")
    up = PackedGGUFWeight(RV["expert_up"], (f, d), "Q5_K")
    down = PackedGGUFWeight(RV["expert_down"], (d, f), "Q6_K")
    expert = PackedExpertFFNInference(upload(gate, cuda), upload(up, cuda), upload(down, cuda))
    got = expert.forward(torch.from_numpy(RV["expert_x"]).to(cuda)).cpu().numpy()
    np.testing.assert_allclose(got, RV["expert_out"], rtol=3e-5, atol=2e-4 * np.abs(RV["expert_out"]).max())


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K", "BF16"])
@pytest.mark.parametrize("shape", [(4096, 4096), (1024, 4096), (4096, 14336)])
def test_8b_projection_shapes_linearity_and_row_checks(cuda, fmt, shape):
    """Full-size shapes: spot rows against the oracle plus linearity in x (size-independent)."""
    announce("linear 8B shape", fmt, shape)
    n, k = shape
    w = synthetic.packed_weight(fmt, (n, k), 106)
    dev = upload(w, cuda)
    rng = np.random.default_rng(103)
    x = rng.standard_normal((2, k), dtype=np.float32)
    xd = torch.from_numpy(x).to(cuda)
    y = quantized_linear(xd, dev)
    # linearity: W(a*x0 + b*x1) == a*W x0 + b*W x1 up to fp32 rounding
    combo = torch.from_numpy((0.5 * x[0] - 0.25 * x[1])[None]).to(cuda)
    yc = quantized_linear(combo, dev)
    lin = 0.5 * y[0] - 0.25 * y[1]
    assert rel_l2(yc[0].cpu().numpy(), lin.cpu().numpy()) <= 3e-5
    rows = rng.choice(n, 24, replace=False)
    sub = PackedGGUFWeight(w.data.reshape(n, -1)[rows].copy(), (len(rows), k), fmt)
    want = R.linear(x, *triple(sub))
    got = y.cpu().numpy()[:, rows]
    assert rel_l2(got, want) <= 3e-5  # two tokens: MFMA path, 16-bit operand splits


LAYER_8B = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K", "Q5_K", "Q4_K"])
def test_full_8b_layer_in_one_batch_single_token(cuda, fmt):
    """The benchmark's launch: the seven full-size projections of one layer through one
    qmoe_linear_batch call at M = 1, activations shared per data-flow group (q/k/v | o | gate/up |
    down).  Sampled rows of every problem against the oracle, the first and the last rows included;
    a second call must give the same bits (the launch leaves no state behind)."""
    announce("8B layer batch", fmt)
    rng = np.random.default_rng(103)
    xs = {name: torch.from_numpy(rng.standard_normal((1, k), dtype=np.float32)).to(cuda)
          for name, k in (("qkv", 4096), ("o", 4096), ("gateup", 4096), ("down", 14336))}
    groups = ["qkv", "qkv", "qkv", "o", "gateup", "gateup", "down"]
    weights = [synthetic.packed_weight(fmt, shape, 106 + i) for i, shape in enumerate(LAYER_8B)]
    problems = [(xs[g], upload(w, cuda)) for g, w in zip(groups, weights)]
    outs = quantized_linear_batch(problems)
    again = quantized_linear_batch(problems)
    for i, (w, (n, k)) in enumerate(zip(weights, LAYER_8B)):
        got = outs[i].cpu().numpy()
        assert got.shape == (1, n)
        assert np.array_equal(got.view(np.uint32), again[i].cpu().numpy().view(np.uint32))
        # whole stretches of rows across 64-row boundaries (the first and last 64 rows, 130 rows
        # around three boundaries inside the matrix) plus scattered single rows
        inner = [64 * int(b) for b in rng.choice(np.arange(2, n // 64 - 2), 3, replace=False)]
        rows = np.unique(np.concatenate([np.arange(64), np.arange(n - 64, n), rng.choice(n, 40, replace=False)]
                                        + [np.arange(b - 65, b + 65) for b in inner]))
        sub = PackedGGUFWeight(w.data.reshape(n, -1)[rows].copy(), (len(rows), k), fmt)
        want = R.linear(xs[groups[i]].cpu().numpy(), *triple(sub))
        assert rel_l2(got[:, rows], want) <= 2e-6, (i, n, k)
        np.testing.assert_allclose(got[:, rows], want, rtol=0, atol=2e-5 * np.abs(want).max())
        assert np.isfinite(got).all()


@pytest.mark.parametrize("fmt,tokens", [("Q8_0", 4), ("Q8_0", 16), ("Q8_0", 64), ("Q6_K", 16), ("Q5_K", 16)])
@pytest.mark.parametrize("shape", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)])
def test_8b_projection_shapes_at_small_token_counts(cuda, fmt, tokens, shape):
    """Every projection shape of the 8B layer, the wide gate/up one included, at the token counts
    the small-batch kernels are tuned for: sampled rows (first and last among them) against the
    oracle for every token."""
    announce("linear 8B shape small M", fmt, tokens, shape)
    n, k = shape
    w = synthetic.packed_weight(fmt, (n, k), 206)
    rng = np.random.default_rng(203)
    x = rng.standard_normal((tokens, k), dtype=np.float32)
    y = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    assert y.shape == (tokens, n) and np.isfinite(y).all()
    rows = np.unique(np.concatenate([[0, 1, n - 2, n - 1], rng.choice(n, 28, replace=False)]))
    sub = PackedGGUFWeight(w.data.reshape(n, -1)[rows].copy(), (len(rows), k), fmt)
    assert rel_l2(y[:, rows], R.linear(x, *triple(sub))) <= 3e-5


def test_four_host_threads_on_their_own_streams_give_identical_bits(cuda):
    """Four threads, each on a stream of its own, twelve calls each of the single-token and the
    small-batch linear: every result carries the bits of a single-threaded call (the reference pins
    the same for its native backend, tests/test_0106e_cpu_packed_and_gpu_swaps.py:78-88)."""
    import threading
    announce("threads x streams linear")
    w8 = upload(synthetic.packed_weight("Q8_0", (1024, 4096), 1), cuda)
    w6 = upload(synthetic.packed_weight("Q6_K", (512, 2048), 2), cuda)
    x1 = torch.from_numpy(synthetic.activations((1, 4096), 3)).to(cuda)
    x16 = torch.from_numpy(synthetic.activations((16, 2048), 4)).to(cuda)
    want1, want16 = quantized_linear(x1, w8), quantized_linear(x16, w6)
    want_batch = quantized_linear_batch([(x1, w8), (x1, w8)])
    torch.cuda.synchronize()
    failures = []

    def work():
        try:
            stream = torch.cuda.Stream(device=cuda)
            with torch.cuda.stream(stream):
                for _ in range(12):
                    a, b = quantized_linear(x1, w8), quantized_linear(x16, w6)
                    c = quantized_linear_batch([(x1, w8), (x1, w8)])
                    stream.synchronize()
                    if not (torch.equal(a, want1) and torch.equal(b, want16) and torch.equal(c[1], want_batch[1])):
                        failures.append("bits differ")
        except Exception as exc:          # surfaced below: a thread's exception is otherwise lost
            failures.append(repr(exc))

    threads = [threading.Thread(target=work) for _ in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[:3]


@pytest.mark.parametrize("shape", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("tokens", [1, 16])
def test_bf16_weights_at_the_8b_projection_shapes(cuda, shape, tokens):
    """BF16 weights ~ N(0, 0.02) at every projection shape of the 8B layer, one token and sixteen:
    stretches of rows (first, last, across a 64-row boundary) against the oracle for every token."""
    announce("linear 8B shape BF16", shape, tokens)
    n, k = shape
    w = synthetic.packed_weight("BF16", (n, k), 506)
    rng = np.random.default_rng(503)
    x = rng.standard_normal((tokens, k), dtype=np.float32)
    y = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    assert y.shape == (tokens, n) and np.isfinite(y).all()
    mid = 64 * (n // 128)
    rows = np.unique(np.concatenate([np.arange(40), np.arange(n - 40, n), np.arange(mid - 20, mid + 20), rng.choice(n, 24, replace=False)]))
    sub = PackedGGUFWeight(w.data.reshape(n, -1)[rows].copy(), (len(rows), k), "BF16")
    assert rel_l2(y[:, rows], R.linear(x, *triple(sub))) <= (2e-6 if tokens == 1 else 3e-5)


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6_K"])
def test_output_projection_of_the_vocabulary_at_full_shape(cuda, fmt):
    """The output projection of the reference's model at its real shape, 151 936 x 2048
    (mini_llm/external/qwen3next_model.py:291-293), one token: 311 M weights through the
    single-token streaming kernel; stretches of rows at the start, across the middle and up to the
    very last row against the oracle, and every output finite."""
    announce("linear vocabulary projection", fmt)
    n, k = 151936, 2048
    w = synthetic.packed_weight(fmt, (n, k), 606)
    rng = np.random.default_rng(603)
    x = rng.standard_normal((1, k), dtype=np.float32)
    y = quantized_linear(torch.from_numpy(x).to(cuda), upload(w, cuda)).cpu().numpy()
    assert y.shape == (1, n) and np.isfinite(y).all()
    rows = np.unique(np.concatenate([np.arange(70), np.arange(n - 70, n), np.arange(n // 2 - 35, n // 2 + 35),
                                     rng.choice(n, 200, replace=False)]))
    sub = PackedGGUFWeight(w.data.reshape(n, -1)[rows].copy(), (len(rows), k), fmt)
    want = R.linear(x, *triple(sub))
    assert rel_l2(y[:, rows], want) <= 2e-6
    np.testing.assert_allclose(y[:, rows], want, rtol=0, atol=2e-5 * np.abs(want).max())
