"""Pins the oracle's operators (linear, SwiGLU, expert, router, dispatch/combine, MoE step)
against closed forms, brute-force fp64 loops, the reference's recorded native outputs and its
router / ordered-sum fixtures."""
import os

import numpy as np
import pytest

from oracle import native, reference_np as R
from mylocal_llm_amd import synthetic

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FV = np.load(os.path.join(GOLDEN, "format_vectors.npz"))
RV = np.load(os.path.join(GOLDEN, "ref_native_vectors.npz"))


def triple(w):
    return (w.data, w.shape, w.quant_type)


@pytest.mark.parametrize("fmt", ["Q8_0", "Q5_K", "Q6_K", "Q4_K", "Q3_K", "Q4_0", "BF16"])
@pytest.mark.parametrize("shape", [(3, 512), (2, 3, 512)])
def test_linear_is_fp32_matmul_of_dequantised_matrix(fmt, shape):
    w = synthetic.packed_weight(fmt, (7, 512), 11)
    x = np.random.default_rng(103).normal(size=shape).astype(np.float32)
    y = R.linear(x, *triple(w))
    dense = R.dequantize(*triple(w)).astype(np.float64)
    expect = x.reshape(-1, 512).astype(np.float64) @ dense.T
    assert y.shape == shape[:-1] + (7,) and y.dtype == np.float32
    np.testing.assert_allclose(y.reshape(-1, 7), expect, rtol=1e-6, atol=2e-5)
    # the C restatement rounds the exact dot product once
    np.testing.assert_array_equal(native.c_linear(x, *triple(w)), expect.astype(np.float32))


def test_linear_q8_0_closed_form_exact():
    # reference vector: q = row%15-7, d = .125, x = (arange(32)+t)/32 -> every partial sum exact
    rows = 2048
    q = np.broadcast_to((np.arange(rows) % 15 - 7).astype(np.int8)[:, None], (rows, 32)).copy()
    raw = np.concatenate((np.full((rows, 1), .125, "<f2").view(np.uint8), q.view(np.uint8)), axis=1).reshape(-1)
    hidden = np.stack([(np.arange(32, dtype=np.float32) + t) / 32 for t in range(2)])
    expected = hidden.sum(axis=1, keepdims=True) * (q[:, 0].astype(np.float32) * .125)[None]
    np.testing.assert_array_equal(R.linear(hidden, raw, (rows, 32), "Q8_0"), expected)
    np.testing.assert_array_equal(native.c_linear(hidden, raw, (rows, 32), "Q8_0"), expected)


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
def test_linear_preserves_dtype_and_rejects_bad_shapes(dtype):
    w = synthetic.packed_weight("Q8_0", (5, 64), 3)
    x = np.ones((2, 64), dtype)
    assert R.linear(x, *triple(w)).dtype == dtype
    with pytest.raises(ValueError, match="Input K"):
        R.linear(np.zeros((2, 32), dtype), *triple(w))
    with pytest.raises(ValueError, match="Expected x"):
        R.linear(np.zeros(64, dtype), *triple(w))


@pytest.mark.parametrize("fmt", ["Q8_0", "Q4_0", "Q4_K", "Q3_K", "Q5_K", "Q6_K"])
def test_linear_matches_reference_native_gemv_vectors(fmt):
    blocks, x, y = RV[fmt + "_blocks"], RV[fmt + "_x"], RV[fmt + "_gemv"]
    shape = (y.shape[1], x.shape[1])
    scale = np.abs(y).max()
    # tolerance of the reference's own native-vs-NumPy test (rtol 3e-5, atol 2e-4 at unit scale)
    np.testing.assert_allclose(R.linear(x, blocks, shape, fmt), y, rtol=3e-5, atol=2e-4 * max(scale, 1))
    np.testing.assert_allclose(native.c_linear(x, blocks, shape, fmt), y, rtol=3e-5, atol=2e-4 * max(scale, 1))


def test_swiglu_and_expert_closed_form_fp64():
    gate = synthetic.packed_weight("Q5_K", (256, 256), 1)
    up = synthetic.packed_weight("Q8_0", (256, 256), 2)
    down = synthetic.packed_weight("Q6_K", (256, 256), 3)
    x = np.random.default_rng(4).normal(0, 1, (3, 256)).astype(np.float32)
    g = x.astype(np.float64) @ R.dequantize(*triple(gate)).astype(np.float64).T
    u = x.astype(np.float64) @ R.dequantize(*triple(up)).astype(np.float64).T
    h = g / (1 + np.exp(-g)) * u
    np.testing.assert_allclose(R.swiglu(x, triple(gate), triple(up)), h, rtol=3e-5, atol=1e-6)
    y = h.astype(np.float32).astype(np.float64) @ R.dequantize(*triple(down)).astype(np.float64).T
    np.testing.assert_allclose(R.expert_ffn(x, triple(gate), triple(up), triple(down)), y, rtol=3e-4, atol=1e-6)
    np.testing.assert_allclose(native.c_expert(x, triple(gate), triple(up), triple(down)), y, rtol=3e-4, atol=1e-6)
    assert R.swiglu(x.astype(np.float16), triple(gate), triple(up)).dtype == np.float16


def test_expert_matches_reference_native_expert_vector():
    d, f = RV["expert_x"].shape[1], RV["expert_gate"].shape[0] * 256 // RV["expert_x"].shape[1]
    gate = (RV["expert_gate"], (f, d), "Q5_K")
    up = (RV["expert_up"], (f, d), "Q5_K")
    down = (RV["expert_down"], (d, f), "Q6_K")
    expect = RV["expert_out"]
    scale = np.abs(expect).max()
    np.testing.assert_allclose(R.expert_ffn(RV["expert_x"], gate, up, down), expect, rtol=3e-5, atol=2e-4 * scale)
    np.testing.assert_allclose(native.c_expert(RV["expert_x"], gate, up, down), expect, rtol=3e-5, atol=2e-4 * scale)


# ---- router -------------------------------------------------------------------------------
@pytest.mark.parametrize("i", range(7))
def test_router_tie_inf_nan_fixtures(i):
    row, ids = FV[f"router_row{i}"], FV[f"router_row{i}_ids"]
    k = min(4, row.size)
    w, got = R.router_topk(row[None], k, floor=2.0 ** -14)
    np.testing.assert_array_equal(got[0], ids)
    wc, idc = native.c_router_topk(row[None], k, 2.0 ** -14)
    np.testing.assert_array_equal(idc[0], ids)
    np.testing.assert_allclose(wc, w, rtol=2e-7, atol=2e-7, equal_nan=True)


@pytest.mark.parametrize("n,k", [(1, 1), (3, 2), (32, 4), (512, 10), (4096, 32)])
@pytest.mark.parametrize("floor", [2.0 ** -14, .9, 2.0])
def test_router_definition_and_invariants(n, k, floor):
    z = np.random.default_rng(n).normal(0, 5, (3, n)).astype(np.float32)
    w, ids = R.router_topk(z, k, floor=floor)
    z64 = z.astype(np.float64)
    p = np.exp(z64 - z64.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    for t in range(3):
        brute = sorted(range(n), key=lambda i: (-z[t, i], i))[:k]
        assert list(ids[t]) == brute
        sel = p[t, brute]
        np.testing.assert_allclose(w[t], sel / max(sel.sum(), floor), rtol=2e-6, atol=2e-7)
        assert len(set(ids[t])) == k
        if sel.sum() >= floor:
            assert abs(float(w[t].sum()) - 1) < 1e-6
    wc, idc = native.c_router_topk(z, k, floor)
    np.testing.assert_array_equal(idc, ids)
    np.testing.assert_allclose(wc, w, rtol=2e-6, atol=2e-7)
    assert ids.dtype == np.int64 and w.dtype == np.float32


def test_router_without_renormalisation_is_plain_softmax_gather():
    z = np.random.default_rng(9).normal(0, 2, (4, 64)).astype(np.float32)
    w, ids = R.router_topk(z, 5, renormalize=False)
    p = np.exp(z - z.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    np.testing.assert_allclose(w, np.take_along_axis(p, ids, -1), rtol=1e-6)
    with pytest.raises(ValueError):
        R.router_topk(z, 65)


# ---- plan / dispatch / combine ---------------------------------------------------------------
def test_routing_plan_groups_by_expert():
    ids = np.array([[3, 0], [1, 3], [0, 2]])
    token, slot, order, offsets = R.routing_plan(ids, 5)
    np.testing.assert_array_equal(offsets, [0, 2, 3, 4, 6, 6])
    np.testing.assert_array_equal(token, [0, 2, 1, 2, 0, 1])
    np.testing.assert_array_equal(slot, [1, 0, 0, 1, 0, 1])
    np.testing.assert_array_equal(ids.reshape(-1)[order], [0, 0, 1, 2, 3, 3])


def test_combine_is_ascending_expert_order_not_slot_order():
    # expert outputs 1e20, -1e20, 3 for experts 0, 1, 2; slots arrive as (2, 0, 1):
    # expert order gives (1e20 - 1e20) + 3 = 3, slot order would give 0.
    x = np.ones((1, 3), np.float32)
    values = {0: 4e20, 1: -8e20, 2: 6.0}
    weights = np.array([[.5, .25, .125]], np.float32)
    ids = np.array([[2, 0, 1]])
    out = R.experts_forward(x, weights, ids, 3, lambda e, rows: np.full_like(rows, values[e]))
    np.testing.assert_array_equal(out, np.full((1, 3), 3, np.float32))


def test_grouped_decode_order_storage_boundaries_and_slots():
    experts = [tuple(triple(synthetic.packed_weight(fmt, shp, 50 + 3 * e + j))
                     for j, (fmt, shp) in enumerate([("Q8_0", (64, 256)), ("Q5_K", (64, 256)), ("Q8_0", (256, 64))]))
               for e in range(3)]
    x = np.random.default_rng(106).normal(0, .05, (1, 256)).astype(np.float32)
    routes = np.array([.7, -.2, .3], np.float32)
    out = np.zeros((1, 256), np.float32)
    for (g, u, d), r in zip(experts, routes):
        gd, ud, dd = (R.dequantize(*w).astype(np.float64) for w in (g, u, d))
        gate, up = x.astype(np.float64) @ gd.T, x.astype(np.float64) @ ud.T
        hidden = ((gate / (1 + np.exp(-gate))) * up).astype(np.float32)
        res = (hidden.astype(np.float64) @ dd.T).astype(np.float32)
        out = out + np.multiply(res, r, dtype=np.float32)
    got = R.grouped_decode(x, experts, routes)
    np.testing.assert_allclose(got, out, rtol=4e-4, atol=8e-6)
    slots = [2, 0, 1]
    np.testing.assert_array_equal(R.grouped_decode(x, experts, routes, slots),
                                  R.grouped_decode(x, experts, routes[slots]))


def test_ordered_sum_cancellation_fixture():
    # terms 1e8, 1, -1e8, 3 summed sequentially from zero give 3 (a tree gives 4 or 0)
    terms = [1e8, 1.0, -1e8, 3.0]
    acc = np.float32(0)
    for t in terms:
        acc = np.float32(acc + np.float32(t))
    assert acc == 3
    x = np.ones((1, 1), np.float32)
    ids = np.array([[0, 1, 2, 3]])
    w = np.ones((1, 4), np.float32)
    out = R.experts_forward(x, w, ids, 4, lambda e, rows: np.full_like(rows, terms[e]))
    assert out[0, 0] == 3


def moe_fp64(hidden, logits, k, dense, shared_dense, shared_gate):
    """Independent per-token fp64 loop (after the reference's test oracle for the layer)."""
    x = hidden.astype(np.float64)
    z = logits.astype(np.float64)
    p = np.exp(z - z.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    ids = np.stack([sorted(range(z.shape[1]), key=lambda i: (-z[t, i], i))[:k] for t in range(z.shape[0])])
    sel = np.take_along_axis(p, ids, -1)
    sel /= sel.sum(-1, keepdims=True)
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        for s, e in enumerate(ids[t]):
            g, u, d = dense[e]
            a, b = g @ x[t], u @ x[t]
            out[t] += sel[t, s] * (d @ (a / (1 + np.exp(-a)) * b))
        g, u, d = shared_dense
        a, b = g @ x[t], u @ x[t]
        out[t] += (d @ (a / (1 + np.exp(-a)) * b)) * np.exp(-np.logaddexp(0, -float(shared_gate @ x[t])))
    return out, ids, sel


def small_moe(seed=77, e=8, d=256, f=256, fsh=512, t=5):
    rng = np.random.default_rng(seed)
    experts = [tuple(triple(synthetic.packed_weight(fmt, shp, seed + 10 * i + j))
                     for j, (fmt, shp) in enumerate([("Q8_0", (f, d)), ("Q8_0", (f, d)), ("Q6_K", (d, f))]))
               for i in range(e)]
    shared = tuple(triple(synthetic.packed_weight(fmt, shp, seed + 1000 + j))
                   for j, (fmt, shp) in enumerate([("Q5_K", (fsh, d)), ("Q5_K", (fsh, d)), ("Q6_K", (d, fsh))]))
    # scale the synthetic weights' effect: hidden ~ N(0, .3)
    hidden = rng.normal(0, .3, (t, d)).astype(np.float32)
    logits = rng.normal(0, 1, (t, e)).astype(np.float32)
    gate_vec = rng.normal(0, .1, d).astype(np.float32)
    return experts, shared, hidden, logits, gate_vec


def test_moe_forward_against_independent_fp64_loop():
    experts, shared, hidden, logits, gate_vec = small_moe()
    dense = [tuple(R.dequantize(*w).astype(np.float64) for w in ex) for ex in experts]
    shared_dense = tuple(R.dequantize(*w).astype(np.float64) for w in shared)
    expect, ids, sel = moe_fp64(hidden, logits, 2, dense, shared_dense, gate_vec.astype(np.float64))
    out, w, got_ids = R.moe_forward(hidden, logits, 2, len(experts),
                                    lambda e, rows: R.expert_ffn(rows, *experts[e]), shared, gate_vec)
    np.testing.assert_array_equal(got_ids, ids)
    np.testing.assert_allclose(w, sel, rtol=2e-6, atol=2e-7)
    scale = np.abs(expect).max()
    np.testing.assert_allclose(out, expect, rtol=3e-4, atol=3e-5 * scale)
    # zero admission vector -> sigmoid(0) = 0.5 exactly
    expect0, _, _ = moe_fp64(hidden, logits, 2, dense, shared_dense, np.zeros(hidden.shape[1]))
    out0, _, _ = R.moe_forward(hidden, logits, 2, len(experts),
                               lambda e, rows: R.expert_ffn(rows, *experts[e]), shared, np.zeros_like(gate_vec))
    np.testing.assert_allclose(out0, expect0, rtol=3e-4, atol=3e-5 * scale)
    np.testing.assert_array_equal(R.shared_gate_sigmoid(hidden, np.zeros_like(gate_vec)), np.full(hidden.shape[0], .5, np.float32))


def test_rmsnorm_closed_forms_and_fp64():
    d = 96
    gamma = np.linspace(0.5, 1.5, d).astype(np.float32)
    for c, eps in ((3.0, 1e-6), (-0.25, 1e-5), (1e-3, 1e-6)):
        row = np.full((2, d), c, np.float32)
        want = gamma.astype(np.float64) * c / np.sqrt(c * c + eps)
        np.testing.assert_allclose(R.rmsnorm(row, gamma, eps)[1], want, rtol=3e-7)
    x = np.random.default_rng(3).standard_normal((5, d)).astype(np.float32)
    np.testing.assert_allclose(R.rmsnorm(4.0 * x, gamma, 0.0), R.rmsnorm(x, gamma, 0.0), rtol=1e-6)   # scale invariance at eps = 0
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt(np.mean(x64 * x64, axis=-1, keepdims=True) + 1e-6) * gamma
    got = R.rmsnorm(x, gamma, 1e-6)
    assert got.dtype == np.float32
    np.testing.assert_allclose(got, want, rtol=1e-6)
    # a dropped eps, a mean taken as a sum or gamma left out each fail one of the above
    assert not np.allclose(R.rmsnorm(np.full((1, d), 1e-3, np.float32), gamma, 1e-6), gamma)


def test_router_logits_against_fp64():
    rng = np.random.default_rng(4)
    x, w, b = rng.standard_normal((3, 128)).astype(np.float32), rng.standard_normal((16, 128)).astype(np.float32), rng.standard_normal(16).astype(np.float32)
    np.testing.assert_allclose(R.router_logits(x, w, b), x.astype(np.float64) @ w.astype(np.float64).T + b, rtol=1e-5, atol=1e-5)
    assert R.router_logits(x, w).shape == (3, 16)
