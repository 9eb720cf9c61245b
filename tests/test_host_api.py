"""Host-side logic that needs no GPU: the packed container, the ABI surface of the built
library, and argument validation that returns before any kernel would be launched."""
import ctypes
import os
import re

import numpy as np
import pytest

from mylocal_llm_amd import _lib, synthetic
from mylocal_llm_amd.quantized_weight import BLOCK_FORMATS, PackedGGUFWeight

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_block_format_table():
    assert BLOCK_FORMATS["Q8_0"] == (32, 34)
    assert BLOCK_FORMATS["Q5_K"] == (256, 176)
    assert BLOCK_FORMATS["Q6_K"] == (256, 210)
    assert BLOCK_FORMATS["Q4_K"] == (256, 144)
    assert BLOCK_FORMATS["Q4_0"] == (32, 18)


@pytest.mark.parametrize("fmt", list(BLOCK_FORMATS))
def test_length_alignment_and_type_errors(fmt):
    elems, nbytes = BLOCK_FORMATS[fmt]
    good = np.zeros(2 * nbytes, np.uint8)
    PackedGGUFWeight(good, (1, 2 * elems), fmt)
    with pytest.raises(ValueError, match="expected"):
        PackedGGUFWeight(good[:-1], (1, 2 * elems), fmt)
    if elems > 1:
        with pytest.raises(ValueError, match="innermost"):
            PackedGGUFWeight(good, (1, 2 * elems - 1), fmt)
    with pytest.raises(ValueError, match="Unsupported"):
        PackedGGUFWeight(good, (1, 2 * elems), "Q9_Z")
    with pytest.raises(ValueError, match="positive"):
        PackedGGUFWeight(good, (0, 2 * elems), fmt)
    with pytest.raises(ValueError, match="contiguous"):
        PackedGGUFWeight(np.zeros(4 * nbytes, np.uint8)[::2], (1, 2 * elems), fmt)


def test_select_outer_and_rows_are_zero_copy():
    original = synthetic.packed_weight("Q5_K", (3, 4, 512), 49)
    sample = original.select_outer(1)
    assert sample.shape == (4, 512) and sample.nbytes == 4 * 2 * 176
    assert np.shares_memory(sample.data, original.data)
    np.testing.assert_array_equal(sample.data, original.data[sample.nbytes:2 * sample.nbytes])
    rows = sample.select_rows(1, 3)
    assert rows.shape == (2, 512) and np.shares_memory(rows.data, original.data)
    with pytest.raises(IndexError):
        original.select_outer(3)
    with pytest.raises(ValueError):
        sample.select_outer(0).select_outer(0)


def test_mmap_payload_stays_the_owner(tmp_path):
    w = synthetic.packed_weight("Q6_K", (12, 512), 5)
    path = tmp_path / "q6.bin"
    path.write_bytes(w.data.tobytes())
    mapped = np.memmap(path, dtype=np.uint8, mode="r")
    view = PackedGGUFWeight(mapped, (3, 4, 512), "Q6_K").select_outer(2)
    assert np.shares_memory(view.data, mapped)
    np.testing.assert_array_equal(view.data, w.data[2 * view.nbytes:])


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "qmoe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qmoe_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert set(names) == set(_lib.EXPORTS)
    for name in names:
        assert getattr(lib, name) is not None
    # the header, the binding and the built library agree on the ABI version
    with open(os.path.join(ROOT, "include", "qmoe.h")) as fh:
        declared = int(re.search(r"#define\s+QMOE_ABI_VERSION\s+(\d+)", fh.read()).group(1))
    assert lib.qmoe_abi_version() == declared == _lib.ABI_VERSION


def test_driver_build_entry_checks_the_bound_version():
    """build() of the driver entry module must not pin a version of its own."""
    with open(os.path.join(ROOT, "__graft_entry__.py")) as fh:
        text = fh.read()
    assert "_lib.ABI_VERSION" in text and not re.search(r"qmoe_abi_version\(\)\s*==\s*\d", text)


def test_format_info_matches_table():
    lib = _lib.load()
    e, b = ctypes.c_int(), ctypes.c_int()
    for fmt, (elems, nbytes) in BLOCK_FORMATS.items():
        assert lib.qmoe_format_info(_lib.FORMAT_ID[fmt], ctypes.byref(e), ctypes.byref(b)) == 0
        assert (e.value, b.value) == (elems, nbytes)
    assert lib.qmoe_format_info(77, ctypes.byref(e), ctypes.byref(b)) == 1
    assert b"unknown" in lib.qmoe_last_error()


def test_invalid_arguments_return_codes_before_any_launch():
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    fake = ctypes.c_void_p(4096)  # never dereferenced: validation fails first
    assert lib.qmoe_linear(null, 0, 4, 32, fake, 0, 1, fake, 0, null) == 1
    assert lib.qmoe_linear(fake, 0, 4, 33, fake, 0, 1, fake, 0, null) == 1      # K not a block multiple
    assert b"multiple" in lib.qmoe_last_error()
    assert lib.qmoe_linear(fake, 0, 4, 32, fake, 0, 0, fake, 0, null) == 1      # no tokens
    assert lib.qmoe_linear(fake, 3, 4, 384, fake, 0, 1, fake, 0, null) == 1     # Q3_K: K not a multiple of 256
    assert lib.qmoe_linear(fake, 42, 4, 256, fake, 0, 1, fake, 0, null) == 1    # unknown format
    assert lib.qmoe_linear(fake, 0, 4, 32, fake, 9, 1, fake, 0, null) == 1      # unknown dtype
    assert lib.qmoe_dequantize(fake, 5, 2, 100, fake, null) == 1
    assert lib.qmoe_swiglu(fake, 0, null, 0, 4, 32, fake, 0, 1, fake, 0, null) == 1
    assert lib.qmoe_expert(fake, 0, fake, 0, fake, 0, 32, 32, fake, 0, 1, fake, 0, null, null) == 4
    assert lib.qmoe_router_topk(fake, 1, 5000, 2, 1e-6, 1, fake, fake, null) == 2
    assert lib.qmoe_router_topk(fake, 1, 16, 33, 1e-6, 1, fake, fake, null) == 2
    assert lib.qmoe_router_topk(fake, 1, 16, 3, 1e-50, 1, fake, fake, null) == 1
    assert lib.qmoe_grouped_decode(fake, fake, 0, 0, 0, 0, 32, 32, fake, 1, null, fake, fake, null) == 1
    assert lib.qmoe_moe_forward(None, null, 0, null) == 1


def test_listed_grouped_decode_rejects_bad_arguments_before_any_launch():
    """qmoe_grouped_decode_listed reads its expert list on the host: every rejection below happens
    before anything is launched (no GPU needed), with the status code the header names."""
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    fake = ctypes.c_void_p(4096)
    table = (ctypes.c_void_p * 6)(4096, 8192, 12288, 16384, 20480, 24576)
    listed = ctypes.cast(table, ctypes.c_void_p)
    call = lambda **kw: lib.qmoe_grouped_decode_listed(*[kw.get(name, default) for name, default in (
        ("x", fake), ("experts", listed), ("n", 2), ("gf", 0), ("uf", 0), ("df", 0), ("d", 256), ("f", 256), ("routes", fake),
        ("stride", 1), ("slots", null), ("out", fake), ("ws", fake), ("stream", null))])
    assert call(x=null) == 1 and call(experts=null) == 1 and call(routes=null) == 1 and call(out=null) == 1
    assert call(ws=null) == 4 and call(ws=ctypes.c_void_p(4100)) == 4           # workspace missing / not 16-byte aligned
    assert b"workspace" in lib.qmoe_last_error()
    assert call(n=0) == 1
    assert call(n=17) == 2 and b"qmoe_grouped_decode" in lib.qmoe_last_error()    # beyond a host list: the device-table entry
    assert call(d=0) == 1 and call(f=-256) == 1
    assert call(gf=42) == 1 and b"unknown" in lib.qmoe_last_error()
    assert call(d=200) == 1 and b"block multiple" in lib.qmoe_last_error()          # Q8_0: K not a multiple of 32
    holes = (ctypes.c_void_p * 6)(4096, 0, 12288, 16384, 20480, 24576)
    assert call(experts=ctypes.cast(holes, ctypes.c_void_p)) == 1 and b"null projection" in lib.qmoe_last_error()
    odd = (ctypes.c_void_p * 6)(4097, 8192, 12288, 16384, 20480, 24576)
    assert call(experts=ctypes.cast(odd, ctypes.c_void_p)) == 1 and b"2-byte aligned" in lib.qmoe_last_error()
    negative = (ctypes.c_int32 * 2)(0, -1)
    assert call(slots=ctypes.cast(negative, ctypes.c_void_p)) == 1 and b"route position" in lib.qmoe_last_error()


def test_wait_limit_and_abi_version_are_plain_host_calls():
    lib = _lib.load()
    assert lib.qmoe_abi_version() == _lib.ABI_VERSION == 5
    lib.qmoe_set_wait_limit(12345)     # stored for the next launches; nothing touches a device
    lib.qmoe_set_wait_limit(0)         # back to the default


def test_moe_workspace_size_is_monotone_and_aligned():
    lib = _lib.load()
    a = lib.qmoe_moe_workspace_bytes(1, 10, 512, 2048, 512, 2048)
    b = lib.qmoe_moe_workspace_bytes(16, 10, 512, 2048, 512, 2048)
    assert 0 < a < b and a % 256 == 0 and b % 256 == 0
    assert lib.qmoe_moe_workspace_bytes(1, 0, 512, 2048, 512, 0) == 0


def test_host_and_device_operands_do_not_mix():
    """NumPy activations go with host-packed weights (computed by the library's host twins);
    nothing else is accepted in their place, and uploading needs a device."""
    torch = pytest.importorskip("torch")
    from mylocal_llm_amd.quantized_linear import quantized_linear, quantized_swiglu, packed_to_device
    w = synthetic.packed_weight("Q4_K", (2, 256), 1)
    assert quantized_linear(np.zeros((2, 256), np.float32), w).shape == (2, 2)
    assert quantized_swiglu(np.zeros((2, 256), np.float32), w, w).shape == (2, 2)
    with pytest.raises(TypeError, match="NumPy"):
        quantized_linear([[0] * 256], w)
    with pytest.raises(TypeError, match="NumPy"):
        quantized_linear(torch.zeros((2, 256)), w)      # a host tensor is not a NumPy array
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="HIP device"):
            packed_to_device(w)


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "mylocal_llm_amd")
    for base, _, files in os.walk(pkg):
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(base, name)).read()
                assert "oracle" not in text.replace("no oracle", ""), os.path.join(base, name)


@pytest.mark.parametrize("tokens,n_experts,k", [(2500, 512, 10), (1900, 512, 1), (929, 512, 4), (70000, 8, 2)])
def test_routing_plan_of_token_chunks_is_the_plan_of_the_whole_batch(tokens, n_experts, k, monkeypatch):
    """Batches beyond what one plan-kernel call covers are planned in token chunks and joined with
    index arithmetic: with the kernel call replaced by the oracle's plan of each chunk (host tensors),
    the joined plan must be the oracle's plan of the whole batch, Zipf-skewed routing included."""
    import torch
    from oracle import reference_np as R
    from mylocal_llm_amd import routing_plan as rp, synthetic

    calls = []

    def oracle_call(ids, w, kk, e):
        n = ids.shape[0]
        calls.append(n)
        assert n <= min(512, rp.max_tokens_per_plan_call(e)) and ids.is_contiguous() and w.is_contiguous()
        token, _, order, offsets = R.routing_plan(ids.numpy(), e)
        pos = np.empty(n * kk, dtype=np.int32)
        pos[order] = np.arange(n * kk, dtype=np.int32)
        as_i32 = lambda a: torch.from_numpy(np.asarray(a, dtype=np.int32))
        return (as_i32(offsets), as_i32(order), as_i32(token), torch.from_numpy(w.numpy().reshape(-1)[order].copy()),
                torch.from_numpy(pos), torch.zeros(1, dtype=torch.int32))

    logits = synthetic.router_logits(tokens, n_experts, 5, zipf=1.1)
    w, ids = R.router_topk(logits, k, floor=2.0 ** -14)
    plan = rp.RoutingPlan._build(torch.from_numpy(ids.reshape(1, tokens, k)), torch.from_numpy(w.reshape(1, tokens, k)), k, n_experts, oracle_call)
    assert len(calls) == -(-tokens // 512) > 1 and sum(calls) == tokens
    token, slot, order, offsets = R.routing_plan(ids, n_experts)
    assert plan.expert_offsets == tuple(int(v) for v in offsets)
    np.testing.assert_array_equal(plan.order.numpy(), order)
    np.testing.assert_array_equal(plan.token_indices.numpy(), token)
    np.testing.assert_array_equal(plan.slot_indices.numpy(), slot)
    np.testing.assert_array_equal(plan.expert_indices.numpy(), ids.reshape(-1)[order])
    np.testing.assert_array_equal(plan.weights.numpy(), w.reshape(-1)[order])
    np.testing.assert_array_equal(order[plan.position_of_assignment.numpy().reshape(-1)], np.arange(tokens * k))
    assert plan.active_expert_ids() == tuple(int(i) for i in np.nonzero(np.bincount(ids.reshape(-1), minlength=n_experts))[0])


def test_routing_plan_of_token_chunks_reports_invalid_routing(monkeypatch):
    """A chunk whose plan is flagged (and may hold anything) makes the joined plan raise; no look-up
    of the join leaves its arrays on the way."""
    import torch
    from mylocal_llm_amd import routing_plan as rp

    def flagged(ids, w, kk, e):
        n = ids.shape[0] * kk
        junk = torch.full((n,), 2 ** 31 - 1, dtype=torch.int32)
        return (torch.zeros(e + 1, dtype=torch.int32), junk, junk.clone(), torch.zeros(n), -junk, torch.ones(1, dtype=torch.int32))

    ids = torch.zeros((1, 2000, 2), dtype=torch.int64)
    with pytest.raises(ValueError, match="Invalid routing"):
        rp.RoutingPlan._build(ids, torch.zeros((1, 2000, 2)), 2, 512, flagged)
