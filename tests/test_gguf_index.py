"""GGUF container reader and the Qwen3-Next expert index (host logic, no GPU).

The index tests follow the reference's own (tests/test_0106f_qwen3next_gguf.py): duck-typed
readers, zero-copy expert views, fused and separate gate/up tensors, error cases.
"""
import os
import struct

import numpy as np
import pytest

from mylocal_llm_amd import synthetic
from mylocal_llm_amd.gguf_file import GGUFFile
from mylocal_llm_amd.gguf_tensor import decode_gguf_dense
from mylocal_llm_amd.moe import Qwen3NextMoESpec
from mylocal_llm_amd.quantized_weight import BLOCK_FORMATS, PackedGGUFWeight
from mylocal_llm_amd.qwen3next_gguf import ExpertKey, Qwen3NextGGUFIndex, _row_range
from oracle import reference_np as R

from gguf_writer import write_gguf

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FV = np.load(os.path.join(GOLDEN, "format_vectors.npz"))


def test_reader_parses_a_hand_assembled_file(tmp_path):
    """Every byte of this file is written out here, field by field, after the container
    specification: magic, version 3, 1 tensor, 3 metadata entries (string, u32, array of
    strings), one Q8_0 tensor [2, 32] (GGML dims 32, 2), payload at the next multiple of 32."""
    payload = bytes(range(68))
    def s(text):
        return struct.pack("<Q", len(text)) + text.encode()
    blob = b"GGUF" + struct.pack("<I", 3) + struct.pack("<Q", 1) + struct.pack("<Q", 3)
    blob += s("general.architecture") + struct.pack("<I", 8) + s("qwen3next")
    blob += s("qwen3next.block_count") + struct.pack("<I", 4) + struct.pack("<I", 48)
    blob += s("tokenizer.tokens") + struct.pack("<I", 9) + struct.pack("<I", 8) + struct.pack("<Q", 2) + s("a") + s("bc")
    blob += s("blk.0.w") + struct.pack("<I", 2) + struct.pack("<Q", 32) + struct.pack("<Q", 2)
    blob += struct.pack("<I", 8) + struct.pack("<Q", 0)          # ggml type 8 = Q8_0, offset 0
    start = (len(blob) + 31) // 32 * 32
    blob += b"\0" * (start - len(blob)) + payload
    path = tmp_path / "tiny.gguf"
    path.write_bytes(blob)
    with GGUFFile(path) as f:
        assert f.version == 3 and f.alignment == 32 and f.data_offset == start
        assert f.fields["general.architecture"].contents(0) == "qwen3next"
        assert f.fields["qwen3next.block_count"].contents(0) == 48
        assert f.fields["tokenizer.tokens"].contents(1) == "bc"
        (t,) = f.tensors
        assert (t.name, t.shape, t.tensor_type.name) == ("blk.0.w", (32, 2), "Q8_0")
        assert t.data.dtype == np.uint8 and bytes(t.data) == payload
        assert not t.data.flags.owndata and not t.data.flags.writeable


def test_reader_round_trip_types_and_alignment(tmp_path):
    f32 = np.arange(12, dtype=np.float32).reshape(3, 4)
    f16 = np.linspace(-2, 2, 10, dtype=np.float16).reshape(2, 5)
    bf16 = FV["bf16_bytes_blocks"]
    q6 = synthetic.packed_weight("Q6_K", (3, 256), 5)
    path = tmp_path / "types.gguf"
    write_gguf(path, {"general.architecture": "test", "x.flag": True, "x.ids": [3, 1, 2]},
               [("a", f32.shape, "F32", f32), ("b", f16.shape, "F16", f16),
                ("c", (bf16.size // 2,), "BF16", bf16), ("d", q6.shape, "Q6_K", q6.data)], alignment=64)
    with GGUFFile(path) as f:
        assert f.alignment == 64 and f.fields["x.flag"].contents(0) is True
        assert f.fields["x.ids"].contents() == [3, 1, 2]
        t = {x.name: x for x in f.tensors}
        assert all(x.data_offset % 64 == 0 for x in f.tensors)
        np.testing.assert_array_equal(decode_gguf_dense(t["a"]), f32)
        np.testing.assert_array_equal(decode_gguf_dense(t["b"]), f16)
        np.testing.assert_array_equal(decode_gguf_dense(t["c"]).view(np.uint32), FV["bf16_bytes_expected_bits"])
        np.testing.assert_array_equal(t["d"].data, q6.data)
        with pytest.raises(NotImplementedError):
            decode_gguf_dense(t["d"])


@pytest.mark.parametrize("blob,match", [(b"GGML" + b"\0" * 60, "not a GGUF"),
                                        (b"GGUF" + struct.pack("<I", 1) + b"\0" * 56, "version 1"),
                                        (b"GGUF" + struct.pack("<IQQ", 3, 1, 0), "truncated")])
def test_reader_rejects_bad_files(tmp_path, blob, match):
    path = tmp_path / "bad.gguf"
    path.write_bytes(blob)
    with pytest.raises(ValueError, match=match):
        GGUFFile(path)


# ---- duck-typed reader, as in the reference's tests ---------------------------------------------
class Field:
    def __init__(self, value): self.value = value
    def contents(self, index): return self.value


class Kind:
    def __init__(self, name): self.name = name


class Tensor:
    def __init__(self, name, shape, kind="Q4_0", seed=None):
        self.name, self.shape, self.tensor_type = name, tuple(reversed(shape)), Kind(kind)
        qk, qb = BLOCK_FORMATS[kind]
        n = int(np.prod(shape)) // qk * qb
        self.data = np.zeros(n, np.uint8) if seed is None else np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


class Reader:
    def __init__(self, fused=False, kind="Q4_0", seed=None):
        self.fields = {k: Field(v) for k, v in {
            "general.architecture": "qwen3next", "qwen3next.block_count": 2, "qwen3next.embedding_length": 256,
            "qwen3next.expert_count": 3, "qwen3next.expert_used_count": 2}.items()}
        self.tensors = []
        for i in range(2):
            stem = f"blk.{i}."
            self.tensors += [Tensor(stem + "ffn_down_exps.weight", (3, 256, 256), kind, seed),
                             Tensor(stem + "ffn_gate_inp.weight", (3, 256), kind)]
            if fused:
                self.tensors.append(Tensor(stem + "ffn_gate_up_exps.weight", (3, 512, 256), kind, seed))
            else:
                self.tensors += [Tensor(stem + "ffn_gate_exps.weight", (3, 256, 256), kind, seed),
                                 Tensor(stem + "ffn_up_exps.weight", (3, 256, 256), kind, seed)]


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("fmt", ["Q4_0", "Q3_K", "Q8_0"])
def test_index_expert_provider_is_zero_copy(fused, fmt):
    reader = Reader(fused, fmt, seed=3)
    idx = Qwen3NextGGUFIndex(reader)
    w = idx.provider(ExpertKey("test", 1, 2))
    assert len(w) == 3 and all(isinstance(x, PackedGGUFWeight) for x in w)
    assert [x.shape for x in w] == [(256, 256)] * 3
    assert all(not x.data.flags.owndata for x in w)
    by_name = {t.name: t for t in reader.tensors}
    qk, qb = BLOCK_FORMATS[fmt]
    mat = 256 * 256 // qk * qb
    np.testing.assert_array_equal(w[2].data, by_name["blk.1.ffn_down_exps.weight"].data[2 * mat:3 * mat])
    if fused:  # gate rows [0, F) then up rows [F, 2F) of the expert
        src = by_name["blk.1.ffn_gate_up_exps.weight"].data
        np.testing.assert_array_equal(w[0].data, src[4 * mat:5 * mat])
        np.testing.assert_array_equal(w[1].data, src[5 * mat:6 * mat])
    else:
        np.testing.assert_array_equal(w[1].data, by_name["blk.1.ffn_up_exps.weight"].data[2 * mat:3 * mat])
    stats = idx.report(device_budget_gib=0.001)
    assert stats["layers"] == 2 and stats["estimated_device_cache_experts"] > 0
    assert not stats["full_model_decode_available"]


def test_row_range_checks():
    w = synthetic.packed_weight("Q8_0", (8, 64), 1)
    part = _row_range(w, 2, 5)
    assert part.shape == (3, 64)
    np.testing.assert_array_equal(R.dequantize(part.data, part.shape, "Q8_0"), R.dequantize(w.data, w.shape, "Q8_0")[2:5])
    for first, last in ((-1, 2), (3, 3), (0, 9)):
        with pytest.raises(ValueError):
            _row_range(w, first, last)


def test_bad_architecture_missing_layers_formats_and_indices():
    reader = Reader()
    reader.fields["general.architecture"] = Field("llama")
    with pytest.raises(ValueError, match="Expected Qwen3-Next"):
        Qwen3NextGGUFIndex(reader)
    reader = Reader()
    reader.tensors = reader.tensors[4:]
    with pytest.raises(ValueError, match="Missing blk.0"):
        Qwen3NextGGUFIndex(reader)
    reader = Reader()
    next(t for t in reader.tensors if t.name == "blk.0.ffn_down_exps.weight").tensor_type = Kind("IQ1_S")
    idx = Qwen3NextGGUFIndex(reader)
    assert idx.report()["unsupported_routed_formats"]["IQ1_S"] == 1
    with pytest.raises(NotImplementedError, match="IQ1_S"):
        idx.expert_weights(0, 0)
    idx = Qwen3NextGGUFIndex(Reader())
    for layer, expert in ((-1, 0), (0, 3), (2, 0)):
        with pytest.raises(IndexError):
            idx.expert_weights(layer, expert)
    with pytest.raises(TypeError):
        idx.provider((0, 0))
    with pytest.raises(ValueError, match="routed expert banks"):
        idx.non_expert_weight("blk.0.ffn_down_exps.weight")


def moe_file(path, *, fused, fmt="Q8_0", shared=("Q8_0", "Q8_0", "BF16"), e=4, d=256, f=256, fsh=256, k=2, seed=11):
    """One-layer Qwen3-Next MoE block written as a GGUF file; returns the host tensors."""
    gate = synthetic.packed_weight(fmt, (e, f, d), seed)
    up = synthetic.packed_weight(fmt, (e, f, d), seed + 1)
    down = synthetic.packed_weight(fmt, (e, d, f), seed + 2)
    sh = [synthetic.packed_weight(kind, shape, seed + 3 + i) for i, (kind, shape) in
          enumerate(zip(shared, ((fsh, d), (fsh, d), (d, fsh))))]
    rng = np.random.default_rng(seed)
    router = rng.standard_normal((e, d), dtype=np.float32)
    sgate = rng.standard_normal(d, dtype=np.float32) * np.float32(0.1)
    tensors = [("blk.0.ffn_down_exps.weight", down.shape, fmt, down.data),
               ("blk.0.ffn_gate_inp.weight", router.shape, "F32", router),
               ("blk.0.ffn_gate_inp_shexp.weight", sgate.shape, "F32", sgate)]
    if fused:
        rows = BLOCK_FORMATS[fmt][1] * d // BLOCK_FORMATS[fmt][0]
        both = np.concatenate([gate.data.reshape(e, f * rows), up.data.reshape(e, f * rows)], axis=1)
        tensors.append(("blk.0.ffn_gate_up_exps.weight", (e, 2 * f, d), fmt, both))
    else:
        tensors += [("blk.0.ffn_gate_exps.weight", gate.shape, fmt, gate.data), ("blk.0.ffn_up_exps.weight", up.shape, fmt, up.data)]
    for name, w in zip(("ffn_gate_shexp", "ffn_up_shexp", "ffn_down_shexp"), sh):
        tensors.append((f"blk.0.{name}.weight", w.shape, w.quant_type, w.data))
    write_gguf(path, {"general.architecture": "qwen3next", "qwen3next.block_count": 1, "qwen3next.embedding_length": d,
                      "qwen3next.expert_count": e, "qwen3next.expert_used_count": k,
                      "qwen3next.expert_shared_feed_forward_length": fsh, "qwen3next.expert_feed_forward_length": f}, tensors)
    return gate, up, down, sh, router, sgate


@pytest.mark.parametrize("fused", [True, False])
def test_index_over_a_written_file_and_spec(tmp_path, fused):
    path = tmp_path / "moe.gguf"
    gate, up, down, sh, router, sgate = moe_file(path, fused=fused)
    idx = Qwen3NextGGUFIndex.open(path)
    assert (idx.layers, idx.d_model, idx.d_ff, idx.expert_count, idx.experts_per_token) == (1, 256, 256, 4, 2)
    g, u, dn = idx.expert_weights(0, 3)
    np.testing.assert_array_equal(g.data, gate.select_outer(3).data)
    np.testing.assert_array_equal(u.data, up.select_outer(3).data)
    np.testing.assert_array_equal(dn.data, down.select_outer(3).data)
    np.testing.assert_array_equal(idx.non_expert_weight("blk.0.ffn_gate_inp.weight"), router)
    bf = idx.projection("blk.0.ffn_down_shexp.weight")
    assert isinstance(bf, PackedGGUFWeight) and bf.quant_type == "BF16" and bf.shape == (256, 256)
    np.testing.assert_array_equal(bf.data, sh[2].data)
    spec = Qwen3NextMoESpec.from_index(idx, 0)
    assert (spec.d_model, spec.d_ff, spec.shared_d_ff, spec.n_experts, spec.top_k) == (256, 256, 256, 4, 2)
    with pytest.raises(IndexError):
        Qwen3NextMoESpec.from_index(idx, 1)
    with pytest.raises(TypeError):
        Qwen3NextMoESpec.from_index(idx, True)
    idx.reader.fields["qwen3next.expert_group_count"] = Field(2)
    with pytest.raises(NotImplementedError, match="expert_group_count"):
        Qwen3NextMoESpec.from_index(idx, 0)


# ---- single rows of an embedding-like tensor (the reference's tests/test_0106p_gguf_rows.py) ------
def _row_tensor(kind):
    from types import SimpleNamespace
    values = (np.arange(5 * 32).reshape(5, 32) % 17 - 8).astype(np.float32) / 16
    if kind == "Q8_0":
        codes = (values * 16).astype(np.int8)
        scale = np.full((5, 1), 1 / 16, dtype="<f2")
        data = np.concatenate((scale.view(np.uint8), codes.view(np.uint8)), axis=1)
    elif kind == "BF16":
        data = (values.view(np.uint32) >> 16).astype("<u2").view(np.uint8)
    else:
        data = values.astype(np.float16 if kind == "F16" else np.float32)
    return SimpleNamespace(name="embedding", shape=(32, 5), data=data, tensor_type=SimpleNamespace(name=kind)), values


@pytest.mark.parametrize("kind", ["F32", "F16", "BF16", "Q8_0"])
def test_single_rows_decode_only_the_row_and_leave_the_owner_alone(kind, monkeypatch):
    from mylocal_llm_amd.gguf_tensor import decode_gguf_row
    weight, expected = _row_tensor(kind)
    before, writable = weight.data.copy(), weight.data.flags.writeable
    decoded_shapes = []
    whole = PackedGGUFWeight.dequantize_reference

    def only_rows(self):
        decoded_shapes.append(self.shape)
        assert self.shape == (32,), "the whole table must never be expanded"
        return whole(self)

    monkeypatch.setattr(PackedGGUFWeight, "dequantize_reference", only_rows)
    for row in (4, 0, 2):
        np.testing.assert_array_equal(decode_gguf_row(weight, row), expected[row])
    assert len(decoded_shapes) == (3 if kind == "Q8_0" else 0)
    np.testing.assert_array_equal(weight.data, before)
    assert weight.data.flags.writeable == writable


@pytest.mark.parametrize("row,error", [(-1, IndexError), (5, IndexError), (True, TypeError), (1.0, TypeError)])
def test_single_row_index_is_validated(row, error):
    from mylocal_llm_amd.gguf_tensor import decode_gguf_row
    with pytest.raises(error):
        decode_gguf_row(_row_tensor("Q8_0")[0], row)


def test_single_row_of_big_endian_bf16_words_and_a_short_payload():
    from mylocal_llm_amd.gguf_tensor import decode_gguf_row
    weight, expected = _row_tensor("BF16")
    weight.data = weight.data.view("<u2").astype(">u2")
    np.testing.assert_array_equal(decode_gguf_row(weight, 3), expected[3])
    weight.data = weight.data[:-1]
    with pytest.raises(ValueError, match="payload"):
        decode_gguf_row(weight, 0)
    weight3 = _row_tensor("F32")[0]
    weight3.shape = (32, 5, 1)
    with pytest.raises(ValueError, match="positive matrix"):
        decode_gguf_row(weight3, 0)
