"""The emitted gfx950 assembly of the LDS-DMA kernels keeps the wait states their inline assembly
hides from the compiler (mylocal_llm_amd/_asm_check.py).  Needs hipcc, no GPU."""
import shutil
from concurrent.futures import ThreadPoolExecutor

import pytest

from mylocal_llm_amd import _asm_check

pytestmark = pytest.mark.skipif(not (shutil.which("hipcc") or shutil.which("/opt/rocm/bin/hipcc")), reason="hipcc not installed")


def test_scanner_sees_what_it_is_meant_to_see():
    text = """
_Z1kv:
	v_readfirstlane_b32 s5, v1
	v_readfirstlane_b32 s4, v0
	s_add_i32 s9, s9, 8
	global_load_lds_dwordx4 v7, s[4:5] offset:0
	s_mov_b32 m0, s3
	global_load_lds_dwordx4 v7, s[10:11] offset:0
	v_readfirstlane_b32 s20, v0
	s_nop 4
	global_load_dword v1, v0, s[20:21]
	s_mov_b32 m0, s3
	s_nop 0
	global_load_lds_dword v[2:3], off
"""
    found = _asm_check.scan(text)
    assert dict(found["_Z1kv"]) == {"sgpr_base_after_valu": 1, "m0_back_to_back": 1}


@pytest.fixture(scope="module")
def findings():
    with ThreadPoolExecutor(max_workers=2) as pool:
        texts = list(pool.map(_asm_check.device_asm, _asm_check.SOURCES))
    names = {source: _asm_check.kernels(text) for source, text in zip(_asm_check.SOURCES, texts)}
    # what the checks below talk about is there: sixteen span kernels, half of them plain-row, and the decode kernels
    assert sum(_asm_check.plain_row_span_kernel(k) for k in names["qmoe_span.hip"]) == 8
    assert sum("span_kernel" in k for k in names["qmoe_span.hip"]) == 16
    assert sum("pairs2_kernel" in k for k in names["qmoe_decode2.hip"]) == 4 and sum("down2_kernel" in k for k in names["qmoe_decode2.hip"]) == 4
    return {source: _asm_check.scan(text) for source, text in zip(_asm_check.SOURCES, texts)}


def test_no_base_register_is_read_within_five_slots_of_its_vector_write(findings):
    """The plain-row instantiations of span_kernel and both MoE decode kernels compute every base of
    a memory instruction with scalar instructions (or address through vector registers): none reads a
    scalar register that a vector instruction wrote fewer than five slots earlier.  Versions of
    span_kernel that had such sites in their plain-row instantiations faulted on the GPU."""
    span = findings["qmoe_span.hip"]
    offenders = {k: v["sgpr_base_after_valu"] for k, v in span.items() if _asm_check.plain_row_span_kernel(k) and v["sgpr_base_after_valu"]}
    assert not offenders, offenders
    decode = {k: v["sgpr_base_after_valu"] for k, v in findings["qmoe_decode2.hip"].items() if v["sgpr_base_after_valu"]}
    assert not decode, decode


def test_decode_kernels_keep_the_wait_state_behind_an_m0_write(findings):
    """No LDS-DMA of the MoE decode kernels follows its M0 write back to back."""
    offenders = {k: v["m0_back_to_back"] for k, v in findings["qmoe_decode2.hip"].items() if v["m0_back_to_back"]}
    assert not offenders, offenders


def test_multiply_high_division_is_exact_where_the_decode_plans_allow_it():
    """The MoE decode kernels divide item and piece numbers by run-time constants with one
    multiply-high: q / d = (q * (floor(2^32 / d) + 1)) >> 32.  The host plans admit a launch only
    while dividend x divisor < 2^32 (csrc/qmoe_decode2.hip: pairs2_plan, down2_plan); inside that
    bound the quotient is exact -- checked here at the bound's edge for every divisor the plans can
    produce and on random dividends below it."""
    import numpy as np
    rng = np.random.default_rng(5)
    divisors = sorted(set(range(1, 600)) | {1024, 2048, 4096, 7168, 14336, 65536, 151936})
    for d in divisors:
        if d == 1:
            continue                                  # (k == 1 is special-cased in the kernel: the magic number overflows)
        magic = (1 << 32) // d + 1
        assert magic < (1 << 32)
        limit = ((1 << 32) - 1) // d                  # largest dividend with q * d < 2^32
        q = np.unique(np.concatenate([np.arange(0, min(limit, 4096) + 1), np.arange(max(0, limit - 4096), limit + 1),
                                      rng.integers(0, limit + 1, 4096)])).astype(np.uint64)
        got = (q * np.uint64(magic)) >> np.uint64(32)
        assert np.array_equal(got, q // np.uint64(d)), d
