"""Wait-state check of the emitted gfx950 assembly of the LDS-DMA kernels.

The kernels of csrc/qmoe_span.hip and csrc/qmoe_decode2.hip issue their LDS-DMA from inline
assembly, which the compiler's hazard recogniser does not look into.  Two rules of the ISA
manual that the compiler keeps for its own instructions are therefore this package's to keep:

* five wait states between a vector instruction that writes a scalar register (v_readfirstlane,
  v_readlane: what ``uniform()`` becomes when a value lives in vector registers) and a memory
  instruction that reads that register as its base;
* one wait state between a scalar write of M0 and an LDS-DMA that reads it.

``scan`` counts, per kernel, the memory instructions that follow such a write too closely.
Versions of span_kernel whose plain-row instantiations had sites of the first kind faulted on
the GPU; the versions that run have none there (every base is computed by scalar instructions).

    python -m mylocal_llm_amd._asm_check            # prints the counts for both sources
"""
import re
import subprocess
from collections import Counter

from ._build import CSRC, HIPCC_FLAGS, _hipcc

SOURCES = ("qmoe_span.hip", "qmoe_decode2.hip")
_MEMORY = re.compile(r"(global|flat|buffer|scratch)_(load|store|atomic)")
_LDS_DMA = re.compile(r"(global|buffer)_load_lds")
_VALU_TO_SGPR = re.compile(r"v_(readfirstlane|readlane)_b32 s(\d+),")
_SGPR_RANGE = re.compile(r"\bs\[(\d+):(\d+)\]")
_M0_WRITE = re.compile(r"s_\w+ m0,")
_NOP = re.compile(r"s_nop (\d+)")


def device_asm(source):
    """gfx950 assembly text of one source of csrc/, with the flags the library is built with."""
    import os
    cmd = [_hipcc(), *HIPCC_FLAGS, "--cuda-device-only", "-S", os.path.join(CSRC, source), "-o", "-"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode:
        raise RuntimeError(f"hipcc failed on {source}:\n{proc.stderr[-3000:]}")
    return proc.stdout


def _instructions(asm):
    """(text, kernel) of every instruction, labels and directives dropped."""
    kernel = None
    for line in asm.splitlines():
        text = line.split(";")[0].strip()      # (a label may carry a trailing comment)
        if not text:
            continue
        if text.endswith(":") and not text.startswith("."):
            if text.startswith("_Z"):
                kernel = text[:-1]
            continue
        if text.startswith("."):
            continue
        yield text, kernel


def kernels(asm):
    """Names (mangled) of the kernels and device functions the assembly defines."""
    return sorted({kernel for _, kernel in _instructions(asm) if kernel})


def scan(asm):
    """{kernel: Counter(sgpr_base_after_valu=..., m0_back_to_back=...)} for every kernel with a finding."""
    code = list(_instructions(asm))
    found = {}
    for at, (text, kernel) in enumerate(code):
        if not _MEMORY.match(text):
            continue
        bases = _SGPR_RANGE.search(text)
        if bases:
            registers = set(range(int(bases.group(1)), int(bases.group(2)) + 1))
            waited, back = 0, at - 1
            while back >= 0 and waited < 5:
                earlier = code[back][0]
                nop = _NOP.match(earlier)
                waited += 1 + (int(nop.group(1)) if nop else 0)
                write = _VALU_TO_SGPR.match(earlier)
                if write and int(write.group(2)) in registers and waited <= 5:
                    found.setdefault(kernel, Counter())["sgpr_base_after_valu"] += 1
                    break
                back -= 1
        if _LDS_DMA.match(text) and at and _M0_WRITE.match(code[at - 1][0]):
            found.setdefault(kernel, Counter())["m0_back_to_back"] += 1
    return found


def plain_row_span_kernel(name):
    """True for span_kernel<FMT, false, PD> (mangled): the instantiations without gate/up pairing."""
    return bool(re.match(r"_ZN4qmoe11span_kernelILi\d+ELb0ELi\d+EEE", name or ""))


if __name__ == "__main__":
    for source in SOURCES:
        findings = scan(device_asm(source))
        print(source)
        for kernel in sorted(findings, key=str):
            print("   ", kernel, dict(findings[kernel]))
        if not findings:
            print("    (no findings)")
