"""Writes tests/golden/ref_native_vectors.npz with outputs of the reference's own native
packed CPU library (mini_llm/ops/native_packed_cpu.cpp, built by oracle/Makefile into
oracle/_ref/) on small seeded inputs:
  <fmt>_blocks / <fmt>_dense   packed rows and mylocal_packed_gemv applied to identity rows,
                               i.e. every decoded coefficient as the reference decodes it
  <fmt>_x / <fmt>_gemv         random activations and the reference's GEMV result
  expert_*                     one Q5_K/Q5_K/Q6_K SwiGLU expert through mylocal_packed_expert
  (formats: Q8_0, Q4_0, Q4_K, Q5_K, Q6_K, Q3_K)
Only this container has the reference checkout; the vectors travel, the reference does not.
Run from the repository root after `make -C oracle`: python tests/golden/make_ref_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import native  # noqa: E402


def main():
    if native.load_ref() is None:
        raise SystemExit("oracle/_ref/libref_packed_cpu.so not built (reference checkout absent?)")
    sizes = {"Q8_0": 34, "Q4_0": 18, "Q4_K": 144, "Q5_K": 176, "Q6_K": 210}
    elems = {"Q8_0": 32, "Q4_0": 32, "Q4_K": 256, "Q5_K": 256, "Q6_K": 256}
    scale_at = {"Q8_0": [0], "Q4_0": [0], "Q4_K": [0, 2], "Q5_K": [0, 2], "Q6_K": [208]}
    out = {}
    rng = np.random.default_rng(20251)
    for fmt in sizes:
        rows, k = 6, 512
        nblocks = rows * k // elems[fmt]
        blk = rng.integers(0, 256, (nblocks, sizes[fmt]), dtype=np.uint8)
        for at in scale_at[fmt]:  # finite, modest scales incl. one fp16 subnormal and a negative one
            s = rng.normal(0, 0.01, nblocks).astype("<f2")
            s[0] = np.float16(3e-6)
            blk[:, at:at + 2] = s.view(np.uint8).reshape(nblocks, 2)
        dense = native.ref_gemv(np.eye(k, dtype=np.float32), blk, (rows, k), fmt).T.copy()
        x = rng.standard_normal((3, k), dtype=np.float32)
        out[f"{fmt}_blocks"] = blk
        out[f"{fmt}_dense"] = dense
        out[f"{fmt}_x"] = x
        out[f"{fmt}_gemv"] = native.ref_gemv(x, blk, (rows, k), fmt)
    d, f = 256, 256
    def bank(fmt, n, k):
        nb = n * k // elems[fmt]
        b = rng.integers(0, 256, (nb, sizes[fmt]), dtype=np.uint8)
        for at in scale_at[fmt]:
            b[:, at:at + 2] = np.abs(rng.normal(2e-3, 2e-4, nb)).astype("<f2").view(np.uint8).reshape(nb, 2)
        return b
    gate, up, down = bank("Q5_K", f, d), bank("Q5_K", f, d), bank("Q6_K", d, f)
    x = rng.standard_normal((2, d), dtype=np.float32) * 0.5
    out["expert_gate"], out["expert_up"], out["expert_down"], out["expert_x"] = gate, up, down, x
    out["expert_out"] = native.ref_expert(x, (gate, (f, d), "Q5_K"), (up, (f, d), "Q5_K"), (down, (d, f), "Q6_K"))
    # Q3_K, from a generator of its own so that the vectors above stay as they were
    rng3 = np.random.default_rng(20253)
    rows, k = 6, 512
    nblocks = rows * k // 256
    blk = rng3.integers(0, 256, (nblocks, 110), dtype=np.uint8)
    s = rng3.normal(0, 0.01, nblocks).astype("<f2")
    s[0] = np.float16(3e-6)
    blk[:, 108:110] = s.view(np.uint8).reshape(nblocks, 2)
    x = rng3.standard_normal((3, k), dtype=np.float32)
    out["Q3_K_blocks"] = blk
    out["Q3_K_dense"] = native.ref_gemv(np.eye(k, dtype=np.float32), blk, (rows, k), "Q3_K").T.copy()
    out["Q3_K_x"] = x
    out["Q3_K_gemv"] = native.ref_gemv(x, blk, (rows, k), "Q3_K")
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_native_vectors.npz"), **out)


if __name__ == "__main__":
    main()
