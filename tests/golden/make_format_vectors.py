"""Writes tests/golden/format_vectors.npz: hand-packed blocks and their exact decoded values.

The cases are the known-answer vectors held by the reference's own tests, re-encoded here
as data (packed bytes in, fp32 values out):
  q4_0_nibbles      tests/test_0106a_packed_gguf.py:18-25   d=.5, every byte 0x83
  q4_k_scales       tests/test_0106a_packed_gguf.py:28-33   d=1, dmin=0, four groups scale 1
  q3_k_keep / q3_k_minus4  tests/test_0106a_packed_gguf.py:36-43   every scale 33-32=1, every code 2, mask all ones / all zeros
  q5_k_group0       tests/test_0106g_q5k_packed.py:23-35    8.25 x32 then zeros
  q5_k_group7       tests/test_0106g_q5k_packed.py:37-45    zeros then 9.0 x32
  q6_k_all_codes    tests/test_0106l_q6k_packed.py:25-46    every 6-bit code x 16 signed scales
  bf16_bytes        tests/test_0106l_gguf_bf16.py:47-57     six little-endian words
  router_rows       tests/test_0106v_router_decode.py:44-62 tie / inf / NaN rows (inputs only;
                    expected ids follow the documented order: descending, lower id, NaN last)
Run from the repository root: python tests/golden/make_format_vectors.py
"""
import os

import numpy as np


def f16(v):
    return np.array([v], "<f2").view(np.uint8)


def main():
    out = {}
    # Q4_0: low nibble 3 -> (3-8)*.5 = -2.5 for elements 0..15, high nibble 8 -> 0 for 16..31
    out["q4_0_nibbles_blocks"] = np.concatenate([f16(0.5), np.full(16, 0x83, np.uint8)])
    out["q4_0_nibbles_expected"] = np.array([-2.5] * 16 + [0.0] * 16, np.float32)
    # Q4_K: scales 1,1,1,1,0,0,0,0 ; minima 0 ; every qs byte 0x12
    out["q4_k_scales_blocks"] = np.concatenate(
        [f16(1), f16(0), np.array([1] * 4 + [0] * 8, np.uint8), np.full(128, 0x12, np.uint8)])
    out["q4_k_scales_expected"] = np.array(([2.0] * 32 + [1.0] * 32) * 2 + [0.0] * 128, np.float32)
    # Q3_K: scale bytes 0x11 x8 + 0xAA x4 -> every six-bit scale 33 (= +1), qs 0xAA -> every code 2;
    # mask bit 1 keeps the code, 0 subtracts four
    for name, mask, value in (("q3_k_keep", 0xFF, 2.0), ("q3_k_minus4", 0x00, -2.0)):
        out[name + "_blocks"] = np.concatenate([np.full(32, mask, np.uint8), np.full(64, 0xAA, np.uint8),
                                                np.array([0x11] * 8 + [0xAA] * 4, np.uint8), f16(1)])
        out[name + "_expected"] = np.full(256, value, np.float32)
    # Q5_K group 0: d=.5 dmin=.25 scale0=1 min0=1, high bit of group 0 set, nibbles 0x21
    raw = np.zeros(176, np.uint8)
    raw[0:2], raw[2:4] = f16(0.5), f16(0.25)
    raw[4], raw[8] = 1, 1
    raw[16:48] = 1
    raw[48:176] = 0x21
    out["q5_k_group0_blocks"] = raw.copy()
    out["q5_k_group0_expected"] = np.array([8.25] * 32 + [0.0] * 224, np.float32)
    # Q5_K group 7: high bit 7, scale of group 7 = low nibble of field byte 11, no minimum
    raw[16:48] = 0x80
    raw[4:16] = 0
    raw[15] = 0x01
    out["q5_k_group7_blocks"] = raw.copy()
    out["q5_k_group7_expected"] = np.array([0.0] * 224 + [9.0] * 32, np.float32)
    # Q6_K: codes -32..31 tiled four times, sixteen signed sub-scales incl. -128 and 127
    quants = np.tile(np.arange(-32, 32, dtype=np.int16), 4)
    scales = np.array([-128, -64, -32, -16, -1, 0, 1, 2, 3, 7, 16, 31, 63, 100, 126, 127], np.int8)
    raw = np.zeros(210, np.uint8)
    for half in range(2):
        for lane in range(32):
            q = [int(quants[half * 128 + lane + 32 * g]) + 32 for g in range(4)]
            raw[half * 64 + lane] = (q[0] & 15) | ((q[2] & 15) << 4)
            raw[half * 64 + 32 + lane] = (q[1] & 15) | ((q[3] & 15) << 4)
            raw[128 + half * 32 + lane] = sum((q[g] >> 4) << (2 * g) for g in range(4))
    raw[192:208] = scales.view(np.uint8)
    raw[208:210] = f16(0.03125)
    out["q6_k_all_codes_blocks"] = raw
    out["q6_k_all_codes_expected"] = (np.float32(0.03125) * np.repeat(scales.astype(np.float32), 16)
                                      * quants.astype(np.float32)).astype(np.float32)
    out["bf16_bytes_blocks"] = np.array([0x80, 0x3F, 0x20, 0xC0, 0, 0x80, 0x80, 0x7F, 0x80, 0xFF, 0x81, 0x7F], np.uint8)
    out["bf16_bytes_expected_bits"] = np.array([0x3F800000, 0xC0200000, 0x80000000, 0x7F800000, 0xFF800000, 0x7F810000],
                                               np.uint32)
    rows = [
        [0.0] * 512,
        [2.0, 1.0, 2.0, -1.0, -np.inf, 2.0],
        [1.0, float(np.nextafter(np.float32(1), np.float32(2))), 1.0, -10.0],
        [10000.0, -10000.0, 0.0, 1.0],
        [np.nan, 1.0, -np.inf, 1.0, np.nan],
        [np.inf, 2.0, np.inf, -np.inf],
        [-np.inf] * 4,
    ]
    expected_ids = [[0, 1, 2, 3], [0, 2, 5, 1], [1, 0, 2, 3], [0, 3, 2, 1], [1, 3, 2, 0], [0, 2, 1, 3], [0, 1, 2, 3]]
    for i, (row, ids) in enumerate(zip(rows, expected_ids)):
        out[f"router_row{i}"] = np.array(row, np.float32)
        out[f"router_row{i}_ids"] = np.array(ids, np.int64)
    np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "format_vectors.npz"), **out)


if __name__ == "__main__":
    main()
