// GGUF block formats on the device: per-format "lane units".
//
// A lane unit is the piece of one packed row that a single lane decodes: a fixed
// number of weights (UNIT) whose bytes sit at a lane-uniform offset pattern, and a
// list of GROUPS runs of four consecutive activation elements they multiply.  Every
// decoder keeps the reference's float operation order -- d*q (Q8_0), (d*sc)*q - dmin*mn
// (Q4_K/Q5_K), (d*sc)*q (Q6_K) -- so the decoded weights are bit-identical to
// PackedGGUFWeight.dequantize_reference (mini_llm/ops/quantized_weight.py:208-250).
//
// Block layouts (little-endian):
//   Q8_0  34 B / 32 el : f16 d | i8 q[32]
//   Q4_0  18 B / 32 el : f16 d | u8 qs[16]           (low nibbles el 0..15, high 16..31)
//   Q4_K 144 B /256 el : f16 d | f16 dmin | u8 sc[12] | u8 qs[128]
//   Q3_K 110 B /256 el : u8 hmask[32] | u8 qs[64] | u8 sc[12] | f16 d
//   Q5_K 176 B /256 el : f16 d | f16 dmin | u8 sc[12] | u8 qh[32] | u8 qs[128]
//   Q6_K 210 B /256 el : u8 ql[128] | u8 qh[64] | i8 sc[16] | f16 d
//   BF16   2 B /  1 el
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qmoe.h"

namespace qmoe {

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    // v_cvt_f32_f16 honours subnormals, infinities and NaNs.
    return __half2float(__ushort_as_half((unsigned short)h));
}
__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) { return __uint_as_float(h << 16); }

// Loads that only assume the alignment the format guarantees.
__device__ __forceinline__ uint32_t ld_u16(const uint8_t* p) { return *(const __attribute__((address_space(1))) uint16_t*)p; }
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t* p) {
    return ld_u16(p) | (ld_u16(p + 2) << 16);
}
__device__ __forceinline__ uint32_t ld_u32(const uint8_t* p) { return *(const __attribute__((address_space(1))) uint32_t*)p; }
struct __attribute__((packed, aligned(4))) u32x4_a4 { uint32_t v[4]; };
__device__ __forceinline__ u32x4_a4 ld_u32x4_a4(const uint8_t* p) {
    typedef uint32_t V __attribute__((ext_vector_type(4), aligned(4)));
    const V v = *(const __attribute__((address_space(1))) V*)p;
    return u32x4_a4{{v[0], v[1], v[2], v[3]}};
}

__device__ __forceinline__ float sbyte(uint32_t word, int i) {
    return (float)(int)(int8_t)(word >> (8 * i));
}

// The six-bit scale and minimum of K-quant group g from the 12-byte field held in
// three dwords (mini_llm/ops/quantized_weight.py:225-228).
__device__ __forceinline__ void kquant_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int g,
                                                 uint32_t& sc, uint32_t& mn) {
    if (g < 4) {
        sc = (s0 >> (8 * g)) & 63u;
        mn = (s1 >> (8 * g)) & 63u;
    } else {
        int h = g - 4;
        uint32_t hi = (s2 >> (8 * h)) & 255u;
        sc = (hi & 15u) | (((s0 >> (8 * h + 6)) & 3u) << 4);
        mn = (hi >> 4) | (((s1 >> (8 * h + 6)) & 3u) << 4);
    }
}

template <int FMT> struct Fmt;

template <> struct Fmt<QMOE_FMT_Q8_0> {
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 34;
    static constexpr int UNIT = 64, GROUPS = 16;  // two blocks, 68 bytes, 4-byte aligned
    __device__ static int units_per_row(int k) { return k / 64; }
    __device__ static int xoff(int u, int g) { return u * 64 + 4 * g; }
    __device__ static void decode(const uint8_t* row, int u, float* w) {
        const uint8_t* p = row + (size_t)u * 68;
        uint32_t r[17];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4_a4 v = ld_u32x4_a4(p + 16 * i);
            r[4 * i] = v.v[0]; r[4 * i + 1] = v.v[1]; r[4 * i + 2] = v.v[2]; r[4 * i + 3] = v.v[3];
        }
        r[16] = ld_u32(p + 64);
        float d0 = half_bits_to_float(r[0] & 0xFFFFu);
        float d1 = half_bits_to_float(r[8] >> 16);
        // block 0 quants: bytes 2..33 ; block 1 quants: bytes 36..67
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            int b0 = 2 + i, b1 = 36 + i;
            w[i] = d0 * sbyte(r[b0 >> 2], b0 & 3);
            w[32 + i] = d1 * sbyte(r[b1 >> 2], b1 & 3);
        }
    }
    __device__ static float element(const uint8_t* blk, int i) {
        return half_bits_to_float(ld_u16(blk)) * (float)(int)(int8_t)blk[2 + i];
    }
};

template <> struct Fmt<QMOE_FMT_Q4_0> {
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 18;
    static constexpr int UNIT = 32, GROUPS = 8;  // one block, 2-byte aligned
    __device__ static int units_per_row(int k) { return k / 32; }
    __device__ static int xoff(int u, int g) { return u * 32 + 4 * g; }
    __device__ static void decode(const uint8_t* row, int u, float* w) {
        const uint8_t* p = row + (size_t)u * 18;
        float d = half_bits_to_float(ld_u16(p));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t v = ld_u32_a2(p + 2 + 4 * i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t byte = (v >> (8 * j)) & 255u;
                w[4 * i + j] = d * ((float)(byte & 15u) - 8.0f);
                w[16 + 4 * i + j] = d * ((float)(byte >> 4) - 8.0f);
            }
        }
    }
    __device__ static float element(const uint8_t* blk, int i) {
        uint32_t nib = i < 16 ? (blk[2 + i] & 15u) : (uint32_t)(blk[2 + i - 16] >> 4);
        return half_bits_to_float(ld_u16(blk)) * ((float)nib - 8.0f);
    }
};

// Q4_K and Q5_K: a unit is the four consecutive bytes jj of every 32-byte nibble
// chunk of one block -> 32 weights, four from each of the eight groups.
template <int QS_BASE, bool HIGH, int BYTES> struct FmtK45 {
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = BYTES;
    static constexpr int UNIT = 32, GROUPS = 8;
    __device__ static int units_per_row(int k) { return k / 32; }
    // unit u -> block u/8, byte quad jj = u%8; group g covers elements 32g + 4jj .. +3
    __device__ static int xoff(int u, int g) { return (u >> 3) * 256 + 32 * g + 4 * (u & 7); }
    __device__ static void decode(const uint8_t* row, int u, float* w) {
        const uint8_t* p = row + (size_t)(u >> 3) * BYTES;
        int jj = u & 7;
        uint32_t hdr = ld_u32(p);
        float d = half_bits_to_float(hdr & 0xFFFFu), dmin = half_bits_to_float(hdr >> 16);
        uint32_t s0 = ld_u32(p + 4), s1 = ld_u32(p + 8), s2 = ld_u32(p + 12);
        uint32_t qh = HIGH ? ld_u32(p + 16 + 4 * jj) : 0u;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t qs = ld_u32(p + QS_BASE + 32 * c + 4 * jj);
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                int g = 2 * c + part;
                uint32_t sc, mn;
                kquant_scale_min(s0, s1, s2, g, sc, mn);
                float scale = d * (float)sc, floor_ = dmin * (float)mn;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t q = (qs >> (8 * j + 4 * part)) & 15u;
                    if (HIGH) q |= ((qh >> (8 * j + g)) & 1u) << 4;
                    w[4 * g + j] = scale * (float)q - floor_;
                }
            }
        }
    }
    __device__ static float element(const uint8_t* blk, int i) {
        int g = i >> 5, j = i & 31;
        uint32_t sc, mn;
        kquant_scale_min(ld_u32(blk + 4), ld_u32(blk + 8), ld_u32(blk + 12), g, sc, mn);
        uint32_t q = (blk[QS_BASE + 32 * (g >> 1) + j] >> (4 * (g & 1))) & 15u;
        if (HIGH) q |= ((blk[16 + j] >> g) & 1u) << 4;
        float scale = half_bits_to_float(ld_u16(blk)) * (float)sc;
        float floor_ = half_bits_to_float(ld_u16(blk + 2)) * (float)mn;
        return scale * (float)q - floor_;
    }
};
template <> struct Fmt<QMOE_FMT_Q4_K> : FmtK45<16, false, 144> {};
template <> struct Fmt<QMOE_FMT_Q5_K> : FmtK45<48, true, 176> {};

// Q3_K: a unit is byte quad jj of the 32-byte lanes: one hmask dword and the two qs dwords ->
// 32 weights, four from each 32-element plane.  w = (d*(sc-32)) * (q2 - 4*(1-hbit))
// (mini_llm/ops/quantized_weight.py:251-266, native_packed_cpu.cpp:177-193).
template <> struct Fmt<QMOE_FMT_Q3_K> {
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 110;
    static constexpr int UNIT = 32, GROUPS = 8;
    __device__ static int units_per_row(int k) { return k / 32; }
    __device__ static int xoff(int u, int g) { return (u >> 3) * 256 + 32 * g + 4 * (u & 7); }
    // six-bit scale of 16-element group g, minus 32
    __device__ static int scale_of(const uint8_t* sb, int g) {
        const uint32_t lo = ((uint32_t)sb[g & 7] >> (4 * (g >> 3))) & 15u;
        const uint32_t hi = ((uint32_t)sb[8 + (g & 3)] >> (2 * (g >> 2))) & 3u;
        return (int)(lo | (hi << 4)) - 32;
    }
    __device__ static void decode(const uint8_t* row, int u, float* w) {
        const uint8_t* p = row + (size_t)(u >> 3) * 110;
        const int jj = u & 7;
        const uint32_t hm = ld_u32_a2(p + 4 * jj);
        const uint32_t q0 = ld_u32_a2(p + 32 + 4 * jj), q1 = ld_u32_a2(p + 64 + 4 * jj);
        const float d = half_bits_to_float(ld_u16(p + 108));
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const float scale = d * (float)scale_of(p + 96, 2 * g + (jj >> 2));
            const uint32_t qs = g < 4 ? q0 : q1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int low = (int)((qs >> (8 * j + 2 * (g & 3))) & 3u);
                const int keep = (int)((hm >> (8 * j + g)) & 1u);
                w[4 * g + j] = scale * (float)(low - 4 * (1 - keep));
            }
        }
    }
    __device__ static float element(const uint8_t* blk, int i) {
        const int low = (blk[32 + (i >> 7) * 32 + (i & 31)] >> (2 * ((i & 127) >> 5))) & 3;
        const int keep = (blk[i & 31] >> (i >> 5)) & 1;
        const float scale = half_bits_to_float(ld_u16(blk + 108)) * (float)scale_of(blk + 96, i >> 4);
        return scale * (float)(low - 4 * (1 - keep));
    }
};

// Q6_K: a unit is byte quad jj of one 128-element half h: two ql dwords and one qh
// dword -> 16 weights, four from each 32-element quarter of the half.
template <> struct Fmt<QMOE_FMT_Q6_K> {
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 210;
    static constexpr int UNIT = 16, GROUPS = 4;
    __device__ static int units_per_row(int k) { return k / 16; }
    // unit u -> block u/16, half h = (u/8)%2, quad jj = u%8; group = quarter
    __device__ static int xoff(int u, int g) {
        return (u >> 4) * 256 + ((u >> 3) & 1) * 128 + 32 * g + 4 * (u & 7);
    }
    __device__ static void decode(const uint8_t* row, int u, float* w) {
        const uint8_t* p = row + (size_t)(u >> 4) * 210;
        int h = (u >> 3) & 1, jj = u & 7;
        uint32_t la = ld_u32_a2(p + 64 * h + 4 * jj);
        uint32_t lb = ld_u32_a2(p + 64 * h + 32 + 4 * jj);
        uint32_t hb = ld_u32_a2(p + 128 + 32 * h + 4 * jj);
        float d = half_bits_to_float(ld_u16(p + 208));
        const int8_t* sc = (const int8_t*)(p + 192 + 8 * h + (jj >> 2));
#pragma unroll
        for (int quarter = 0; quarter < 4; ++quarter) {
            float scale = d * (float)(int)sc[2 * quarter];
            uint32_t lo = (quarter & 1) ? lb : la;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t low = (lo >> (8 * j + 4 * (quarter >> 1))) & 15u;
                uint32_t high = (hb >> (8 * j + 2 * quarter)) & 3u;
                w[4 * quarter + j] = scale * (float)((int)(low | (high << 4)) - 32);
            }
        }
    }
    __device__ static float element(const uint8_t* blk, int i) {
        int h = i >> 7, r = i & 127;
        uint32_t low = (blk[64 * h + (i & 63)] >> (4 * (r >> 6))) & 15u;
        uint32_t high = (blk[128 + 32 * h + (i & 31)] >> (2 * (r >> 5))) & 3u;
        float scale = half_bits_to_float(ld_u16(blk + 208)) * (float)(int)(int8_t)blk[192 + (i >> 4)];
        return scale * (float)((int)(low | (high << 4)) - 32);
    }
};

template <> struct Fmt<QMOE_FMT_BF16> {
    static constexpr int BLOCK_ELEMS = 1, BLOCK_BYTES = 2;
    static constexpr int UNIT = 8, GROUPS = 2;  // 16 bytes; rows with k%8 != 0 use the tail path
    __device__ static int units_per_row(int k) { return k / 8; }
    __device__ static int xoff(int u, int g) { return u * 8 + 4 * g; }
    __device__ static void decode(const uint8_t* row, int u, float* w) {
        const uint8_t* p = row + (size_t)u * 16;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t v = ld_u32_a2(p + 4 * i);
            w[2 * i] = bf16_bits_to_float(v & 0xFFFFu);
            w[2 * i + 1] = bf16_bits_to_float(v >> 16);
        }
    }
    __device__ static float element(const uint8_t* blk, int) { return bf16_bits_to_float(ld_u16(blk)); }
};

// Host-side format table.
inline int block_elems(int fmt) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: case QMOE_FMT_Q4_0: return 32;
    case QMOE_FMT_Q4_K: case QMOE_FMT_Q5_K: case QMOE_FMT_Q6_K: case QMOE_FMT_Q3_K: return 256;
    case QMOE_FMT_BF16: return 1;
    default: return 0;
    }
}
inline int block_bytes(int fmt) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: return 34;
    case QMOE_FMT_Q4_0: return 18;
    case QMOE_FMT_Q4_K: return 144;
    case QMOE_FMT_Q3_K: return 110;
    case QMOE_FMT_Q5_K: return 176;
    case QMOE_FMT_Q6_K: return 210;
    case QMOE_FMT_BF16: return 2;
    default: return 0;
    }
}
inline bool format_implemented(int fmt) {
    return fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q4_0 || fmt == QMOE_FMT_Q4_K || fmt == QMOE_FMT_Q3_K ||
           fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_BF16;
}
inline int64_t row_bytes(int fmt, int64_t k) { return k / block_elems(fmt) * block_bytes(fmt); }

}  // namespace qmoe
