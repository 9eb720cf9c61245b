// Single-token weight-streaming engine: one pass over packed rows at HBM speed.
//
// Every format is cut into 64-element lane units.  A lane keeps the 64 activation values
// of its unit position in registers for the whole problem, loads its unit of each row
// straight from global memory with the widest loads the block layout allows, decodes in
// registers and accumulates in fp32; one row (or one gate/up row pair) costs one DPP
// reduction across the lanes that share it.  Rows are never staged in LDS: consecutive
// lanes read consecutive units, so a wave's loads cover one contiguous stretch of the row.
//
//   Q8_0  unit = 2 blocks            68 B  (4 x 16 B + 4 B)
//   Q6_K  unit = quarter block       48 B + 8 B scales + 2 B d   (16-lane runs of 4 quarters)
//   Q5_K  unit = quarter block       40 B + 16 B header          (8-lane runs of 8 groups)
//   Q4_K  unit = quarter block       32 B + 16 B header
//   BF16  unit = 64 elements        128 B
#pragma once
#include "qmoe_common.hpp"
#include "qmoe_formats.hpp"

namespace qmoe {

// ---- DPP reductions -----------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_add(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false);
    return v + __int_as_float(r);
}
// Sum over groups of LR consecutive lanes (LR = 8, 16, 32 or 64).  The total of a group is
// valid in its last lane.
template <int LR>
__device__ __forceinline__ float group_sum(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror: lanes of an 8-group now agree
    if (LR >= 16) v = dpp_add<0x140>(v);        // row_mirror: 16 lanes
    if (LR >= 32) v = dpp_add<0x142, 0xa>(v);   // row_bcast15: lanes 16..31 / 48..63 gain the row before
    if (LR >= 64) v = dpp_add<0x143, 0xc>(v);   // row_bcast31: lanes 32..63 gain lanes 0..31
    return v;
}


__device__ __forceinline__ float ubyte_f(uint32_t w, int i) {
    // v_cvt_f32_ubyte{0..3}
    return (float)((w >> (8 * i)) & 0xFFu);
}

// Activation loader: 4 consecutive elements of any supported type as fp32.
__device__ __forceinline__ float4 load_x4(const void* x, int xdt, int i) {
    if (xdt == QMOE_DT_F32) return Elem<QMOE_DT_F32>::load4(x, i);
    if (xdt == QMOE_DT_F16) return Elem<QMOE_DT_F16>::load4(x, i);
    return Elem<QMOE_DT_BF16>::load4(x, i);
}

// Where a lane's activation values come from: global memory of any supported type, or the
// workgroup's fp32 staging area in LDS.  The staging area carries 4 floats of padding after
// every 64, so that lanes reading consecutive units (272 bytes apart) spread over all banks.
struct GlobalX {
    const void* x;
    int xdt;
    __device__ __forceinline__ float4 operator()(int i) const { return load_x4(x, xdt, i); }
};
struct StagedX {
    const float* xs;
    __device__ __forceinline__ static int at(int i) { return i + 4 * (i >> 6); }
    __device__ __forceinline__ float4 operator()(int i) const { return *(const float4*)(xs + at(i)); }
};

template <int FMT> struct Unit64;

// ---- Q8_0 -----------------------------------------------------------------------------------
template <> struct Unit64<QMOE_FMT_Q8_0> {
    static constexpr int RAW = 17, AUX = 1;
    static constexpr int ROW_ALIGN = 4;
    template <class X> __device__ __forceinline__ static void load_x(const X& x, int u, float* xr, float*) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float4 v = x(u * 64 + 4 * i);
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
    }
    __device__ __forceinline__ static void load_w(const uint8_t* row, int u, uint32_t* r) {
        const uint8_t* p = row + (size_t)u * 68;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32x4_t v = ldg_u32x4<4>(p + 16 * i);
            r[4 * i] = v[0]; r[4 * i + 1] = v[1]; r[4 * i + 2] = v[2]; r[4 * i + 3] = v[3];
        }
        r[16] = ldg<uint32_t>(p + 64);
    }
    __device__ __forceinline__ static float dot(const uint32_t* r, const float* xr, const float*) {
        const float d0 = half_bits_to_float(r[0] & 0xFFFFu), d1 = half_bits_to_float(r[8] >> 16);
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int b0 = 2 + i, b1 = 36 + i;
            s0 += sbyte(r[b0 >> 2], b0 & 3) * xr[i];
            s1 += sbyte(r[b1 >> 2], b1 & 3) * xr[32 + i];
        }
        return d0 * s0 + d1 * s1;
    }
    // the 64 dequantised weights of the unit, in unit order
    __device__ __forceinline__ static void decode(const uint32_t* r, float* w) {
        const float d0 = half_bits_to_float(r[0] & 0xFFFFu), d1 = half_bits_to_float(r[8] >> 16);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int b0 = 2 + i, b1 = 36 + i;
            w[i] = d0 * sbyte(r[b0 >> 2], b0 & 3);
            w[32 + i] = d1 * sbyte(r[b1 >> 2], b1 & 3);
        }
    }
    // column of unit element 8*m (elements 8m..8m+7 are consecutive columns)
    __device__ __forceinline__ static int kstep(int u, int m) { return u * 64 + 8 * m; }
};

// ---- Q6_K -----------------------------------------------------------------------------------
// unit u: block u/4, half h = (u/2)%2, column group c = u%2; element (quarter q, j) of the
// unit is block element 128h + 32q + 16c + j.
template <> struct Unit64<QMOE_FMT_Q6_K> {
    static constexpr int RAW = 15, AUX = 4;
    static constexpr int ROW_ALIGN = 2;
    template <class X> __device__ __forceinline__ static void load_x(const X& x, int u, float* xr, float* aux) {
        const int base = (u >> 2) * 256 + ((u >> 1) & 1) * 128 + (u & 1) * 16;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float4 v = x(base + 32 * q + 4 * i);
                xr[16 * q + 4 * i] = v.x; xr[16 * q + 4 * i + 1] = v.y; xr[16 * q + 4 * i + 2] = v.z; xr[16 * q + 4 * i + 3] = v.w;
                s += (v.x + v.y) + (v.z + v.w);
            }
            aux[q] = 32.0f * s;
        }
    }
    __device__ __forceinline__ static void load_w(const uint8_t* row, int u, uint32_t* r) {
        const uint8_t* b = row + (size_t)(u >> 2) * 210;
        const int h = (u >> 1) & 1, c = u & 1;
        const u32x4_t la = ldg_u32x4<2>(b + 64 * h + 16 * c);
        const u32x4_t lb = ldg_u32x4<2>(b + 64 * h + 32 + 16 * c);
        const u32x4_t hq = ldg_u32x4<2>(b + 128 + 32 * h + 16 * c);
        const u32x2_t sc = ldg_u32x2<2>(b + 192 + 8 * h);
#pragma unroll
        for (int i = 0; i < 4; ++i) { r[i] = la[i]; r[4 + i] = lb[i]; r[8 + i] = hq[i]; }
        // the four sub-block scales of this unit are bytes c, c+2, c+4, c+6 of the half's eight
        const uint32_t s0 = sc[0] >> (8 * c), s1 = sc[1] >> (8 * c);
        r[12] = (s0 & 0xFFu) | ((s0 >> 8) & 0xFF00u);         // scales of quarters 0, 1
        r[13] = (s1 & 0xFFu) | ((s1 >> 8) & 0xFF00u);         // scales of quarters 2, 3
        r[14] = ld_u16(b + 208);
    }
    __device__ __forceinline__ static float dot(const uint32_t* r, const float* xr, const float* aux) {
        const float d = half_bits_to_float(r[14]);
        float total = 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float acc = 0.f;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const uint32_t src = (q & 1) ? r[4 + m] : r[m];
                const uint32_t lo = (q & 2) ? ((src >> 4) & 0x0F0F0F0Fu) : (src & 0x0F0F0F0Fu);
                const uint32_t hi = (r[8 + m] >> (2 * q)) & 0x03030303u;
                const uint32_t code = lo | (hi << 4);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc += ubyte_f(code, j) * xr[16 * q + 4 * m + j];
            }
            const float scale = d * sbyte(r[12 + (q >> 1)], q & 1);
            total += scale * (acc - aux[q]);
        }
        return total;
    }
    __device__ __forceinline__ static void decode(const uint32_t* r, float* w) {
        const float d = half_bits_to_float(r[14]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float scale = d * sbyte(r[12 + (q >> 1)], q & 1);
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const uint32_t src = (q & 1) ? r[4 + m] : r[m];
                const uint32_t lo = (q & 2) ? ((src >> 4) & 0x0F0F0F0Fu) : (src & 0x0F0F0F0Fu);
                const uint32_t hi = (r[8 + m] >> (2 * q)) & 0x03030303u;
                const uint32_t code = lo | (hi << 4);
#pragma unroll
                for (int j = 0; j < 4; ++j) w[16 * q + 4 * m + j] = scale * (ubyte_f(code, j) - 32.0f);
            }
        }
    }
    __device__ __forceinline__ static int kstep(int u, int m) {
        return (u >> 2) * 256 + ((u >> 1) & 1) * 128 + (u & 1) * 16 + 32 * (m >> 1) + 8 * (m & 1);
    }
};

// ---- Q5_K -----------------------------------------------------------------------------------
// unit u: block u/4, byte column c = u%4; element (group g, j) of the unit is block element
// 32g + 8c + j.
template <> struct Unit64<QMOE_FMT_Q5_K> {
    static constexpr int RAW = 14, AUX = 8;
    static constexpr int ROW_ALIGN = 16;
    template <class X> __device__ __forceinline__ static void load_x(const X& x, int u, float* xr, float* aux) {
        const int base = (u >> 2) * 256 + (u & 3) * 8;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            float4 a = x(base + 32 * g), b = x(base + 32 * g + 4);
            xr[8 * g] = a.x; xr[8 * g + 1] = a.y; xr[8 * g + 2] = a.z; xr[8 * g + 3] = a.w;
            xr[8 * g + 4] = b.x; xr[8 * g + 5] = b.y; xr[8 * g + 6] = b.z; xr[8 * g + 7] = b.w;
            aux[g] = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
        }
    }
    __device__ __forceinline__ static void load_w(const uint8_t* row, int u, uint32_t* r) {
        const uint8_t* b = row + (size_t)(u >> 2) * 176;
        const int c = u & 3;
        const uint4 hdr = ldg<uint4>(b);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
        const uint2 qh = ldg<uint2>(b + 16 + 8 * c);
        r[4] = qh.x; r[5] = qh.y;
#pragma unroll
        for (int g2 = 0; g2 < 4; ++g2) {
            const uint2 qs = ldg<uint2>(b + 48 + 32 * g2 + 8 * c);
            r[6 + 2 * g2] = qs.x; r[7 + 2 * g2] = qs.y;
        }
    }
    __device__ __forceinline__ static float dot(const uint32_t* r, const float* xr, const float* aux) {
        const float d = half_bits_to_float(r[0] & 0xFFFFu), dmin = half_bits_to_float(r[0] >> 16);
        // 6-bit scales / minima of the eight groups, four per dword
        const uint32_t sc_lo = r[1] & 0x3F3F3F3Fu, mn_lo = r[2] & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (r[3] & 0x0F0F0F0Fu) | ((r[1] >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((r[3] >> 4) & 0x0F0F0F0Fu) | ((r[2] >> 2) & 0x30303030u);
        float total = 0.f;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            float acc = 0.f;
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const uint32_t qs = r[6 + 2 * (g >> 1) + m];
                const uint32_t lo = (g & 1) ? ((qs >> 4) & 0x0F0F0F0Fu) : (qs & 0x0F0F0F0Fu);
                const uint32_t hb = g < 4 ? ((r[4 + m] << (4 - g)) & 0x10101010u) : ((r[4 + m] >> (g - 4)) & 0x10101010u);
                const uint32_t code = lo | hb;
#pragma unroll
                for (int j = 0; j < 4; ++j) acc += ubyte_f(code, j) * xr[8 * g + 4 * m + j];
            }
            const float sc = ubyte_f(g < 4 ? sc_lo : sc_hi, g & 3), mn = ubyte_f(g < 4 ? mn_lo : mn_hi, g & 3);
            total += (d * sc) * acc - (dmin * mn) * aux[g];
        }
        return total;
    }
    __device__ __forceinline__ static void decode(const uint32_t* r, float* w) {
        const float d = half_bits_to_float(r[0] & 0xFFFFu), dmin = half_bits_to_float(r[0] >> 16);
        const uint32_t sc_lo = r[1] & 0x3F3F3F3Fu, mn_lo = r[2] & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (r[3] & 0x0F0F0F0Fu) | ((r[1] >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((r[3] >> 4) & 0x0F0F0F0Fu) | ((r[2] >> 2) & 0x30303030u);
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const float scale = d * ubyte_f(g < 4 ? sc_lo : sc_hi, g & 3);
            const float floor_ = dmin * ubyte_f(g < 4 ? mn_lo : mn_hi, g & 3);
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const uint32_t qs = r[6 + 2 * (g >> 1) + m];
                const uint32_t lo = (g & 1) ? ((qs >> 4) & 0x0F0F0F0Fu) : (qs & 0x0F0F0F0Fu);
                const uint32_t hb = g < 4 ? ((r[4 + m] << (4 - g)) & 0x10101010u) : ((r[4 + m] >> (g - 4)) & 0x10101010u);
                const uint32_t code = lo | hb;
#pragma unroll
                for (int j = 0; j < 4; ++j) w[8 * g + 4 * m + j] = scale * ubyte_f(code, j) - floor_;
            }
        }
    }
    __device__ __forceinline__ static int kstep(int u, int m) { return (u >> 2) * 256 + (u & 3) * 8 + 32 * m; }
};

// ---- Q4_K -----------------------------------------------------------------------------------
// Q5_K without the fifth bit: unit u = block u/4, byte column c = u%4; element (group g, j) of
// the unit is block element 32g + 8c + j.
template <> struct Unit64<QMOE_FMT_Q4_K> {
    static constexpr int RAW = 12, AUX = 8;
    static constexpr int ROW_ALIGN = 16;
    template <class X> __device__ __forceinline__ static void load_x(const X& x, int u, float* xr, float* aux) {
        Unit64<QMOE_FMT_Q5_K>::load_x(x, u, xr, aux);
    }
    __device__ __forceinline__ static void load_w(const uint8_t* row, int u, uint32_t* r) {
        const uint8_t* b = row + (size_t)(u >> 2) * 144;
        const int c = u & 3;
        const uint4 hdr = ldg<uint4>(b);
        r[0] = hdr.x; r[1] = hdr.y; r[2] = hdr.z; r[3] = hdr.w;
#pragma unroll
        for (int g2 = 0; g2 < 4; ++g2) {
            const uint2 qs = ldg<uint2>(b + 16 + 32 * g2 + 8 * c);
            r[4 + 2 * g2] = qs.x; r[5 + 2 * g2] = qs.y;
        }
    }
    __device__ __forceinline__ static float dot(const uint32_t* r, const float* xr, const float* aux) {
        const float d = half_bits_to_float(r[0] & 0xFFFFu), dmin = half_bits_to_float(r[0] >> 16);
        const uint32_t sc_lo = r[1] & 0x3F3F3F3Fu, mn_lo = r[2] & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (r[3] & 0x0F0F0F0Fu) | ((r[1] >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((r[3] >> 4) & 0x0F0F0F0Fu) | ((r[2] >> 2) & 0x30303030u);
        float total = 0.f;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            float acc = 0.f;
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const uint32_t qs = r[4 + 2 * (g >> 1) + m];
                const uint32_t code = (g & 1) ? ((qs >> 4) & 0x0F0F0F0Fu) : (qs & 0x0F0F0F0Fu);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc += ubyte_f(code, j) * xr[8 * g + 4 * m + j];
            }
            const float sc = ubyte_f(g < 4 ? sc_lo : sc_hi, g & 3), mn = ubyte_f(g < 4 ? mn_lo : mn_hi, g & 3);
            total += (d * sc) * acc - (dmin * mn) * aux[g];
        }
        return total;
    }
    __device__ __forceinline__ static void decode(const uint32_t* r, float* w) {
        const float d = half_bits_to_float(r[0] & 0xFFFFu), dmin = half_bits_to_float(r[0] >> 16);
        const uint32_t sc_lo = r[1] & 0x3F3F3F3Fu, mn_lo = r[2] & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (r[3] & 0x0F0F0F0Fu) | ((r[1] >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((r[3] >> 4) & 0x0F0F0F0Fu) | ((r[2] >> 2) & 0x30303030u);
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const float scale = d * ubyte_f(g < 4 ? sc_lo : sc_hi, g & 3);
            const float floor_ = dmin * ubyte_f(g < 4 ? mn_lo : mn_hi, g & 3);
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const uint32_t qs = r[4 + 2 * (g >> 1) + m];
                const uint32_t code = (g & 1) ? ((qs >> 4) & 0x0F0F0F0Fu) : (qs & 0x0F0F0F0Fu);
#pragma unroll
                for (int j = 0; j < 4; ++j) w[8 * g + 4 * m + j] = scale * ubyte_f(code, j) - floor_;
            }
        }
    }
    __device__ __forceinline__ static int kstep(int u, int m) { return (u >> 2) * 256 + (u & 3) * 8 + 32 * m; }
};

// ---- BF16 -----------------------------------------------------------------------------------
template <> struct Unit64<QMOE_FMT_BF16> {
    static constexpr int RAW = 32, AUX = 1;
    static constexpr int ROW_ALIGN = 16;
    template <class X> __device__ __forceinline__ static void load_x(const X& x, int u, float* xr, float*) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float4 v = x(u * 64 + 4 * i);
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
    }
    __device__ __forceinline__ static void load_w(const uint8_t* row, int u, uint32_t* r) {
        const uint8_t* p = row + (size_t)u * 128;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint4 v = ldg<uint4>(p + 16 * i);
            r[4 * i] = v.x; r[4 * i + 1] = v.y; r[4 * i + 2] = v.z; r[4 * i + 3] = v.w;
        }
    }
    __device__ __forceinline__ static float dot(const uint32_t* r, const float* xr, const float*) {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            s0 += __uint_as_float(r[i] << 16) * xr[2 * i];
            s1 += __uint_as_float(r[i] & 0xFFFF0000u) * xr[2 * i + 1];
        }
        return s0 + s1;
    }
    __device__ __forceinline__ static void decode(const uint32_t* r, float* w) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            w[2 * i] = __uint_as_float(r[i] << 16);
            w[2 * i + 1] = __uint_as_float(r[i] & 0xFFFF0000u);
        }
    }
    __device__ __forceinline__ static int kstep(int u, int m) { return u * 64 + 8 * m; }
};

// ---- problem lists ----------------------------------------------------------------------------
static constexpr int STREAM_THREADS = 256;
static constexpr int STREAM_WAVES = STREAM_THREADS / 64;
static constexpr int STREAM_MAX_PROBLEMS = 16;
static constexpr int STREAM_MAX_K = 16384;  // activations of one problem staged in LDS as fp32
static constexpr int STREAM_XS_FLOATS = STREAM_MAX_K + 4 * (STREAM_MAX_K / 64);

struct StreamProblem {
    const uint8_t* w;   // [n, k] packed rows
    const uint8_t* w2;  // second matrix of a gate/up pair, or null
    const void* x;      // one activation row
    void* y;            // n outputs
    int n, k;
    int fmt;
    int flat_end;       // rows of up to 4096 columns: end of the problem's range of global work items
    int xdt, ydt;
    int first_item;     // start of that range; for wider rows the workgroup that takes the first row
    int xgroup;         // equal for consecutive problems that read the same activation row
};

struct StreamArgs {
    int count;
    int flat_items;     // total work items of the problems with rows of up to 4096 columns
    // Activation rows of the problems with rows of up to 4096 columns, when there are at most
    // STREAM_WAVES different ones: group g is read by problem group_problem[g] (and others) and
    // is fetched into LDS stripe g before the first row is multiplied.
    int groups;
    int group_problem[STREAM_WAVES];
    StreamProblem p[STREAM_MAX_PROBLEMS];
};

// Lanes that share one row of k columns (a power of two, 8..64) and its log2.
__host__ __device__ inline int lanes_per_row(int k) {
    const int units = k >> 6;
    return units <= 8 ? 8 : units <= 16 ? 16 : units <= 32 ? 32 : 64;
}

// ---- device side of the streaming engine ---------------------------------------------------------
__device__ __forceinline__ int64_t row_bytes_dev(int fmt, int k) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: return (int64_t)(k >> 5) * 34;
    case QMOE_FMT_Q5_K: return (int64_t)(k >> 8) * 176;
    case QMOE_FMT_Q4_K: return (int64_t)(k >> 8) * 144;
    case QMOE_FMT_Q6_K: return (int64_t)(k >> 8) * 210;
    default: return (int64_t)k * 2;
    }
}

// One step's worth of raw weight registers for a row (and its partner row of a gate/up pair).
template <int FMT, bool PAIR> struct RowRegs {
    uint32_t a[Unit64<FMT>::RAW];
    uint32_t b[PAIR ? Unit64<FMT>::RAW : 1];
};

// Rows of `LR` lanes each (64/LR rows per wave and step); WR waves share one row (the
// workgroup's four waves then work on 4/WR rows at a time); PD rows are requested ahead of
// the one being reduced.
template <int FMT, bool PAIR, int LR, int WR, int PD>
__device__ __forceinline__ void stream_problem(const StreamProblem& p, float* partial, float* xs, int& staged,
                                               float (&xr)[64], float (&aux)[8], int& xgroup) {
    using U = Unit64<FMT>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int units = p.k >> 6;
    const int64_t rb = row_bytes_dev(FMT, p.k);
    constexpr int RPW = WR > 1 ? STREAM_WAVES / WR : 64 / LR;  // rows per step of a wave (of the workgroup if WR > 1)
    const int sub = WR > 1 ? wave / WR : lane / LR;            // which of those rows this lane works on
    const int part = WR > 1 ? wave % WR : 0;                   // which 4096-column part of the row
    const int u = part * 64 + (lane % LR);
    const bool active = u < units;
    const int uu = active ? u : 0;
    // work items: groups of RPW rows; taken by waves (WR == 1) or by workgroups (WR > 1)
    const int items = (p.n + RPW - 1) / RPW;
    const int workers = WR > 1 ? gridDim.x : gridDim.x * STREAM_WAVES;
    const int me = WR > 1 ? blockIdx.x : blockIdx.x * STREAM_WAVES + wave;
    int item = (me - p.first_item + workers) % workers;
    const bool busy = item < items;

    RowRegs<FMT, PAIR> buf[PD + 1];
    auto fetch = [&](RowRegs<FMT, PAIR>& r, int it) {
        const int row = it * RPW + sub;
        const int64_t rr = row < p.n ? row : p.n - 1;
        U::load_w(p.w + rr * rb, uu, r.a);
        if (PAIR) U::load_w(p.w2 + rr * rb, uu, r.b);
    };
#pragma unroll
    for (int j = 0; j < PD; ++j)
        if (item + j * workers < items) fetch(buf[j], item + j * workers);
    // New activations are staged once per workgroup in LDS (as fp32) while this wave's first
    // rows are already in flight; every wave of the workgroup passes here for every problem.
    if (staged != p.xgroup) {
        // all loads first, then all LDS stores: the loads travel together (a store between two
        // loads would order them, LDS and global pointers are not told apart here), and they
        // travel while the workgroup's other waves are still finishing what reads the old contents
        float4 v[STREAM_MAX_K / (4 * STREAM_THREADS)];
#pragma unroll
        for (int j = 0; j < STREAM_MAX_K / (4 * STREAM_THREADS); ++j) {
            const int i = 4 * threadIdx.x + 4 * STREAM_THREADS * j;
            if (i < p.k) v[j] = load_x4(p.x, p.xdt, i);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < STREAM_MAX_K / (4 * STREAM_THREADS); ++j) {
            const int i = 4 * threadIdx.x + 4 * STREAM_THREADS * j;
            if (i < p.k) *(float4*)(xs + StagedX::at(i)) = v[j];
        }
        __syncthreads();
        staged = p.xgroup;
    }
    if (!busy) return;
    // The activation slice of the lane's unit position stays in registers across problems
    // that read the same activations (xgroup names what is loaded).
    if (xgroup != p.xgroup) {
        U::load_x(StagedX{xs}, uu, xr, aux);
        if (!active) {
#pragma unroll
            for (int i = 0; i < 64; ++i) xr[i] = 0.f;
#pragma unroll
            for (int i = 0; i < U::AUX; ++i) aux[i] = 0.f;
        }
        xgroup = p.xgroup;
    }
    int slot = 0;
    bool done = false;
    while (!done) {
#pragma unroll
        for (int s = 0; s <= PD; ++s) {
            if (done) break;
            const int ahead = item + PD * workers;
            if (ahead < items) fetch(buf[(s + PD) % (PD + 1)], ahead);
            const bool more = item + workers < items;
            const int row = item * RPW + sub;
            const float g = group_sum<LR>(U::dot(buf[s].a, xr, aux));
            float v = g;
            if (PAIR) {
                const float up = group_sum<LR>(U::dot(buf[s].b, xr, aux));
                if (WR == 1) v = silu_mul(g, up);
                else if (lane == 63) {
                    partial[((slot * RPW + sub) * 2) * WR + part] = g;
                    partial[((slot * RPW + sub) * 2 + 1) * WR + part] = up;
                }
            } else if (WR > 1) {
                if (lane == 63) partial[(slot * RPW + sub) * WR + part] = g;
            }
            if (WR == 1) {
                if ((lane % LR) == LR - 1 && row < p.n) store_out(p.y, p.ydt, row, v);
            } else {
                // rows of a workgroup-shared problem: the waves' partial sums meet in LDS
                ++slot;
                if (slot == 32 || !more) {
                    __syncthreads();
                    const int t = threadIdx.x;  // entry t = step t / RPW of this flush, row t % RPW of the step
                    const int r2 = (item - (slot - 1 - t / RPW) * workers) * RPW + t % RPW;
                    if (t < slot * RPW && r2 < p.n) {
                        float sg = 0.f, su = 0.f;
#pragma unroll
                        for (int wv = 0; wv < WR; ++wv) {
                            if (PAIR) { sg += partial[(t * 2) * WR + wv]; su += partial[(t * 2 + 1) * WR + wv]; }
                            else sg += partial[t * WR + wv];
                        }
                        store_out(p.y, p.ydt, r2, PAIR ? silu_mul(sg, su) : sg);
                    }
                    __syncthreads();
                    slot = 0;
                }
            }
            if (!more) done = true;
            item += workers;
        }
    }
}

// Sum over groups of `lr` consecutive lanes, lr known only at run time (uniform).
__device__ __forceinline__ float group_sum_rt(float v, int lr) {
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x141>(v);
    if (lr >= 16) v = dpp_add<0x140>(v);
    if (lr >= 32) v = dpp_add<0x142, 0xa>(v);
    if (lr >= 64) v = dpp_add<0x143, 0xc>(v);
    return v;
}

// Wave-uniform values moved to scalar registers.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const uint8_t* uniform(const uint8_t* p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = (uint32_t)uniform((int)(uint32_t)v), hi = (uint32_t)uniform((int)(uint32_t)(v >> 32));
    return (const uint8_t*)(((uint64_t)hi << 32) | lo);
}

// All problems whose rows fit one wave (k <= 4096), as ONE stream of work items: item g of the
// concatenated ranges [first_item, flat_end).  Wave w takes items w, w + W, ... (all waves
// sweep one window of consecutive rows: best for few, long matrices) or, with `contiguous`,
// one contiguous share (it changes activations as rarely as possible: best for lists of many
// small matrices over several activation rows).  A wave requests
// the rows of its next PD items before it reduces the current one, across problem boundaries,
// so the start of a new matrix does not drain the memory pipeline.
// Activations are fetched coalesced into the wave's private LDS stripe `xw` and read back as
// the lane's 64-value slice; with `xpre` the caller has already put the activations of
// xgroup g into stripe g of that array (same padded layout, stripes `xstride` floats apart) and
// nothing is fetched here.  Items [begin, end) are walked; `probs` covers them in order.
// `between` runs once on every wave, after the wave's first PD row requests have left and before
// anything is read from the stripes: a caller whose activations are still on their way stores
// them (and meets the workgroup's other waves) there, while the rows travel.
struct NothingBetween { __device__ __forceinline__ void operator()() const {} };
template <int FMT, bool PAIR, int PD, class Between = NothingBetween>
__device__ __forceinline__ void stream_flat(const StreamProblem* probs, int count, int begin, int end, bool contiguous, float* xw,
                                            const float* xpre, int xstride = STREAM_XS_FLOATS / STREAM_WAVES,
                                            Between&& between = Between()) {
    using U = Unit64<FMT>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int W = gridDim.x * STREAM_WAVES;
    const int me = blockIdx.x * STREAM_WAVES + wave;
    int g = begin + me, step = W;
    if (contiguous) {
        const int share = (end - begin) / W, extra = (end - begin) % W;
        g = begin + me * share + (me < extra ? me : extra);
        end = g + share + (me < extra ? 1 : 0);
        step = 1;
    }
    if (g >= end) {
        between();
        return;
    }
    RowRegs<FMT, PAIR> buf[PD + 1];
    int bp[PD + 1], bi[PD + 1];
    // the problem the fetch side is in, held in scalar registers
    int cursor = -1, c_begin = 0, c_end = begin, c_n = 1, c_k = 64;
    const uint8_t *c_w = nullptr, *c_w2 = nullptr;
    auto fetch = [&](int gi, bool past, RowRegs<FMT, PAIR>& r, int& rp, int& ri) {
        if (gi >= c_end || cursor < 0) {
            // 64 range ends at a time: one LDS read and a ballot per hop
            ++cursor;
            while (true) {
                const int c = cursor + lane < count ? cursor + lane : count - 1;
                const uint64_t past = __ballot(gi >= probs[c].flat_end && cursor + lane < count - 1);
                const int hop = ~past ? __builtin_ctzll(~past) : 64;
                cursor += hop;
                if (hop < 64) break;
            }
            const StreamProblem& p = probs[cursor];
            c_begin = uniform(p.first_item);
            c_end = uniform(p.flat_end);
            c_n = uniform(p.n);
            c_k = uniform(p.k);
            c_w = uniform(p.w);
            if (PAIR) c_w2 = uniform(p.w2);
        }
        rp = cursor;
        ri = gi - c_begin;
        const int lr = lanes_per_row(c_k), units = c_k >> 6;
        const int u = lane & (lr - 1);
        const int uu = u < units && !past ? u : 0;
        const int row = ri * (64 / lr) + lane / lr;
        const int64_t rr = past ? 0 : row < c_n ? row : (c_n > 0 ? c_n - 1 : 0);
        const int64_t rb = row_bytes_dev(FMT, c_k);
        U::load_w(c_w + rr * rb, uu, r.a);
        if (PAIR) U::load_w(c_w2 + rr * rb, uu, r.b);
    };
    // Every fetch is issued on every path (past the end all lanes request the first bytes of
    // the current matrix: one cache line): the number of loads in flight behind the rows about
    // to be reduced is then the same whichever way the branches go, and the wait before the
    // reduction can leave them in flight.
    const int last = end - 1 - (end - 1 - g) % step;
    auto bounded = [&](int gi) { return gi < end ? gi : last; };
#pragma unroll
    for (int j = 0; j < PD; ++j) fetch(bounded(g + j * step), g + j * step >= end, buf[j], bp[j], bi[j]);
    between();
    float xr[64], aux[8];
    int xgroup = -1;
    bool done = false;
    while (!done) {
#pragma unroll
        for (int s = 0; s <= PD; ++s) {
            if (!done) {
                const int nb = (s + PD) % (PD + 1);
                fetch(bounded(g + PD * step), g + PD * step >= end, buf[nb], bp[nb], bi[nb]);
                const StreamProblem& p = probs[bp[s]];
                const int pk = uniform(p.k), pn = uniform(p.n), pg = uniform(p.xgroup);
                const int lr = lanes_per_row(pk), units = pk >> 6;
                const int u = lane & (lr - 1);
                const bool active = u < units;
                if (xgroup != pg) {
                    const float* xl = xw;
                    if (xpre) {
                        xl = xpre + pg * xstride;
                    } else {
                        const uint8_t* px = uniform((const uint8_t*)p.x);
                        const int pxdt = uniform(p.xdt);
                        float4 v[16];  // all loads first, then all LDS stores
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const int idx = 4 * lane + 256 * i;
                            if (idx < pk) v[i] = load_x4(px, pxdt, idx);
                        }
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const int idx = 4 * lane + 256 * i;
                            if (idx < pk) *(float4*)(xw + StagedX::at(idx)) = v[i];
                        }
                    }
                    U::load_x(StagedX{xl}, active ? u : 0, xr, aux);
                    if (!active) {
#pragma unroll
                        for (int i = 0; i < 64; ++i) xr[i] = 0.f;
#pragma unroll
                        for (int i = 0; i < U::AUX; ++i) aux[i] = 0.f;
                    }
                    xgroup = pg;
                }
                const int row = bi[s] * (64 / lr) + lane / lr;
                float v = group_sum_rt(U::dot(buf[s].a, xr, aux), lr);
                if (PAIR) v = silu_mul(v, group_sum_rt(U::dot(buf[s].b, xr, aux), lr));
                if (u == lr - 1 && row < pn) store_out(p.y, uniform(p.ydt), row, v);
                g += step;
                if (g >= end) done = true;
            }
        }
    }
}

// One matrix (or gate/up pair) of rows of up to 4096 columns multiplied with SEVERAL activation
// rows that lie in LDS stripes (padded layout, `stripe` floats apart): every row is streamed
// once and reduced against each staged activation row in turn; results go to fp32
// y[g * ystride + row].  The caller is worker `me` of `W`; item i belongs to worker i mod W.
template <int FMT, bool PAIR, int PD>
__device__ __forceinline__ void stream_rows_many_x(const uint8_t* w, const uint8_t* w2, int n, int k, const float* xs,
                                                   int stripe, int groups, float* y, int64_t ystride, int me, int W) {
    using U = Unit64<FMT>;
    const int lane = threadIdx.x & 63;
    const int lr = lanes_per_row(k), units = k >> 6;
    const int u = lane & (lr - 1);
    const bool active = u < units;
    const int uu = active ? u : 0;
    const int rpw = 64 / lr;
    const int items = (n + rpw - 1) / rpw;
    const int64_t rb = row_bytes_dev(FMT, k);
    int item = me;
    if (item >= items) return;
    RowRegs<FMT, PAIR> buf[PD + 1];
    auto fetch = [&](int it, RowRegs<FMT, PAIR>& r) {
        const int row = it * rpw + lane / lr;
        const int64_t rr = row < n ? row : n - 1;
        U::load_w(w + rr * rb, uu, r.a);
        if (PAIR) U::load_w(w2 + rr * rb, uu, r.b);
    };
#pragma unroll
    for (int j = 0; j < PD; ++j)
        if (item + j * W < items) fetch(item + j * W, buf[j]);
    bool done = false;
    while (!done) {
#pragma unroll
        for (int s = 0; s <= PD; ++s) {
            if (!done) {
                if (item + PD * W < items) fetch(item + PD * W, buf[(s + PD) % (PD + 1)]);
                const int row = item * rpw + lane / lr;
                for (int g = 0; g < groups; ++g) {
                    float xr[64], aux[8];
                    U::load_x(StagedX{xs + g * stripe}, uu, xr, aux);
                    float a = U::dot(buf[s].a, xr, aux);
                    a = group_sum_rt(active ? a : 0.f, lr);
                    if (PAIR) {
                        float b = U::dot(buf[s].b, xr, aux);
                        a = silu_mul(a, group_sum_rt(active ? b : 0.f, lr));
                    }
                    if (u == lr - 1 && row < n) y[g * ystride + row] = a;
                }
                item += W;
                if (item >= items) done = true;
            }
        }
    }
}

// Rows requested ahead (measured: with eight waves per CU one row ahead keeps the memory system
// busy, and more only lengthens the queues in the vector cache; BF16 units, a cache line per
// lane, and gate/up pairs, two rows per step, do best with none).
template <int FMT, bool PAIR> struct Prefetch {
    static constexpr int DEPTH = (FMT == QMOE_FMT_BF16 || PAIR) ? 0 : FMT == QMOE_FMT_Q8_0 ? 1 : 2;
};

// A whole problem list held in LDS: first the single stream of all problems whose rows fit a
// wave, then, one after the other, the problems with wider rows (four waves per row).
template <int FMT, bool PAIR, bool WIDE = true, class Between = NothingBetween>
__device__ __forceinline__ void stream_run(const StreamProblem* probs, int count, int flat_begin, int flat_end, bool contiguous, float* partial, float* xs,
                                           const float* xpre = nullptr, int xstride = STREAM_XS_FLOATS / STREAM_WAVES,
                                           Between&& between = Between()) {
    constexpr int PD = Prefetch<FMT, PAIR>::DEPTH;
    const int wave = threadIdx.x >> 6;
    if (flat_end > flat_begin)
        stream_flat<FMT, PAIR, PD>(probs, count, flat_begin, flat_end, contiguous, xs + wave * (STREAM_XS_FLOATS / STREAM_WAVES), xpre, xstride, between);
    else
        between();
    if (!WIDE) return;
    float xr[64], aux[8];
    int xgroup = -1, staged = -1;
    for (int i = 0; i < count; ++i) {
        const StreamProblem& p = probs[i];
        if (p.n < 1 || (p.k >> 6) <= 64) continue;
        if ((p.k >> 6) <= 128) stream_problem<FMT, PAIR, 64, 2, PD>(p, partial, xs, staged, xr, aux, xgroup);
        else stream_problem<FMT, PAIR, 64, 4, PD>(p, partial, xs, staged, xr, aux, xgroup);
    }
}

// True if (fmt, shape, alignment) can go through the streaming kernel.
bool stream_supported(int fmt, const void* w, int n, int k, const void* x, int xdt);
// Enqueue args.count (<= STREAM_MAX_PROBLEMS) supported problems as one launch.
int stream_launch(StreamArgs& args, hipStream_t s);

int stream_grid();

// ---- decode-time MoE step (qmoe_decode.hip) -----------------------------------------------------
struct DecodeBuffers {  // workspace regions, all device pointers
    float* weights;
    int64_t* ids;
    int* sorted_ids;
    float* sorted_w;
    float* sig;
    int* status;
    void* problems;
    int* problem_count;
    float* h;
    float* hs;
};
bool decode_supported(const qmoe_moe_args& a, const void* h_ws);
int decode_launch(const qmoe_moe_args& a, const DecodeBuffers& w, hipStream_t s);

}  // namespace qmoe
