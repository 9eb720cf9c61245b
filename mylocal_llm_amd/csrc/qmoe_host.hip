// Host twins of the packed operators: the same arithmetic contract as the device entry points,
// computed on the CPU from host pointers by one thread of plain scalar C++.  They give callers
// that hold NumPy activations and host-packed weights a compute path (the host branch of
// quantized_linear, mini_llm/ops/quantized_linear.py:292-305, and its native backend
// mylocal_packed_gemv / mylocal_packed_expert, native_packed_cpu.cpp:206-246) and a CPU figure
// to quote beside the device kernels.  Nothing here touches the GPU; no kernel is defined.
//
// A block is decoded to fp32 exactly as the device decoders do (d*q, (d*sc)*q - dmin*mn,
// (d*sc)*q), then multiplied into eight interleaved fp32 partial sums per row, which are added
// pairwise at the end.
#include <math.h>
#include <string.h>

#include <vector>

#include "qmoe_common.hpp"
#include "qmoe_formats.hpp"

// The decoders round a product before they subtract from it, as the reference does: a fused
// multiply-add would change the last bit of a weight.
#pragma clang fp contract(off)

namespace {

using qmoe::block_bytes;
using qmoe::block_elems;
using qmoe::fail;
using qmoe::format_implemented;

inline uint16_t u16_at(const uint8_t* p) { uint16_t v; memcpy(&v, p, 2); return v; }
inline float bits_to_float(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }

// IEEE binary16 -> binary32, subnormals, infinities and NaN payloads kept.
inline float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exponent = (h >> 10) & 31u, fraction = h & 1023u;
    if (exponent == 31u) return bits_to_float(sign | 0x7F800000u | (fraction << 13));
    if (exponent) return bits_to_float(sign | ((exponent + 112u) << 23) | (fraction << 13));
    const float magnitude = (float)fraction * 5.9604644775390625e-8f;   // fraction * 2^-24, exact
    return sign ? -magnitude : magnitude;
}

// Six-bit scale and minimum of group g of a Q4_K / Q5_K block (12 bytes at `s`).
inline void scale_min(const uint8_t* s, int g, int& sc, int& mn) {
    if (g < 4) { sc = s[g] & 63; mn = s[4 + g] & 63; return; }
    sc = (s[4 + g] & 15) | ((s[g - 4] >> 6) << 4);
    mn = (s[4 + g] >> 4) | ((s[g] >> 6) << 4);
}

void decode_q8_0(const uint8_t* b, float* w) {
    const float d = half_to_float(u16_at(b));
    for (int i = 0; i < 32; ++i) w[i] = d * (float)(int8_t)b[2 + i];
}
void decode_q4_0(const uint8_t* b, float* w) {
    const float d = half_to_float(u16_at(b));
    for (int i = 0; i < 16; ++i) {
        w[i] = d * ((float)(b[2 + i] & 15) - 8.0f);
        w[16 + i] = d * ((float)(b[2 + i] >> 4) - 8.0f);
    }
}
template <bool FIFTH_BIT> void decode_q45_k(const uint8_t* b, float* w) {
    const float d = half_to_float(u16_at(b)), dmin = half_to_float(u16_at(b + 2));
    const uint8_t* high = b + 16;
    const uint8_t* nibbles = b + (FIFTH_BIT ? 48 : 16);
    for (int g = 0; g < 8; ++g) {
        int sc, mn;
        scale_min(b + 4, g, sc, mn);
        const float scale = d * (float)sc, lowest = dmin * (float)mn;
        const uint8_t* q = nibbles + 32 * (g >> 1);
        for (int j = 0; j < 32; ++j) {
            int code = (q[j] >> (4 * (g & 1))) & 15;
            if (FIFTH_BIT) code |= ((high[j] >> g) & 1) << 4;
            w[32 * g + j] = scale * (float)code - lowest;
        }
    }
}
void decode_q3_k(const uint8_t* b, float* w) {
    const float d = half_to_float(u16_at(b + 108));
    const uint8_t* s = b + 96;
    for (int g = 0; g < 16; ++g) {
        const int six = ((s[g & 7] >> (4 * (g >> 3))) & 15) | (((s[8 + (g & 3)] >> (2 * (g >> 2))) & 3) << 4);
        const float scale = d * (float)(six - 32);
        for (int j = 0; j < 16; ++j) {
            const int i = 16 * g + j;
            const int low = (b[32 + 32 * (i >> 7) + (i & 31)] >> (2 * ((i & 127) >> 5))) & 3;
            const int keep = (b[i & 31] >> (i >> 5)) & 1;
            w[i] = scale * (float)(low - 4 * (1 - keep));
        }
    }
}
void decode_q6_k(const uint8_t* b, float* w) {
    const float d = half_to_float(u16_at(b + 208));
    for (int g = 0; g < 16; ++g) {
        const float scale = d * (float)(int8_t)b[192 + g];
        for (int j = 0; j < 16; ++j) {
            const int i = 16 * g + j, half = i >> 7, r = i & 127;
            const int low = (b[64 * half + (i & 63)] >> (4 * (r >> 6))) & 15;
            const int high = (b[128 + 32 * half + (i & 31)] >> (2 * (r >> 5))) & 3;
            w[i] = scale * (float)((low | (high << 4)) - 32);
        }
    }
}

void decode_block(int fmt, const uint8_t* block, float* w) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: decode_q8_0(block, w); break;
    case QMOE_FMT_Q4_0: decode_q4_0(block, w); break;
    case QMOE_FMT_Q4_K: decode_q45_k<false>(block, w); break;
    case QMOE_FMT_Q5_K: decode_q45_k<true>(block, w); break;
    case QMOE_FMT_Q3_K: decode_q3_k(block, w); break;
    default: decode_q6_k(block, w); break;
    }
}

// One packed row times one activation row.
float row_dot(const uint8_t* row, int fmt, int k, const float* x) {
    float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (fmt == QMOE_FMT_BF16) {
        for (int i = 0; i < k; ++i) part[i & 7] += bits_to_float((uint32_t)u16_at(row + 2 * i) << 16) * x[i];
    } else {
        const int elems = block_elems(fmt), bytes = block_bytes(fmt);
        float w[256];
        for (int at = 0; at < k; at += elems, row += bytes) {
            decode_block(fmt, row, w);
            for (int i = 0; i < elems; ++i) part[i & 7] += w[i] * x[at + i];
        }
    }
    return ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
}

bool matrix_ok(int fmt, int n, int k) {
    return format_implemented(fmt) && n > 0 && k > 0 && k % block_elems(fmt) == 0;
}

inline float silu_times(float g, float u) {
    // the sigmoid in the form that cannot overflow (native_packed_cpu.cpp:236-238)
    const float s = g >= 0.0f ? 1.0f / (1.0f + expf(-g)) : expf(g) / (1.0f + expf(g));
    return (g * s) * u;
}

// Position of a logit in "descending value, NaN last": larger key first; -0 and +0 tie.
inline uint32_t selection_key(float v) {
    if (v != v) return 0u;
    uint32_t bits;
    const float z = v == 0.0f ? 0.0f : v;
    memcpy(&bits, &z, 4);
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

}  // namespace

extern "C" int qmoe_dequantize_cpu(const void* w, int fmt, int64_t n, int64_t k, float* out) {
    if (!w || !out) return fail(QMOE_EINVAL, "qmoe_dequantize_cpu: null pointer");
    if (!format_implemented(fmt)) return fail(QMOE_EUNSUPPORTED, "qmoe_dequantize_cpu: format %d", fmt);
    if (n < 1 || k < 1 || k % block_elems(fmt)) return fail(QMOE_EINVAL, "qmoe_dequantize_cpu: n=%lld k=%lld", (long long)n, (long long)k);
    const int elems = block_elems(fmt), bytes = block_bytes(fmt);
    const uint8_t* block = (const uint8_t*)w;
    const int64_t blocks = n * (k / elems);
    if (fmt == QMOE_FMT_BF16) {
        for (int64_t i = 0; i < blocks; ++i) out[i] = bits_to_float((uint32_t)u16_at(block + 2 * i) << 16);
        return QMOE_OK;
    }
    for (int64_t i = 0; i < blocks; ++i, block += bytes, out += elems) decode_block(fmt, block, out);
    return QMOE_OK;
}

extern "C" int qmoe_linear_cpu(const void* w, int fmt, int n, int k, const float* x, int tokens, float* y) {
    if (!w || !x || !y) return fail(QMOE_EINVAL, "qmoe_linear_cpu: null pointer");
    if (!format_implemented(fmt)) return fail(QMOE_EUNSUPPORTED, "qmoe_linear_cpu: format %d", fmt);
    if (!matrix_ok(fmt, n, k) || tokens < 1)
        return fail(QMOE_EINVAL, "qmoe_linear_cpu: n=%d k=%d tokens=%d for a format of %d-element blocks", n, k, tokens, block_elems(fmt));
    const size_t stride = (size_t)qmoe::row_bytes(fmt, k);
    for (int t = 0; t < tokens; ++t)
        for (int r = 0; r < n; ++r)
            y[(size_t)t * n + r] = row_dot((const uint8_t*)w + stride * r, fmt, k, x + (size_t)t * k);
    return QMOE_OK;
}

extern "C" int qmoe_swiglu_cpu(const void* gate, int gate_fmt, const void* up, int up_fmt, int f, int k,
                               const float* x, int tokens, float* h) {
    if (!gate || !up || !x || !h) return fail(QMOE_EINVAL, "qmoe_swiglu_cpu: null pointer");
    if (!format_implemented(gate_fmt) || !format_implemented(up_fmt))
        return fail(QMOE_EUNSUPPORTED, "qmoe_swiglu_cpu: formats %d, %d", gate_fmt, up_fmt);
    if (!matrix_ok(gate_fmt, f, k) || !matrix_ok(up_fmt, f, k) || tokens < 1)
        return fail(QMOE_EINVAL, "qmoe_swiglu_cpu: f=%d k=%d tokens=%d", f, k, tokens);
    const size_t gs = (size_t)qmoe::row_bytes(gate_fmt, k), us = (size_t)qmoe::row_bytes(up_fmt, k);
    for (int t = 0; t < tokens; ++t) {
        const float* xt = x + (size_t)t * k;
        for (int r = 0; r < f; ++r)
            h[(size_t)t * f + r] = silu_times(row_dot((const uint8_t*)gate + gs * r, gate_fmt, k, xt),
                                              row_dot((const uint8_t*)up + us * r, up_fmt, k, xt));
    }
    return QMOE_OK;
}

extern "C" int qmoe_expert_cpu(const void* gate, int gate_fmt, const void* up, int up_fmt, const void* down,
                               int down_fmt, int d_model, int d_ff, const float* x, int tokens, float* out) {
    if (!gate || !up || !down || !x || !out) return fail(QMOE_EINVAL, "qmoe_expert_cpu: null pointer");
    if (!format_implemented(gate_fmt) || !format_implemented(up_fmt) || !format_implemented(down_fmt))
        return fail(QMOE_EUNSUPPORTED, "qmoe_expert_cpu: formats %d, %d, %d", gate_fmt, up_fmt, down_fmt);
    if (!matrix_ok(gate_fmt, d_ff, d_model) || !matrix_ok(up_fmt, d_ff, d_model) || !matrix_ok(down_fmt, d_model, d_ff) || tokens < 1)
        return fail(QMOE_EINVAL, "qmoe_expert_cpu: d_model=%d d_ff=%d tokens=%d", d_model, d_ff, tokens);
    std::vector<float> hidden((size_t)d_ff);
    const size_t ds = (size_t)qmoe::row_bytes(down_fmt, d_ff);
    for (int t = 0; t < tokens; ++t) {
        const int rc = qmoe_swiglu_cpu(gate, gate_fmt, up, up_fmt, d_ff, d_model, x + (size_t)t * d_model, 1, hidden.data());
        if (rc != QMOE_OK) return rc;
        for (int r = 0; r < d_model; ++r)
            out[(size_t)t * d_model + r] = row_dot((const uint8_t*)down + ds * r, down_fmt, d_ff, hidden.data());
    }
    return QMOE_OK;
}

extern "C" int qmoe_router_topk_cpu(const float* logits, int tokens, int n, int k, float floor_value,
                                    int renormalize, float* weights, int64_t* ids) {
    if (!logits || !weights || !ids) return fail(QMOE_EINVAL, "qmoe_router_topk_cpu: null pointer");
    if (tokens < 1 || n < 1 || k < 1 || k > n) return fail(QMOE_EINVAL, "qmoe_router_topk_cpu: tokens=%d n=%d k=%d", tokens, n, k);
    if (renormalize && !(floor_value > 0.0f)) return fail(QMOE_EINVAL, "qmoe_router_topk_cpu: floor must be positive");
    std::vector<uint32_t> key((size_t)n);
    for (int t = 0; t < tokens; ++t) {
        const float* z = logits + (size_t)t * n;
        // maximum with NaN propagation, then the full softmax denominator in double
        float top = z[0];
        bool has_nan = false;
        for (int i = 0; i < n; ++i) {
            has_nan |= z[i] != z[i];
            if (z[i] > top) top = z[i];
            key[i] = selection_key(z[i]);
            if (!key[i]) key[i] = 1u;            // NaN: below -inf, above "taken"
        }
        if (has_nan) top = NAN;
        double total = 0.0;
        for (int i = 0; i < n; ++i) total += (double)expf(z[i] - top);
        const float denominator = (float)total;
        float mass = 0.0f;
        for (int slot = 0; slot < k; ++slot) {
            int best = 0;
            for (int i = 1; i < n; ++i)
                if (key[i] > key[best]) best = i;
            key[best] = 0u;
            const float p = expf(z[best] - top) / denominator;
            weights[(size_t)t * k + slot] = p;
            ids[(size_t)t * k + slot] = best;
            mass += p;
        }
        if (renormalize) {
            const float norm = mass != mass ? mass : fmaxf(mass, floor_value);
            for (int slot = 0; slot < k; ++slot) weights[(size_t)t * k + slot] /= norm;
        }
    }
    return QMOE_OK;
}
