/* CPU oracle in plain C -- TEST INFRASTRUCTURE ONLY.
 *
 * A scalar, element-at-a-time restatement of the reference's packed-weight
 * arithmetic, written independently of the NumPy restatement in
 * reference_np.py so that the two can be checked against each other (a wrong
 * index or a dropped term in one shows up as a mismatch with the other and with
 * the reference's hand-packed vectors).  Nothing in the product links or loads
 * this file; only tests, the smoke check and the cpu_baseline leg of the bench do.
 *
 * Reference lines restated:
 *   block sizes                      mini_llm/ops/quantized_weight.py:24-37
 *   Q8_0  w = d*q                    mini_llm/ops/quantized_weight.py:208-211
 *   Q4_0  w = d*(nibble-8)           mini_llm/ops/quantized_weight.py:212-216
 *   Q4_K/Q5_K w=(d*sc)*q - dmin*mn   mini_llm/ops/quantized_weight.py:217-237
 *   Q3_K  w = (d*(sc-32))*(q2-4*(1-h)) mini_llm/ops/quantized_weight.py:251-266
 *   Q6_K  w = (d*sc)*q               mini_llm/ops/quantized_weight.py:238-250
 *   BF16  bits<<16                   mini_llm/external/gguf_tensor.py:48-51
 *   host linear x @ W.T (fp32)       mini_llm/ops/quantized_linear.py:303-305
 *   SwiGLU g/(1+exp(-g))*u           mini_llm/ops/quantized_linear.py:367-370
 *   expert FFN                       mini_llm/ops/quantized_linear.py:414-424
 *   top-k order / renormalisation    mini_llm/ops/router_decode.py:19-26, :27-95
 *   C ABI shape, error convention    mini_llm/ops/native_packed_cpu.cpp:206-246
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { F_Q8_0 = 0, F_Q4_0 = 1, F_Q4_K = 2, F_Q3_K = 3, F_Q5_K = 4, F_Q6_K = 5, F_BF16 = 100 };

static int fmt_elems(int f) {
    switch (f) {
    case F_Q8_0: case F_Q4_0: return 32;
    case F_Q4_K: case F_Q5_K: case F_Q6_K: case F_Q3_K: return 256;
    case F_BF16: return 1;
    default: return 0;
    }
}
static int fmt_bytes(int f) {
    switch (f) {
    case F_Q8_0: return 34;
    case F_Q4_0: return 18;
    case F_Q4_K: return 144;
    case F_Q3_K: return 110;
    case F_Q5_K: return 176;
    case F_Q6_K: return 210;
    case F_BF16: return 2;
    default: return 0;
    }
}

/* IEEE binary16 -> binary32, subnormals / inf / NaN included. */
static float half_at(const uint8_t* p) {
    uint32_t h = (uint32_t)p[0] | ((uint32_t)p[1] << 8);
    uint32_t sign = (h >> 15) & 1, ex = (h >> 10) & 31, man = h & 1023;
    uint32_t bits;
    if (ex == 31) bits = 0x7F800000u | (man << 13);
    else if (ex) bits = ((ex + 112) << 23) | (man << 13);
    else if (man) {
        int shift = 0;
        while (!(man & 1024)) { man <<= 1; ++shift; }
        bits = ((uint32_t)(113 - shift) << 23) | ((man & 1023) << 13);
    } else bits = 0;
    bits |= sign << 31;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Element i of one block, decoded on its own from the block's field offsets. */
static float decode_element(int fmt, const uint8_t* b, int i) {
    if (fmt == F_Q8_0) return half_at(b) * (float)(int8_t)b[2 + i];
    if (fmt == F_Q4_0) {
        int nib = i < 16 ? (b[2 + i] & 15) : (b[2 + i - 16] >> 4);
        return half_at(b) * ((float)nib - 8.0f);
    }
    if (fmt == F_Q4_K || fmt == F_Q5_K) {
        int g = i / 32, j = i % 32, sc, mn;
        const uint8_t* s = b + 4;
        if (g < 4) { sc = s[g] & 63; mn = s[4 + g] & 63; }
        else {
            sc = (s[4 + g] & 15) | ((s[g - 4] >> 6) << 4);
            mn = (s[4 + g] >> 4) | ((s[g] >> 6) << 4);
        }
        int base = fmt == F_Q5_K ? 48 : 16;
        int q = (b[base + 32 * (g / 2) + j] >> (4 * (g & 1))) & 15;
        if (fmt == F_Q5_K) q |= ((b[16 + j] >> g) & 1) << 4;
        float scale = half_at(b) * (float)sc;
        float floor_ = half_at(b + 2) * (float)mn;
        return scale * (float)q - floor_;
    }
    if (fmt == F_Q3_K) { /* mini_llm/ops/native_packed_cpu.cpp:177-193, one element at a time */
        int g = i / 16;
        int sc = (int)(((b[96 + g % 8] >> (4 * (g / 8))) & 15) | (((b[104 + g % 4] >> (2 * (g / 4))) & 3) << 4)) - 32;
        int two = (b[32 + (i / 128) * 32 + i % 32] >> (2 * ((i % 128) / 32))) & 3;
        int keep = (b[i % 32] >> (i / 32)) & 1;
        float scale = half_at(b + 108) * (float)sc;
        return scale * (float)(two - 4 * (1 - keep));
    }
    if (fmt == F_Q6_K) {
        int h = i / 128, r = i % 128;
        int lo = (b[64 * h + (i % 64)] >> (4 * (r / 64))) & 15;
        int hi = (b[128 + 32 * h + (i % 32)] >> (2 * (r / 32))) & 3;
        int q = (lo | (hi << 4)) - 32;
        float scale = half_at(b + 208) * (float)(int8_t)b[192 + i / 16];
        return scale * (float)q;
    }
    if (fmt == F_BF16) {
        uint32_t bits = ((uint32_t)b[0] | ((uint32_t)b[1] << 8)) << 16;
        float f;
        memcpy(&f, &bits, 4);
        return f;
    }
    return 0.0f;
}

static int shape_ok(int fmt, long n, long k) {
    int e = fmt_elems(fmt);
    return e > 0 && n > 0 && k > 0 && k % e == 0;
}

int oracle_format_info(int fmt, int* elems, int* bytes) {
    if (!fmt_elems(fmt)) return 1;
    if (elems) *elems = fmt_elems(fmt);
    if (bytes) *bytes = fmt_bytes(fmt);
    return 0;
}

/* out[n*k] fp32 from packed rows.  Nonzero on invalid arguments. */
int oracle_dequantize(const uint8_t* w, int fmt, long n, long k, float* out) {
    if (!w || !out || !shape_ok(fmt, n, k)) return 1;
    int e = fmt_elems(fmt), bb = fmt_bytes(fmt);
    long nblocks = n * k / e;
    for (long blk = 0; blk < nblocks; ++blk)
        for (int i = 0; i < e; ++i)
            out[blk * e + i] = decode_element(fmt, w + blk * bb, i);
    return 0;
}

/* y[t*n+j] = sum_k x[t*k+..] * W[j,..]; products in fp32 as the reference's
 * dense operand would hold them, accumulated in double and rounded once, so the
 * result is the correctly rounded value of the fp32-weight dot product. */
int oracle_linear(const uint8_t* w, int fmt, int n, int k, const float* x, int tokens, float* y) {
    if (!w || !x || !y || !shape_ok(fmt, n, k) || tokens < 1) return 1;
    int e = fmt_elems(fmt), bb = fmt_bytes(fmt);
    long row_bytes = (long)k / e * bb;
    float* row = (float*)malloc(sizeof(float) * (size_t)k);
    if (!row) return 2;
    for (int j = 0; j < n; ++j) {
        const uint8_t* wr = w + (long)j * row_bytes;
        for (int c = 0; c < k; ++c) row[c] = decode_element(fmt, wr + (long)(c / e) * bb, c % e);
        for (int t = 0; t < tokens; ++t) {
            double acc = 0.0;
            const float* xt = x + (long)t * k;
            for (int c = 0; c < k; ++c) acc += (double)row[c] * (double)xt[c];
            y[(long)t * n + j] = (float)acc;
        }
    }
    free(row);
    return 0;
}

static float silu_mul(float g, float u) { return (g / (1.0f + expf(-g))) * u; }

/* h[t*f+j] = silu(x.G[j]) * (x.U[j]) with an fp32 storage boundary at g, u and h. */
int oracle_swiglu(const uint8_t* gate, int gf, const uint8_t* up, int uf, int f, int k,
                  const float* x, int tokens, float* h) {
    if (!h || tokens < 1) return 1;
    float* g = (float*)malloc(sizeof(float) * (size_t)tokens * f);
    float* u = (float*)malloc(sizeof(float) * (size_t)tokens * f);
    int rc = (!g || !u) ? 2 : 0;
    if (!rc) rc = oracle_linear(gate, gf, f, k, x, tokens, g);
    if (!rc) rc = oracle_linear(up, uf, f, k, x, tokens, u);
    if (!rc) for (long i = 0; i < (long)tokens * f; ++i) h[i] = silu_mul(g[i], u[i]);
    free(g); free(u);
    return rc;
}

/* out[t*d_model+..] = down(swiglu(x)); same argument order as the reference's
 * mylocal_packed_expert. */
int oracle_expert(const uint8_t* gate, int gf, const uint8_t* up, int uf, const uint8_t* down, int df,
                  int d_model, int d_ff, const float* x, int tokens, float* out) {
    if (!out || tokens < 1 || d_ff < 1) return 1;
    float* h = (float*)malloc(sizeof(float) * (size_t)tokens * d_ff);
    if (!h) return 2;
    int rc = oracle_swiglu(gate, gf, up, uf, d_ff, d_model, x, tokens, h);
    if (!rc) rc = oracle_linear(down, df, d_model, d_ff, h, tokens, out);
    free(h);
    return rc;
}

/* "a is selected before b": descending value, NaN last, lower id on ties. */
static int before(float a, int ia, float b, int ib) {
    int an = isnan(a), bn = isnan(b);
    if (an || bn) return an == bn ? ia < ib : bn;
    return a > b || (a == b && ia < ib);
}

/* Rows of softmax -> top-k -> optional renormalisation by max(mass, floor). */
int oracle_router_topk(const float* logits, int tokens, int n, int k, float floor_, int renorm,
                       float* weights, int64_t* ids) {
    if (!logits || !weights || !ids || tokens < 0 || n < 1 || k < 1 || k > n) return 1;
    uint8_t* used = (uint8_t*)malloc((size_t)n);
    if (!used) return 2;
    for (int t = 0; t < tokens; ++t) {
        const float* z = logits + (long)t * n;
        float m = -INFINITY;
        for (int i = 0; i < n; ++i) m = (isnan(z[i]) || isnan(m)) ? NAN : fmaxf(m, z[i]);
        double denom = 0.0;
        for (int i = 0; i < n; ++i) denom += (double)expf(z[i] - m);
        float den = (float)denom;
        memset(used, 0, (size_t)n);
        float mass = 0.0f;
        for (int s = 0; s < k; ++s) {
            int best = -1;
            for (int i = 0; i < n; ++i)
                if (!used[i] && (best < 0 || before(z[i], i, z[best], best))) best = i;
            used[best] = 1;
            ids[(long)t * k + s] = best;
            float p = expf(z[best] - m) / den;
            weights[(long)t * k + s] = p;
            mass += p;
        }
        if (renorm) {
            float norm = isnan(mass) ? mass : fmaxf(mass, floor_);
            for (int s = 0; s < k; ++s) weights[(long)t * k + s] /= norm;
        }
    }
    free(used);
    return 0;
}
