// Dequantise, dequant-fused linear, fused gate/up SwiGLU and single packed expert.
//
// General kernels: one wave (64 lanes) per output row, lanes stride over the row's
// lane units, fp32 accumulate, xor-shuffle reduction, result rounded once to the
// output type.  Any format, any K that is a block multiple, any token count (token
// chunks of MT re-read the row, which then comes from L2).
#include <stdarg.h>
#include <string.h>

#include "qmoe_few.hpp"
#include "qmoe_gemm.hpp"
#include "qmoe_rowdot.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

// ---- error plumbing ----------------------------------------------------------------------
static thread_local char g_error[512];
char* error_buffer() { return g_error; }
int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return status;
}
int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(QMOE_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return QMOE_OK;
}

// ---- dequantise ----------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ w, int64_t n, int64_t k,
                                                      int64_t row_bytes, bool fast, float* __restrict__ out) {
    using F = Fmt<FMT>;
    const int64_t units_row = fast ? F::units_per_row((int)k) : 0;
    const int64_t tail = k - units_row * F::UNIT;
    const int64_t per_row = units_row + tail;  // work items per row
    const int64_t total = n * per_row;
    for (int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; item < total;
         item += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = item / per_row, c = item % per_row;
        const uint8_t* row = w + r * row_bytes;
        float* orow = out + r * k;
        if (c < units_row) {
            float v[F::UNIT];
            F::decode(row, (int)c, v);
#pragma unroll
            for (int g = 0; g < F::GROUPS; ++g)
                *(float4*)(orow + F::xoff((int)c, g)) = make_float4(v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3]);
        } else {
            const int64_t i = units_row * F::UNIT + (c - units_row);
            orow[i] = F::element(row + (i / F::BLOCK_ELEMS) * F::BLOCK_BYTES, (int)(i % F::BLOCK_ELEMS));
        }
    }
}

template <int FMT>
static int launch_dequant(const void* w, int64_t n, int64_t k, float* out, hipStream_t s) {
    const int64_t rb = row_bytes(FMT, k);
    const bool fast = rows_fast(FMT, w, rb, k) && ((uintptr_t)out % 16 == 0);
    const int64_t units_row = fast ? k / Fmt<FMT>::UNIT : 0;
    const int64_t per_row = units_row + (k - units_row * Fmt<FMT>::UNIT);
    int64_t blocks = (n * per_row + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(dequant_kernel<FMT>, dim3((unsigned)blocks), dim3(256), 0, s, (const uint8_t*)w, n, k, rb, fast, out);
    return check_launch("qmoe_dequantize");
}

// ---- linear ---------------------------------------------------------------------------------
template <int XDT, int MT>
__global__ __launch_bounds__(256) void linear_kernel(const uint8_t* __restrict__ w, int fmt, int n, int k,
                                                     int64_t row_bytes, bool fast, const void* __restrict__ x,
                                                     int tokens, void* __restrict__ y, int ydt) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const uint8_t* wr = w + (int64_t)row * row_bytes;
    for (int t0 = 0; t0 < tokens; t0 += MT) {
        size_t xbase[MT];
        float acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            int t = t0 + m < tokens ? t0 + m : tokens - 1;
            xbase[m] = (size_t)t * k;
            acc[m] = 0.0f;
        }
        row_dot<XDT, MT>(fmt, wr, k, fast, x, xbase, lane, acc);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float v = wave_sum(acc[m]);
            if (lane == m && t0 + m < tokens) store_out(y, ydt, (size_t)(t0 + m) * n + row, v);
        }
    }
}

template <int XDT>
static void launch_linear_mt(const void* w, int fmt, int n, int k, bool fast, const void* x, int tokens, void* y,
                             int ydt, hipStream_t s) {
    const dim3 grid((n + 3) / 4), block(256);
    const int64_t rb = row_bytes(fmt, k);
    if (tokens == 1)
        hipLaunchKernelGGL((linear_kernel<XDT, 1>), grid, block, 0, s, (const uint8_t*)w, fmt, n, k, rb, fast, x, tokens, y, ydt);
    else if (tokens <= 4)
        hipLaunchKernelGGL((linear_kernel<XDT, 4>), grid, block, 0, s, (const uint8_t*)w, fmt, n, k, rb, fast, x, tokens, y, ydt);
    else
        hipLaunchKernelGGL((linear_kernel<XDT, 8>), grid, block, 0, s, (const uint8_t*)w, fmt, n, k, rb, fast, x, tokens, y, ydt);
}

static int validate_matrix(const char* who, const void* w, int fmt, int64_t n, int64_t k) {
    if (!w) return fail(QMOE_EINVAL, "%s: null weight pointer", who);
    if (!block_elems(fmt)) return fail(QMOE_EINVAL, "%s: unknown packed format id %d", who, fmt);
    if (!format_implemented(fmt)) return fail(QMOE_EUNSUPPORTED, "%s: packed format id %d has no kernel", who, fmt);
    if (n <= 0 || k <= 0) return fail(QMOE_EINVAL, "%s: matrix dimensions must be positive (n=%lld k=%lld)", who, (long long)n, (long long)k);
    if (k % block_elems(fmt)) return fail(QMOE_EINVAL, "%s: K=%lld is not a multiple of the %d-element block", who, (long long)k, block_elems(fmt));
    if ((uintptr_t)w % 2) return fail(QMOE_EINVAL, "%s: packed weights must be 2-byte aligned", who);
    return QMOE_OK;
}
static int validate_dtype(const char* who, const char* what, int dt) {
    if (!dtype_size(dt)) return fail(QMOE_EINVAL, "%s: unknown %s element type %d", who, what, dt);
    return QMOE_OK;
}

int linear_impl(const void* w, int fmt, int n, int k, const void* x, int xdt, int tokens, void* y, int ydt,
                hipStream_t s) {
    int rc = validate_matrix("qmoe_linear", w, fmt, n, k);
    if (rc) return rc;
    if (!x || !y) return fail(QMOE_EINVAL, "qmoe_linear: null activation or output pointer");
    if (tokens < 1) return fail(QMOE_EINVAL, "qmoe_linear: tokens must be >= 1 (got %d)", tokens);
    if ((rc = validate_dtype("qmoe_linear", "input", xdt)) || (rc = validate_dtype("qmoe_linear", "output", ydt))) return rc;
    if ((uintptr_t)x % dtype_size(xdt) || (uintptr_t)y % dtype_size(ydt))
        return fail(QMOE_EINVAL, "qmoe_linear: activation/output pointer not aligned to its element type");
    if (tokens == 1 && stream_supported(fmt, w, n, k, x, xdt)) {
        StreamArgs args{};
        args.count = 1;
        args.p[0] = StreamProblem{(const uint8_t*)w, nullptr, x, y, n, k, fmt, 0, xdt, ydt, 0, 0};
        return stream_launch(args, s);
    }
    // two to four tokens over Q8_0 rows of up to 4096 columns: streamed once, 4x4x4 MFMA products
    if (few_supported(fmt, w, n, k, x, xdt, tokens)) {
        FewArgs f{};
        f.count = 1;
        f.tokens = tokens;
        f.xdt = xdt;
        f.p[0] = FewProblem{(const uint8_t*)w, x, y, n, k, ydt};
        return few_launch(f, s);
    }
    // token batches: the token-tile GEMM (it splits K over the waves of a workgroup when the matrix
    // alone would leave most of the chip idle); the general kernel where its rules do not hold
    // (one token whose row is too long for the streaming kernel's LDS goes the same way if Q8_0;
    // the K-quants' single token is faster in the general kernel than in the GEMM's K-split loop)
    const bool tile_ok = (tokens >= 2 || fmt == QMOE_FMT_Q8_0) && gemm_supported(fmt, w, 0, n, k, x, xdt, k);
    if (tile_ok) {
        GemmDenseArgs d{};
        d.count = 1;
        d.tokens = tokens;
        d.p[0] = GemmDenseProblem{(const uint8_t*)w, x, y, n, k, ydt, 0};
        return gemm_dense_launch(fmt, xdt, d, s);
    }
    const bool fast = rows_fast(fmt, w, row_bytes(fmt, k), k) && x_fast(x, xdt, k);
    if (xdt == QMOE_DT_F32) launch_linear_mt<QMOE_DT_F32>(w, fmt, n, k, fast, x, tokens, y, ydt, s);
    else if (xdt == QMOE_DT_F16) launch_linear_mt<QMOE_DT_F16>(w, fmt, n, k, fast, x, tokens, y, ydt, s);
    else launch_linear_mt<QMOE_DT_BF16>(w, fmt, n, k, fast, x, tokens, y, ydt, s);
    return check_launch("qmoe_linear");
}

// ---- fused gate/up SwiGLU --------------------------------------------------------------------
template <int XDT, int MT>
__global__ __launch_bounds__(256) void swiglu_kernel(const uint8_t* __restrict__ gate, int gf, int64_t grb, bool gfast,
                                                     const uint8_t* __restrict__ up, int uf, int64_t urb, bool ufast,
                                                     int f, int k, const void* __restrict__ x, int tokens,
                                                     void* __restrict__ h, int hdt) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= f) return;
    for (int t0 = 0; t0 < tokens; t0 += MT) {
        size_t xbase[MT];
        float ga[MT], ua[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            int t = t0 + m < tokens ? t0 + m : tokens - 1;
            xbase[m] = (size_t)t * k;
            ga[m] = ua[m] = 0.0f;
        }
        row_dot<XDT, MT>(gf, gate + (int64_t)row * grb, k, gfast, x, xbase, lane, ga);
        row_dot<XDT, MT>(uf, up + (int64_t)row * urb, k, ufast, x, xbase, lane, ua);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float g = wave_sum(ga[m]), u = wave_sum(ua[m]);
            if (lane == m && t0 + m < tokens) store_out(h, hdt, (size_t)(t0 + m) * f + row, silu_mul(g, u));
        }
    }
}

template <int XDT>
static void launch_swiglu_mt(const void* gate, int gf, bool gfast, const void* up, int uf, bool ufast, int f, int k,
                             const void* x, int tokens, void* h, int hdt, hipStream_t s) {
    const dim3 grid((f + 3) / 4), block(256);
    const int64_t grb = row_bytes(gf, k), urb = row_bytes(uf, k);
    if (tokens == 1)
        hipLaunchKernelGGL((swiglu_kernel<XDT, 1>), grid, block, 0, s, (const uint8_t*)gate, gf, grb, gfast, (const uint8_t*)up, uf, urb, ufast, f, k, x, tokens, h, hdt);
    else
        hipLaunchKernelGGL((swiglu_kernel<XDT, 4>), grid, block, 0, s, (const uint8_t*)gate, gf, grb, gfast, (const uint8_t*)up, uf, urb, ufast, f, k, x, tokens, h, hdt);
}

int swiglu_impl(const void* gate, int gf, const void* up, int uf, int f, int k, const void* x, int xdt, int tokens,
                void* h, int hdt, hipStream_t s) {
    int rc = validate_matrix("qmoe_swiglu(gate)", gate, gf, f, k);
    if (!rc) rc = validate_matrix("qmoe_swiglu(up)", up, uf, f, k);
    if (rc) return rc;
    if (!x || !h) return fail(QMOE_EINVAL, "qmoe_swiglu: null activation or output pointer");
    if (tokens < 1) return fail(QMOE_EINVAL, "qmoe_swiglu: tokens must be >= 1 (got %d)", tokens);
    if ((rc = validate_dtype("qmoe_swiglu", "input", xdt)) || (rc = validate_dtype("qmoe_swiglu", "output", hdt))) return rc;
    if ((uintptr_t)x % dtype_size(xdt) || (uintptr_t)h % dtype_size(hdt))
        return fail(QMOE_EINVAL, "qmoe_swiglu: activation/output pointer not aligned to its element type");
    if (tokens == 1 && gf == uf && stream_supported(gf, gate, f, k, x, xdt) && stream_supported(uf, up, f, k, x, xdt)) {
        StreamArgs args{};
        args.count = 1;
        args.p[0] = StreamProblem{(const uint8_t*)gate, (const uint8_t*)up, x, h, f, k, gf, 0, xdt, hdt, 0, 0};
        return stream_launch(args, s);
    }
    if (tokens >= 2 && gf == uf && gemm_supported(gf, gate, 0, f, k, x, xdt, k) && gemm_supported(uf, up, 0, f, k, x, xdt, k)) {
        GemmArgs g{};  // token batch: gate and up rows multiplied together on MFMA
        g.w = (const uint8_t*)gate;
        g.w2 = (const uint8_t*)up;
        g.n = f;
        g.k = k;
        g.a0 = x;
        g.a_stride = k;
        g.dense_tokens = tokens;
        g.out0 = h;
        g.out_dt = hdt;
        return gemm_launch(gf, true, xdt, g, (tokens + GEMM_CHUNK - 1) / GEMM_CHUNK, tokens, s);
    }
    const bool xf = x_fast(x, xdt, k);
    const bool gfast = xf && rows_fast(gf, gate, row_bytes(gf, k), k);
    const bool ufast = xf && rows_fast(uf, up, row_bytes(uf, k), k);
    if (xdt == QMOE_DT_F32) launch_swiglu_mt<QMOE_DT_F32>(gate, gf, gfast, up, uf, ufast, f, k, x, tokens, h, hdt, s);
    else if (xdt == QMOE_DT_F16) launch_swiglu_mt<QMOE_DT_F16>(gate, gf, gfast, up, uf, ufast, f, k, x, tokens, h, hdt, s);
    else launch_swiglu_mt<QMOE_DT_BF16>(gate, gf, gfast, up, uf, ufast, f, k, x, tokens, h, hdt, s);
    return check_launch("qmoe_swiglu");
}

}  // namespace qmoe

using namespace qmoe;

extern "C" {

int qmoe_abi_version(void) { return QMOE_ABI_VERSION; }
const char* qmoe_last_error(void) { return error_buffer(); }

int qmoe_format_info(int fmt, int* elems, int* bytes) {
    if (!block_elems(fmt)) return fail(QMOE_EINVAL, "qmoe_format_info: unknown packed format id %d", fmt);
    if (elems) *elems = block_elems(fmt);
    if (bytes) *bytes = block_bytes(fmt);
    return QMOE_OK;
}

int qmoe_dequantize(const void* w, int fmt, int64_t n, int64_t k, float* out, void* stream) {
    int rc = validate_matrix("qmoe_dequantize", w, fmt, n, k);
    if (rc) return rc;
    if (!out || (uintptr_t)out % 4) return fail(QMOE_EINVAL, "qmoe_dequantize: output pointer null or misaligned");
    hipStream_t s = (hipStream_t)stream;
    switch (fmt) {
    case QMOE_FMT_Q8_0: return launch_dequant<QMOE_FMT_Q8_0>(w, n, k, out, s);
    case QMOE_FMT_Q4_0: return launch_dequant<QMOE_FMT_Q4_0>(w, n, k, out, s);
    case QMOE_FMT_Q3_K: return launch_dequant<QMOE_FMT_Q3_K>(w, n, k, out, s);
    case QMOE_FMT_Q4_K: return launch_dequant<QMOE_FMT_Q4_K>(w, n, k, out, s);
    case QMOE_FMT_Q5_K: return launch_dequant<QMOE_FMT_Q5_K>(w, n, k, out, s);
    case QMOE_FMT_Q6_K: return launch_dequant<QMOE_FMT_Q6_K>(w, n, k, out, s);
    default: return launch_dequant<QMOE_FMT_BF16>(w, n, k, out, s);
    }
}

int qmoe_linear(const void* w, int fmt, int n, int k, const void* x, int x_dtype, int tokens, void* y, int y_dtype,
                void* stream) {
    return linear_impl(w, fmt, n, k, x, x_dtype, tokens, y, y_dtype, (hipStream_t)stream);
}

int qmoe_linear_batch(const qmoe_linear_problem* problems, int count, void* stream) {
    if (!problems || count < 1) return fail(QMOE_EINVAL, "qmoe_linear_batch: need at least one problem");
    // Validate everything before the first launch so that an error leaves all outputs untouched.
    for (int i = 0; i < count; ++i) {
        const qmoe_linear_problem& p = problems[i];
        int rc = validate_matrix("qmoe_linear_batch", p.w, p.fmt, p.n, p.k);
        if (rc) return rc;
        if (!p.x || !p.y || p.tokens < 1 || !dtype_size(p.x_dtype) || !dtype_size(p.y_dtype))
            return fail(QMOE_EINVAL, "qmoe_linear_batch: problem %d has a null pointer, no tokens or a bad element type", i);
    }
    // Single-token problems the streaming kernel covers share launches (up to
    // STREAM_MAX_PROBLEMS each), and so do token batches of one size the token-tile GEMM covers
    // (up to GEMM_MAX_PROBLEMS each); anything else goes through linear_impl in order.
    StreamArgs args{};
    GemmDenseArgs dense{};
    int dense_fmt = 0, dense_xdt = 0;
    auto flush_stream = [&]() -> int {
        if (!args.count) return QMOE_OK;
        const int rc = stream_launch(args, (hipStream_t)stream);
        args.count = 0;
        return rc;
    };
    auto flush_dense = [&]() -> int {
        if (!dense.count) return QMOE_OK;
        const int rc = gemm_dense_launch(dense_fmt, dense_xdt, dense, (hipStream_t)stream);
        dense.count = 0;
        return rc;
    };
    FewArgs few{};
    auto flush_few = [&]() -> int {
        if (!few.count) return QMOE_OK;
        const int rc = few_launch(few, (hipStream_t)stream);
        few.count = 0;
        return rc;
    };
    for (int i = 0; i < count; ++i) {
        const qmoe_linear_problem& p = problems[i];
        const bool aligned = (uintptr_t)p.x % dtype_size(p.x_dtype) == 0 && (uintptr_t)p.y % dtype_size(p.y_dtype) == 0;
        const bool streams = aligned && p.tokens == 1 && stream_supported(p.fmt, p.w, p.n, p.k, p.x, p.x_dtype);
        const bool fews = aligned && !streams && few_supported(p.fmt, p.w, p.n, p.k, p.x, p.x_dtype, p.tokens);
        const bool tiles = aligned && !streams && !fews && (p.tokens >= 2 || p.fmt == QMOE_FMT_Q8_0) &&
                           gemm_supported(p.fmt, p.w, 0, p.n, p.k, p.x, p.x_dtype, p.k);
        int rc;
        if (fews) {
            if ((rc = flush_stream()) || (rc = flush_dense())) return rc;
            if (few.count && (few.tokens != p.tokens || few.xdt != p.x_dtype || few.count == FEW_MAX_PROBLEMS ||
                              few_is_wide(few.p[0].k) != few_is_wide(p.k)) && (rc = flush_few())) return rc;
            few.tokens = p.tokens;
            few.xdt = p.x_dtype;
            few.p[few.count++] = FewProblem{(const uint8_t*)p.w, p.x, p.y, p.n, p.k, p.y_dtype};
        } else if (streams) {
            if ((rc = flush_dense()) || (rc = flush_few())) return rc;
            if (args.count && (args.p[0].fmt != p.fmt || args.count == STREAM_MAX_PROBLEMS) && (rc = flush_stream())) return rc;
            args.p[args.count++] = StreamProblem{(const uint8_t*)p.w, nullptr, p.x, p.y, p.n, p.k, p.fmt, 0,
                                                 p.x_dtype, p.y_dtype, 0, 0};
        } else if (tiles) {
            if ((rc = flush_stream()) || (rc = flush_few())) return rc;
            if (dense.count && (dense_fmt != p.fmt || dense_xdt != p.x_dtype || dense.tokens != p.tokens ||
                                dense.count == GEMM_MAX_PROBLEMS) && (rc = flush_dense())) return rc;
            dense_fmt = p.fmt;
            dense_xdt = p.x_dtype;
            dense.tokens = p.tokens;
            dense.p[dense.count++] = GemmDenseProblem{(const uint8_t*)p.w, p.x, p.y, p.n, p.k, p.y_dtype, 0};
        } else {
            if ((rc = flush_stream()) || (rc = flush_dense()) || (rc = flush_few())) return rc;
            if ((rc = linear_impl(p.w, p.fmt, p.n, p.k, p.x, p.x_dtype, p.tokens, p.y, p.y_dtype, (hipStream_t)stream))) return rc;
        }
    }
    int rc;
    if ((rc = flush_stream()) || (rc = flush_dense()) || (rc = flush_few())) return rc;
    return QMOE_OK;
}

int qmoe_swiglu(const void* gate, int gate_fmt, const void* up, int up_fmt, int f, int k, const void* x, int x_dtype,
                int tokens, void* h, int h_dtype, void* stream) {
    return swiglu_impl(gate, gate_fmt, up, up_fmt, f, k, x, x_dtype, tokens, h, h_dtype, (hipStream_t)stream);
}

int qmoe_expert(const void* gate, int gate_fmt, const void* up, int up_fmt, const void* down, int down_fmt,
                int d_model, int d_ff, const void* x, int x_dtype, int tokens, void* out, int out_dtype,
                float* workspace, void* stream) {
    if (!workspace || (uintptr_t)workspace % 16)
        return fail(QMOE_EWORKSPACE, "qmoe_expert: workspace of tokens*d_ff floats (16-byte aligned) required");
    // Validate the down projection before anything is launched.
    int rc = validate_matrix("qmoe_expert(down)", down, down_fmt, d_model, d_ff);
    if (rc) return rc;
    if (!out || !dtype_size(out_dtype)) return fail(QMOE_EINVAL, "qmoe_expert: bad output pointer or element type");
    rc = swiglu_impl(gate, gate_fmt, up, up_fmt, d_ff, d_model, x, x_dtype, tokens, workspace, QMOE_DT_F32, (hipStream_t)stream);
    if (rc) return rc;
    return linear_impl(down, down_fmt, d_model, d_ff, workspace, QMOE_DT_F32, tokens, out, out_dtype, (hipStream_t)stream);
}

}  // extern "C"
