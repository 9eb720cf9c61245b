// Token-tile GEMM on MFMA for batches of tokens (prefill): grouped per-expert gate/up + SwiGLU,
// grouped down scaled by the route, and the same two steps for one dense (shared) expert.
//
// A workgroup owns one chunk of up to 32 tokens of one expert and 64 (gate/up pair) or 128
// weight rows.  K is walked in passes of 256 columns:
//   * the chunk's activations of the pass are staged once per workgroup in LDS as bf16 terms
//     (fp32 / fp16 input is split hi + lo while it is staged, bf16 input is copied, the
//     SwiGLU output of the previous step arrives already split), rows padded to 528 bytes so
//     that the 16 token lanes of an MFMA operand read 16 different bank groups;
//   * every lane (n = lane % 16, g = lane / 16) streams unit 4*pass + g of its weight row
//     with the streaming engine's unit loads, dequantises it exactly as the reference does
//     and splits it into two bf16 terms in registers: that is the B operand of the unit's
//     eight v_mfma_f32_16x16x32_bf16 steps, with no LDS round trip for weights;
//   * hi*hi + lo*hi + hi*lo accumulate in fp32 (lo*lo is below 2^-32 of the product).
// Rows of the next pass (weights and activations) are requested before the current pass is
// multiplied.
#include "qmoe_gemm.hpp"

#include "qmoe_mfma.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

static constexpr int GEMM_THREADS = 256;
static constexpr int GEMM_A_STRIDE = 528;                       // bytes of one staged token row
static constexpr int GEMM_TERM_BYTES = GEMM_CHUNK * GEMM_A_STRIDE;  // one bf16 term of the chunk

template <int AKIND> struct AStage {
    static constexpr int WORDS = (AKIND == GEMM_A_F32 || AKIND == GEMM_A_PAIR) ? 2 : 1;
};

// Eight consecutive columns of one activation row, as they lie in memory; a position outside
// the chunk or the row reads (valid) element 0 instead and is replaced by zeros.
template <int AKIND>
__device__ __forceinline__ void stage_load(uint4& r0, uint4& r1, const GemmArgs& a, int64_t row, int col, bool valid) {
    const int64_t at = valid ? row * a.a_stride + col : 0;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    if (AKIND == GEMM_A_F32) {
        r0 = *(const uint4*)((const float*)a.a0 + at);
        r1 = *(const uint4*)((const float*)a.a0 + at + 4);
    } else if (AKIND == GEMM_A_PAIR) {
        r0 = *(const uint4*)((const uint16_t*)a.a0 + at);
        r1 = *(const uint4*)((const uint16_t*)a.a1 + at);
    } else {
        r0 = *(const uint4*)((const uint16_t*)a.a0 + at);
        r1 = zero;
    }
    if (!valid) { r0 = zero; r1 = zero; }
}

// ... and their bf16 terms into the staged tile (hi at `dst`, lo one term further).
template <int AKIND>
__device__ __forceinline__ void stage_store(const uint4 r0, const uint4 r1, uint8_t* dst) {
    if (AKIND == GEMM_A_BF16) {
        *(uint4*)dst = r0;
    } else if (AKIND == GEMM_A_PAIR) {
        *(uint4*)dst = r0;
        *(uint4*)(dst + GEMM_TERM_BYTES) = r1;
    } else {
        float v[8];
        if (AKIND == GEMM_A_F32) {
            v[0] = __uint_as_float(r0.x); v[1] = __uint_as_float(r0.y); v[2] = __uint_as_float(r0.z); v[3] = __uint_as_float(r0.w);
            v[4] = __uint_as_float(r1.x); v[5] = __uint_as_float(r1.y); v[6] = __uint_as_float(r1.z); v[7] = __uint_as_float(r1.w);
        } else {
            v[0] = half_bits_to_float(r0.x & 0xFFFFu); v[1] = half_bits_to_float(r0.x >> 16);
            v[2] = half_bits_to_float(r0.y & 0xFFFFu); v[3] = half_bits_to_float(r0.y >> 16);
            v[4] = half_bits_to_float(r0.z & 0xFFFFu); v[5] = half_bits_to_float(r0.z >> 16);
            v[6] = half_bits_to_float(r0.w & 0xFFFFu); v[7] = half_bits_to_float(r0.w >> 16);
        }
        OperandBits hi, lo;
        split_terms(v, hi, lo);
        *(uint4*)dst = make_uint4(hi.u[0], hi.u[1], hi.u[2], hi.u[3]);
        *(uint4*)(dst + GEMM_TERM_BYTES) = make_uint4(lo.u[0], lo.u[1], lo.u[2], lo.u[3]);
    }
}

// One chunk (expert e, sorted positions start .. start+count) x this workgroup's rows.
template <int FMT, int AKIND, bool PAIR, int MT>
__device__ __forceinline__ void tile_gemm_chunk(const GemmArgs& a, int e, int start, int count, uint8_t* lds) {
    using U = Unit64<FMT>;
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2, NB = BTerms<FMT>::N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int units = a.k >> 6, passes = (units + 3) >> 2;
    const int64_t rb = row_bytes_dev(FMT, a.k);
    // two matrices per wave: gate and up rows of the same index, or two 16-row tiles
    int rows[2];
    const uint8_t* rp[2];
    if (PAIR) {
        rows[0] = rows[1] = blockIdx.x * 64 + wave * 16 + col;
        const int64_t rr = rows[0] < a.n ? rows[0] : a.n - 1;
        rp[0] = a.w + (int64_t)e * a.stride + rr * rb;
        rp[1] = a.w2 + (int64_t)e * a.stride2 + rr * rb;
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            rows[j] = blockIdx.x * 128 + wave * 32 + 16 * j + col;
            const int64_t rr = rows[j] < a.n ? rows[j] : a.n - 1;
            rp[j] = a.w + (int64_t)e * a.stride + rr * rb;
        }
    }
    floatx4 acc[2][MT];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[j][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    // staging share of this thread: column chunk c8 of token rows tid/32 + 8*j
    constexpr int NS = 2 * MT;
    const int c8 = tid & 31;
    int64_t arow[NS];
    bool avalid[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int r = (tid >> 5) + 8 * j;
        avalid[j] = r < count;
        arow[j] = avalid[j] ? (a.gather ? a.gather[start + r] : start + r) : 0;
    }
    uint4 st0[NS], st1[NS];
    uint32_t raw[2][U::RAW];
    {
        const int u = g < units ? g : 0;
#pragma unroll
        for (int j = 0; j < 2; ++j) U::load_w(rp[j], u, raw[j]);
#pragma unroll
        for (int j = 0; j < NS; ++j) stage_load<AKIND>(st0[j], st1[j], a, arow[j], 8 * c8, avalid[j] && 8 * c8 < a.k);
    }
    for (int p = 0; p < passes; ++p) {
        __syncthreads();  // the previous pass has been multiplied
#pragma unroll
        for (int j = 0; j < NS; ++j) stage_store<AKIND>(st0[j], st1[j], lds + ((tid >> 5) + 8 * j) * GEMM_A_STRIDE + 16 * c8);
        __syncthreads();
        const int unit = 4 * p + g;
        const bool live = unit < units;
        const int uu = live ? unit : 0;
        const int un = unit + 4 < units ? unit + 4 : 0;
        if (p + 1 < passes) {
            const int c0 = 256 * (p + 1) + 8 * c8;
#pragma unroll
            for (int j = 0; j < NS; ++j) stage_load<AKIND>(st0[j], st1[j], a, arow[j], c0, avalid[j] && c0 < a.k);
        }
        // a unit past the end of the row multiplies as zeros: all-zero bytes decode to 0.0 in
        // every format (zero scales)
        if (!live) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < U::RAW; ++i) raw[j][i] = 0u;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                // the eight weights of step s only: the rest of the unit's decode is dead code
                // here and is dropped, so few registers stay live between the MFMAs
                OperandBits bt[NB];
                {
                    float wf[64];
                    U::decode(raw[j], wf);
                    if (NB == 2) split_terms(wf + 8 * s, bt[0], bt[NB - 1]);
                    else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) bt[0].u[i] = pack_exact_bf16(wf[8 * s + 2 * i], wf[8 * s + 2 * i + 1]);
                    }
                }
                const int koff = (U::kstep(uu, s) - 256 * p) * 2;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const uint8_t* ap = lds + (16 * mt + col) * GEMM_A_STRIDE + koff;
                    OperandBits a0, a1;
                    const uint4 t0 = *(const uint4*)ap;
                    a0.u[0] = t0.x; a0.u[1] = t0.y; a0.u[2] = t0.z; a0.u[3] = t0.w;
                    floatx4 c = acc[j][mt];
                    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, bt[0].v, c, 0, 0, 0);
                    if (NA == 2) {
                        const uint4 t1 = *(const uint4*)(ap + GEMM_TERM_BYTES);
                        a1.u[0] = t1.x; a1.u[1] = t1.y; a1.u[2] = t1.z; a1.u[3] = t1.w;
                        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, bt[0].v, c, 0, 0, 0);
                    }
                    if (NB == 2) c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, bt[NB - 1].v, c, 0, 0, 0);
                    acc[j][mt] = c;
                }
            }
            // this matrix's unit of the next pass takes the registers that just became free
            if (p + 1 < passes) U::load_w(rp[j], un, raw[j]);
        }
    }
    // lane (col, g) holds outputs of tokens 16*mt + 4*g + i, row index col of each matrix
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tk = 16 * mt + 4 * g + i;
            if (tk >= count) continue;
            const size_t pos = (size_t)(start + tk);
            if (PAIR) {
                if (rows[0] < a.n) {
                    // SwiGLU, left as two bf16 terms for the down step's A operand
                    const float v = silu_mul(acc[0][mt][i], acc[1][mt][i]);
                    const uint16_t hi = float_to_bf16_bits(v);
                    const uint16_t lo = float_to_bf16_bits(v - __uint_as_float((uint32_t)hi << 16));
                    ((uint16_t*)a.out0)[pos * a.n + rows[0]] = hi;
                    ((uint16_t*)a.out1)[pos * a.n + rows[0]] = lo;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (rows[j] >= a.n) continue;
                    const float v = acc[j][mt][i];
                    // the routed product is rounded on its own, as the reference stores it
                    ((float*)a.out0)[pos * a.n + rows[j]] = a.scale ? mul_unfused(v, a.scale[pos]) : v;
                }
            }
        }
}

template <int FMT, int AKIND, bool PAIR>
__global__ __launch_bounds__(GEMM_THREADS, 2) void tile_gemm_kernel(const GemmArgs a) {
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    __shared__ __attribute__((aligned(16))) uint8_t lds[NA * GEMM_TERM_BYTES];
    const int c = blockIdx.y;
    int e = 0, start, count;
    if (a.chunk_expert) {
        if (c >= *a.n_chunks) return;
        e = a.chunk_expert[c];
        start = a.chunk_start[c];
        count = a.chunk_count[c];
    } else {
        start = c * GEMM_CHUNK;
        count = a.dense_tokens - start < GEMM_CHUNK ? a.dense_tokens - start : GEMM_CHUNK;
    }
    if (count <= 0) return;
    if (count <= 16) tile_gemm_chunk<FMT, AKIND, PAIR, 1>(a, e, start, count, lds);
    else tile_gemm_chunk<FMT, AKIND, PAIR, 2>(a, e, start, count, lds);
}

// ---- host side ------------------------------------------------------------------------------------
bool gemm_supported(int fmt, const void* w, int64_t stride, int n, int k, const void* a0, int a_kind, int64_t a_stride) {
    if (!stream_supported(fmt, w, n, k, nullptr, QMOE_DT_F32)) return false;  // unit loads: same format and alignment rules
    const int align = fmt == QMOE_FMT_Q8_0 ? 4 : fmt == QMOE_FMT_Q6_K ? 2 : 16;
    if (stride % align) return false;
    const int esize = a_kind == GEMM_A_F32 ? 4 : 2;
    return (uintptr_t)a0 % 16 == 0 && (a_stride * esize) % 16 == 0;
}

template <int FMT, bool PAIR>
static void gemm_launch_f(const GemmArgs& a, int a_kind, dim3 grid, hipStream_t s) {
    const dim3 block(GEMM_THREADS);
    switch (a_kind) {
    case GEMM_A_F32: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_F32, PAIR>), grid, block, 0, s, a); break;
    case GEMM_A_F16: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_F16, PAIR>), grid, block, 0, s, a); break;
    case GEMM_A_BF16: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_BF16, PAIR>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_PAIR, PAIR>), grid, block, 0, s, a); break;
    }
}

int gemm_launch(int fmt, bool pair, int a_kind, const GemmArgs& a, int chunks, hipStream_t s) {
    const int rows_per_wg = pair ? 64 : 128;
    const dim3 grid((a.n + rows_per_wg - 1) / rows_per_wg, chunks);
#define QMOE_GEMM_F(F)                                                  \
    if (pair) gemm_launch_f<F, true>(a, a_kind, grid, s);               \
    else gemm_launch_f<F, false>(a, a_kind, grid, s)
    switch (fmt) {
    case QMOE_FMT_Q8_0: QMOE_GEMM_F(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_GEMM_F(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_GEMM_F(QMOE_FMT_Q5_K); break;
    default: QMOE_GEMM_F(QMOE_FMT_BF16); break;
    }
#undef QMOE_GEMM_F
    return check_launch("token-tile GEMM");
}

}  // namespace qmoe
