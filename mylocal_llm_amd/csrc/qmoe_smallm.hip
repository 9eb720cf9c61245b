// Small-batch (2..64 tokens) dequant-fused linear on MFMA: the weights are streamed once, with
// the streaming engine's coalesced 64-element unit loads, and every unit feeds eight
// v_mfma_f32_16x16x32_bf16 steps per token tile.
//
// Operands: weights are dequantised in registers exactly as the reference does (fp32) and
// split into two bf16 terms (hi + lo, 16 significant bits) -- never rounded once to bf16;
// fp32 / fp16 activations are split the same way, bf16 activations are used as they are.
// hi*hi + lo*hi + hi*lo accumulate in the MFMA's fp32 accumulator.  A workgroup owns a tile
// of 16*RT rows; its four waves take every fourth group of units and meet in LDS at the end.
#include "qmoe_mfma.hpp"
#include "qmoe_rowdot.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

static constexpr int SM_THREADS = 256;
static constexpr int SM_WAVES = 4;

// The eight activation values k0..k0+7 of one token as MFMA A operands: one bf16 term for
// bf16 input, else hi + lo (rounded remainder): 16 significant bits.
template <int XDT>
__device__ __forceinline__ void load_a_terms(const void* x, size_t index, bool valid, OperandBits* terms) {
    if (XDT == QMOE_DT_BF16) {
        uint4 raw = valid ? *(const uint4*)((const uint16_t*)x + index) : make_uint4(0, 0, 0, 0);
        terms[0].u[0] = raw.x; terms[0].u[1] = raw.y; terms[0].u[2] = raw.z; terms[0].u[3] = raw.w;
        return;
    }
    float v[8];
    if (XDT == QMOE_DT_F32) {
        float4 a = valid ? *(const float4*)((const float*)x + index) : make_float4(0, 0, 0, 0);
        float4 b = valid ? *(const float4*)((const float*)x + index + 4) : make_float4(0, 0, 0, 0);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        float4 a = valid ? Elem<QMOE_DT_F16>::load4(x, index) : make_float4(0, 0, 0, 0);
        float4 b = valid ? Elem<QMOE_DT_F16>::load4(x, index + 4) : make_float4(0, 0, 0, 0);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    split_terms(v, terms[0], terms[1]);
}

template <int XDT> struct ATerms { static constexpr int N = XDT == QMOE_DT_BF16 ? 1 : 2; };

// MT token tiles of 16, RT row tiles of 16 per workgroup item.  Lane (n = l%16, g = l/16) of
// wave w owns unit 16*step + 4*w + g of row n: it loads the unit with the streaming engine's
// unit loads, dequantises it, splits it into bf16 terms, and feeds the unit's eight K-steps
// (8 consecutive columns each) to the MFMA as the B operand; the A operand holds the same
// columns of the activations.  hi*hi + lo*hi + hi*lo are accumulated (lo*lo is below 2^-32).
template <int FMT, int XDT, int MT, int RT>
__global__ __launch_bounds__(SM_THREADS, 2) void smallm_kernel(const uint8_t* __restrict__ w, int n, int k,
                                                             const void* __restrict__ x, int m,
                                                             void* __restrict__ y, int ydt) {
    using U = Unit64<FMT>;
    __shared__ float red[SM_WAVES][MT * RT][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int units = k >> 6;
    const int64_t rb = row_bytes_dev(FMT, k);
    const int items = (n + 16 * RT - 1) / (16 * RT);
    constexpr int NA = ATerms<XDT>::N, NB = BTerms<FMT>::N;
    for (int item = blockIdx.x; item < items; item += gridDim.x) {
        const uint8_t* rp[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            int row = (item * RT + rt) * 16 + col;
            row = row < n ? row : n - 1;
            rp[rt] = w + (int64_t)row * rb;
        }
        floatx4 acc[MT][RT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) acc[mt][rt] = floatx4{0.f, 0.f, 0.f, 0.f};
        uint32_t raw[RT][U::RAW], nxt[RT][U::RAW];
        int u = wave * 4 + g;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) U::load_w(rp[rt], u < units ? u : 0, raw[rt]);
        for (int u0 = 0; u0 < units; u0 += 16) {
            u = u0 + wave * 4 + g;
            const bool live = u < units;
            const int uu = live ? u : 0;
            const int un = u + 16 < units ? u + 16 : 0;
            if (u0 + 16 < units) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) U::load_w(rp[rt], un, nxt[rt]);
            }
            OperandBits bt[RT][8][NB];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                float wf[64];
                U::decode(raw[rt], wf);
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    if (NB == 2) split_terms(wf + 8 * s, bt[rt][s][0], bt[rt][s][NB - 1]);
                    else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) bt[rt][s][0].u[i] = pack_exact_bf16(wf[8 * s + 2 * i], wf[8 * s + 2 * i + 1]);
                    }
                    if (!live) {
#pragma unroll
                        for (int tb = 0; tb < NB; ++tb)
#pragma unroll
                            for (int i = 0; i < 4; ++i) bt[rt][s][tb].u[i] = 0u;
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int k0 = U::kstep(uu, s);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const int token = mt * 16 + col;
                    OperandBits a[NA];
                    load_a_terms<XDT>(x, (size_t)(token < m ? token : 0) * k + k0, token < m, a);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        floatx4 c = acc[mt][rt];
                        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[0].v, bt[rt][s][0].v, c, 0, 0, 0);
                        if (NA == 2) c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[NA - 1].v, bt[rt][s][0].v, c, 0, 0, 0);
                        if (NB == 2) c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[0].v, bt[rt][s][NB - 1].v, c, 0, 0, 0);
                        acc[mt][rt] = c;
                    }
                }
            }
            if (u0 + 16 < units) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                    for (int i = 0; i < U::RAW; ++i) raw[rt][i] = nxt[rt][i];
            }
        }
        // the four waves hold disjoint columns of the same outputs
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave][mt * RT + rt][lane][i] = acc[mt][rt][i];
        __syncthreads();
        for (int p = wave; p < MT * RT; p += SM_WAVES) {
            const int mt = p / RT, rt = p % RT;
            const int row = (item * RT + rt) * 16 + col;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float v = (red[0][p][lane][i] + red[1][p][lane][i]) + (red[2][p][lane][i] + red[3][p][lane][i]);
                const int token = mt * 16 + 4 * g + i;
                if (token < m && row < n) store_out(y, ydt, (size_t)token * n + row, v);
            }
        }
        __syncthreads();
    }
}

bool smallm_supported(int fmt, const void* w, int n, int k, const void* x, int xdt, int tokens) {
    if (tokens < 2 || tokens > 64) return false;
    return stream_supported(fmt, w, n, k, x, xdt);  // same unit loads, same alignment rules
}

template <int FMT, int XDT>
static void smallm_launch_fx(const void* w, int n, int k, const void* x, int tokens, void* y, int ydt, hipStream_t s) {
    const int cap = stream_grid();  // two workgroups per CU
    const int tiles = (n + 15) / 16;
    const int mt = (tokens + 15) / 16;
    // pairs of row tiles reuse the activation operands; taken when tiles are plentiful and the
    // registers allow (two token tiles at most)
    const bool two = mt <= 2 && tiles >= 2 * cap;
    const int items = two ? (tiles + 1) / 2 : tiles;
    const dim3 grid(items < cap ? items : cap), block(SM_THREADS);
#define QMOE_SM(MT, RT) hipLaunchKernelGGL((smallm_kernel<FMT, XDT, MT, RT>), grid, block, 0, s, (const uint8_t*)w, n, k, x, tokens, y, ydt)
    if (two) {
        if (mt == 1) QMOE_SM(1, 2); else QMOE_SM(2, 2);
    } else {
        if (mt == 1) QMOE_SM(1, 1); else if (mt == 2) QMOE_SM(2, 1); else if (mt == 3) QMOE_SM(3, 1); else QMOE_SM(4, 1);
    }
#undef QMOE_SM
}

template <int FMT>
static void smallm_launch_f(const void* w, int n, int k, const void* x, int xdt, int tokens, void* y, int ydt,
                            hipStream_t s) {
    if (xdt == QMOE_DT_F32) smallm_launch_fx<FMT, QMOE_DT_F32>(w, n, k, x, tokens, y, ydt, s);
    else if (xdt == QMOE_DT_F16) smallm_launch_fx<FMT, QMOE_DT_F16>(w, n, k, x, tokens, y, ydt, s);
    else smallm_launch_fx<FMT, QMOE_DT_BF16>(w, n, k, x, tokens, y, ydt, s);
}

int smallm_launch(int fmt, const void* w, int n, int k, const void* x, int xdt, int tokens, void* y, int ydt,
                  hipStream_t s) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: smallm_launch_f<QMOE_FMT_Q8_0>(w, n, k, x, xdt, tokens, y, ydt, s); break;
    case QMOE_FMT_Q6_K: smallm_launch_f<QMOE_FMT_Q6_K>(w, n, k, x, xdt, tokens, y, ydt, s); break;
    case QMOE_FMT_Q5_K: smallm_launch_f<QMOE_FMT_Q5_K>(w, n, k, x, xdt, tokens, y, ydt, s); break;
    case QMOE_FMT_Q4_K: smallm_launch_f<QMOE_FMT_Q4_K>(w, n, k, x, xdt, tokens, y, ydt, s); break;
    default: smallm_launch_f<QMOE_FMT_BF16>(w, n, k, x, xdt, tokens, y, ydt, s); break;
    }
    return check_launch("small-batch linear");
}

}  // namespace qmoe
