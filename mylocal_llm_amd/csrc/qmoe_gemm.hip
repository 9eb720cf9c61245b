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
// multiplied.  Q8_0 takes its own loop (q8_tile_loop below): whole weight tiles go through LDS
// and the integer codes themselves are the B operand.
#include "qmoe_gemm.hpp"

#include <type_traits>

#include "qmoe_mfma.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

static constexpr int GEMM_THREADS = 256;
// measured choices (512-expert step at T = 512 and the 8B layer at 4..64 tokens):
static constexpr int GEMM_SLIM_WGS = 3;        // workgroups a CU where a kernel's LDS and registers allow a third
static constexpr int GEMM_Q8_PLAIN_TILES = 1;  // row tiles per wave of the grouped Q8_0 kernel over plain rows
static constexpr int GEMM_A_STRIDE = 528;                       // bytes of one staged token row
static constexpr int GEMM_TERM_BYTES = GEMM_CHUNK * GEMM_A_STRIDE;  // one bf16 term of the chunk

// Eight consecutive columns of one activation row, as they lie in memory; a position outside
// the chunk or the row reads (valid) element 0 instead.  The caller zeroes such a position when
// it stores, so that no load has to be waited for where it is issued.
template <int AKIND>
__device__ __forceinline__ void stage_fetch(uint4& r0, uint4& r1, const GemmArgs& a, int64_t row, int col, bool valid) {
    const int64_t at = valid ? row * a.a_stride + col : 0;
    if (AKIND == GEMM_A_F32) {
        r0 = ldg<uint4>((const float*)a.a0 + at);
        r1 = ldg<uint4>((const float*)a.a0 + at + 4);
    } else if (AKIND == GEMM_A_PAIR) {
        r0 = ldg<uint4>((const uint16_t*)a.a0 + at);
        r1 = ldg<uint4>((const uint16_t*)a.a1 + at);
    } else {
        r0 = ldg<uint4>((const uint16_t*)a.a0 + at);
        r1 = make_uint4(0, 0, 0, 0);
    }
}

// ... and their bf16 terms into the staged tile (hi at `dst`, lo TERM bytes further).
template <int AKIND, int TERM>
__device__ __forceinline__ void stage_store(const uint4 r0, const uint4 r1, uint8_t* dst) {
    if (AKIND == GEMM_A_BF16) {
        *(uint4*)dst = r0;
    } else if (AKIND == GEMM_A_PAIR) {
        *(uint4*)dst = r0;
        *(uint4*)(dst + TERM) = r1;
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
        *(uint4*)(dst + TERM) = make_uint4(lo.u[0], lo.u[1], lo.u[2], lo.u[3]);
    }
}

// The two bf16 terms of eight staged columns, as 16 bytes each.
template <int AKIND>
__device__ __forceinline__ void stage_terms(const uint4 r0, const uint4 r1, uint4& hi, uint4& lo) {
    if (AKIND == GEMM_A_BF16) {
        hi = r0;
        lo = make_uint4(0, 0, 0, 0);
    } else if (AKIND == GEMM_A_PAIR) {
        hi = r0;
        lo = r1;
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
        OperandBits h, l;
        split_terms(v, h, l);
        hi = make_uint4(h.u[0], h.u[1], h.u[2], h.u[3]);
        lo = make_uint4(l.u[0], l.u[1], l.u[2], l.u[3]);
    }
}

// ---- Q8_0: weight tiles through LDS, integer codes as the MFMA operand ---------------------------
// A Q8_0 weight is d * q with q an int8, and every int8 is a bf16 exactly.  So the B operand is
// the codes themselves (one bf16 term, one conversion per code) and the block scale multiplies
// the 32-column partial product afterwards: acc += d[row, block] * sum_k q[row, k] * x[token, k],
// which is the same sum the dequantised weights give.  The workgroup copies the 272 bytes that
// hold 256 columns of each of its rows from global memory to LDS with 16-byte loads that cover
// whole cache lines once, and every wave takes its operands from there.
// Within a block of 32 columns lane group g multiplies columns 4g..4g+3 and 16+4g..16+4g+3: two
// dwords of codes per lane that the four groups of a row read from neighbouring LDS banks.
// The staged activations are laid out to match (Q8Perm).
static constexpr int Q8_SEG = 272;   // bytes of 256 columns of one row
static constexpr int Q8_ROW = 272;   // bytes between staged rows in LDS
template <int NM> struct Q8Tile {
    static constexpr int ROWS = 64 * NM, CHUNKS = ROWS * 17, SLOTS = (CHUNKS + GEMM_THREADS - 1) / GEMM_THREADS;
    static constexpr int BYTES = ROWS * Q8_ROW;
};

// four int8 codes -> four bf16 (exact)
__device__ __forceinline__ void q8_codes_to_bf16(uint32_t q, uint32_t& lo2, uint32_t& hi2) {
    const float f0 = (float)(int)(int8_t)(q & 0xFF), f1 = (float)(int)(int8_t)((q >> 8) & 0xFF);
    const float f2 = (float)(int)(int8_t)((q >> 16) & 0xFF), f3 = (float)(int)(int8_t)(q >> 24);
    lo2 = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
    hi2 = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
}

// emit(rowblock) stores the finished block.  (A workgroup walking two or four row blocks of its
// chunk with the prefetch carried across measured slower on the 512-expert step: fewer, longer
// workgroups.)
template <int AKIND, bool PAIR, int NM, int MT, class Emit>
__device__ __forceinline__ void q8_tile_loop(const GemmArgs& a, int e, int start, int count, int rowblock, uint8_t* lds,
                                             floatx4 (&acc)[NM][MT], Emit emit) {
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    constexpr int TERM = GEMM_TERM_BYTES;
    using TL = Q8Tile<NM>;
    uint8_t* wt = lds + NA * GEMM_TERM_BYTES;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int passes = (a.k + 255) >> 8;
    const int rb = (a.k >> 5) * 34;
    // this thread's 16-byte pieces of the weight tile: piece tid + 256*i lies 16 bytes a piece in LDS
    // (272 = 17 * 16) and comes from byte woff[i] + piece[i] behind the matrix of its row
    const uint8_t* const base0 = a.w + (int64_t)e * a.stride;
    const uint8_t* const base1 = PAIR ? a.w2 + (int64_t)e * a.stride2 : base0;
    uint32_t woff[TL::SLOTS];
    // (recomputed where they are needed: registers are scarcer than the few operations)
    auto lrow_of = [&](int i) -> int {
        const int c = tid + GEMM_THREADS * i;
        const int lr = c < TL::CHUNKS ? c / 17 : 0;
        return PAIR ? (lr & 63) : lr;
    };
    auto piece_of = [&](int i) -> int {
        const int c = tid + GEMM_THREADS * i;
        return c < TL::CHUNKS ? 16 * (c % 17) : 0;
    };
#pragma unroll
    for (int i = 0; i < TL::SLOTS; ++i) {   // (a matrix stays below 4 GB)
        const int row = rowblock * (PAIR ? 64 : TL::ROWS) + lrow_of(i);
        woff[i] = (uint32_t)(row < a.n ? row : a.n - 1) * (uint32_t)rb + piece_of(i);
    }
    // Every piece is loaded without a condition, so that the loads of a pass leave together and
    // nothing waits for them before they are stored.  A piece that reaches past the end of its
    // row is loaded `shift` bytes earlier (always the 16 bytes that end the row) and moved into
    // place, zeros behind it, when it is stored.
    auto wshift = [&](int i, int p) -> int {
        const int over = piece_of(i) + 16 - (rb - Q8_SEG * p);
        return over < 0 ? 0 : over;
    };
    int lrow[NM];
#pragma unroll
    for (int j = 0; j < NM; ++j) lrow[j] = PAIR ? j * 64 + wave * 16 + col : wave * (16 * NM) + 16 * j + col;
    // staging share of this thread: column chunk c8 of token rows tid/32 + 8*j
    constexpr int NS = 2 * MT;
    const int c8 = tid & 31, r0 = tid >> 5;
    // columns 8*c8 .. +7 are columns 8*(c8&3) .. of block c8>>2: two runs of four that belong to
    // lane groups 2*(c8&1) and 2*(c8&1)+1, in the first or second half of their eight columns
    const int adst = 64 * (c8 >> 2) + 32 * (c8 & 1) + 8 * ((c8 >> 1) & 1);
    uint4 st0[NS], st1[NS];
    u32x4_t wreg[TL::SLOTS];
    auto request_w = [&](int p) {
#pragma unroll
        for (int i = 0; i < TL::SLOTS; ++i) {
            const uint8_t* base = (PAIR && GEMM_THREADS * i >= 64 * 17) ? base1
                                  : (PAIR && GEMM_THREADS * (i + 1) > 64 * 17 && tid + GEMM_THREADS * i >= 64 * 17) ? base1 : base0;
            wreg[i] = ldg_u32x4<4>(base + (woff[i] + (uint32_t)(Q8_SEG * p - wshift(i, p))));
        }
    };
    // the first weights leave before the chunk's activation rows are known
    request_w(0);
    int arow[NS];
    bool avalid[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int r = r0 + 8 * j;
        avalid[j] = r < count;
        arow[j] = avalid[j] ? (a.gather ? ldg<int>(a.gather + start + r) : start + r) : 0;
    }
    auto request_a = [&](int p) {
        const int c0 = 256 * p + 8 * c8;
#pragma unroll
        for (int j = 0; j < NS; ++j) stage_fetch<AKIND>(st0[j], st1[j], a, arow[j], c0, avalid[j] && c0 < a.k);
    };
    request_a(0);
    auto multiply = [&]() {
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            OperandBits af[MT][NA];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < NA; ++t) {
                    const uint4 v = *(const uint4*)(lds + t * TERM + (16 * mt + col) * GEMM_A_STRIDE + 64 * b + 16 * g);
                    af[mt][t].u[0] = v.x; af[mt][t].u[1] = v.y; af[mt][t].u[2] = v.z; af[mt][t].u[3] = v.w;
                }
#pragma unroll
            for (int j = 0; j < NM; ++j) {
                const uint8_t* rp = wt + lrow[j] * Q8_ROW;
                const uint32_t* dw = (const uint32_t*)rp;
                const float d = half_bits_to_float(*(const uint16_t*)(rp + 34 * b));
                uint32_t q0, q1;
                if (b & 1) {
                    // codes start on a dword
                    const int at = (34 * b + 2) / 4;
                    q0 = dw[at + g];
                    q1 = dw[at + 4 + g];
                } else {
                    const int at = (34 * b) / 4;
                    q0 = __builtin_amdgcn_alignbit(dw[at + g + 1], dw[at + g], 16);
                    q1 = __builtin_amdgcn_alignbit(dw[at + g + 5], dw[at + g + 4], 16);
                }
                OperandBits bt;
                q8_codes_to_bf16(q0, bt.u[0], bt.u[1]);
                q8_codes_to_bf16(q1, bt.u[2], bt.u[3]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    floatx4 c = floatx4{0.f, 0.f, 0.f, 0.f};
                    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt][0].v, bt.v, c, 0, 0, 0);
                    if (NA == 2) c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt][NA - 1].v, bt.v, c, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[j][mt][i] = fmaf(d, c[i], acc[j][mt][i]);
                }
            }
        }
    };
    for (int p = 0; p < passes; ++p) {
        __syncthreads();   // the previous pass has been multiplied
        const bool ragged = rb - Q8_SEG * p < Q8_SEG;   // the rows end inside this pass
#pragma unroll
        for (int i = 0; i < TL::SLOTS; ++i) {
            u32x4_t v = wreg[i];
            if (ragged) {
                const int sh = (wshift(i, p) < 16 ? wshift(i, p) : 16) >> 2;   // dwords
                const u32x4_t t = v;
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const int from = d + sh;
                    v[d] = from == 0 ? t[0] : from == 1 ? t[1] : from == 2 ? t[2] : from == 3 ? t[3] : 0u;
                }
            }
            if (tid + GEMM_THREADS * i < TL::CHUNKS) *(uint4*)(wt + 16 * (tid + GEMM_THREADS * i)) = make_uint4(v[0], v[1], v[2], v[3]);
        }
        const bool cols_live = 256 * p + 8 * c8 < a.k;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            uint4 hi, lo;
            stage_terms<AKIND>(st0[j], st1[j], hi, lo);
            if (!(avalid[j] && cols_live)) hi = lo = make_uint4(0, 0, 0, 0);
            uint8_t* dst = lds + (r0 + 8 * j) * GEMM_A_STRIDE + adst;
            *(uint2*)dst = make_uint2(hi.x, hi.y);
            *(uint2*)(dst + 16) = make_uint2(hi.z, hi.w);
            if (NA == 2) {
                *(uint2*)(dst + TERM) = make_uint2(lo.x, lo.y);
                *(uint2*)(dst + TERM + 16) = make_uint2(lo.z, lo.w);
            }
        }
        __syncthreads();
        if (p + 1 < passes) {
            request_w(p + 1);
            request_a(p + 1);
        }
        multiply();
    }
    emit(rowblock);
}

// ---- Q4_K / Q5_K: the same scheme with the 4- and 5-bit codes as the operand ----------------------
// w = (d * sc) * q - dmin * m for the 32 columns of a group, so with S = the sum of the group's
// activations   sum_k w x = (d * sc) * sum_k q x  -  (dmin * m) * S :
// one MFMA per group and activation term over the codes (exact in bf16), two FMAs per output.
// A pass is one 256-column block of every row (144 / 176 bytes, 9 / 11 pieces of 16 bytes, rows
// in LDS as they lie in memory); S comes from the activation staging, one value per token and
// group.  Lane group g takes columns 4g..4g+3 and 16+4g..16+4g+3 of a group as for Q8_0: the
// nibbles of one dword each, and (Q5_K) bit `group` of the bytes of one dword of the high plane.
template <int FMT, int NM> struct K45Tile {
    static constexpr int SEG = FMT == QMOE_FMT_Q5_K ? 176 : 144;
    static constexpr int QS = FMT == QMOE_FMT_Q5_K ? 48 : 16;
    static constexpr int PIECES = SEG / 16;
    static constexpr int ROWS = 64 * NM, CHUNKS = ROWS * PIECES, SLOTS = (CHUNKS + GEMM_THREADS - 1) / GEMM_THREADS;
    static constexpr int SUMS = 8 * GEMM_CHUNK * 4;          // S[group][token], fp32
    static constexpr int BYTES = ROWS * SEG + SUMS;
};

// four unsigned byte codes -> four bf16 (exact)
__device__ __forceinline__ void byte_codes_to_bf16(uint32_t q, uint32_t& lo2, uint32_t& hi2) {
    const float f0 = (float)(q & 0xFFu), f1 = (float)((q >> 8) & 0xFFu), f2 = (float)((q >> 16) & 0xFFu), f3 = (float)(q >> 24);
    lo2 = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
    hi2 = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
}

// sum of the eight staged columns as the GEMM sees them (the value of hi + lo)
template <int AKIND>
__device__ __forceinline__ float stage_sum(const uint4 r0, const uint4 r1) {
    auto two = [](uint32_t w) { return __uint_as_float(w << 16) + __uint_as_float(w & 0xFFFF0000u); };
    if (AKIND == GEMM_A_F32) {
        return ((__uint_as_float(r0.x) + __uint_as_float(r0.y)) + (__uint_as_float(r0.z) + __uint_as_float(r0.w))) +
               ((__uint_as_float(r1.x) + __uint_as_float(r1.y)) + (__uint_as_float(r1.z) + __uint_as_float(r1.w)));
    } else if (AKIND == GEMM_A_F16) {
        auto h2 = [](uint32_t w) { return half_bits_to_float(w & 0xFFFFu) + half_bits_to_float(w >> 16); };
        return (h2(r0.x) + h2(r0.y)) + (h2(r0.z) + h2(r0.w));
    } else if (AKIND == GEMM_A_PAIR) {
        return ((two(r0.x) + two(r0.y)) + (two(r0.z) + two(r0.w))) + ((two(r1.x) + two(r1.y)) + (two(r1.z) + two(r1.w)));
    } else {
        return (two(r0.x) + two(r0.y)) + (two(r0.z) + two(r0.w));
    }
}

template <int FMT, int AKIND, bool PAIR, int NM, int MT, class Emit>
__device__ __forceinline__ void k45_tile_loop(const GemmArgs& a, int e, int start, int count, int rowblock, uint8_t* lds,
                                              floatx4 (&acc)[NM][MT], Emit emit) {
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    constexpr int TERM = GEMM_TERM_BYTES;
    using TL = K45Tile<FMT, NM>;
    uint8_t* wt = lds + NA * GEMM_TERM_BYTES;
    float* sums = (float*)(wt + TL::ROWS * TL::SEG);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int passes = a.k >> 8;
    const int rb = passes * TL::SEG;
    const uint8_t* const base0 = a.w + (int64_t)e * a.stride;
    const uint8_t* const base1 = PAIR ? a.w2 + (int64_t)e * a.stride2 : base0;
    // this thread's 16-byte pieces of the weight tile: piece tid + 256*i lies 16 bytes a piece in LDS
    uint32_t woff[TL::SLOTS];
#pragma unroll
    for (int i = 0; i < TL::SLOTS; ++i) {
        const int c = tid + GEMM_THREADS * i;
        const int lr = c < TL::CHUNKS ? c / TL::PIECES : 0;
        const int piece = c < TL::CHUNKS ? c % TL::PIECES : 0;
        const int row = PAIR ? rowblock * 64 + (lr & 63) : rowblock * TL::ROWS + lr;
        woff[i] = (uint32_t)(row < a.n ? row : a.n - 1) * (uint32_t)rb + 16 * piece;   // (a matrix stays below 4 GB)
    }
    int lrow[NM];
#pragma unroll
    for (int j = 0; j < NM; ++j) lrow[j] = PAIR ? j * 64 + wave * 16 + col : wave * (16 * NM) + 16 * j + col;
    constexpr int NS = 2 * MT;
    const int c8 = tid & 31, r0 = tid >> 5;
    const int adst = 64 * (c8 >> 2) + 32 * (c8 & 1) + 8 * ((c8 >> 1) & 1);
    uint4 st0[NS], st1[NS];
    u32x4_t wreg[TL::SLOTS];
    auto request_w = [&](int p) {
#pragma unroll
        for (int i = 0; i < TL::SLOTS; ++i) {
            constexpr int HALF = 64 * TL::PIECES;   // pieces of the first matrix of a pair
            const uint8_t* base = (PAIR && GEMM_THREADS * i >= HALF) ? base1
                                  : (PAIR && GEMM_THREADS * (i + 1) > HALF && tid + GEMM_THREADS * i >= HALF) ? base1 : base0;
            wreg[i] = ldg_u32x4<16>(base + (woff[i] + (uint32_t)(TL::SEG * p)));
        }
    };
    request_w(0);
    int arow[NS];
    bool avalid[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int r = r0 + 8 * j;
        avalid[j] = r < count;
        arow[j] = avalid[j] ? (a.gather ? ldg<int>(a.gather + start + r) : start + r) : 0;
    }
    auto request_a = [&](int p) {
        const int c0 = 256 * p + 8 * c8;
#pragma unroll
        for (int j = 0; j < NS; ++j) stage_fetch<AKIND>(st0[j], st1[j], a, arow[j], c0, avalid[j]);
    };
    request_a(0);
    for (int p = 0; p < passes; ++p) {
        __syncthreads();   // the previous pass has been multiplied
#pragma unroll
        for (int i = 0; i < TL::SLOTS; ++i)
            if (tid + GEMM_THREADS * i < TL::CHUNKS)
                *(uint4*)(wt + 16 * (tid + GEMM_THREADS * i)) = make_uint4(wreg[i][0], wreg[i][1], wreg[i][2], wreg[i][3]);
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            uint4 hi, lo;
            stage_terms<AKIND>(st0[j], st1[j], hi, lo);
            float part = stage_sum<AKIND>(st0[j], st1[j]);
            if (!avalid[j]) { hi = lo = make_uint4(0, 0, 0, 0); part = 0.f; }
            uint8_t* dst = lds + (r0 + 8 * j) * GEMM_A_STRIDE + adst;
            *(uint2*)dst = make_uint2(hi.x, hi.y);
            *(uint2*)(dst + 16) = make_uint2(hi.z, hi.w);
            if (NA == 2) {
                *(uint2*)(dst + TERM) = make_uint2(lo.x, lo.y);
                *(uint2*)(dst + TERM + 16) = make_uint2(lo.z, lo.w);
            }
            // the four threads c8 = 4G .. 4G+3 hold the 32 columns of group G of this token
            part += __shfl_xor(part, 1, 64);
            part += __shfl_xor(part, 2, 64);
            if ((c8 & 3) == 0) sums[(c8 >> 2) * GEMM_CHUNK + r0 + 8 * j] = part;
        }
        __syncthreads();
        if (p + 1 < passes) {
            request_w(p + 1);
            request_a(p + 1);
        }
        // d, dmin and the packed scales of this lane's rows
        float dd[NM], dm[NM];
        uint32_t s0[NM], s1[NM], s2[NM];
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            const uint4 h = *(const uint4*)(wt + lrow[j] * TL::SEG);
            dd[j] = half_bits_to_float(h.x & 0xFFFFu);
            dm[j] = half_bits_to_float(h.x >> 16);
            s0[j] = h.y; s1[j] = h.z; s2[j] = h.w;
        }
#pragma unroll
        for (int G = 0; G < 8; ++G) {
            OperandBits af[MT][NA];
            floatx4 sx[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int t = 0; t < NA; ++t) {
                    const uint4 v = *(const uint4*)(lds + t * TERM + (16 * mt + col) * GEMM_A_STRIDE + 64 * G + 16 * g);
                    af[mt][t].u[0] = v.x; af[mt][t].u[1] = v.y; af[mt][t].u[2] = v.z; af[mt][t].u[3] = v.w;
                }
                sx[mt] = *(const floatx4*)(sums + G * GEMM_CHUNK + 16 * mt + 4 * g);
            }
#pragma unroll
            for (int j = 0; j < NM; ++j) {
                const uint32_t* dw = (const uint32_t*)(wt + lrow[j] * TL::SEG);
                uint32_t q0 = (dw[TL::QS / 4 + 8 * (G >> 1) + g] >> (4 * (G & 1))) & 0x0F0F0F0Fu;
                uint32_t q1 = (dw[TL::QS / 4 + 8 * (G >> 1) + 4 + g] >> (4 * (G & 1))) & 0x0F0F0F0Fu;
                if (FMT == QMOE_FMT_Q5_K) {
                    q0 |= ((dw[4 + g] >> G) & 0x01010101u) << 4;
                    q1 |= ((dw[8 + g] >> G) & 0x01010101u) << 4;
                }
                OperandBits bt;
                byte_codes_to_bf16(q0, bt.u[0], bt.u[1]);
                byte_codes_to_bf16(q1, bt.u[2], bt.u[3]);
                uint32_t sc, mn;
                kquant_scale_min(s0[j], s1[j], s2[j], G, sc, mn);
                const float scale = dd[j] * (float)sc, floor_ = dm[j] * (float)mn;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    floatx4 c = floatx4{0.f, 0.f, 0.f, 0.f};
                    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt][0].v, bt.v, c, 0, 0, 0);
                    if (NA == 2) c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt][NA - 1].v, bt.v, c, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[j][mt][i] = fmaf(-floor_, sx[mt][i], fmaf(scale, c[i], acc[j][mt][i]));
                }
            }
        }
    }
    emit(rowblock);
}

// ---- Q6_K: 6-bit codes as the operand, 16 columns a scale --------------------------------------
// w = (d * sc) * (q - 32) for the 16 columns of a group.  With bit 5 of a code flipped and the code
// shifted up by two, its byte read as an int8 is 4 * (q - 32): that is the operand (exact in
// bf16), and the group's partial product is scaled by (d * sc) / 4 -- no offset term.
// One v_mfma_f32_16x16x16_bf16 per group and activation term (lane group g multiplies columns
// 4g..4g+3 of the group: the nibbles of one dword and two bits of the bytes of one dword of the
// high plane), activations staged in their natural order.  The 210-byte blocks are only 2-byte
// aligned in memory: a row's block goes to LDS as 13 pieces of 16 bytes plus its scale `d`,
// rows 240 bytes apart (the 16 rows of a fragment then start in 16 different bank groups).
template <int NM> struct Q6Tile {
    static constexpr int SEG = 210, ROW = 240, PIECES = 13;
    static constexpr int ROWS = 64 * NM, CHUNKS = ROWS * PIECES, SLOTS = (CHUNKS + GEMM_THREADS - 1) / GEMM_THREADS;
    static constexpr int BYTES = ROWS * ROW;
};
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;

template <int AKIND, bool PAIR, int NM, int MT, class Emit>
__device__ __forceinline__ void q6_tile_loop(const GemmArgs& a, int e, int start, int count, int rowblock, uint8_t* lds,
                                             floatx4 (&acc)[NM][MT], Emit emit) {
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    constexpr int TERM = GEMM_TERM_BYTES;
    using TL = Q6Tile<NM>;
    static_assert(TL::ROWS <= GEMM_THREADS, "one thread a row fetches its scale");
    uint8_t* wt = lds + NA * GEMM_TERM_BYTES;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int passes = a.k >> 8;
    const int rb = passes * TL::SEG;
    const uint8_t* const base0 = a.w + (int64_t)e * a.stride;
    const uint8_t* const base1 = PAIR ? a.w2 + (int64_t)e * a.stride2 : base0;
    auto row_off = [&](int lr) -> uint32_t {   // (a matrix stays below 4 GB)
        const int row = PAIR ? rowblock * 64 + (lr & 63) : rowblock * TL::ROWS + lr;
        return (uint32_t)(row < a.n ? row : a.n - 1) * (uint32_t)rb;
    };
    uint32_t woff[TL::SLOTS];
    int wdst[TL::SLOTS];
#pragma unroll
    for (int i = 0; i < TL::SLOTS; ++i) {
        const int c = tid + GEMM_THREADS * i;
        const int lr = c < TL::CHUNKS ? c / TL::PIECES : 0;
        const int piece = c < TL::CHUNKS ? c % TL::PIECES : 0;
        woff[i] = row_off(lr) + 16 * piece;
        wdst[i] = lr * TL::ROW + 16 * piece;
    }
    const int drow = tid < TL::ROWS ? tid : 0;   // the row whose `d` this thread fetches
    const uint32_t doff = row_off(drow) + 208;
    const uint8_t* const dbase = (PAIR && drow >= 64) ? base1 : base0;
    int lrow[NM];
#pragma unroll
    for (int j = 0; j < NM; ++j) lrow[j] = PAIR ? j * 64 + wave * 16 + col : wave * (16 * NM) + 16 * j + col;
    constexpr int NS = 2 * MT;
    const int c8 = tid & 31, r0 = tid >> 5;
    uint4 st0[NS], st1[NS];
    u32x4_t wreg[TL::SLOTS];
    uint32_t dreg;
    auto request_w = [&](int p) {
#pragma unroll
        for (int i = 0; i < TL::SLOTS; ++i) {
            constexpr int HALF = 64 * TL::PIECES;   // pieces of the first matrix of a pair
            const uint8_t* base = (PAIR && GEMM_THREADS * i >= HALF) ? base1
                                  : (PAIR && GEMM_THREADS * (i + 1) > HALF && tid + GEMM_THREADS * i >= HALF) ? base1 : base0;
            wreg[i] = ldg_u32x4<2>(base + (woff[i] + (uint32_t)(TL::SEG * p)));
        }
        dreg = ld_u16(dbase + (doff + (uint32_t)(TL::SEG * p)));
    };
    request_w(0);
    int arow[NS];
    bool avalid[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int r = r0 + 8 * j;
        avalid[j] = r < count;
        arow[j] = avalid[j] ? (a.gather ? ldg<int>(a.gather + start + r) : start + r) : 0;
    }
    auto request_a = [&](int p) {
        const int c0 = 256 * p + 8 * c8;
#pragma unroll
        for (int j = 0; j < NS; ++j) stage_fetch<AKIND>(st0[j], st1[j], a, arow[j], c0, avalid[j]);
    };
    request_a(0);
    for (int p = 0; p < passes; ++p) {
        __syncthreads();   // the previous pass has been multiplied
#pragma unroll
        for (int i = 0; i < TL::SLOTS; ++i)
            if (tid + GEMM_THREADS * i < TL::CHUNKS) *(uint4*)(wt + wdst[i]) = make_uint4(wreg[i][0], wreg[i][1], wreg[i][2], wreg[i][3]);
        if (tid < TL::ROWS) *(uint32_t*)(wt + tid * TL::ROW + 208) = dreg;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            uint4 hi, lo;
            stage_terms<AKIND>(st0[j], st1[j], hi, lo);
            if (!avalid[j]) hi = lo = make_uint4(0, 0, 0, 0);
            uint8_t* dst = lds + (r0 + 8 * j) * GEMM_A_STRIDE + 16 * c8;
            *(uint4*)dst = hi;
            if (NA == 2) *(uint4*)(dst + TERM) = lo;
        }
        __syncthreads();
        if (p + 1 < passes) {
            request_w(p + 1);
            request_a(p + 1);
        }
        float dd[NM];
        uint4 scw[NM];
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            const uint8_t* rp = wt + lrow[j] * TL::ROW;
            dd[j] = half_bits_to_float(*(const uint16_t*)(rp + 208));
            scw[j] = *(const uint4*)(rp + 192);
        }
#pragma unroll
        for (int G = 0; G < 16; ++G) {
            const int h = G >> 3, Q = (G >> 1) & 3, L = G & 1;
            union { bf16x4 v; uint2 u; } af[MT][NA];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < NA; ++t) af[mt][t].u = *(const uint2*)(lds + t * TERM + (16 * mt + col) * GEMM_A_STRIDE + 32 * G + 8 * g);
#pragma unroll
            for (int j = 0; j < NM; ++j) {
                const uint32_t* dw = (const uint32_t*)(wt + lrow[j] * TL::ROW);
                const uint32_t ql = dw[16 * h + 8 * (Q & 1) + 4 * L + g];
                const uint32_t qh = dw[32 + 8 * h + 4 * L + g];
                const uint32_t code = ((ql >> (4 * (Q >> 1))) & 0x0F0F0F0Fu) | (((qh >> (2 * Q)) & 0x03030303u) << 4);
                union { bf16x4 v; uint2 u; } bt;
                q8_codes_to_bf16((code ^ 0x20202020u) << 2, bt.u.x, bt.u.y);   // bytes <= 63: no carry between them
                const uint32_t sw = (G >> 2) == 0 ? scw[j].x : (G >> 2) == 1 ? scw[j].y : (G >> 2) == 2 ? scw[j].z : scw[j].w;
                const float scale = (0.25f * dd[j]) * (float)(int)(int8_t)((sw >> (8 * (G & 3))) & 0xFFu);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    floatx4 c = floatx4{0.f, 0.f, 0.f, 0.f};
                    c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(af[mt][0].v, bt.v, c, 0, 0, 0);
                    if (NA == 2) c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(af[mt][NA - 1].v, bt.v, c, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[j][mt][i] = fmaf(scale, c[i], acc[j][mt][i]);
                }
            }
        }
    }
    emit(rowblock);
}

// One chunk (expert e, sorted positions start .. start+count) x this workgroup's rows.
// NM matrices per wave: the gate and up rows of the same index (PAIR, NM == 2) or NM tiles of
// 16 rows; `rowblock` counts blocks of 64 (pair) or 64 * NM rows.
// With SOLO (one token tile, long rows) the four waves share the same 16 * NM rows and split K:
// wave w walks its quarter of the passes, stages its own activations in its own part of the
// LDS tile without waiting for the others, and the partial sums meet in LDS at the end.  A
// matrix with few rows and many columns then has four times as many, four times shorter,
// work items.
template <int FMT, int AKIND, bool PAIR, int NM, int MT, bool SOLO>
__device__ __forceinline__ void tile_gemm_chunk(const GemmArgs& a, int e, int start, int count, int rowblock, uint8_t* lds) {
    static_assert(!PAIR || NM == 2, "a pair is two matrices");
    static_assert(!SOLO || MT == 1, "a wave stages one token tile on its own");
    using U = Unit64<FMT>;
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2, NB = BTerms<FMT>::N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int units = a.k >> 6, all_passes = (units + 3) >> 2;
    const int share = SOLO ? (all_passes + 3) >> 2 : all_passes;
    const int p_begin = SOLO ? wave * share : 0;
    const int passes = p_begin + share < all_passes ? p_begin + share : all_passes;  // end of this wave's range
    const int64_t rb = row_bytes_dev(FMT, a.k);
    int rows[NM];
    const uint8_t* rp[NM];
    if (PAIR) {
        rows[0] = rows[NM - 1] = SOLO ? rowblock * 16 + col : rowblock * 64 + wave * 16 + col;
        const int64_t rr = rows[0] < a.n ? rows[0] : a.n - 1;
        rp[0] = a.w + (int64_t)e * a.stride + rr * rb;
        rp[NM - 1] = a.w2 + (int64_t)e * a.stride2 + rr * rb;
    } else {
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            rows[j] = SOLO ? rowblock * (16 * NM) + 16 * j + col : rowblock * (64 * NM) + wave * (16 * NM) + 16 * j + col;
            const int64_t rr = rows[j] < a.n ? rows[j] : a.n - 1;
            rp[j] = a.w + (int64_t)e * a.stride + rr * rb;
        }
    }
    floatx4 acc[NM][MT];
#pragma unroll
    for (int j = 0; j < NM; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[j][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    // lane (col, g) holds outputs of tokens 16*mt + 4*g + i, row index col of each matrix
    auto emit = [&](int block) {
        int rows[NM];
        if (PAIR) rows[0] = rows[NM - 1] = SOLO ? block * 16 + col : block * 64 + wave * 16 + col;
        else {
#pragma unroll
            for (int j = 0; j < NM; ++j) rows[j] = SOLO ? block * (16 * NM) + 16 * j + col : block * (64 * NM) + wave * (16 * NM) + 16 * j + col;
        }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tk = 16 * mt + 4 * g + i;
            if (tk >= count) continue;
            const size_t pos = (size_t)(start + tk);
            if (PAIR) {
                if (rows[0] < a.n) {
                    // SwiGLU, left as two bf16 terms for the down step's A operand when a second array is given
                    const float v = silu_mul(acc[0][mt][i], acc[NM - 1][mt][i]);
                    if (a.out1) {
                        const uint16_t hi = float_to_bf16_bits(v);
                        const uint16_t lo = float_to_bf16_bits(v - __uint_as_float((uint32_t)hi << 16));
                        ((uint16_t*)a.out0)[pos * a.n + rows[0]] = hi;
                        ((uint16_t*)a.out1)[pos * a.n + rows[0]] = lo;
                    } else {
                        store_out(a.out0, a.out_dt, pos * a.n + rows[0], v);  // a caller's SwiGLU output
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < NM; ++j) {
                    if (rows[j] >= a.n) continue;
                    const float v = acc[j][mt][i];
                    // the routed product is rounded on its own, as the reference stores it
                    if (a.scale) ((float*)a.out0)[pos * a.n + rows[j]] = mul_unfused(v, a.scale[pos]);
                    else store_out(a.out0, a.out_dt, pos * a.n + rows[j], v);
                }
            }
        }
    };
    if constexpr (FMT == QMOE_FMT_Q8_0 && !SOLO) {
        q8_tile_loop<AKIND, PAIR, NM, MT>(a, e, start, count, rowblock, lds, acc, emit);
        return;
    } else if constexpr ((FMT == QMOE_FMT_Q4_K || FMT == QMOE_FMT_Q5_K) && !SOLO) {
        k45_tile_loop<FMT, AKIND, PAIR, NM, MT>(a, e, start, count, rowblock, lds, acc, emit);
        return;
    } else if constexpr (FMT == QMOE_FMT_Q6_K && !SOLO) {
        q6_tile_loop<AKIND, PAIR, NM, MT>(a, e, start, count, rowblock, lds, acc, emit);
        return;
    } else {
    // staging share of this thread: column chunk c8 of token rows tid/32 + 8*j (of the wave's
    // own copy: rows lane/32 + 2*j)
    constexpr int NS = SOLO ? 8 : 2 * MT;
    constexpr int RSTEP = SOLO ? 2 : 8;
    const int c8 = tid & 31;
    const int r0 = SOLO ? (lane >> 5) : (tid >> 5);
    if (SOLO) lds += wave * ((AKIND == GEMM_A_BF16 ? 1 : 2) * 16 * GEMM_A_STRIDE);
    constexpr int TERM = SOLO ? 16 * GEMM_A_STRIDE : GEMM_TERM_BYTES;
    int64_t arow[NS];
    bool avalid[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int r = r0 + RSTEP * j;
        avalid[j] = r < count;
        arow[j] = avalid[j] ? (a.gather ? a.gather[start + r] : start + r) : 0;
    }
    uint4 st0[NS], st1[NS];
    uint32_t raw[NM][U::RAW];
    {
        const int u = 4 * p_begin + g < units ? 4 * p_begin + g : 0;
        const int c0 = 256 * p_begin + 8 * c8;
#pragma unroll
        for (int j = 0; j < NM; ++j) U::load_w(rp[j], u, raw[j]);
#pragma unroll
        for (int j = 0; j < NS; ++j) stage_fetch<AKIND>(st0[j], st1[j], a, arow[j], c0, avalid[j] && c0 < a.k);
    }
    for (int p = p_begin; p < passes; ++p) {
        // the previous pass has been multiplied (LDS operations of one wave stay in order)
        if (SOLO) __builtin_amdgcn_wave_barrier(); else __syncthreads();
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            // (a position outside the chunk or the row was fetched from a valid place: zeros instead)
            const bool live = avalid[j] && 256 * p + 8 * c8 < a.k;
            const uint4 zero = make_uint4(0, 0, 0, 0);
            stage_store<AKIND, TERM>(live ? st0[j] : zero, live ? st1[j] : zero, lds + (r0 + RSTEP * j) * GEMM_A_STRIDE + 16 * c8);
        }
        if (SOLO) __builtin_amdgcn_wave_barrier(); else __syncthreads();
        const int unit = 4 * p + g;
        const bool live = unit < units;
        const int uu = live ? unit : 0;
        const int un = unit + 4 < units ? unit + 4 : 0;
        if (p + 1 < passes) {
            const int c0 = 256 * (p + 1) + 8 * c8;
#pragma unroll
            for (int j = 0; j < NS; ++j) stage_fetch<AKIND>(st0[j], st1[j], a, arow[j], c0, avalid[j] && c0 < a.k);
        }
        // a unit past the end of the row multiplies as zeros: all-zero bytes decode to 0.0 in
        // every format (zero scales)
        if (!live) {
#pragma unroll
            for (int j = 0; j < NM; ++j)
#pragma unroll
                for (int i = 0; i < U::RAW; ++i) raw[j][i] = 0u;
        }
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            // Every dword of the unit becomes a value of its own here.  Without this, hipcc 7.2
            // kept the unit in its 128-bit load tuples and, in the K-split variant, assigned a
            // conversion result to a register of a tuple whose other bytes were still unread
            // (wrong sums, caught by tests/test_gpu_linear.py).
#pragma unroll
            for (int i = 0; i < U::RAW; ++i) asm volatile("" : "+v"(raw[j][i]));
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
                        const uint4 t1 = *(const uint4*)(ap + TERM);
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
    }
    if (SOLO) {
        // partial sums of the four K ranges: every wave leaves its own in its own LDS part
        floatx4* mine = (floatx4*)lds;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < NM; ++j) mine[j * 64 + lane] = acc[j][0];
        __syncthreads();
        if (wave != 0) return;
        constexpr int PART = (AKIND == GEMM_A_BF16 ? 1 : 2) * 16 * GEMM_A_STRIDE / (int)sizeof(floatx4);
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            const floatx4 b = mine[PART + j * 64 + lane], c = mine[2 * PART + j * 64 + lane], d = mine[3 * PART + j * 64 + lane];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[j][0][i] = (acc[j][0][i] + b[i]) + (c[i] + d[i]);
        }
    }
    emit(rowblock);
}

// Row tiles per wave and workgroups per CU of the grouped kernel.  Q8_0 keeps a workgroup's LDS and
// registers small enough for three workgroups a CU where it can (bf16 activations: one staged
// term; plain rows: one row tile per wave): the kernel waits for memory most of the time and
// a third workgroup fills part of that.
template <int FMT, int NM> struct WeightTile {
    static constexpr int BYTES = FMT == QMOE_FMT_Q8_0 ? Q8Tile<NM>::BYTES
                                 : (FMT == QMOE_FMT_Q4_K || FMT == QMOE_FMT_Q5_K) ? K45Tile<FMT, NM>::BYTES
                                 : FMT == QMOE_FMT_Q6_K ? Q6Tile<NM>::BYTES : 0;
};
template <int FMT, int AKIND, bool PAIR> struct GroupedShape {
    static constexpr int NM = (FMT == QMOE_FMT_Q8_0 && !PAIR) ? GEMM_Q8_PLAIN_TILES : 2;
    static constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    static constexpr int LDS = NA * GEMM_TERM_BYTES + WeightTile<FMT, NM>::BYTES;
    static constexpr int WGS = (WeightTile<FMT, NM>::BYTES != 0 && LDS * 3 <= 160 * 1024) ? GEMM_SLIM_WGS : 2;
};

// A launch may carry a second, dense problem of the same kinds (`side`: the shared expert beside
// the routed ones): its token chunks come first in blockIdx.y, each cut into `side_parts` parts
// of gridDim.x row blocks, so that the two problems need not have the same number of rows and
// the long workgroups of the dense problem start first.
template <int FMT, int AKIND, bool PAIR>
__global__ __launch_bounds__(GEMM_THREADS, (GroupedShape<FMT, AKIND, PAIR>::WGS)) void tile_gemm_kernel(const GemmArgs main_args, const GemmArgs side,
                                                                                                       int side_chunks, int side_parts) {
    using GS = GroupedShape<FMT, AKIND, PAIR>;
    __shared__ __attribute__((aligned(16))) uint8_t lds[GS::LDS];
    constexpr int ROWS_PER_WG = PAIR ? 64 : 64 * GS::NM;
    int c = blockIdx.y, rowblock = blockIdx.x;
    const bool on_side = c < side_chunks * side_parts;
    const GemmArgs& a = on_side ? side : main_args;
    if (on_side) {
        rowblock += (c % side_parts) * gridDim.x;
        c /= side_parts;
    } else {
        c -= side_chunks * side_parts;
    }
    if (rowblock * ROWS_PER_WG >= a.n) return;
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
    if (count <= 16) tile_gemm_chunk<FMT, AKIND, PAIR, GS::NM, 1, false>(a, e, start, count, rowblock, lds);
    else tile_gemm_chunk<FMT, AKIND, PAIR, GS::NM, 2, false>(a, e, start, count, rowblock, lds);
}

// Chunks of at most 16 tokens with K split over the four waves of a workgroup (16 rows, or 16
// gate/up row pairs, a workgroup): the steps of a few tokens whose matrices have too few 64-row
// blocks to fill the chip.
template <int FMT, int AKIND, bool PAIR>
__global__ __launch_bounds__(GEMM_THREADS, 2) void tile_gemm_split_kernel(const GemmArgs a) {
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    __shared__ __attribute__((aligned(16))) uint8_t lds[4 * NA * 16 * GEMM_A_STRIDE];
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
    tile_gemm_chunk<FMT, AKIND, PAIR, PAIR ? 2 : 1, 1, true>(a, e, start, count, blockIdx.x, lds);
}

template <int FMT, bool PAIR>
static void gemm_split_f(const GemmArgs& a, int a_kind, dim3 grid, hipStream_t s) {
    const dim3 block(GEMM_THREADS);
    switch (a_kind) {
    case GEMM_A_F32: hipLaunchKernelGGL((tile_gemm_split_kernel<FMT, GEMM_A_F32, PAIR>), grid, block, 0, s, a); break;
    case GEMM_A_F16: hipLaunchKernelGGL((tile_gemm_split_kernel<FMT, GEMM_A_F16, PAIR>), grid, block, 0, s, a); break;
    case GEMM_A_BF16: hipLaunchKernelGGL((tile_gemm_split_kernel<FMT, GEMM_A_BF16, PAIR>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((tile_gemm_split_kernel<FMT, GEMM_A_PAIR, PAIR>), grid, block, 0, s, a); break;
    }
}

// Several dense matrices (y = W x for `tokens` rows of x each) in one launch: blockIdx.x walks
// the row blocks of all problems, blockIdx.y the token chunks.
template <int FMT, int AKIND, int NM>
__global__ __launch_bounds__(GEMM_THREADS, (FMT == QMOE_FMT_Q8_0 && AKIND == GEMM_A_BF16) ? GEMM_SLIM_WGS : 2) void tile_gemm_dense_kernel(const GemmDenseArgs d) {
    constexpr int NA = AKIND == GEMM_A_BF16 ? 1 : 2;
    // four solo tiles, or one shared tile (Q8_0: and the weight tile behind it)
    constexpr int SHARED = NA * GEMM_TERM_BYTES + WeightTile<FMT, NM>::BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t lds[SHARED > 2 * NA * GEMM_TERM_BYTES ? SHARED : 2 * NA * GEMM_TERM_BYTES];
    int i = 0;
    while (i + 1 < d.count && (int)blockIdx.x >= d.block_start[i + 1]) ++i;
    const bool ksplit = d.p[i].ksplit != 0;
    const int chunk = ksplit ? 16 : GEMM_CHUNK;
    const int start = blockIdx.y * chunk;
    const int count = d.tokens - start < chunk ? d.tokens - start : chunk;
    if (count <= 0) return;
    GemmArgs a{};
    a.w = d.p[i].w;
    a.n = d.p[i].n;
    a.k = d.p[i].k;
    a.a0 = d.p[i].x;
    a.a_stride = d.p[i].k;
    a.out0 = d.p[i].y;
    a.out_dt = d.p[i].ydt;
    const int rowblock = blockIdx.x - d.block_start[i];
    if (ksplit) tile_gemm_chunk<FMT, AKIND, false, NM, 1, true>(a, 0, start, count, rowblock, lds);
    else if (count <= 16) tile_gemm_chunk<FMT, AKIND, false, NM, 1, false>(a, 0, start, count, rowblock, lds);
    else tile_gemm_chunk<FMT, AKIND, false, NM, 2, false>(a, 0, start, count, rowblock, lds);
}

// ---- host side ------------------------------------------------------------------------------------
int stream_grid();

bool gemm_supported(int fmt, const void* w, int64_t stride, int n, int k, const void* a0, int a_kind, int64_t a_stride) {
    // the streaming kernel's formats and alignment rules (same unit loads), rows of any length
    if (!(fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q4_K || fmt == QMOE_FMT_BF16)) return false;
    if (k % 64 || n < 1 || k > (1 << 24)) return false;
    if ((fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q4_K) && (k % 256)) return false;
    const int align = fmt == QMOE_FMT_Q8_0 ? 4 : fmt == QMOE_FMT_Q6_K ? 2 : 16;
    if ((uintptr_t)w % align || row_bytes(fmt, k) % align || stride % align) return false;
    // (the tile loops address a matrix with 32-bit offsets)
    if (fmt != QMOE_FMT_BF16 && (int64_t)n * row_bytes(fmt, k) >= (1ll << 32)) return false;
    const int esize = a_kind == GEMM_A_F32 ? 4 : 2;
    return (uintptr_t)a0 % 16 == 0 && (a_stride * esize) % 16 == 0;
}

template <int FMT, bool PAIR>
static void gemm_launch_f(const GemmArgs& a, const GemmArgs& side, int side_chunks, int side_parts, int a_kind, dim3 grid, hipStream_t s) {
    const dim3 block(GEMM_THREADS);
    switch (a_kind) {
    case GEMM_A_F32: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_F32, PAIR>), grid, block, 0, s, a, side, side_chunks, side_parts); break;
    case GEMM_A_F16: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_F16, PAIR>), grid, block, 0, s, a, side, side_chunks, side_parts); break;
    case GEMM_A_BF16: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_BF16, PAIR>), grid, block, 0, s, a, side, side_chunks, side_parts); break;
    default: hipLaunchKernelGGL((tile_gemm_kernel<FMT, GEMM_A_PAIR, PAIR>), grid, block, 0, s, a, side, side_chunks, side_parts); break;
    }
}

static bool gemm_splits_k(const GemmArgs& a, int chunks, int max_count) {
    return max_count <= 16 && a.k >= 1024 && (int64_t)((a.n + 63) / 64) * chunks < stream_grid() / 2;
}

bool gemm_side_fits(const GemmArgs& a, int chunks, const GemmArgs& side, int side_chunks, int max_count) {
    return !gemm_splits_k(a, chunks, max_count) && !gemm_splits_k(side, side_chunks, max_count) && !side.chunk_expert && side.n >= 1;
}

int gemm_launch(int fmt, bool pair, int a_kind, const GemmArgs& a, int chunks, int max_count, hipStream_t s,
                const GemmArgs* side, int side_chunks) {
    // few tokens: the K-split kernel where 64-row workgroups would not fill half the chip
    const bool split = !side && gemm_splits_k(a, chunks, max_count);
    if (split) {
        const dim3 sgrid((a.n + 15) / 16, chunks);
#define QMOE_SPLIT_F(F)                                              \
    if (pair) gemm_split_f<F, true>(a, a_kind, sgrid, s);            \
    else gemm_split_f<F, false>(a, a_kind, sgrid, s)
        switch (fmt) {
        case QMOE_FMT_Q8_0: QMOE_SPLIT_F(QMOE_FMT_Q8_0); break;
        case QMOE_FMT_Q6_K: QMOE_SPLIT_F(QMOE_FMT_Q6_K); break;
        case QMOE_FMT_Q5_K: QMOE_SPLIT_F(QMOE_FMT_Q5_K); break;
        case QMOE_FMT_Q4_K: QMOE_SPLIT_F(QMOE_FMT_Q4_K); break;
        default: QMOE_SPLIT_F(QMOE_FMT_BF16); break;
        }
#undef QMOE_SPLIT_F
        return check_launch("token-tile GEMM (K split)");
    }
    const int rows_per_wg = pair ? 64 : fmt == QMOE_FMT_Q8_0 ? 64 * GEMM_Q8_PLAIN_TILES : 128;
    const int rowblocks = (a.n + rows_per_wg - 1) / rows_per_wg;
    // the side problem's row blocks in parts of the main problem's grid width
    const int side_parts = side ? ((side->n + rows_per_wg - 1) / rows_per_wg + rowblocks - 1) / rowblocks : 0;
    const GemmArgs none{};
    const GemmArgs& sd = side ? *side : none;
    const int sc = side ? side_chunks : 0;
    const dim3 grid(rowblocks, chunks + sc * side_parts);
#define QMOE_GEMM_F(F)                                                          \
    if (pair) gemm_launch_f<F, true>(a, sd, sc, side_parts, a_kind, grid, s);   \
    else gemm_launch_f<F, false>(a, sd, sc, side_parts, a_kind, grid, s)
    switch (fmt) {
    case QMOE_FMT_Q8_0: QMOE_GEMM_F(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_GEMM_F(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_GEMM_F(QMOE_FMT_Q5_K); break;
    case QMOE_FMT_Q4_K: QMOE_GEMM_F(QMOE_FMT_Q4_K); break;
    default: QMOE_GEMM_F(QMOE_FMT_BF16); break;
    }
#undef QMOE_GEMM_F
    return check_launch("token-tile GEMM");
}

template <int FMT, int NM>
static void gemm_dense_f(const GemmDenseArgs& d, int a_kind, dim3 grid, hipStream_t s) {
    const dim3 block(GEMM_THREADS);
    switch (a_kind) {
    case GEMM_A_F32: hipLaunchKernelGGL((tile_gemm_dense_kernel<FMT, GEMM_A_F32, NM>), grid, block, 0, s, d); break;
    case GEMM_A_F16: hipLaunchKernelGGL((tile_gemm_dense_kernel<FMT, GEMM_A_F16, NM>), grid, block, 0, s, d); break;
    default: hipLaunchKernelGGL((tile_gemm_dense_kernel<FMT, GEMM_A_BF16, NM>), grid, block, 0, s, d); break;
    }
}

// Row blocks of 128 rows when that still fills the chip, else of 64.
int gemm_dense_launch(int fmt, int a_kind, GemmDenseArgs& d, hipStream_t s) {
    const int chunks = (d.tokens + GEMM_CHUNK - 1) / GEMM_CHUNK;
    int blocks128 = 0;
    for (int i = 0; i < d.count; ++i) blocks128 += (d.p[i].n + 127) / 128;
    // The formats whose workgroup keeps a weight tile in flight take two row tiles per wave already
    // where that fills half the chip: more bytes on their way per CU outweigh the idle places.
    const int enough = fmt != QMOE_FMT_BF16 ? stream_grid() / 2 : stream_grid();
    const int nm = blocks128 * chunks >= enough ? 2 : 1;
    // Rows of 8192 columns and more are shared by the four waves of a workgroup (K split, 16 rows
    // and 16 tokens a workgroup); so is every matrix of a launch that would not fill half the chip
    // with 64-row workgroups (a lone attention projection: 64 workgroups walking 16 passes each).
    int blocks64 = 0;
    for (int i = 0; i < d.count; ++i) blocks64 += (d.p[i].n + 63) / 64;
    const bool sparse = (int64_t)blocks64 * chunks < stream_grid() / 2;
    int at = 0, ychunks = chunks;
    for (int i = 0; i < d.count; ++i) {
        d.p[i].ksplit = d.p[i].k >= 8192 || (sparse && d.p[i].k >= 1024);
        const int rows_per_block = d.p[i].ksplit ? 16 * nm : 64 * nm;
        d.block_start[i] = at;
        at += (d.p[i].n + rows_per_block - 1) / rows_per_block;
        if (d.p[i].ksplit && (d.tokens + 15) / 16 > ychunks) ychunks = (d.tokens + 15) / 16;
    }
    d.block_start[d.count] = at;
    const dim3 grid(at, ychunks);
#define QMOE_DENSE_F(F)                                        \
    if (nm == 2) gemm_dense_f<F, 2>(d, a_kind, grid, s);      \
    else gemm_dense_f<F, 1>(d, a_kind, grid, s)
    switch (fmt) {
    case QMOE_FMT_Q8_0: QMOE_DENSE_F(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_DENSE_F(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_DENSE_F(QMOE_FMT_Q5_K); break;
    case QMOE_FMT_Q4_K: QMOE_DENSE_F(QMOE_FMT_Q4_K); break;
    default: QMOE_DENSE_F(QMOE_FMT_BF16); break;
    }
#undef QMOE_DENSE_F
    return check_launch("token-tile GEMM (dense)");
}

}  // namespace qmoe
