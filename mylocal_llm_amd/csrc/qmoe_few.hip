// Two to four tokens against Q8_0 matrices with rows of up to 4096 columns, streamed like the
// single-token kernel: the weights are read once, at HBM pace, and the products of all tokens
// come from v_mfma_f32_4x4x4 (sixteen independent 4x4x4 blocks a wave).
//
// Lane l = 4 b + j of a wave streams 64-column unit b (of the wave's 1024-column chunk) of row
// j of a group of four rows, and holds the activations of token j for the same unit as bf16
// hi / lo terms (16 significant bits).  For four columns at a time the instruction gives lane l
//     D[i] = sum_k A[lane 4 b + i][k] * B[lane l][k],   i = 0..3
// (operand layout measured on the part), i.e. with the lane's int8 codes as B (exact in bf16)
// and the activations as A, the partial products of row j with every token i.  The block scale
// multiplies the partial sum of its 32 columns, as the dequantised weights would give.  Wave w of
// a workgroup takes chunk w of every row (a lane's unit position never changes, so its
// activations stay in registers for a whole matrix); the partial sums of the 16 units and the
// up to four chunks meet in LDS every FEW_SLOTS row groups.
#include "qmoe_few.hpp"

#include "qmoe_mfma.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

static constexpr int FEW_NARROW_WGS = 2;   // workgroups a CU of the four-wave form (three measured slower)
static constexpr int FEW_SLOTS = 8;   // row groups between two meetings of the workgroup's partial sums

template <int CTRL>
__device__ __forceinline__ float dpp_row_add(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// WAVES waves a workgroup; wave w takes the 1024-column chunks w, w + WAVES, ... (CPW of them at
// most) of every row.  Four waves with one chunk each cover rows of up to 4096 columns at two
// workgroups a CU; eight waves with two chunks each, one workgroup a CU, rows of up to 16384.
template <int XDT, int WAVES, int CPW>
__global__ __launch_bounds__(64 * WAVES, (WAVES == 4 ? FEW_NARROW_WGS : 1)) void few_tokens_kernel(const FewArgs args) {
    using U = Unit64<QMOE_FMT_Q8_0>;
    // [slot][wave][unit row of 16 lanes][row j][token i]
    __shared__ float partial[FEW_SLOTS][WAVES][4][4][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 3, b = lane >> 2;
    const int tokens = args.tokens;
    const int total = args.group_start[args.count];
    uint32_t x_hi[CPW][32], x_lo[CPW][32];
    int held = -1;        // problem whose activations the registers hold (the next may read the same ones)
    const void* held_x = nullptr;
    int held_k = 0;
    int slot = 0;
    int first_group = 0;   // row group in slot 0; slot s holds first_group + s * gridDim.x
    uint32_t raw0[CPW][U::RAW], raw1[CPW][U::RAW];

    // Two cursors over the problem list, both uniform and both only ever moving forward: the one
    // the row requests follow and the one the arithmetic follows.  Their fields sit in registers;
    // the argument block is read again only when a cursor enters the next problem.
    struct Cursor {
        int pi, lo, hi, n, k;
        const uint8_t* w;
    };
    auto enter = [&](Cursor& c, int pi) {
        c.pi = pi;
        c.lo = args.group_start[pi];
        c.hi = args.group_start[pi + 1];
        c.n = args.p[pi].n;
        c.k = args.p[pi].k;
        c.w = args.p[pi].w;
    };
    auto advance = [&](Cursor& c, int g) {
        while (g >= c.hi && c.pi + 1 < args.count) enter(c, c.pi + 1);
    };
    Cursor fc, cc;
    enter(fc, 0);
    enter(cc, 0);
    // chunk c of this wave, or chunk 0 (read and ignored) where the row has no such chunk
    auto fetch = [&](int g, uint32_t (&r)[CPW][U::RAW]) {
        advance(fc, g);
        const int chunks = fc.k >> 10;
        const int row = 4 * (g - fc.lo) + j;
        const int64_t rr = row < fc.n ? row : fc.n - 1;
        const uint8_t* rp = fc.w + rr * ((int64_t)(fc.k >> 5) * 34);
#pragma unroll
        for (int c = 0; c < CPW; ++c) {
            const int chunk = wave + WAVES * c;
            U::load_w(rp, chunk < chunks ? 16 * chunk + b : b, r[c]);
        }
    };
    // the partial sums of the filled slots -> outputs of the problem the arithmetic is in; every
    // thread of the workgroup passes here
    auto flush = [&]() {
        __syncthreads();
        const int t = threadIdx.x;   // entry t: slot t / 16, row j2 = t % 4, token i2 = (t / 4) % 4
        const int s = t >> 4, j2 = t & 3, i2 = (t >> 2) & 3;
        if (s < slot && i2 < tokens) {
            float sum = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
                for (int r = 0; r < 4; ++r) sum += partial[s][wv][r][j2][i2];
            // slot s holds row group first_group + s * gridDim.x
            const int row = 4 * (first_group + s * (int)gridDim.x - cc.lo) + j2;
            if (row < cc.n) store_out(args.p[cc.pi].y, args.p[cc.pi].ydt, (size_t)i2 * cc.n + row, sum);
        }
        __syncthreads();
        slot = 0;
    };

    int g = blockIdx.x;
    if (g >= total) return;
    fetch(g, raw0);
    // one row group: `r` holds its rows, `rn` receives the next group's
    auto step = [&](uint32_t (&r)[CPW][U::RAW], uint32_t (&rn)[CPW][U::RAW]) -> bool {
        advance(cc, g);
        const int chunks = cc.k >> 10;
        const int next = g + gridDim.x;
        if (held != cc.pi && (args.p[cc.pi].x != held_x || cc.k != held_k)) {
            // token j's activations of this lane's units, as bf16 hi / lo pairs
            const void* x = args.p[cc.pi].x;
            const int tj = j < tokens ? j : 0;
#pragma unroll
            for (int c = 0; c < CPW; ++c) {
                const int chunk = wave + WAVES * c;
                const bool mine = chunk < chunks && j < tokens;
                const int u = chunk < chunks ? 16 * chunk + b : b;
                // every load is issued on every lane (a lane without a token or a chunk reads valid
                // memory and drops it): the sixteen requests leave together
                float4 v[16];
#pragma unroll
                for (int q = 0; q < 16; ++q) v[q] = Elem<XDT>::load4(x, (size_t)tj * cc.k + 64 * u + 4 * q);
#pragma unroll
                for (int q = 0; q < 16; q += 2) {
                    const float f[8] = {mine ? v[q].x : 0.f, mine ? v[q].y : 0.f, mine ? v[q].z : 0.f, mine ? v[q].w : 0.f,
                                        mine ? v[q + 1].x : 0.f, mine ? v[q + 1].y : 0.f, mine ? v[q + 1].z : 0.f, mine ? v[q + 1].w : 0.f};
                    OperandBits hi, lo;
                    split_terms(f, hi, lo);
#pragma unroll
                    for (int m = 0; m < 4; ++m) { x_hi[c][2 * q + m] = hi.u[m]; x_lo[c][2 * q + m] = lo.u[m]; }
                }
            }
            held_x = x;
            held_k = cc.k;
        }
        held = cc.pi;
        // The next group's rows are requested on every path (past the end: this group's again), so
        // that the wait for `r` below can leave exactly these loads in flight.
        fetch(next < total ? next : g, rn);
        if (slot == 0) first_group = g;
        // a unit: two blocks of 32 codes, eight steps of four columns each.  A chunk the row does
        // not have multiplies activations that were stored as zeros.
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < CPW; ++c) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float d = h == 0 ? half_bits_to_float(r[c][0] & 0xFFFFu) : half_bits_to_float(r[c][8] >> 16);
                float4v acc4 = {0.f, 0.f, 0.f, 0.f}, low4 = {0.f, 0.f, 0.f, 0.f};   // two chains: no MFMA waits for the one before it
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) {
                    // four codes from byte 2 + 34 h + 4 kk of the unit
                    const int at = 2 + 34 * h + 4 * kk;
                    const uint32_t q = (at & 3) ? __builtin_amdgcn_alignbit(r[c][(at >> 2) + 1], r[c][at >> 2], 16) : r[c][at >> 2];
                    const float f0 = (float)(int)(int8_t)(q & 0xFF), f1 = (float)(int)(int8_t)((q >> 8) & 0xFF);
                    const float f2 = (float)(int)(int8_t)((q >> 16) & 0xFF), f3 = (float)(int)(int8_t)(q >> 24);
                    union { uint32_t u[2]; short4v v; } wb, ah, al;
                    wb.u[0] = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
                    wb.u[1] = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
                    ah.u[0] = x_hi[c][16 * h + 2 * kk]; ah.u[1] = x_hi[c][16 * h + 2 * kk + 1];
                    al.u[0] = x_lo[c][16 * h + 2 * kk]; al.u[1] = x_lo[c][16 * h + 2 * kk + 1];
                    acc4 = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(ah.v, wb.v, acc4, 0, 0, 0);
                    if (XDT != QMOE_DT_BF16) low4 = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(al.v, wb.v, low4, 0, 0, 0);   // bf16 input has no low term
                }
                // a scale read from a chunk the row does not have may be anything: its sum is zero
                // unless the scale is not finite, so such a chunk is left out
                if (wave + WAVES * c < chunks) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[i] = fmaf(d, XDT != QMOE_DT_BF16 ? acc4[i] + low4[i] : acc4[i], acc[i]);
                }
            }
        }
        // units of the same row inside a row of 16 lanes: lanes j, j + 4, j + 8, j + 12
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = acc[i];
            v = dpp_row_add<0x124>(v);   // row_ror:4
            v = dpp_row_add<0x128>(v);   // row_ror:8
            if ((lane & 15) < 4) partial[slot][wave][lane >> 4][j][i] = v;
        }
        ++slot;
        g = next;
        const bool last = g >= total;
        if (slot == FEW_SLOTS || last || g >= cc.hi) flush();
        return last;
    };
    while (true) {
        if (step(raw0, raw1)) break;
        if (step(raw1, raw0)) break;
    }
}

static bool few_common(int fmt, const void* w, int n, int k, const void* x, int xdt, int tokens) {
    if (fmt != QMOE_FMT_Q8_0 || tokens < 2 || tokens > 4 || n < 1) return false;
    if (k < 1024 || k % 1024) return false;
    if ((uintptr_t)w % 4) return false;
    const int esize = xdt == QMOE_DT_F32 ? 4 : 2;
    return (uintptr_t)x % 16 == 0 && ((int64_t)k * esize) % 16 == 0;
}

bool few_supported(int fmt, const void* w, int n, int k, const void* x, int xdt, int tokens) {
    return few_common(fmt, w, n, k, x, xdt, tokens) && k <= 16384;
}

bool few_is_wide(int k) { return k > 4096; }

// All problems of a launch are wide (rows of more than 4096 columns) or none is.
int few_launch(FewArgs& a, hipStream_t s) {
    int at = 0;
    for (int i = 0; i < a.count; ++i) {
        a.group_start[i] = at;
        at += (a.p[i].n + 3) / 4;
    }
    a.group_start[a.count] = at;
    const bool wide = few_is_wide(a.p[0].k);
    const int slots = wide ? stream_grid() / 2 : stream_grid() / 2 * FEW_NARROW_WGS;   // workgroups the chip holds at once
    const dim3 g(slots < at ? slots : at), b(wide ? 512 : 256);
#define QMOE_FEW(XDT)                                                                      \
    if (wide) hipLaunchKernelGGL((few_tokens_kernel<XDT, 8, 2>), g, b, 0, s, a);          \
    else hipLaunchKernelGGL((few_tokens_kernel<XDT, 4, 1>), g, b, 0, s, a)
    if (a.xdt == QMOE_DT_F32) { QMOE_FEW(QMOE_DT_F32); }
    else if (a.xdt == QMOE_DT_F16) { QMOE_FEW(QMOE_DT_F16); }
    else { QMOE_FEW(QMOE_DT_BF16); }
#undef QMOE_FEW
    return check_launch("few-token streaming kernel");
}

}  // namespace qmoe
