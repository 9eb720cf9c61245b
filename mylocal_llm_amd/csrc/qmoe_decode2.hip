// Packed-expert MoE decode step, rows through LDS by LDS-DMA: the two launches of a step of a few
// tokens, written for the case where a launch is a handful of microseconds long and every phase of
// it is a memory round trip.  Both kernels run one workgroup of eight waves per CU and fetch
// weight rows with global_load_lds_dwordx4 (consecutive lanes, consecutive 16 bytes, straight into
// LDS: no register holds a byte in flight, every cache line is requested once), so a wave can put
// everything it will need in flight the moment it knows the addresses.
//
//   pairs2_kernel   routing + gate/up, up to four tokens.  The first T waves of every workgroup
//                   route a token each; the other waves meanwhile stage the tokens' activations
//                   and request and multiply rows of the shared expert, which need no routing.
//                   After the workgroup's one barrier all waves walk the item stream (shared
//                   expert rows first, then token by token the selected experts) through a ring
//                   of LDS slots.  A slot holds the gate rows of an item in its first half and the
//                   up rows in its second, so one pass of a wave over a slot yields silu(g) * u.
//   down2_kernel    down projection, ordered combine, shared expert, residual: up to sixteen
//                   tokens.  A wave owns one or two output rows for ALL tokens: the shared
//                   expert's row is fetched once, the selected experts' rows token after token
//                   into a two-deep ring, and the token's SwiGLU activations are staged once per
//                   workgroup by DMA.  Lanes are laid out [expert slot][row part] plus a group for
//                   the shared expert; the wave adds the products in ascending expert id (product
//                   rounded, then added) and finally shared * sigmoid.
//
// The kernels' waits are counted by hand (s_waitcnt vmcnt with the number of newer requests), so
// while requests are in flight every fetch is a DMA into LDS: a load into registers that the
// compiler can see makes it wait for everything outstanding, and one it cannot see (inline
// assembly) is unsafe as soon as its result is copied or merged at a branch before the data has
// arrived.  Stores only make the counted waits conservative.
#include "qmoe_decode.hpp"
#include "qmoe_rowdot.hpp"
#include "qmoe_span.hpp"

namespace qmoe {

static constexpr int D2_WAVES = 8;
static constexpr int D2_THREADS = D2_WAVES * 64;
static constexpr int D2_LDS = 160 * 1024;

// Per-wave time stamps of the two kernels' phases, for builds with -DQMOE_TIMELINE only (the
// measurement build of `python -m mylocal_llm_amd._build --timeline`; bench.py --only moe_timeline
// reads them): stamp i of wave w of kernel k is the 100 MHz device counter when the wave got there.
#ifdef QMOE_TIMELINE
static constexpr int TL_WAVES = 4096, TL_STAMPS = 8;
static __device__ unsigned long long timeline[2][TL_WAVES][TL_STAMPS];
#define QMOE_STAMP(kernel, index)                                                                          \
    do {                                                                                                   \
        const int w_ = blockIdx.x * D2_WAVES + (threadIdx.x >> 6);                                         \
        if ((threadIdx.x & 63) == 0 && w_ < TL_WAVES) timeline[kernel][w_][index] = wall_clock64();        \
    } while (0)
#else
#define QMOE_STAMP(kernel, index) ((void)0)
#endif

// 16 bytes per lane from a per-lane 64-bit address into LDS at m0 + 16 lane.
__device__ __forceinline__ void dma16_at(const uint8_t* lane_address) {
    asm volatile("global_load_lds_dwordx4 %0, off" ::"v"(lane_address) : "memory");
}
// 4 bytes per lane into LDS at m0 + 4 lane
__device__ __forceinline__ void dma4_at(const void* lane_address) {
    asm volatile("global_load_lds_dword %0, off" ::"v"(lane_address) : "memory");
}
__device__ __forceinline__ void dma4_at_masked(const void* lane_address, uint64_t mask) {
    uint64_t save;
    mask = ((uint64_t)(uint32_t)uniform((int)(mask >> 32)) << 32) | (uint32_t)uniform((int)(uint32_t)mask);
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %2\n\tglobal_load_lds_dword %1, off\n\ts_mov_b64 exec, %0"
                 : "=&s"(save) : "v"(lane_address), "s"(mask) : "memory");
}
// ... on the lanes of `mask` only (a wave-uniform 64-bit lane mask, not zero)
__device__ __forceinline__ void dma16_at_masked(const uint8_t* lane_address, uint64_t mask) {
    uint64_t save;
    mask = ((uint64_t)(uint32_t)uniform((int)(mask >> 32)) << 32) | (uint32_t)uniform((int)(uint32_t)mask);
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %2\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b64 exec, %0"
                 : "=&s"(save) : "v"(lane_address), "s"(mask) : "memory");
}
// s_waitcnt vmcnt(n) for a wave-uniform n known only at run time (the count is an immediate).
__device__ __forceinline__ void wait_vmcnt_rt(int n) {
    switch (n) {
#define QMOE_W(N) case N: wait_vmcnt<N>(); break;
        QMOE_W(1) QMOE_W(2) QMOE_W(3) QMOE_W(4) QMOE_W(5) QMOE_W(6) QMOE_W(7) QMOE_W(8) QMOE_W(9) QMOE_W(10)
        QMOE_W(11) QMOE_W(12) QMOE_W(13) QMOE_W(14) QMOE_W(15) QMOE_W(16) QMOE_W(17) QMOE_W(18) QMOE_W(19) QMOE_W(20)
        QMOE_W(21) QMOE_W(22) QMOE_W(23) QMOE_W(24) QMOE_W(25) QMOE_W(26) QMOE_W(27) QMOE_W(28) QMOE_W(29) QMOE_W(30)
#undef QMOE_W
    default: wait_vmcnt<0>(); break;
    }
}

__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = (uint32_t)uniform((int)(uint32_t)v), hi = (uint32_t)uniform((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Sum over groups of `lpe` consecutive lanes (1, 2, 4, 8 or 16), the total in every lane of a group.
__device__ __forceinline__ float part_sum_rt(float v, int lpe) {
    if (lpe >= 2) v = dpp_add<0xB1>(v);
    if (lpe >= 4) v = dpp_add<0x4E>(v);
    if (lpe >= 8) v = dpp_add<0x141>(v);
    if (lpe >= 16) v = dpp_add<0x140>(v);
    return v;
}

// ================================================================================================
// down projection
// ================================================================================================
static constexpr int DOWN2_MAX_TOKENS = 16;
static constexpr int DOWN2_CI = 8, DOWN2_CH = 4;   // most DMA instructions per row image / per wave for the activations

struct Down2Args {
    const uint8_t* down;         // bank base, [E, D, F]
    int64_t down_stride;
    const uint8_t* shared_down;  // [D, Fsh] or null
    const float* h;              // [T*k, F] in sorted-slot order
    const float* hs;             // [T, Fsh]
    const int* sorted_ids;       // [T, k]
    const float* sorted_w;       // [T, k]
    const float* sig;            // [T]
    void* out;                   // [T, D]
    const float* residual;       // [T, D] or null
    int odt, k, d, f, fsh;
    int rows;                    // output rows per wave
    int lpe;                     // lanes per expert row: f / 128
    int ppr, pps;                // 16-byte pieces of the LDS image of one routed row / of the shared row
    uint32_t ppr_magic;          // floor(2^32 / ppr) + 1: p / ppr by mulhi, exact for the few hundred pieces of an image
    int ci, ch;                  // DMA instructions per row image, per wave for the activations
    int image;                   // LDS bytes of a row image: the k routed rows, then the shared row
    int hbytes;                  // LDS bytes of the staged activations, whole KB
};

// One workgroup = one token x 8 waves x `rows` output rows.  A row's image -- row r of each of the
// token's k experts, then row r of the shared expert -- is one request (DMA instructions of 64
// pieces, the last one on the lanes that are left); a wave keeps two images in flight: as soon as
// an image's bytes are in registers its slot is requested into again, so two rows are on their way
// while one is multiplied.
// LDS: [staged activations | per wave: expert ids | dump | per wave: two row images]
template <int FMT>
__global__ __launch_bounds__(D2_THREADS, 1) void down2_kernel(const Down2Args a, const ListedExperts listed) {
    using U = Unit64<FMT>;
    using S = SpanFmt<FMT>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = uniform((int)(threadIdx.x >> 6));
    const int k = a.k, R = a.rows, t = blockIdx.y;
    uint8_t* const hbuf = lds;
    int* const tab_ids = (int*)(lds + a.hbytes + wave * 256);   // this wave's copy of the token's routing: 16 ids, 16 weights, the gate
    uint8_t* const dump = lds + a.hbytes + D2_WAVES * 256;
    uint8_t* const ring = dump + 1024 + wave * (2 * a.image);
    const int row0 = (blockIdx.x * D2_WAVES + wave) * R;   // first output row of this wave
    const int64_t rb_r = row_bytes_dev(FMT, a.f), rb_s = row_bytes_dev(FMT, a.fsh);
    auto clamp_row = [&](int i) { return row0 + i < a.d ? row0 + i : a.d - 1; };
    QMOE_STAMP(1, 0);

    // ---- 1. the token's routing, by DMA into this wave's table (no register waits for a load) ------
    // one request: lanes 0..15 fetch the expert ids (entries past k repeat entry k - 1), lanes
    // 16..31 the weights, the rest the sigmoid gate
    {
        const int kk = (lane & 15) < k ? (lane & 15) : k - 1;
        const void* const from = lane < 16 ? (const void*)(a.sorted_ids + t * k + kk)
                               : lane < 32 ? (const void*)(a.sorted_w + t * k + kk) : (const void*)(a.sig + t);
        set_m0((uint32_t)(uintptr_t)tab_ids);
        dma4_at(from);
    }

    // ---- 2. the token's activations: [h of its k slots | hs], swizzled while they travel --------
    // LDS granule P = 64 chunk + lane receives source granule swizzled(P); a wave brings chunks
    // wave, wave + 8, ...; chunks past the end fetch into the dump.
    const int nr = k * a.f, n_gran = (nr + (a.shared_down ? a.fsh : 0)) >> 2;
    {
        const uint8_t* const hr = (const uint8_t*)(a.h + (size_t)t * nr);
        const uint8_t* const hsr = (const uint8_t*)(a.hs + (size_t)t * a.fsh);
#pragma unroll
        for (int i = 0; i < DOWN2_CH; ++i)
            if (i < a.ch) {
                const int chunk = wave + D2_WAVES * i;
                const int P = 64 * chunk + lane;
                const int g = swizzled_granule(P);
                const bool valid = P < n_gran, from_hs = valid && 4 * g >= nr;
                const uint32_t off = valid ? (uint32_t)(from_hs ? 4 * g - nr : 4 * g) * 4u : 0u;
                set_m0((uint32_t)(uintptr_t)(64 * chunk < n_gran ? hbuf + 1024 * chunk : dump));
                dma16_at(from_hs ? hsr + off : hr + off);
            }
    }

    // ---- 3. where piece p = lane + 64 c of a row image comes from ---------------------------------
    // p < k ppr: piece p % ppr of expert slot p / ppr; then the pieces of the shared row.  What does
    // not depend on the routing is worked out while the routing travels: row 0's address without
    // the expert's offset, and the bytes between consecutive rows.
    const uint8_t* src[DOWN2_CI];
    uint32_t stride[DOWN2_CI];
    uint32_t slot_of = 0;   // 4 bits per instruction: the expert slot of a routed piece
    uint32_t is_routed = 0;
    const int routed_pieces = k * a.ppr, pieces = routed_pieces + a.pps;
#pragma unroll
    for (int c = 0; c < DOWN2_CI; ++c) {
        const int p = lane + 64 * c;
        src[c] = a.down;
        stride[c] = 0u;
        if (p < routed_pieces) {
            const int j = (int)__umulhi((uint32_t)p, a.ppr_magic), q = p - j * a.ppr;
            src[c] = a.down + S::src(q);
            stride[c] = (uint32_t)rb_r;
            slot_of |= (uint32_t)j << (4 * c);
            is_routed |= 1u << c;
        } else if (p < pieces) {
            src[c] = a.shared_down + S::src(p - routed_pieces);
            stride[c] = (uint32_t)rb_s;
        }
    }
    const int last_lanes = pieces - 64 * (a.ci - 1);   // lanes of the last instruction, 1..64
    const uint64_t last_mask = last_lanes >= 64 ? ~0ull : ((1ull << last_lanes) - 1);
    wait_vmcnt_rt(a.ch);
    QMOE_STAMP(1, 6);
    const float route_w = lane < k ? __int_as_float(tab_ids[16 + lane]) : 0.f;   // lane j holds weight j
    const float sg = __int_as_float(tab_ids[32]);
#pragma unroll
    for (int c = 0; c < DOWN2_CI; ++c)
        if ((is_routed >> c) & 1u) {
            const int e = tab_ids[(slot_of >> (4 * c)) & 15u];
            if (listed.count) src[c] = listed.down[e >= 0 && e < listed.count ? e : 0] + (src[c] - a.down);   // ("ids" are list positions)
            else src[c] += (int64_t)(e >= 0 ? e : 0) * a.down_stride;
        }
    // With a residual, its value of the row travels with the row, behind the image (an ordinary
    // load here would make the compiler wait for everything in flight).
    const float* const res_row = a.residual ? a.residual + (size_t)t * a.d : nullptr;
    auto request = [&](int i) {   // row i of this wave into slot i & 1
        const uint32_t row = (uint32_t)clamp_row(i);
        uint8_t* const img = ring + (i & 1) * a.image;
#pragma unroll
        for (int c = 0; c < DOWN2_CI; ++c)
            if (c < a.ci) {
                const uint8_t* const from = src[c] + (uint64_t)row * stride[c];
                set_m0((uint32_t)(uintptr_t)(img + 1024 * c));
                if (c + 1 < a.ci) dma16_at(from);
                else dma16_at_masked(from, last_mask);
            }
        if (res_row) {
            set_m0((uint32_t)(uintptr_t)(img + pieces * 16));
            dma4_at_masked(res_row + row, 1ull);
        }
    };
    const int per_request = a.ci + (res_row ? 1 : 0);
    QMOE_STAMP(1, 7);
    request(0);
    if (R > 1) request(1);
    QMOE_STAMP(1, 1);

    // ---- lane layout of the multiplication -------------------------------------------------------
    const int lpe = a.lpe;
    const int shared_parts = a.shared_down ? a.fsh >> 7 : 0;
    const bool routed = lane < k * lpe;
    const bool shared = lane >= 48 && lane - 48 < shared_parts;
    const int slot = routed ? lane / lpe : 0;
    const int part = routed ? lane % lpe : (shared ? lane - 48 : 0);
    const int ux = shared ? (nr >> 6) + 2 * part : slot * (a.f >> 6) + 2 * part;
    const uint32_t row_at = shared ? routed_pieces * 16 : slot * a.ppr * 16;
    const uint32_t unit_at0 = row_at + S::unit_offset(2 * part), unit_at1 = row_at + S::unit_offset(2 * part + 1);
    const bool live = (routed && tab_ids[slot] >= 0) || shared;

    // the activations have arrived (this wave's share; the barrier covers the others')
    wait_vmcnt_rt((R > 1 ? 2 : 1) * per_request);
    QMOE_STAMP(1, 2);
    __syncthreads();
    QMOE_STAMP(1, 3);
    float x0[64], x1[64], aux0[U::AUX], aux1[U::AUX];
    U::load_x(SwizzledX{hbuf}, ux, x0, aux0);
    U::load_x(SwizzledX{hbuf}, ux + 1, x1, aux1);

    for (int i = 0; i < R; ++i) {
        if (i + 1 < R) wait_vmcnt_rt(per_request);
        else wait_vmcnt<0>();
        if (i == 0) QMOE_STAMP(1, 4);
        const uint8_t* const img = ring + (i & 1) * a.image;
        uint32_t r0[U::RAW], r1[U::RAW];
        S::read(img + unit_at0, 2 * part, r0);
        S::read(img + unit_at1, 2 * part + 1, r1);
        const float before = res_row ? *(const float*)(img + pieces * 16) : 0.f;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the image is in registers: its slot is free
        if (i + 2 < R) request(i + 2);
        float v = U::dot(r0, x0, aux0) + U::dot(r1, x1, aux1);
        if (!live) v = 0.f;   // idle lanes decoded whatever lies at the start of the image
        const float ys = group_sum<16>(v);      // lanes 48..63 are one DPP row: the shared expert's total
        const float yr = part_sum_rt(v, lpe);   // every slot's total in each of its lanes
        float acc = 0.f;
        for (int j = 0; j < k; ++j) {
            const float yj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(yr), j * lpe));
            const float wj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(route_w), j));
            acc = add_product(acc, yj, wj);
        }
        if (a.shared_down) {
            const float y63 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ys), 63));
            acc = add_product(acc, y63, sg);
        }
        const int row = row0 + i;
        if (lane == 0 && row < a.d) {
            if (a.residual) acc = before + acc;
            store_out(a.out, a.odt, (size_t)t * a.d + row, acc);
        }
    }
    QMOE_STAMP(1, 5);
}

// ================================================================================================
// routing + gate/up
// ================================================================================================
static constexpr int PAIRS2_MAX_TOKENS = 4;         // tokens a workgroup routes and holds activations of
static constexpr int PAIRS2_MAX_STEP_TOKENS = 16;   // tokens of a launch: groups of up to four
static constexpr int PAIRS2_MAX_EXPERTS = 1024;   // a router row of 4 KB fits the ring slots it is staged in
static constexpr int PAIRS2_MAX_K = 16;
static constexpr int PAIRS2_PD = 2;               // slots requested ahead of the one being multiplied

struct Pairs2Shape {
    int lr;            // lanes per row (8, 16 or 32)
    int ri;            // rows of an item: 32 / lr (a slot holds ri gate rows, then the same ri up rows)
    int row_image;     // LDS bytes of one row's image
    int pph;           // 16-byte pieces of half a slot: ri rows
    int ipe, ish;      // items per expert pair (f / ri), of the shared pair (fsh / ri)
    int total;         // ish + tokens * k * ipe
    uint32_t ipe_magic, k_magic;   // floor(2^32 / d) + 1: exact quotients by mulhi for the sizes taken here
    int xs_bytes;      // LDS bytes of the staged activations (tokens of a group * d * 4)
    int groups;        // token groups of the launch: ceil(tokens / 4)
    int group_tokens;  // tokens per group (the last group may have fewer)
    int nv;            // router values per lane: 8 (up to 512 experts) or 16
};

// What the two waves that route a token leave in LDS: the row's maximum and softmax denominator.
struct RouteShare {
    float m, denom;
};

// A router row in LDS (value i at byte 4 i), NV values per lane (value j of a lane is expert
// lane + 64 j).  Keys: order_key with every NaN raised to 1 (below -inf, above 0 = "taken or
// absent"); a round is one DPP maximum of the lanes' best keys; ties go to the lower id.
template <int NV>
__device__ __forceinline__ void row_select(const uint8_t* row, int n, int k, uint32_t& my_key, int& my_id) {
    const int lane = threadIdx.x & 63;
    uint32_t key[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const uint32_t ok = order_key(*(const float*)(row + 256 * j + 4 * lane));
        key[j] = lane + 64 * j < n ? (ok ? ok : 1u) : 0u;
    }
    for (int slot = 0; slot < k; ++slot) {
        uint32_t c = 0u;
#pragma unroll
        for (int j = 0; j < NV; ++j) c = key[j] > c ? key[j] : c;
        const uint32_t win = wave_max_u32(c);
        int wj = -1;   // owner: first j with a holder, then the lowest lane holding it there
        unsigned long long holders = 0ull;
#pragma unroll
        for (int j = NV - 1; j >= 0; --j) {
            const unsigned long long b = __ballot(key[j] == win);
            if (b) { wj = j; holders = b; }
        }
        const int wl = __builtin_ctzll(holders);
#pragma unroll
        for (int j = 0; j < NV; ++j)
            if (j == wj) key[j] = lane == wl ? 0u : key[j];
        if (lane == slot) { my_key = win; my_id = wl + 64 * wj; }
    }
}
// The row's maximum (NaN if the row holds one, as the portable graph computes it) and the softmax
// denominator sum exp(v - max), accumulated in double.
template <int NV>
__device__ __forceinline__ void row_softmax_sum(const uint8_t* row, int n, float& m, float& denom) {
    const int lane = threadIdx.x & 63;
    float v[NV];
    uint32_t best = 0u;
    bool nan_seen = false;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        v[j] = *(const float*)(row + 256 * j + 4 * lane);
        const bool valid = lane + 64 * j < n;
        const uint32_t ok = order_key(v[j]);
        const uint32_t key = valid ? (ok ? ok : 1u) : 0u;
        nan_seen |= valid && ok == 0u;
        best = key > best ? key : best;
    }
    m = __any(nan_seen) ? __uint_as_float(0x7FC00000u) : key_value(wave_max_u32(best));
    double part = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j)
        if (lane + 64 * j < n) part += (double)expf(v[j] - m);
    denom = (float)wave_sum_f64(part);
}

template <int FMT> struct Pairs2Slot {
    static constexpr int CH = SpanSlot<FMT>::CHUNKS;    // DMA instructions per slot
    static constexpr int BYTES = CH * 1024;             // (whole instructions: no lane mask)
};

// LDS: [activations fp32, swizzled | sorted ids per token | dump | rings: 8 waves x 3 slots]
template <int FMT>
__global__ __launch_bounds__(D2_THREADS, 1) void pairs2_kernel(const DecodeRouteArgs step, const Pairs2Shape shape, const ListedExperts listed) {
    using U = Unit64<FMT>;
    using S = SpanFmt<FMT>;
    using SL = Pairs2Slot<FMT>;
    constexpr int PD = PAIRS2_PD, NS = PD + 1, CH = SL::CH;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    QMOE_STAMP(0, 7);
    const int lane = threadIdx.x & 63, wave = uniform((int)(threadIdx.x >> 6));
    // More than four tokens are cut into groups of up to four; the workgroups are dealt out to the
    // groups in turn, and each group is a step of its own on its share of the chip: `a`, `x`, `wg` and
    // `wgs` below are that step (its tokens, its outputs, this workgroup's place in it).
    DecodeRouteArgs a = step;
    Pairs2Shape x = shape;
    const int wg_index = blockIdx.x / shape.groups, wgs = (gridDim.x - blockIdx.x % shape.groups + shape.groups - 1) / shape.groups;
    {
        const int q = blockIdx.x % shape.groups, token0 = q * shape.group_tokens;
        const int mine = step.tokens - token0 < shape.group_tokens ? step.tokens - token0 : shape.group_tokens;
        a.tokens = mine;
        a.hidden = (const uint8_t*)step.hidden + (size_t)token0 * step.d * (step.xdt == QMOE_DT_F32 ? 4 : 2);
        if (step.logits) a.logits = step.logits + (size_t)token0 * step.n_experts;
        if (step.in_ids) a.in_ids = step.in_ids + (size_t)token0 * step.k;
        if (step.in_weights) a.in_weights = step.in_weights + (size_t)token0 * step.k;
        if (step.out_weights) a.out_weights = step.out_weights + (size_t)token0 * step.k;
        if (step.out_ids) a.out_ids = step.out_ids + (size_t)token0 * step.k;
        a.sorted_ids = step.sorted_ids + (size_t)token0 * step.k;
        a.sorted_w = step.sorted_w + (size_t)token0 * step.k;
        a.sig = step.sig + token0;
        a.h = step.h + (size_t)token0 * step.k * step.f;
        a.hs = step.hs + (size_t)token0 * step.fsh;
        x.total = x.ish + mine * step.k * x.ipe;
    }
    const int T = a.tokens, k = a.k;
    uint8_t* const xs = lds;
    int64_t* const sid = (int64_t*)(lds + x.xs_bytes);                  // [PAIRS2_MAX_TOKENS][32]
    uint8_t* const dump = (uint8_t*)(sid + PAIRS2_MAX_TOKENS * 32) + PAIRS2_MAX_TOKENS * sizeof(RouteShare);
    uint8_t* const ring = dump + 1024 + wave * (NS * SL::BYTES);
    const int64_t rb = row_bytes_dev(FMT, a.d);
    const int lr = x.lr, units = a.d >> 6;
    const int u = lane & (lr - 1), sub = lane / lr;
    const bool active = u < units;
    const uint32_t lane_off = sub * x.row_image + S::unit_offset(active ? u : 0);

    // where piece p = lane + 64 c of a slot comes from: half (gate / up rows) and offset inside it
    uint32_t p_off[CH];
    uint32_t p_up = 0;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int p = lane + 64 * c;
        const bool up = p >= x.pph, valid = p < 2 * x.pph;
        p_off[c] = valid ? (uint32_t)S::src(up ? p - x.pph : p) : 0u;
        p_up |= (up && valid ? 1u : 0u) << c;
    }

    struct Item {
        const uint8_t *g, *u;   // first gate / up row of the item
        float* y;               // where row r0 of the result goes (token 0 of a shared item)
        int t;                  // token, -1 for the shared expert (all tokens)
        int r0;
        bool live;
    };
    auto decode = [&](int g) {
        Item it;
        it.g = it.u = a.gate;
        it.y = nullptr;
        it.t = 0;
        it.r0 = 0;
        it.live = false;
        if (g < x.ish) {
            it.r0 = g * x.ri;
            it.g = a.shared_gate_w + (int64_t)it.r0 * rb;
            it.u = a.shared_up_w + (int64_t)it.r0 * rb;
            it.y = a.hs + it.r0;
            it.t = -1;
            it.live = true;
        } else if (g < x.total) {
            const uint32_t q = (uint32_t)(g - x.ish);
            const uint32_t tj = __umulhi(q, x.ipe_magic);
            const uint32_t t = k == 1 ? tj : __umulhi(tj, x.k_magic);
            it.r0 = (int)(q - tj * (uint32_t)x.ipe) * x.ri;
            it.t = (int)t;
            const int64_t e = uniform64(sid[t * 32 + (tj - t * (uint32_t)k)]);
            if (e >= 0 && listed.count) {   // (listed experts: the "id" is the list position)
                it.g = listed.gate[e] + (int64_t)it.r0 * rb;
                it.u = listed.up[e] + (int64_t)it.r0 * rb;
                it.y = a.h + (size_t)tj * a.f + it.r0;
                it.live = true;
            } else if (e >= 0) {
                it.g = a.gate + e * a.gate_stride + (int64_t)it.r0 * rb;
                it.u = a.up + e * a.up_stride + (int64_t)it.r0 * rb;
                it.y = a.h + (size_t)tj * a.f + it.r0;
                it.live = true;
            }
        }
        it.g = uniform(it.g);
        it.u = uniform(it.u);
        return it;
    };
    auto request = [&](int slot, const Item& it) {
        uint8_t* const at = ring + slot * SL::BYTES;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            set_m0((uint32_t)(uintptr_t)(at + 1024 * c));
            // (an item past the end fetches one line, sixty-four times the same 16 bytes)
            dma16_at(it.live ? (((p_up >> c) & 1u) ? it.u + p_off[c] : it.g + p_off[c]) : it.g);
        }
    };
    float xr[64], aux[8];
    int held = -1;   // the token whose slice of the activations is in xr
    auto multiply = [&](int slot, const Item& it) {
        uint32_t r[U::RAW];
        S::read(ring + slot * SL::BYTES + lane_off, u, r);
        const int t0 = it.t < 0 ? 0 : it.t, t1 = it.t < 0 ? T : it.t + 1;
        for (int t = t0; t < t1; ++t) {
            if (held != t) {
                U::load_x(SwizzledX{xs + (size_t)t * a.d * 4}, active ? u : 0, xr, aux);
                held = t;
            }
            float v = U::dot(r, xr, aux);
            v = group_sum_rt(active ? v : 0.f, lr);           // (a lane without a unit has read bytes of another one)
            const float partner = __shfl_xor(v, 32, 64);      // the up row's total, for the lanes of the gate row
            if (lane < 32 && u == lr - 1) {
                float* const y = it.t < 0 ? it.y + (size_t)t * a.fsh : it.y;
                stg<float>(y + sub, silu_mul(v, partner));
            }
        }
    };

    // ---- routing, activations, and a first row pair of the shared expert ---------------------------
    // Two waves route a token, side by side: wave 2 t picks the k best of the row (ten serial rounds
    // of a wave-wide maximum: the long pole), wave 2 t + 1 meanwhile finds the row's maximum and the
    // softmax denominator.  All waves stage the tokens' activations and request a first row pair
    // of the shared expert, which needs no routing.  Everything fetched here travels by DMA into
    // LDS (router rows and 16-bit activations into the wave's own ring slots, which are free until
    // the barrier; fp32 activations straight to their place): no register waits for a load, and the
    // row pair on its way is waited for by nothing.
    QMOE_STAMP(0, 0);
    const int n = a.n_experts;
    const int token = wave >> 1;                     // the token this wave helps to route, if < T
    const bool routes = token < T, selects = routes && !(wave & 1);
    const bool from_logits = a.logits != nullptr;
    RouteShare* const share = (RouteShare*)(sid + PAIRS2_MAX_TOKENS * 32) + token;
    // The waves that publish the routing (the selecting waves of workgroup 0) take no items: they
    // have the admission gate to compute, with ordinary loads, which must not meet requests in
    // flight.  All other waves share the item stream.
    const bool publishes = wg_index == 0 && selects;
    // (a) the routing given by the caller (ordinary loads, waited for before anything else is issued)
    float weight = 0.f;
    int64_t id = 0;
    if (selects && !from_logits) {
        const int kk = lane < k ? lane : k - 1;
        if (listed.count) {   // listed experts: position kk of the list, its weight from the caller's routes
            id = kk;
            weight = listed.routes[(int64_t)listed.slot[kk] * listed.route_stride];
        } else {
            id = a.in_ids[(size_t)token * k + kk];
            weight = a.in_weights[(size_t)token * k + kk];
        }
        asm volatile("" ::"v"((uint32_t)id), "v"((uint32_t)((uint64_t)id >> 32)), "v"(weight) : "memory");
    }
    // ... or the router row, into the second slot of this wave's ring (and on into the third)
    uint8_t* const lds_logits = ring + SL::BYTES;              // value i at byte 4 i, up to 4 KB
    uint8_t* const lds_xraw = ring + NS * SL::BYTES - 2048;    // this wave's 16-bit chunks, 512 bytes each
    int n_loads = 0;
    if (routes && from_logits) {
        const float* const row = a.logits + (size_t)token * n;
        for (int j = 0; j < x.nv; ++j) {
            const int at = lane + 64 * j;
            set_m0((uint32_t)(uintptr_t)(lds_logits + 256 * j));
            dma4_at(row + (at < n ? at : n - 1));
            ++n_loads;
        }
    }
    const int n_logit_loads = n_loads;
    // (b) this wave's share of the tokens' activations: 256-column chunks wave, wave + 8, ... of all tokens
    const int per_token = a.d >> 8, chunks = T * per_token;
    if (a.xdt == QMOE_DT_F32) {
        for (int c = wave; c < chunks; c += D2_WAVES) {
            const int t = c / per_token, cc = c - t * per_token;
            // LDS granule 64 cc + lane receives source granule swizzled(64 cc + lane)
            const float* const src = (const float*)a.hidden + (size_t)t * a.d + 4 * swizzled_granule(64 * cc + lane);
            set_m0((uint32_t)(uintptr_t)(xs + (size_t)t * a.d * 4 + 1024 * cc));
            dma16_at((const uint8_t*)src);
            ++n_loads;
        }
    } else {
        for (int q = 0; 2 * q * D2_WAVES + wave < chunks; ++q) {   // two chunks per instruction: lanes 0..31, 32..63
            const int c = wave + D2_WAVES * (2 * q + (lane >> 5));
            const uint16_t* const src = (const uint16_t*)a.hidden + 256 * (size_t)(c < chunks ? c : wave) + 8 * (lane & 31);
            set_m0((uint32_t)(uintptr_t)(lds_xraw + 1024 * q));
            dma16_at((const uint8_t*)src);
            ++n_loads;
        }
    }
    n_loads -= n_logit_loads;   // (requests newer than the router row)
    // (c) a row pair of the shared expert, if the wave's first item is one
    const int W = wgs * D2_WAVES - T;                             // waves of this group that take items
    const int before = (wave + 1) >> 1;                           // publishing waves of the group's first workgroup ahead of this one
    const int me = wg_index * D2_WAVES + wave - (wg_index == 0 ? (before < T ? before : T) : T);
    const int g0 = publishes ? x.total : me;                      // this wave's items are g0, g0 + W, ...
    const bool early = g0 < x.ish;   // the first item is a shared one, requested before the routing is known
    Item it[NS];
    if (early) {
        it[0] = decode(g0);
        request(0, it[0]);
        n_loads += CH;
    }
    // (d) the row's k best on one wave, its maximum and denominator on the other
    wait_vmcnt_rt(n_loads);
    uint32_t sel_key = 0u;
    int sel_id = 0;
    if (routes && from_logits) {
        if (selects) {
            if (x.nv <= 8) row_select<8>(lds_logits, n, k, sel_key, sel_id);
            else row_select<16>(lds_logits, n, k, sel_key, sel_id);
        } else {
            float m, denom;
            if (x.nv <= 8) row_softmax_sum<8>(lds_logits, n, m, denom);
            else row_softmax_sum<16>(lds_logits, n, m, denom);
            if (lane == 0) {
                share->m = m;
                share->denom = denom;
            }
        }
    }
    // (e) activations into LDS as fp32 (they have long arrived; only the row pair may still travel)
    wait_vmcnt_rt(early ? CH : 0);
    if (a.xdt != QMOE_DT_F32) {
        for (int i = 0; wave + D2_WAVES * i < chunks; ++i) {
            const int c = wave + D2_WAVES * i;
            const uint2 w = *(const uint2*)(lds_xraw + 512 * i + 8 * lane);
            float4 f;
            if (a.xdt == QMOE_DT_BF16) {
                f = make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u),
                                __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xFFFF0000u));
            } else {
                f = make_float4(__half2float(__ushort_as_half((unsigned short)(w.x & 0xFFFFu))), __half2float(__ushort_as_half((unsigned short)(w.x >> 16))),
                                __half2float(__ushort_as_half((unsigned short)(w.y & 0xFFFFu))), __half2float(__ushort_as_half((unsigned short)(w.y >> 16))));
            }
            const int t = c / per_token, gran = 64 * (c - t * per_token) + lane;
            *(float4*)(xs + (size_t)t * a.d * 4 + 16 * swizzled_granule(gran)) = f;
        }
    }
    QMOE_STAMP(0, 1);
    __syncthreads();
    // (f) the selecting wave: probabilities, renormalisation, the selections sorted by expert id
    if (selects) {
        if (from_logits) {
            const float m = share->m, denom = share->denom;
            id = sel_id;
            // probabilities in parallel; their sum in selection order
            const float p = lane < k ? expf(key_value(sel_key) - m) / denom : 0.0f;
            float mass = 0.0f;
            for (int slot = 0; slot < k; ++slot) mass += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), slot));
            float norm = 1.0f;
            if (a.renorm) norm = isnan(mass) ? mass : fmaxf(mass, a.floor_value);
            weight = a.renorm ? p / norm : p;
        }
        // rank of a selection in ascending expert id; equal ids keep slot order.  An id outside the
        // bank, or an expert the token has named in an earlier slot already, contributes nothing.
        int rank = 0;
        bool again = false;
        for (int j = 0; j < k; ++j) {   // (listed experts: ids are 0 .. k - 1, rank = position, nothing repeats)
            const int64_t other = readlane_i64(id, j);
            rank += (other < id) || (other == id && j < lane);
            again |= other == id && j < lane;
        }
        if (lane < k) {
            const bool in_range = id >= 0 && id < n, ok = in_range && !again;
            sid[token * 32 + rank] = ok ? id : -1;
            if (publishes) {   // for the down kernel and the caller
                if (!ok && a.status_out) atomicOr(a.status_out, (in_range ? 0 : 1) | (again ? 2 : 0));
                if (a.out_weights) {
                    a.out_weights[(size_t)token * k + lane] = weight;
                    a.out_ids[(size_t)token * k + lane] = id;
                }
                a.sorted_ids[(size_t)token * k + rank] = ok ? (int)id : -1;
                a.sorted_w[(size_t)token * k + rank] = weight;
            }
        }
    }
    QMOE_STAMP(0, 3);
    __syncthreads();
    QMOE_STAMP(0, 4);
    // the sigmoid admission gate of the shared expert, by the publishing waves (which request nothing
    // and end here), from the staged rows
    if (publishes) {
        float adm = 0.f;
        if (a.shared_gate) {
            for (int c = lane; c < (a.d >> 2); c += 64) {
                const float4 h = *(const float4*)(xs + (size_t)token * a.d * 4 + 16 * swizzled_granule(c));
                const float4 gv = ldg<float4>(a.shared_gate + 4 * c);
                adm += (h.x * gv.x + h.y * gv.y) + (h.z * gv.z + h.w * gv.w);
            }
            adm = wave_sum(adm);
        }
        // sigmoid(hidden . g) without overflow
        if (lane == 0) a.sig[token] = a.shared_gate ? (adm >= 0.f ? 1.f / (1.f + expf(-adm)) : expf(adm) / (1.f + expf(adm))) : 1.f;
        return;
    }

    // ---- the item stream through the ring --------------------------------------------------------
    int g = g0;
    if (g >= x.total) return;   // (only where there are fewer items than waves: such a wave has requested nothing)
#pragma unroll
    for (int j = 0; j < PD; ++j)
        if (j > 0 || !early) {
            it[j] = decode(g + j * W);
            request(j, it[j]);
        }
    bool done = false;
    while (!done) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (!done) {
                const int nb = (s + PD) % NS;
                it[nb] = decode(g + PD * W);
                request(nb, it[nb]);
                wait_vmcnt<PD * CH>();
                if (g == g0) QMOE_STAMP(0, 5);
                if (it[s].live) multiply(s, it[s]);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot may be requested into again
                g += W;
                if (g >= x.total) done = true;
            }
        }
    }
    wait_vmcnt<0>();
    QMOE_STAMP(0, 6);
}

// ---- host side ---------------------------------------------------------------------------------
static bool span_format(int fmt) {
    return fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q4_K;
}
static int pieces_per_256(int fmt) {
    return fmt == QMOE_FMT_Q8_0 ? 17 : fmt == QMOE_FMT_Q6_K ? 14 : fmt == QMOE_FMT_Q5_K ? 11 : 9;
}
static int kb(int bytes) { return (bytes + 1023) & ~1023; }

static uint32_t magic_of(int d) { return (uint32_t)(0x100000000ull / (uint32_t)d) + 1u; }

// Fills `out` if the down step of this MoE step is one down2_kernel takes.
static bool down2_plan(const qmoe_moe_args& m, const DecodeBuffers& w, int cus, Down2Args* out) {
    const qmoe_expert_bank& b = m.bank;
    const bool has_shared = m.shared_down_w != nullptr;
    if (!span_format(b.down_fmt) || (has_shared && m.shared_down_fmt != b.down_fmt)) return false;
    if (m.tokens < 1 || m.tokens > DOWN2_MAX_TOKENS || m.tokens > cus || m.top_k > 16) return false;
    const int lpe = b.d_ff >> 7;
    if (b.d_ff % 256 || (lpe & (lpe - 1)) || lpe > 16 || m.top_k * lpe > 48) return false;
    if (has_shared && (m.d_ff_shared % 256 || (m.d_ff_shared >> 7) > 16)) return false;
    const int align = b.down_fmt == QMOE_FMT_Q6_K ? 2 : 16;
    if ((uintptr_t)b.down % align || b.down_stride % align || (has_shared && (uintptr_t)m.shared_down_w % align)) return false;
    if ((uintptr_t)w.h % 16 || (uintptr_t)w.hs % 16) return false;
    Down2Args a{};
    const int row_blocks = cus / m.tokens;   // workgroups per token
    a.rows = (b.d_model + row_blocks * D2_WAVES - 1) / (row_blocks * D2_WAVES);
    const int pp4 = pieces_per_256(b.down_fmt);
    a.ppr = (b.d_ff >> 8) * pp4;
    a.pps = has_shared ? (m.d_ff_shared >> 8) * pp4 : 0;
    a.ppr_magic = magic_of(a.ppr);
    if (m.residual && (uintptr_t)m.residual % 4) return false;
    const int pieces = m.top_k * a.ppr + a.pps;
    a.ci = (pieces + 63) / 64;
    a.image = pieces * 16 + 16;   // (+ the residual's value)
    const int floats = m.top_k * b.d_ff + (has_shared ? m.d_ff_shared : 0);
    const int chunks = (floats / 4 + 63) / 64;
    a.ch = (chunks + D2_WAVES - 1) / D2_WAVES;
    if (a.ci > DOWN2_CI || a.ch > DOWN2_CH) return false;
    a.hbytes = chunks * 1024;
    if (a.hbytes + D2_WAVES * 256 + 1024 + D2_WAVES * 2 * a.image > D2_LDS) return false;
    a.down = (const uint8_t*)b.down;
    a.down_stride = b.down_stride;
    a.shared_down = (const uint8_t*)m.shared_down_w;
    a.h = w.h;
    a.hs = w.hs;
    a.sorted_ids = w.sorted_ids;
    a.sorted_w = w.sorted_w;
    a.sig = w.sig;
    a.out = m.out;
    a.residual = m.residual;
    a.odt = m.out_dtype;
    a.k = m.top_k;
    a.d = b.d_model;
    a.f = b.d_ff;
    a.fsh = has_shared ? m.d_ff_shared : 0;
    a.lpe = lpe;
    if (out) *out = a;
    return true;
}

template <int FMT>
static int down2_launch_as(const Down2Args& a, int tokens, const ListedExperts& listed, hipStream_t s) {
    static bool configured = false;   // (benign if two threads both set it)
    if (!configured) {
        if (hipFuncSetAttribute((const void*)down2_kernel<FMT>, hipFuncAttributeMaxDynamicSharedMemorySize, D2_LDS) != hipSuccess)
            return fail(QMOE_ELAUNCH, "MoE decode (down): cannot reserve %d bytes of LDS", D2_LDS);
        configured = true;
    }
    const int per_wg = D2_WAVES * a.rows;
    hipLaunchKernelGGL(down2_kernel<FMT>, dim3((a.d + per_wg - 1) / per_wg, tokens), dim3(D2_THREADS), D2_LDS, s, a, listed);
    return check_launch("qmoe_moe_forward(down)");
}

bool decode2_down_supported(const qmoe_moe_args& m, const DecodeBuffers& w) { return down2_plan(m, w, stream_grid() / 2, nullptr); }

int decode2_down_launch(const qmoe_moe_args& m, const DecodeBuffers& w, hipStream_t s, const ListedExperts* listed) {
    ListedExperts l{};
    if (listed) l = *listed;
    Down2Args a;
    if (!down2_plan(m, w, stream_grid() / 2, &a)) return fail(QMOE_EUNSUPPORTED, "MoE decode (down): shape not taken");
    switch (m.bank.down_fmt) {
    case QMOE_FMT_Q8_0: return down2_launch_as<QMOE_FMT_Q8_0>(a, m.tokens, l, s);
    case QMOE_FMT_Q6_K: return down2_launch_as<QMOE_FMT_Q6_K>(a, m.tokens, l, s);
    case QMOE_FMT_Q5_K: return down2_launch_as<QMOE_FMT_Q5_K>(a, m.tokens, l, s);
    default: return down2_launch_as<QMOE_FMT_Q4_K>(a, m.tokens, l, s);
    }
}



static bool pairs2_plan(const qmoe_moe_args& m, int waves, Pairs2Shape* out) {
    const qmoe_expert_bank& b = m.bank;
    const bool has_shared = m.shared_gate_w != nullptr;
    if (m.tokens < 1 || m.tokens > PAIRS2_MAX_STEP_TOKENS || m.top_k > PAIRS2_MAX_K) return false;
    if (!span_format(b.gate_fmt) || b.up_fmt != b.gate_fmt) return false;
    if (has_shared && (m.shared_gate_fmt != b.gate_fmt || m.shared_up_fmt != b.gate_fmt)) return false;
    if (m.logits && b.n_experts > PAIRS2_MAX_EXPERTS) return false;
    if (b.d_model % 256 || b.d_model > 2048) return false;
    const int align = b.gate_fmt == QMOE_FMT_Q6_K ? 2 : 16;
    const void* bases[4] = {b.gate, b.up, m.shared_gate_w, m.shared_up_w};
    for (int i = 0; i < (has_shared ? 4 : 2); ++i)
        if ((uintptr_t)bases[i] % align) return false;
    if (b.gate_stride % align || b.up_stride % align) return false;
    if (!x_fast(m.hidden, m.hidden_dtype, b.d_model)) return false;
    Pairs2Shape x{};
    x.lr = lanes_per_row(b.d_model);
    x.ri = 32 / x.lr;
    if (b.d_ff % x.ri || (has_shared && m.d_ff_shared % x.ri)) return false;
    x.row_image = (b.d_model >> 8) * pieces_per_256(b.gate_fmt) * 16;
    x.pph = x.ri * (b.d_model >> 8) * pieces_per_256(b.gate_fmt);
    x.ipe = b.d_ff / x.ri;
    x.ish = has_shared ? m.d_ff_shared / x.ri : 0;
    x.groups = (m.tokens + PAIRS2_MAX_TOKENS - 1) / PAIRS2_MAX_TOKENS;
    x.group_tokens = (m.tokens + x.groups - 1) / x.groups;
    if (x.groups * 8 > waves / D2_WAVES) return false;   // (a group wants a few workgroups at least)
    const long total = (long)x.ish + (long)x.group_tokens * m.top_k * x.ipe;
    // quotients by mulhi are exact while dividend x divisor stays below 2^32
    if ((uint64_t)(total + 3L * waves) * (uint64_t)(x.ipe > m.top_k ? x.ipe : m.top_k) >= (1ull << 32)) return false;
    x.total = (int)total;
    x.ipe_magic = magic_of(x.ipe);
    x.k_magic = magic_of(m.top_k);
    x.xs_bytes = x.group_tokens * b.d_model * 4;
    x.nv = b.n_experts <= 512 ? 8 : 16;
    if (x.group_tokens * (b.d_model >> 8) > 4 * D2_WAVES) return false;   // a wave's 16-bit chunks fit the end of its ring
    if (out) *out = x;
    return true;
}

template <int FMT>
static int pairs2_launch_as(const DecodeRouteArgs& r, const Pairs2Shape& x, int grid, const ListedExperts& listed, hipStream_t s) {
    static bool configured = false;   // (benign if two threads both set it)
    if (!configured) {
        if (hipFuncSetAttribute((const void*)pairs2_kernel<FMT>, hipFuncAttributeMaxDynamicSharedMemorySize, D2_LDS) != hipSuccess)
            return fail(QMOE_ELAUNCH, "MoE decode (gate/up): cannot reserve %d bytes of LDS", D2_LDS);
        configured = true;
    }
    static_assert(PAIRS2_MAX_TOKENS * 2048 * 4 + PAIRS2_MAX_TOKENS * 32 * 8 + PAIRS2_MAX_TOKENS * sizeof(RouteShare) + 1024 +
                  D2_WAVES * (PAIRS2_PD + 1) * Pairs2Slot<FMT>::BYTES <= D2_LDS, "LDS layout of the gate/up kernel");
    hipLaunchKernelGGL(pairs2_kernel<FMT>, dim3(grid), dim3(D2_THREADS), D2_LDS, s, r, x, listed);
    return check_launch("qmoe_moe_forward(route + gate/up)");
}

bool decode2_pairs_supported(const qmoe_moe_args& m) { return pairs2_plan(m, (stream_grid() / 2) * D2_WAVES, nullptr); }

int decode2_pairs_launch(const qmoe_moe_args& m, const DecodeRouteArgs& r, hipStream_t s, const ListedExperts* listed) {
    ListedExperts l{};
    if (listed) l = *listed;
    const int grid = stream_grid() / 2;
    Pairs2Shape x;
    if (!pairs2_plan(m, grid * D2_WAVES, &x)) return fail(QMOE_EUNSUPPORTED, "MoE decode (gate/up): shape not taken");
    switch (m.bank.gate_fmt) {
    case QMOE_FMT_Q8_0: return pairs2_launch_as<QMOE_FMT_Q8_0>(r, x, grid, l, s);
    case QMOE_FMT_Q6_K: return pairs2_launch_as<QMOE_FMT_Q6_K>(r, x, grid, l, s);
    case QMOE_FMT_Q5_K: return pairs2_launch_as<QMOE_FMT_Q5_K>(r, x, grid, l, s);
    default: return pairs2_launch_as<QMOE_FMT_Q4_K>(r, x, grid, l, s);
    }
}


int decode2_listed(const float* x, const ListedExperts& listed, int gate_fmt, int up_fmt, int down_fmt, int d_model, int d_ff,
                   float* out, float* workspace, hipStream_t s) {
    const int e = listed.count;
    if (e < 1 || e > LISTED_MAX) return fail(QMOE_EUNSUPPORTED, "listed experts: %d experts (1..%d)", e, LISTED_MAX);
    // the step as the two kernels see it: one token, top_k = the list, "expert ids" = list positions
    qmoe_moe_args m{};
    m.hidden = x;
    m.hidden_dtype = QMOE_DT_F32;
    m.tokens = 1;
    m.top_k = e;
    m.bank.gate = listed.gate[0];
    m.bank.up = listed.up[0];
    m.bank.down = listed.down[0];
    m.bank.gate_fmt = gate_fmt;
    m.bank.up_fmt = up_fmt;
    m.bank.down_fmt = down_fmt;
    m.bank.n_experts = e;
    m.bank.d_model = d_model;
    m.bank.d_ff = d_ff;
    m.out = out;
    m.out_dtype = QMOE_DT_F32;
    const int align_gu = gate_fmt == QMOE_FMT_Q6_K ? 2 : 16, align_d = down_fmt == QMOE_FMT_Q6_K ? 2 : 16;
    for (int i = 0; i < e; ++i)
        if ((uintptr_t)listed.gate[i] % align_gu || (uintptr_t)listed.up[i] % align_gu || (uintptr_t)listed.down[i] % align_d)
            return fail(QMOE_EUNSUPPORTED, "listed experts: expert %d is not aligned for the streaming kernels", i);
    // workspace: [e * d_ff] SwiGLU activations, then the routing as the down kernel reads it
    DecodeBuffers w{};
    w.h = workspace;
    w.hs = workspace;   // (no shared expert: never read)
    float* const tail = workspace + (size_t)e * d_ff;
    w.sorted_ids = (int*)tail;
    w.sorted_w = tail + LISTED_MAX;
    w.sig = tail + 2 * LISTED_MAX;
    if ((size_t)e * d_model < 3 * LISTED_MAX) return fail(QMOE_EUNSUPPORTED, "listed experts: workspace too small for the routing");
    if (!decode2_pairs_supported(m) || !decode2_down_supported(m, w)) return fail(QMOE_EUNSUPPORTED, "listed experts: shape not taken");
    DecodeRouteArgs r{};
    r.sorted_ids = w.sorted_ids;
    r.sorted_w = w.sorted_w;
    r.sig = w.sig;
    r.hidden = x;
    r.gate = listed.gate[0];
    r.up = listed.up[0];
    r.h = w.h;
    r.hs = w.hs;
    r.n_experts = e;
    r.k = e;
    r.d = d_model;
    r.f = d_ff;
    r.fmt = gate_fmt;
    r.xdt = QMOE_DT_F32;
    r.tokens = 1;
    if (int rc = decode2_pairs_launch(m, r, s, &listed)) return rc;
    return decode2_down_launch(m, w, s, &listed);
}

}  // namespace qmoe

#ifdef QMOE_TIMELINE
// Copies the stamps of both kernels to `out` (2 x 4096 x 8 unsigned 64-bit values) after the device is idle.
extern "C" int qmoe_timeline_read(unsigned long long* out) {
    if (hipDeviceSynchronize() != hipSuccess) return QMOE_ELAUNCH;
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(qmoe::timeline), sizeof(qmoe::timeline)) == hipSuccess ? QMOE_OK : QMOE_ELAUNCH;
}
#endif
