// Packed-expert MoE step for a handful of tokens (decode): three launches, no host round trip.
//
//   1. route   one wave per token: softmax / top-k (or the given routing), the token's experts
//              sorted by id, the sigmoid admission gate of the shared expert, and the token's
//              entries of the device-side problem list (one gate/up pair per selected expert
//              plus the shared expert's pair).
//   2. pairs   the streaming engine walks that list: h = silu(G x) * (U x) for every selected
//              expert and the shared expert, activations kept in registers per token.
//   3. down    one workgroup per (token, 4 or 8 output rows): lanes are laid out as
//              [expert slot][part of the row] plus a group for the shared expert, each lane
//              keeps its slice of h in registers, streams its part of the down rows, and the
//              wave adds the experts' products in ascending expert id (product stored, then
//              added; no FMA, no tree) and finally shared * sigmoid.  Nothing else combines.
#include "qmoe_decode.hpp"
#include "qmoe_rowdot.hpp"

namespace qmoe {

static constexpr int DECODE_MAX_TOKENS = 16;
static constexpr int LIST_STAGE = 96;  // problem descriptors held in LDS at a time
// rows the down kernel requests ahead of the one it reduces (a BF16 unit needs twice the registers)
template <int FMT> struct DownDepth { static constexpr int ROWS_AHEAD = FMT == QMOE_FMT_BF16 ? 0 : 2; };
// the down kernel's LDS row: k*F <= 48*128 routed columns plus up to 2048 shared ones, padded
static constexpr int DOWN_XS_FLOATS = 8192 + 4 * (8192 / 64);

// Entry j of token t's part of the problem list: the gate/up pair of its j-th expert in
// ascending id (j < k) or of the shared expert (j == k).
__device__ __forceinline__ StreamProblem decode_problem(const DecodeRouteArgs& a, int t, int j, int64_t e) {
    const bool shared_listed = a.shared_gate_w && !a.shared_apart;
    const int k = a.k;
    const int units = a.d >> 6;
    const int rpw = 64 / lanes_per_row(a.d);
    const int items_r = (a.f + rpw - 1) / rpw, items_s = shared_listed ? (a.fsh + rpw - 1) / rpw : 0;
    const int wide = units > 64 ? STREAM_WAVES : 1;
    const int64_t xbytes = (int64_t)a.d * (a.xdt == QMOE_DT_F32 ? 4 : 2);
    const long cursor = ((long)t * ((long)k * items_r + items_s) + (long)j * items_r) * wide;
    StreamProblem p;
    p.x = (const uint8_t*)a.hidden + (size_t)t * xbytes;
    p.k = a.d;
    p.fmt = a.fmt;
    p.xdt = a.xdt;
    p.ydt = QMOE_DT_F32;
    p.xgroup = t;
    if (j < k) {
        const bool ok = e >= 0 && e < a.n_experts;
        const int64_t ee = ok ? e : 0;
        p.w = a.gate + ee * a.gate_stride;
        p.w2 = a.up + ee * a.up_stride;
        p.y = a.h + ((size_t)t * k + j) * a.f;
        p.n = ok ? a.f : 0;  // an out-of-range id contributes nothing (its h stays unused)
    } else {
        p.w = a.shared_gate_w;
        p.w2 = a.shared_up_w;
        p.y = a.hs + (size_t)t * a.fsh;
        p.n = a.fsh;
    }
    if (units > 64) {
        p.first_item = (int)((cursor / STREAM_WAVES) % (a.workers / STREAM_WAVES));
        p.flat_end = 0;
    } else {
        p.first_item = (int)cursor;
        p.flat_end = (int)cursor + (j < k ? items_r : items_s);
    }
    return p;
}

template <int MAXNV>
__global__ __launch_bounds__(64) void decode_route_kernel(const DecodeRouteArgs a) {
    __shared__ int64_t sid[32];
    const int t = blockIdx.x, lane = threadIdx.x;
    route_token<MAXNV>(a, t, true, sid, [] {});
    __syncthreads();
    const int per_token = a.k + (a.shared_gate_w && !a.shared_apart ? 1 : 0);
    if (lane == 0 && t == 0) *a.problem_count = a.tokens * per_token;
    if (lane < per_token) a.problems[(size_t)t * per_token + lane] = decode_problem(a, t, lane, lane < a.k ? sid[lane] : 0);
}

// Activation rows of tokens t0 .. t0 + nt - 1 into padded LDS stripes, by the whole workgroup.
// A token's loads are issued together, then stored (a store between two loads orders them).
// (All tokens' loads ahead of all stores measured slower.)
__device__ __forceinline__ void stage_tokens(const DecodeRouteArgs& a, float* xs, int stripe, int t0, int nt) {
    for (int i = 0; i < nt; ++i) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = 4 * threadIdx.x + 4 * STREAM_THREADS * j;
            if (c < a.d) v[j] = load_x4(a.hidden, a.xdt, (t0 + i) * a.d + c);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = 4 * threadIdx.x + 4 * STREAM_THREADS * j;
            if (c < a.d) *(float4*)(xs + i * stripe + StagedX::at(c)) = v[j];
        }
    }
}

// The shared expert's gate/up rows for all tokens of the step.  The tokens are cut into groups
// whose activations fit the LDS stripes together; workgroup `wg` of `wgs` serves group
// wg % groups: it stages that group's tokens and shares the rows with the other workgroups of
// the group, every row streamed once per group and reduced against each staged token in turn.
// A wave's chain (row fetch, then one reduction per token of its group) is pure latency, so
// the tokens are cut into more groups than LDS asks for as long as that gives waves a row that
// would have none.  Workgroup-uniform; ends with the LDS free again.
template <int FMT>
__device__ __forceinline__ void shared_pairs_phase(const DecodeRouteArgs& a, float* xs, int wg, int wgs) {
    const int stripe = a.d + 4 * (a.d >> 6);
    const int fit = STREAM_XS_FLOATS / stripe;
    const int wave = threadIdx.x >> 6;
    const int rpw = 64 / lanes_per_row(a.d);
    const long items = (a.fsh + rpw - 1) / rpw;
    int groups = (a.tokens + fit - 1) / fit;
    while (2 * groups <= a.tokens && 2 * groups <= wgs && items * 2 * groups <= (long)wgs * STREAM_WAVES * 21 / 20) groups *= 2;
    const int per = (a.tokens + groups - 1) / groups;
    for (int g = wg % groups; g < groups; g += wgs) {
        const int t0 = g * per;
        const int nt = a.tokens - t0 < per ? a.tokens - t0 : per;
        if (nt <= 0) break;
        const int serving = wgs >= groups ? (wgs - g + groups - 1) / groups : 1;   // workgroups of this group
        const int mine = wgs >= groups ? wg / groups : 0;
        __syncthreads();
        stage_tokens(a, xs, stripe, t0, nt);
        __syncthreads();
        stream_rows_many_x<FMT, true, Prefetch<FMT, true>::DEPTH>(a.shared_gate_w, a.shared_up_w, a.fsh, a.d, xs, stripe, nt,
                                                                 a.hs + (size_t)t0 * a.fsh, a.fsh,
                                                                 mine * STREAM_WAVES + wave, serving * STREAM_WAVES);
    }
    __syncthreads();
}

// Routing and the shared expert's gate/up rows in one launch (the rows need no routing):
// workgroup t < tokens routes token t with its first wave, as decode_route_kernel does; all
// other workgroups stream.  The launch is as long as the longer of the two.
template <int FMT>
__global__ __launch_bounds__(STREAM_THREADS, 2) void decode_front_kernel(const DecodeRouteArgs a) {
    __shared__ int64_t sid[32];
    __shared__ __attribute__((aligned(16))) float xs[STREAM_XS_FLOATS];
    if ((int)blockIdx.x < a.tokens) {
        if (threadIdx.x >= 64) return;
        const int t = blockIdx.x, lane = threadIdx.x;
        route_token<16>(a, t, true, sid, [] {});
        __builtin_amdgcn_wave_barrier();   // one wave: its LDS accesses complete in order
        if (lane == 0 && t == 0) *a.problem_count = a.tokens * a.k;
        if (lane < a.k) a.problems[(size_t)t * a.k + lane] = decode_problem(a, t, lane, sid[lane]);
        return;
    }
    shared_pairs_phase<FMT>(a, xs, blockIdx.x - a.tokens, gridDim.x - a.tokens);
}

// The streaming engine over a problem list that lives in device memory.
template <int FMT, bool PAIR>
__global__ __launch_bounds__(STREAM_THREADS, 2) void stream_list_kernel(const StreamProblem* __restrict__ list,
                                                                       const int* __restrict__ count,
                                                                       const DecodeRouteArgs a) {
    __shared__ float partial[32 * 2 * 4];
    __shared__ StreamProblem staged[LIST_STAGE];
    __shared__ __attribute__((aligned(16))) float xs[STREAM_XS_FLOATS];
    if (a.shared_apart && !a.shared_in_front) shared_pairs_phase<FMT>(a, xs, blockIdx.x, gridDim.x);
    const int n = *count;
    const int units = a.d >> 6;
    if (units <= 64) {
        // Rows that fit a wave: tokens are taken in groups whose activations fit the LDS stripes
        // (eight tokens of 2048 columns) and whose descriptors fit the staging array; inside a
        // group the waves sweep the item stream together (item w, w + W, ...), as in the fused
        // kernel, instead of each wave walking a stretch of its own.
        const int per_token = a.k + ((a.shared_gate_w && !a.shared_apart) ? 1 : 0);
        const int stripe = a.d + 4 * units;
        int group = STREAM_XS_FLOATS / stripe;
        if (group > LIST_STAGE / per_token) group = LIST_STAGE / per_token;
        for (int t0 = 0; t0 < a.tokens; t0 += group) {
            const int nt = a.tokens - t0 < group ? a.tokens - t0 : group;
            const int base = t0 * per_token;
            int m = nt * per_token;
            if (base + m > n) m = n - base;
            if (m <= 0) break;
            __syncthreads();
            const uint4* src = (const uint4*)(list + base);
            uint4* dst = (uint4*)staged;
            for (int i = threadIdx.x; i < m * 4; i += STREAM_THREADS) dst[i] = src[i];
            stage_tokens(a, xs, stripe, t0, nt);
            __syncthreads();
            if ((int)threadIdx.x < m) staged[threadIdx.x].xgroup -= t0;   // stripe of the token inside this group
            __syncthreads();
            stream_run<FMT, PAIR, false>(staged, m, staged[0].first_item, staged[m - 1].flat_end, false, partial, xs, xs, stripe);
        }
        return;
    }
    // wider rows: descriptors are fetched a stage at a time by the whole workgroup, four waves a row
    for (int base = 0; base < n; base += LIST_STAGE) {
        const int m = n - base < LIST_STAGE ? n - base : LIST_STAGE;
        __syncthreads();
        const uint4* src = (const uint4*)(list + base);
        uint4* dst = (uint4*)staged;
        for (int i = threadIdx.x; i < m * 4; i += STREAM_THREADS) dst[i] = src[i];
        __syncthreads();
        stream_run<FMT, PAIR>(staged, m, 0, 0, true, partial, xs);
    }
}

// Routing fused into the gate/up launch (up to FUSED_MAX_TOKENS tokens of up to 4096
// columns): every workgroup routes the tokens itself (one wave per token), so the problem
// list never leaves LDS and no launch sits between the logits and the first expert byte.
// While the routing loads travel, the workgroup also fetches the tokens' activations into
// LDS, stripe t for token t, where the streaming loop picks them up.  Workgroup 0 publishes
// the routing for the down kernel.
static constexpr int FUSED_MAX_TOKENS = 4;
static constexpr int FUSED_MAX_EXPERTS = 1024;  // wider rows need more registers than the streaming loop leaves
static constexpr int FUSED_MAX_SLOTS = 12;      // top_k + shared expert

template <int FMT>
__global__ __launch_bounds__(STREAM_THREADS, 2) void decode_pairs_fused_kernel(const DecodeRouteArgs a) {
    __shared__ StreamProblem staged[FUSED_MAX_TOKENS * FUSED_MAX_SLOTS];
    __shared__ __attribute__((aligned(16))) float xs[STREAM_XS_FLOATS];
    __shared__ int64_t sid[FUSED_MAX_TOKENS][32];
    constexpr int STRIPE = STREAM_XS_FLOATS / STREAM_WAVES;
    const int wave = threadIdx.x >> 6;
    const int k = a.k, tokens = a.tokens;
    // this thread's share of the tokens' activations: columns 4*tid + 1024*i of every token
    float4 xv[FUSED_MAX_TOKENS][4];
    auto fetch_x = [&] {
#pragma unroll
        for (int t = 0; t < FUSED_MAX_TOKENS; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = 4 * threadIdx.x + 1024 * i;
                if (t < tokens && col < a.d) xv[t][i] = load_x4(a.hidden, a.xdt, t * a.d + col);
            }
    };
    constexpr int PD = Prefetch<FMT, true>::DEPTH;
    const int idle = STREAM_WAVES - tokens;   // waves with no token to route
    if (idle > 0) {
        // The routing waves only route.  Every other wave stages the activations of all tokens
        // (each of them writes every value, the same ones, so none waits for another) and takes
        // its share of the shared expert's gate/up rows, which need no routing: that work
        // is over by the time the selection rounds are.
        if (wave < tokens) {
            route_token<FUSED_MAX_EXPERTS / 64>(a, wave, blockIdx.x == 0, sid[wave], [] {});
        } else {
            const int lane = threadIdx.x & 63;
            for (int t = 0; t < tokens; ++t) {
                float4 v[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int col = 4 * lane + 256 * i;
                    if (col < a.d) v[i] = load_x4(a.hidden, a.xdt, t * a.d + col);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int col = 4 * lane + 256 * i;
                    if (col < a.d) *(float4*)(xs + t * STRIPE + StagedX::at(col)) = v[i];
                }
            }
            if (a.shared_gate_w)
                stream_rows_many_x<FMT, true, PD>(a.shared_gate_w, a.shared_up_w, a.fsh, a.d, xs, STRIPE, tokens, a.hs, a.fsh,
                                                  blockIdx.x * idle + (wave - tokens), gridDim.x * idle);
        }
        __syncthreads();
    } else {
        route_token<FUSED_MAX_EXPERTS / 64>(a, wave, blockIdx.x == 0, sid[wave], fetch_x);
#pragma unroll
        for (int t = 0; t < FUSED_MAX_TOKENS; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = 4 * threadIdx.x + 1024 * i;
                if (t < tokens && col < a.d) *(float4*)(xs + t * STRIPE + StagedX::at(col)) = xv[t][i];
            }
        __syncthreads();
        // the shared expert's rows once for all tokens
        if (a.shared_gate_w)
            stream_rows_many_x<FMT, true, PD>(a.shared_gate_w, a.shared_up_w, a.fsh, a.d, xs, STRIPE, tokens, a.hs, a.fsh,
                                              blockIdx.x * STREAM_WAVES + wave, gridDim.x * STREAM_WAVES);
    }
    const int count = tokens * k;
    if ((int)threadIdx.x < count) {
        const int t = threadIdx.x / k, j = threadIdx.x % k;
        staged[threadIdx.x] = decode_problem(a, t, j, sid[t][j]);
    }
    __syncthreads();
    stream_run<FMT, true, false>(staged, count, 0, staged[count - 1].flat_end, tokens > 1, nullptr, xs, xs);
}

template <int LPE>
__device__ __forceinline__ float part_sum(float v) {
    if (LPE >= 2) v = dpp_add<0xB1>(v);
    if (LPE >= 4) v = dpp_add<0x4E>(v);
    if (LPE >= 8) v = dpp_add<0x141>(v);
    if (LPE >= 16) v = dpp_add<0x140>(v);
    return v;
}

struct DecodeDownArgs {
    const uint8_t* down;        // bank base, [E, D, F]
    int64_t down_stride;
    const uint8_t* shared_down; // [D, Fsh] or null
    const float* h;             // [T*k, F] in sorted-slot order
    const float* hs;            // [T, Fsh]
    const int* sorted_ids;      // [T, k]
    const float* sorted_w;      // [T, k]
    const float* sig;           // [T]
    void* out;                  // [T, D]
    const float* residual;      // [T, D] added to the block's output, or null
    int odt, k, d, f, fsh, rows_per_wave;
};

// Lane layout of a wave: lanes [0, k*LPE) = expert slot j = lane / LPE, part = lane % LPE of
// the F/128 column parts of its down row; lanes [48, 48 + Fsh/128) = the shared expert's row
// parts.  Every lane owns two 64-element units (128 columns) of its expert's h, fetched once
// per workgroup into padded LDS (coalesced) and kept in registers while the wave walks
// `rows_per_wave` consecutive output rows with DownDepth rows requested ahead.
template <int FMT, int LPE>
__global__ __launch_bounds__(256, 2) void decode_down_kernel(const DecodeDownArgs a) {
    using U = Unit64<FMT>;
    constexpr int PD = DownDepth<FMT>::ROWS_AHEAD;
    __shared__ __attribute__((aligned(16))) float xs[DOWN_XS_FLOATS];
    const int t = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int k = a.k;
    const int shared_parts = a.shared_down ? a.fsh >> 7 : 0;
    const bool routed = lane < k * LPE;
    const bool shared = lane >= 48 && lane - 48 < shared_parts;
    const int slot = routed ? lane / LPE : 0;
    const int part = routed ? lane % LPE : (shared ? lane - 48 : 0);
    // lanes with nothing to do read what lane 0 reads (its expert, part 0): no cache line of their own
    const int e = a.sorted_ids[(size_t)t * k + slot];
    const float route_w = lane < k ? a.sorted_w[(size_t)t * k + lane] : 0.f;  // lane j holds weight j
    const bool live = (routed && e >= 0) || shared;
    const int kk = shared ? a.fsh : a.f;
    const int64_t rbytes = row_bytes_dev(FMT, kk);
    const uint8_t* base = shared ? a.shared_down : a.down + (int64_t)(e >= 0 ? e : 0) * a.down_stride;
    const int row0 = (blockIdx.x * 4 + wave) * a.rows_per_wave;
    const int nrows = a.d - row0 < a.rows_per_wave ? a.d - row0 : a.rows_per_wave;
    uint32_t buf[PD + 1][2][U::RAW];
    auto fetch = [&](int r, uint32_t (&b)[2][U::RAW]) {
        const uint8_t* rp = base + (int64_t)(row0 + r) * rbytes;
        U::load_w(rp, 2 * part, b[0]);
        U::load_w(rp, 2 * part + 1, b[1]);
    };
#pragma unroll
    for (int j = 0; j < PD; ++j)
        if (j < nrows) fetch(j, buf[j]);
    // this token's h of every slot, then the shared expert's, as one padded fp32 row in LDS
    const int nr = k * a.f, total = nr + (a.shared_down ? a.fsh : 0);
    const float* hr = a.h + (size_t)t * nr;
    const float* hsh = a.hs + (size_t)t * a.fsh;
    {
        // all loads first, then the LDS stores (a store between two loads orders them)
        constexpr int NV = 8192 / (4 * 256);
        float4 v[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = 4 * threadIdx.x + 4 * 256 * j;
            if (i < total) v[j] = i < nr ? ldg<float4>(hr + i) : ldg<float4>(hsh + (i - nr));
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = 4 * threadIdx.x + 4 * 256 * j;
            if (i < total) *(float4*)(xs + StagedX::at(i)) = v[j];
        }
    }
    __syncthreads();
    const int ux = shared ? (nr >> 6) + 2 * part : slot * (a.f >> 6) + 2 * part;
    float x0[64], x1[64], aux0[U::AUX], aux1[U::AUX];
    U::load_x(StagedX{xs}, ux, x0, aux0);
    U::load_x(StagedX{xs}, ux + 1, x1, aux1);
    if (!live) {
#pragma unroll
        for (int i = 0; i < 64; ++i) { x0[i] = 0.f; x1[i] = 0.f; }
#pragma unroll
        for (int i = 0; i < U::AUX; ++i) { aux0[i] = 0.f; aux1[i] = 0.f; }
    }
    const float sg = a.sig[t];
    int r = 0;
    bool done = nrows <= 0;
    while (!done) {
#pragma unroll
        for (int s = 0; s <= PD; ++s) {
            if (!done) {
                if (r + PD < nrows) fetch(r + PD, buf[(s + PD) % (PD + 1)]);
                float v = U::dot(buf[s][0], x0, aux0) + U::dot(buf[s][1], x1, aux1);
                if (!live) v = 0.f;  // idle lanes decoded whatever bytes sit at the base address
                const float ys = group_sum<16>(v);   // lanes 48..63 are one DPP row: the shared expert's total
                const float yr = part_sum<LPE>(v);   // every slot's total in each of its lanes
                float acc = 0.f;
                for (int j = 0; j < k; ++j) {
                    const float yj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(yr), j * LPE));
                    const float wj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(route_w), j));
                    acc = add_product(acc, yj, wj);
                }
                if (a.shared_down) {
                    const float y63 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ys), 63));
                    acc = add_product(acc, y63, sg);
                }
                if (lane == 0) {
                    if (a.residual) acc = a.residual[(size_t)t * a.d + row0 + r] + acc;
                    store_out(a.out, a.odt, (size_t)t * a.d + row0 + r, acc);
                }
                ++r;
                if (r >= nrows) done = true;
            }
        }
    }
}

// ---- host side ------------------------------------------------------------------------------------
static bool stream_format(int fmt) {
    return fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q4_K || fmt == QMOE_FMT_BF16;
}

// May this MoE step take the three-launch decode path?
bool decode_supported(const qmoe_moe_args& a, const void* h_ws) {
    const qmoe_expert_bank& b = a.bank;
    if (a.tokens < 1 || a.tokens > DECODE_MAX_TOKENS) return false;
    if (b.gate_fmt != b.up_fmt || !stream_format(b.gate_fmt) || !stream_format(b.down_fmt)) return false;
    const bool has_shared = a.shared_gate_w != nullptr;
    if (has_shared && (a.shared_gate_fmt != b.gate_fmt || a.shared_up_fmt != b.gate_fmt || a.shared_down_fmt != b.down_fmt)) return false;
    const int lpe = b.d_ff >> 7;
    if (b.d_ff % 128 || (lpe & (lpe - 1)) || lpe > 16 || a.top_k * lpe > 48) return false;
    if (has_shared && (a.d_ff_shared % 128 || (a.d_ff_shared >> 7) > 16)) return false;
    const bool kq = b.down_fmt == QMOE_FMT_Q6_K || b.down_fmt == QMOE_FMT_Q5_K || b.down_fmt == QMOE_FMT_Q4_K;
    if (kq && (b.d_ff % 256 || (has_shared && a.d_ff_shared % 256))) return false;
    const int ga = b.gate_fmt == QMOE_FMT_Q8_0 ? 4 : b.gate_fmt == QMOE_FMT_Q6_K ? 2 : 16;
    const int da = b.down_fmt == QMOE_FMT_Q8_0 ? 4 : b.down_fmt == QMOE_FMT_Q6_K ? 2 : 16;
    if (b.gate_stride % ga || b.up_stride % ga || b.down_stride % da) return false;
    if (!stream_supported(b.gate_fmt, b.gate, b.d_ff, b.d_model, a.hidden, a.hidden_dtype)) return false;
    if (!stream_supported(b.up_fmt, b.up, b.d_ff, b.d_model, a.hidden, a.hidden_dtype)) return false;
    if (!stream_supported(b.down_fmt, b.down, b.d_model, b.d_ff, h_ws, QMOE_DT_F32)) return false;
    if (has_shared) {
        if (!stream_supported(b.gate_fmt, a.shared_gate_w, a.d_ff_shared, b.d_model, a.hidden, a.hidden_dtype)) return false;
        if (!stream_supported(b.gate_fmt, a.shared_up_w, a.d_ff_shared, b.d_model, a.hidden, a.hidden_dtype)) return false;
        if (!stream_supported(b.down_fmt, a.shared_down_w, b.d_model, a.d_ff_shared, h_ws, QMOE_DT_F32)) return false;
    }
    return true;
}

int stream_grid();

int decode_launch(const qmoe_moe_args& a, const DecodeBuffers& w, hipStream_t s) {
    const qmoe_expert_bank& b = a.bank;
    const bool has_shared = a.shared_gate_w != nullptr;
    const int grid = stream_grid();
    DecodeRouteArgs r{};
    r.logits = a.logits;
    r.in_weights = a.in_weights;
    r.in_ids = a.in_ids;
    r.out_weights = a.out_weights ? a.out_weights : w.weights;
    r.out_ids = a.out_ids ? a.out_ids : w.ids;
    r.sorted_ids = w.sorted_ids;
    r.sorted_w = w.sorted_w;
    r.sig = w.sig;
    r.status = w.status;
    r.status_out = a.status_out;
    r.problems = (StreamProblem*)w.problems;
    r.problem_count = w.problem_count;
    r.hidden = a.hidden;
    r.shared_gate = has_shared ? a.shared_gate : nullptr;
    r.gate = (const uint8_t*)b.gate;
    r.up = (const uint8_t*)b.up;
    r.gate_stride = b.gate_stride;
    r.up_stride = b.up_stride;
    r.shared_gate_w = (const uint8_t*)a.shared_gate_w;
    r.shared_up_w = (const uint8_t*)a.shared_up_w;
    r.h = w.h;
    r.hs = w.hs;
    r.floor_value = a.floor_value;
    r.renorm = a.renormalize;
    r.n_experts = b.n_experts;
    r.k = a.top_k;
    r.d = b.d_model;
    r.f = b.d_ff;
    r.fsh = has_shared ? a.d_ff_shared : 0;
    r.fmt = b.gate_fmt;
    r.xdt = a.hidden_dtype;
    r.tokens = a.tokens;
    r.workers = grid * STREAM_WAVES;
    int rc;
    const bool fused = a.tokens <= FUSED_MAX_TOKENS && a.top_k + 1 <= FUSED_MAX_SLOTS && b.d_model <= 4096 &&
                       (!a.logits || b.n_experts <= FUSED_MAX_EXPERTS);
    if (decode2_pairs_supported(a)) {
        if ((rc = decode2_pairs_launch(a, r, s))) return rc;
    } else if (fused) {
        r.shared_apart = has_shared;   // streamed once for all tokens, beside the routing
        const dim3 fg(grid), fb(STREAM_THREADS);
        switch (b.gate_fmt) {
        case QMOE_FMT_Q8_0: hipLaunchKernelGGL(decode_pairs_fused_kernel<QMOE_FMT_Q8_0>, fg, fb, 0, s, r); break;
        case QMOE_FMT_Q6_K: hipLaunchKernelGGL(decode_pairs_fused_kernel<QMOE_FMT_Q6_K>, fg, fb, 0, s, r); break;
        case QMOE_FMT_Q5_K: hipLaunchKernelGGL(decode_pairs_fused_kernel<QMOE_FMT_Q5_K>, fg, fb, 0, s, r); break;
        case QMOE_FMT_Q4_K: hipLaunchKernelGGL(decode_pairs_fused_kernel<QMOE_FMT_Q4_K>, fg, fb, 0, s, r); break;
        default: hipLaunchKernelGGL(decode_pairs_fused_kernel<QMOE_FMT_BF16>, fg, fb, 0, s, r); break;
        }
        if ((rc = check_launch("qmoe_moe_forward(route + gate/up)"))) return rc;
    } else {
    r.shared_apart = has_shared && b.d_model <= 4096 && a.tokens >= 2;
    r.shared_in_front = r.shared_apart && (!a.logits || b.n_experts <= 1024) && grid > 2 * a.tokens;
    if (r.shared_in_front) {
        const dim3 fg(grid), fb(STREAM_THREADS);
        switch (b.gate_fmt) {
        case QMOE_FMT_Q8_0: hipLaunchKernelGGL(decode_front_kernel<QMOE_FMT_Q8_0>, fg, fb, 0, s, r); break;
        case QMOE_FMT_Q6_K: hipLaunchKernelGGL(decode_front_kernel<QMOE_FMT_Q6_K>, fg, fb, 0, s, r); break;
        case QMOE_FMT_Q5_K: hipLaunchKernelGGL(decode_front_kernel<QMOE_FMT_Q5_K>, fg, fb, 0, s, r); break;
        case QMOE_FMT_Q4_K: hipLaunchKernelGGL(decode_front_kernel<QMOE_FMT_Q4_K>, fg, fb, 0, s, r); break;
        default: hipLaunchKernelGGL(decode_front_kernel<QMOE_FMT_BF16>, fg, fb, 0, s, r); break;
        }
    } else
    // the narrow instance is a fraction of the code: a kernel that runs once per step fetches
    // its instructions cold
    if (!a.logits || b.n_experts <= 1024) hipLaunchKernelGGL(decode_route_kernel<16>, dim3(a.tokens), dim3(64), 0, s, r);
    else hipLaunchKernelGGL(decode_route_kernel<64>, dim3(a.tokens), dim3(64), 0, s, r);
    if ((rc = check_launch("qmoe_moe_forward(route)"))) return rc;
#define QMOE_LIST(F) hipLaunchKernelGGL((stream_list_kernel<F, true>), dim3(grid), dim3(STREAM_THREADS), 0, s, \
                                        (const StreamProblem*)w.problems, (const int*)w.problem_count, r)
    switch (b.gate_fmt) {
    case QMOE_FMT_Q8_0: QMOE_LIST(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_LIST(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_LIST(QMOE_FMT_Q5_K); break;
    case QMOE_FMT_Q4_K: QMOE_LIST(QMOE_FMT_Q4_K); break;
    default: QMOE_LIST(QMOE_FMT_BF16); break;
    }
#undef QMOE_LIST
    if ((rc = check_launch("qmoe_moe_forward(gate/up)"))) return rc;
    }
    if (decode2_down_supported(a, w)) return decode2_down_launch(a, w, s);
    DecodeDownArgs d{};
    d.down = (const uint8_t*)b.down;
    d.down_stride = b.down_stride;
    d.shared_down = has_shared ? (const uint8_t*)a.shared_down_w : nullptr;
    d.h = w.h;
    d.hs = w.hs;
    d.sorted_ids = w.sorted_ids;
    d.sorted_w = w.sorted_w;
    d.sig = w.sig;
    d.out = a.out;
    d.residual = a.residual;
    d.odt = a.out_dtype;
    d.k = a.top_k;
    d.d = b.d_model;
    d.f = b.d_ff;
    d.fsh = r.fsh;
    // enough workgroups to fill the chip at one token; longer walks (activations reused) beyond
    const long want = (long)a.tokens * b.d_model / 2048;
    d.rows_per_wave = want >= 8 ? 8 : want >= 4 ? 4 : want >= 2 ? 2 : 1;
    const int rows_per_wg = 4 * d.rows_per_wave;
    const dim3 dgrid((b.d_model + rows_per_wg - 1) / rows_per_wg, a.tokens), dblock(256);
    const int lpe = b.d_ff >> 7;
#define QMOE_DOWN_L(F, L) hipLaunchKernelGGL((decode_down_kernel<F, L>), dgrid, dblock, 0, s, d)
#define QMOE_DOWN_F(F)                                                                     \
    switch (lpe) {                                                                         \
    case 1: QMOE_DOWN_L(F, 1); break;                                                      \
    case 2: QMOE_DOWN_L(F, 2); break;                                                      \
    case 4: QMOE_DOWN_L(F, 4); break;                                                      \
    case 8: QMOE_DOWN_L(F, 8); break;                                                      \
    default: QMOE_DOWN_L(F, 16); break;                                                    \
    }
    switch (b.down_fmt) {
    case QMOE_FMT_Q8_0: QMOE_DOWN_F(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_DOWN_F(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_DOWN_F(QMOE_FMT_Q5_K); break;
    case QMOE_FMT_Q4_K: QMOE_DOWN_F(QMOE_FMT_Q4_K); break;
    default: QMOE_DOWN_F(QMOE_FMT_BF16); break;
    }
#undef QMOE_DOWN_F
#undef QMOE_DOWN_L
    return check_launch("qmoe_moe_forward(down)");
}

}  // namespace qmoe
