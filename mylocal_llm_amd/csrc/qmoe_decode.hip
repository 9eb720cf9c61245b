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
#include "qmoe_router.hpp"
#include "qmoe_rowdot.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

static constexpr int DECODE_MAX_TOKENS = 16;
// rows of the output one wave produces in the down kernel (a BF16 unit needs twice the registers)
template <int FMT> struct DownRows { static constexpr int PER_WAVE = FMT == QMOE_FMT_BF16 ? 1 : 2; };

struct DecodeRouteArgs {
    const float* logits;       // [T, E] or null
    const float* in_weights;   // [T, k] when logits == null
    const int64_t* in_ids;     // [T, k] when logits == null
    float* out_weights;        // [T, k] routing weights in selection order (workspace or caller's)
    int64_t* out_ids;          // [T, k]
    int* sorted_ids;           // [T, k] ascending expert id
    float* sorted_w;           // [T, k]
    float* sig;                // [T] sigmoid admission gate (1 when ungated)
    int* status;
    StreamProblem* problems;   // [T * (k + 1)]
    int* problem_count;
    const void* hidden;        // [T, D]
    const float* shared_gate;  // [D] or null
    const uint8_t *gate, *up;  // bank bases
    int64_t gate_stride, up_stride;
    const uint8_t *shared_gate_w, *shared_up_w;  // or null
    float* h;                  // [T*k, F]
    float* hs;                 // [T, Fsh]
    float floor_value;
    int renorm, n_experts, k, d, f, fsh, fmt, xdt, tokens, workers;
};

__global__ __launch_bounds__(64) void decode_route_kernel(const DecodeRouteArgs a) {
    extern __shared__ uint32_t keys[];  // n_experts words when routing from logits
    __shared__ int64_t ids_sel[32];
    __shared__ float w_sel[32];
    __shared__ int order[32];
    const int t = blockIdx.x, lane = threadIdx.x;
    const int k = a.k;
    // admission gate first: its loads are in flight while the row is routed
    float adm = 0.f;
    if (a.shared_gate) {
        for (int i = 4 * lane; i < a.d; i += 256) {
            const float4 hv = load_x4(a.hidden, a.xdt, t * a.d + i);
            const float4 gv = *(const float4*)(a.shared_gate + i);
            adm += (hv.x * gv.x + hv.y * gv.y) + (hv.z * gv.z + hv.w * gv.w);
        }
    }
    if (a.logits) {
        router_row(a.logits + (size_t)t * a.n_experts, a.n_experts, k, a.floor_value, a.renorm, keys, w_sel, ids_sel);
    } else if (lane < k) {
        ids_sel[lane] = a.in_ids[(size_t)t * k + lane];
        w_sel[lane] = a.in_weights[(size_t)t * k + lane];
    }
    __syncthreads();
    if (lane < k) {
        if (a.out_weights) {
            a.out_weights[(size_t)t * k + lane] = w_sel[lane];
            a.out_ids[(size_t)t * k + lane] = ids_sel[lane];
        }
        // rank of this selection in ascending expert id; equal ids keep slot order
        const int64_t mine = ids_sel[lane];
        int rank = 0;
        for (int j = 0; j < k; ++j) rank += (ids_sel[j] < mine) || (ids_sel[j] == mine && j < lane);
        order[rank] = lane;
    }
    __syncthreads();
    if (a.shared_gate) adm = wave_sum(adm);
    if (lane == 0) {
        // sigmoid(hidden . g) without overflow
        a.sig[t] = a.shared_gate ? (adm >= 0.f ? 1.f / (1.f + expf(-adm)) : expf(adm) / (1.f + expf(adm))) : 1.f;
        if (t == 0) *a.problem_count = a.tokens * (k + (a.shared_gate_w ? 1 : 0));
    }
    // this token's problems, in sorted-slot order, then the shared expert
    const int units = a.d >> 6;
    const int lr = units <= 8 ? 8 : units <= 16 ? 16 : units <= 32 ? 32 : 64;
    const int rpw = 64 / lr;
    const int items_r = (a.f + rpw - 1) / rpw, items_s = a.shared_gate_w ? (a.fsh + rpw - 1) / rpw : 0;
    const int per_token = k + (a.shared_gate_w ? 1 : 0);
    const int64_t xbytes = (int64_t)a.d * (a.xdt == QMOE_DT_F32 ? 4 : 2);
    const long token_cursor = (long)t * ((long)k * items_r + items_s) * (units > 64 ? STREAM_WAVES : 1);
    if (lane <= k && lane < per_token) {
        StreamProblem p;
        p.x = (const uint8_t*)a.hidden + (size_t)t * xbytes;
        p.k = a.d;
        p.fmt = a.fmt;
        p.fmt2 = a.fmt;
        p.xdt = a.xdt;
        p.ydt = QMOE_DT_F32;
        p.xgroup = t;
        long cursor;
        if (lane < k) {
            const int s = order[lane];
            const int64_t e = ids_sel[s];
            const bool ok = e >= 0 && e < a.n_experts;
            if (!ok) *a.status = 1;
            const int64_t ee = ok ? e : 0;
            p.w = a.gate + ee * a.gate_stride;
            p.w2 = a.up + ee * a.up_stride;
            p.y = a.h + ((size_t)t * k + lane) * a.f;
            p.n = ok ? a.f : 0;  // an out-of-range id contributes nothing (its h stays unused)
            a.sorted_ids[(size_t)t * k + lane] = ok ? (int)e : -1;
            a.sorted_w[(size_t)t * k + lane] = w_sel[s];
            cursor = token_cursor + (long)lane * items_r * (units > 64 ? STREAM_WAVES : 1);
        } else {
            p.w = a.shared_gate_w;
            p.w2 = a.shared_up_w;
            p.y = a.hs + (size_t)t * a.fsh;
            p.n = a.fsh;
            cursor = token_cursor + (long)k * items_r * (units > 64 ? STREAM_WAVES : 1);
        }
        p.first_item = units > 64 ? (int)((cursor / STREAM_WAVES) % (a.workers / STREAM_WAVES)) : (int)(cursor % a.workers);
        a.problems[(size_t)t * per_token + lane] = p;
    }
}

static constexpr int LIST_STAGE = 48;  // problem descriptors held in LDS at a time

// The streaming engine over a problem list that lives in device memory.
template <int FMT, bool PAIR>
__global__ __launch_bounds__(STREAM_THREADS, 2) void stream_list_kernel(const StreamProblem* __restrict__ list,
                                                                       const int* __restrict__ count) {
    __shared__ float partial[32 * 2 * 4];
    __shared__ StreamProblem staged[LIST_STAGE];
    __shared__ __attribute__((aligned(16))) float xs[STREAM_XS_FLOATS];
    float xr[64], aux[8];
    int xgroup = -1, xstaged = -1;
    const int n = *count;
    // descriptors are fetched a stage at a time by the whole workgroup, not one dependent
    // load per problem
    for (int base = 0; base < n; base += LIST_STAGE) {
        const int m = n - base < LIST_STAGE ? n - base : LIST_STAGE;
        __syncthreads();
        const uint4* src = (const uint4*)(list + base);
        uint4* dst = (uint4*)staged;
        for (int i = threadIdx.x; i < m * 4; i += STREAM_THREADS) dst[i] = src[i];
        __syncthreads();
        for (int i = 0; i < m; ++i) {
            if (staged[i].n > 0) stream_dispatch_shape<FMT, PAIR>(staged[i], partial, xs, xstaged, xr, aux, xgroup);
        }
    }
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
    int odt, k, d, f, fsh;
};

// Lane layout of a wave: lanes [0, k*LPE) = expert slot j = lane / LPE, part = lane % LPE of
// the F/128 column parts of its down row; lanes [48, 48 + Fsh/128) = the shared expert's row
// parts.  Every lane owns two 64-element units (128 columns).
template <int FMT, int LPE>
__global__ __launch_bounds__(256, 2) void decode_down_kernel(const DecodeDownArgs a) {
    using U = Unit64<FMT>;
    const int t = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int k = a.k;
    const int shared_parts = a.shared_down ? a.fsh >> 7 : 0;
    const bool routed = lane < k * LPE;
    const bool shared = lane >= 48 && lane - 48 < shared_parts;
    const int slot = routed ? lane / LPE : 0;
    const int part = routed ? lane % LPE : (shared ? lane - 48 : 0);
    const int e = routed ? a.sorted_ids[(size_t)t * k + slot] : 0;
    const float route_w = lane < k ? a.sorted_w[(size_t)t * k + lane] : 0.f;  // lane j holds weight j
    const bool live = (routed && e >= 0) || shared;
    const int kk = shared ? a.fsh : a.f;
    const int64_t rbytes = row_bytes_dev(FMT, kk);
    const uint8_t* base = shared ? a.shared_down : a.down + (int64_t)(e >= 0 ? e : 0) * a.down_stride;
    const float* xsrc = shared ? a.hs + (size_t)t * a.fsh : a.h + ((size_t)t * k + slot) * a.f;
    constexpr int ROWS = DownRows<FMT>::PER_WAVE;
    const int row0 = (blockIdx.x * 4 + wave) * ROWS;
    uint32_t ra[ROWS][2][U::RAW];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int row = row0 + r < a.d ? row0 + r : a.d - 1;
        const uint8_t* rp = base + (int64_t)row * rbytes;
        U::load_w(rp, 2 * part, ra[r][0]);
        U::load_w(rp, 2 * part + 1, ra[r][1]);
    }
    float x0[64], x1[64], aux0[U::AUX], aux1[U::AUX];
    U::load_x(GlobalX{xsrc, QMOE_DT_F32}, 2 * part, x0, aux0);
    U::load_x(GlobalX{xsrc, QMOE_DT_F32}, 2 * part + 1, x1, aux1);
    if (!live) {
#pragma unroll
        for (int i = 0; i < 64; ++i) { x0[i] = 0.f; x1[i] = 0.f; }
#pragma unroll
        for (int i = 0; i < U::AUX; ++i) { aux0[i] = 0.f; aux1[i] = 0.f; }
    }
    const float sg = a.sig[t];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        float v = U::dot(ra[r][0], x0, aux0) + U::dot(ra[r][1], x1, aux1);
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
        if (lane == 0 && row0 + r < a.d) store_out(a.out, a.odt, (size_t)t * a.d + row0 + r, acc);
    }
}

// ---- host side ------------------------------------------------------------------------------------
static bool stream_format(int fmt) {
    return fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_BF16;
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
    const bool kq = b.down_fmt == QMOE_FMT_Q6_K || b.down_fmt == QMOE_FMT_Q5_K;
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
    hipLaunchKernelGGL(decode_route_kernel, dim3(a.tokens), dim3(64), a.logits ? (size_t)b.n_experts * 4 : 0, s, r);
    int rc = check_launch("qmoe_moe_forward(route)");
    if (rc) return rc;
#define QMOE_LIST(F) hipLaunchKernelGGL((stream_list_kernel<F, true>), dim3(grid), dim3(STREAM_THREADS), 0, s, \
                                        (const StreamProblem*)w.problems, (const int*)w.problem_count)
    switch (b.gate_fmt) {
    case QMOE_FMT_Q8_0: QMOE_LIST(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_LIST(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_LIST(QMOE_FMT_Q5_K); break;
    default: QMOE_LIST(QMOE_FMT_BF16); break;
    }
#undef QMOE_LIST
    if ((rc = check_launch("qmoe_moe_forward(gate/up)"))) return rc;
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
    d.odt = a.out_dtype;
    d.k = a.top_k;
    d.d = b.d_model;
    d.f = b.d_ff;
    d.fsh = r.fsh;
    const int rows_per_wg = 4 * (b.down_fmt == QMOE_FMT_BF16 ? DownRows<QMOE_FMT_BF16>::PER_WAVE : DownRows<QMOE_FMT_Q8_0>::PER_WAVE);
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
    default: QMOE_DOWN_F(QMOE_FMT_BF16); break;
    }
#undef QMOE_DOWN_F
#undef QMOE_DOWN_L
    return check_launch("qmoe_moe_forward(down)");
}

}  // namespace qmoe
