// Routing of one token by one wave, shared by the decode-time MoE kernels: softmax / top-k (or the
// caller's routing), the token's experts sorted by id, the sigmoid admission gate of the shared
// expert.
#pragma once
#include "qmoe_router.hpp"
#include "qmoe_stream.hpp"

namespace qmoe {

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
    int* status_out;   // the caller's word, or null
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
    int shared_apart;          // the shared expert's gate/up is not in the problem list: its rows are
                               // streamed once for all tokens by a phase of its own
    int shared_in_front;       // ... and that phase runs beside the routing, in the routing launch
};

// hidden[t] . g for the shared expert's admission gate, 2048 columns at a time: issue() only
// puts the loads in flight, reduce() adds this lane's products to acc.
struct AdmissionRegs {
    float4 h[8], g[8];
    __device__ __forceinline__ void issue(const void* hidden, int xdt, int t, int d, const float* gate, int lane, int base) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = base + 4 * lane + 256 * j;
            const bool in = i < d;
            h[j] = in ? load_x4(hidden, xdt, t * d + i) : make_float4(0, 0, 0, 0);
            g[j] = in ? *(const float4*)(gate + i) : make_float4(0, 0, 0, 0);
        }
    }
    __device__ __forceinline__ float reduce(float acc) const {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += (h[j].x * g[j].x + h[j].y * g[j].y) + (h[j].z * g[j].z + h[j].w * g[j].w);
        return acc;
    }
};

__device__ __forceinline__ int64_t readlane_i64(int64_t v, int lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), lane);
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// One wave routes token t: the row's loads first, then the admission gate's (and whatever
// `more_loads` issues), then the selection.  The token's selections leave sorted by expert
// id in sid[0..k) (LDS); with `publish` the wave also writes the routing outputs, the sorted
// routing and the admission gate for the down kernel.
template <int MAXNV, typename MoreLoads>
__device__ __forceinline__ void route_token(const DecodeRouteArgs& a, int t, bool publish, int64_t* sid, MoreLoads&& more_loads) {
    const int lane = threadIdx.x & 63, k = a.k;
    AdmissionRegs ar;
    auto issue = [&] {
        if (a.shared_gate && publish) ar.issue(a.hidden, a.xdt, t, a.d, a.shared_gate, lane, 0);
        more_loads();
    };
    float w = 0.f;
    int64_t id = 0;
    if (a.logits) {
        router_row<MAXNV>(a.logits + (size_t)t * a.n_experts, a.n_experts, k, a.floor_value, a.renorm, w, id, issue);
    } else {
        if (lane < k) {
            id = a.in_ids[(size_t)t * k + lane];
            w = a.in_weights[(size_t)t * k + lane];
        }
        issue();
    }
    // rank of this selection in ascending expert id; equal ids keep slot order.  An id outside the
    // bank, or an expert the token has named in an earlier slot already, contributes nothing.
    int rank = 0;
    bool again = false;
    for (int j = 0; j < k; ++j) {
        const int64_t other = readlane_i64(id, j);
        rank += (other < id) || (other == id && j < lane);
        again |= other == id && j < lane;
    }
    if (lane < k) {
        const bool in_range = id >= 0 && id < a.n_experts, ok = in_range && !again;
        sid[rank] = ok ? id : -1;
        if (publish) {
            if (!ok) {
                const int bits = (in_range ? 0 : 1) | (again ? 2 : 0);
                if (a.status_out) atomicOr(a.status_out, bits);
            }
            if (a.out_weights) {
                a.out_weights[(size_t)t * k + lane] = w;
                a.out_ids[(size_t)t * k + lane] = id;
            }
            a.sorted_ids[(size_t)t * k + rank] = ok ? (int)id : -1;
            a.sorted_w[(size_t)t * k + rank] = w;
        }
    }
    if (publish) {
        float adm = 0.f;
        if (a.shared_gate) {
            adm = ar.reduce(adm);
            for (int base = 2048; base < a.d; base += 2048) {
                ar.issue(a.hidden, a.xdt, t, a.d, a.shared_gate, lane, base);
                adm = ar.reduce(adm);
            }
            adm = wave_sum(adm);
        }
        // sigmoid(hidden . g) without overflow
        if (lane == 0) a.sig[t] = a.shared_gate ? (adm >= 0.f ? 1.f / (1.f + expf(-adm)) : expf(adm) / (1.f + expf(adm))) : 1.f;
    }
}

// The experts of a single token given one by one instead of as ids into a bank (the grouped
// decode call): pointers and route positions travel in the kernel arguments, in the order the
// experts are summed.  count == 0: no table, the step addresses a bank.
static constexpr int LISTED_MAX = 16;
struct ListedExperts {
    const uint8_t* gate[LISTED_MAX];
    const uint8_t* up[LISTED_MAX];
    const uint8_t* down[LISTED_MAX];
    int slot[LISTED_MAX];     // position of each expert's weight in `routes`
    const float* routes;      // device, fp32
    int64_t route_stride;     // elements between route positions
    int count;
};

// The LDS-DMA kernels of the decode step (qmoe_decode2.hip): routing + gate/up for up to four
// tokens, down + combine for up to sixteen; each says whether it takes a step's shapes.
bool decode2_pairs_supported(const qmoe_moe_args& m);
int decode2_pairs_launch(const qmoe_moe_args& m, const DecodeRouteArgs& r, hipStream_t s, const ListedExperts* listed = nullptr);
bool decode2_down_supported(const qmoe_moe_args& m, const DecodeBuffers& w);
int decode2_down_launch(const qmoe_moe_args& m, const DecodeBuffers& w, hipStream_t s, const ListedExperts* listed = nullptr);
// A single token through listed experts: out[d] = sum in list order of fp32(down_e(swiglu_e(x))[d] * route_e);
// QMOE_EUNSUPPORTED (nothing launched) for shapes the two kernels do not take.
int decode2_listed(const float* x, const ListedExperts& listed, int gate_fmt, int up_fmt, int down_fmt, int d_model, int d_ff,
                   float* out, float* workspace, hipStream_t s);

}  // namespace qmoe
