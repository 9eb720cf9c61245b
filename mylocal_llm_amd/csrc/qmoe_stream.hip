// Persistent single-token streaming kernel over a list of problems.
//
// One launch walks a list of independent problems (y = W x, or h = silu(G x) * (U x)) with a
// fixed grid of 2 workgroups per CU.  Inside a problem every wave keeps taking the next
// unprocessed row (or group of short rows) in round-robin order that continues across
// problem boundaries, so the HBM stream never drains between matrices; the activation
// slice of a new problem is fetched together with that problem's first rows.
#include "qmoe_stream.hpp"
#include "qmoe_rowdot.hpp"

namespace qmoe {

__device__ __forceinline__ int64_t row_bytes_dev(int fmt, int k) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: return (int64_t)(k >> 5) * 34;
    case QMOE_FMT_Q5_K: return (int64_t)(k >> 8) * 176;
    case QMOE_FMT_Q6_K: return (int64_t)(k >> 8) * 210;
    default: return (int64_t)k * 2;
    }
}

// One step's worth of raw weight registers for a row (and its partner row of a gate/up pair).
template <int FMT, bool PAIR> struct RowRegs {
    uint32_t a[Unit64<FMT>::RAW];
    uint32_t b[PAIR ? Unit64<FMT>::RAW : 1];
};

// Rows of `LR` lanes each (64/LR rows per wave and step); WR waves share one row; PD rows
// are requested ahead of the one being reduced.
template <int FMT, bool PAIR, int LR, int WR, int PD>
__device__ __forceinline__ void stream_problem(const StreamProblem& p, float* partial, float (&xr)[64], float (&aux)[8],
                                               int& xgroup) {
    using U = Unit64<FMT>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int units = p.k >> 6;
    const int64_t rb = row_bytes_dev(FMT, p.k);
    constexpr int RPW = 64 / LR;                 // rows per wave step
    const int sub = lane / LR;                   // which of the wave's rows this lane works on
    const int u = (WR > 1 ? wave * 64 : 0) + (lane % LR);
    const bool active = u < units;
    const int uu = active ? u : 0;
    // work items: groups of RPW rows; taken by waves (WR == 1) or by workgroups (WR > 1)
    const int items = (p.n + RPW - 1) / RPW;
    const int workers = WR > 1 ? gridDim.x : gridDim.x * STREAM_WAVES;
    const int me = WR > 1 ? blockIdx.x : blockIdx.x * STREAM_WAVES + wave;
    int item = (me - p.first_item + workers) % workers;
    if (item >= items) return;

    RowRegs<FMT, PAIR> buf[PD + 1];
    auto fetch = [&](RowRegs<FMT, PAIR>& r, int it) {
        const int row = it * RPW + sub;
        const int64_t rr = row < p.n ? row : p.n - 1;
        U::load_w(p.w + rr * rb, uu, r.a);
        if (PAIR) U::load_w(p.w2 + rr * rb, uu, r.b);
    };
#pragma unroll
    for (int j = 0; j < PD; ++j)
        if (item + j * workers < items) fetch(buf[j], item + j * workers);
    // The activation slice of the lane's unit position stays in registers across problems
    // that read the same activations (xgroup names what is loaded).
    if (xgroup != p.xgroup) {
        U::load_x(p.x, p.xdt, uu, xr, aux);
        if (!active) {
#pragma unroll
            for (int i = 0; i < 64; ++i) xr[i] = 0.f;
#pragma unroll
            for (int i = 0; i < U::AUX; ++i) aux[i] = 0.f;
        }
        xgroup = p.xgroup;
    }
    int slot = 0;
    bool done = false;
    while (!done) {
#pragma unroll
        for (int s = 0; s <= PD; ++s) {
            if (done) break;
            const int ahead = item + PD * workers;
            if (ahead < items) fetch(buf[(s + PD) % (PD + 1)], ahead);
            const bool more = item + workers < items;
            const int row = item * RPW + sub;
            const float g = group_sum<LR>(U::dot(buf[s].a, xr, aux));
            float v = g;
            if (PAIR) {
                const float up = group_sum<LR>(U::dot(buf[s].b, xr, aux));
                if (WR == 1) v = silu_mul(g, up);
                else if (lane == 63) { partial[(slot * 2) * WR + wave] = g; partial[(slot * 2 + 1) * WR + wave] = up; }
            } else if (WR > 1) {
                if (lane == 63) partial[slot * WR + wave] = g;
            }
            if (WR == 1) {
                if ((lane % LR) == LR - 1 && row < p.n) store_out(p.y, p.ydt, row, v);
            } else {
                // rows of a workgroup-shared problem: the waves' partial sums meet in LDS
                ++slot;
                if (slot == 32 || !more) {
                    __syncthreads();
                    const int t = threadIdx.x;
                    if (t < slot) {
                        const int r2 = item - (slot - 1 - t) * workers;  // RPW == 1 when WR > 1
                        float sg = 0.f, su = 0.f;
#pragma unroll
                        for (int wv = 0; wv < WR; ++wv) {
                            if (PAIR) { sg += partial[(t * 2) * WR + wv]; su += partial[(t * 2 + 1) * WR + wv]; }
                            else sg += partial[t * WR + wv];
                        }
                        store_out(p.y, p.ydt, r2, PAIR ? silu_mul(sg, su) : sg);
                    }
                    __syncthreads();
                    slot = 0;
                }
            }
            if (!more) done = true;
            item += workers;
        }
    }
}

template <int FMT, bool PAIR>
__device__ __forceinline__ void stream_dispatch_shape(const StreamProblem& p, float* partial, float (&xr)[64],
                                                      float (&aux)[8], int& xgroup) {
    const int units = p.k >> 6;
    // rows requested ahead: bounded by the 256-VGPR budget (a BF16 unit is 32 dwords per row)
    constexpr int PD = FMT == QMOE_FMT_BF16 ? (PAIR ? 0 : 1) : (PAIR ? 1 : 2);
    if (units <= 8) stream_problem<FMT, PAIR, 8, 1, PD>(p, partial, xr, aux, xgroup);
    else if (units <= 16) stream_problem<FMT, PAIR, 16, 1, PD>(p, partial, xr, aux, xgroup);
    else if (units <= 32) stream_problem<FMT, PAIR, 32, 1, PD>(p, partial, xr, aux, xgroup);
    else if (units <= 64) stream_problem<FMT, PAIR, 64, 1, PD>(p, partial, xr, aux, xgroup);
    else if (units <= 128) stream_problem<FMT, PAIR, 64, 2, PD>(p, partial, xr, aux, xgroup);
    else stream_problem<FMT, PAIR, 64, 4, PD>(p, partial, xr, aux, xgroup);
}

// All problems of one launch share the packed format and are all plain rows or all gate/up
// pairs.  Two waves per SIMD (at most 256 VGPRs).
template <int FMT, bool PAIR>
__global__ __launch_bounds__(STREAM_THREADS, 2) void stream_kernel(const StreamArgs args) {
    __shared__ float partial[32 * 2 * 4];
    float xr[64], aux[8];
    int xgroup = -1;
    for (int i = 0; i < args.count; ++i) stream_dispatch_shape<FMT, PAIR>(args.p[i], partial, xr, aux, xgroup);
}

// ---- host side ---------------------------------------------------------------------------------
bool stream_supported(int fmt, const void* w, int n, int k, const void* x, int xdt) {
    if (!(fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_BF16)) return false;
    if (k % 64 || k > 256 * 64 || n < 1) return false;
    if ((fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K) && (k % 256)) return false;
    const int align = fmt == QMOE_FMT_Q8_0 ? 4 : fmt == QMOE_FMT_Q6_K ? 2 : 16;
    if ((uintptr_t)w % align || row_bytes(fmt, k) % align) return false;
    return x_fast(x, xdt, k);
}

static int stream_grid() {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 512;
        cus = prop.multiProcessorCount;
    }
    return cus * 2;
}

// Enqueue up to STREAM_MAX_PROBLEMS problems of ONE packed format -- all plain or all gate/up
// pairs -- as one launch.  All entries must satisfy stream_supported (pairs: both matrices).
int stream_launch(StreamArgs& args, hipStream_t s) {
    const int grid = stream_grid();
    const int waves = grid * STREAM_WAVES;
    long cursor = 0;  // next free worker, counted in waves
    int group = 0;
    for (int i = 0; i < args.count; ++i) {
        StreamProblem& p = args.p[i];
        const int units = p.k >> 6;
        const int lr = units <= 8 ? 8 : units <= 16 ? 16 : units <= 32 ? 32 : 64;
        const int items = (p.n + 64 / lr - 1) / (64 / lr);
        if (units > 64) {  // rows shared by the waves of a workgroup: workgroup-granular round robin
            p.first_item = (int)((cursor / STREAM_WAVES) % grid);
            cursor += (long)items * STREAM_WAVES;
        } else {
            p.first_item = (int)(cursor % waves);
            cursor += items;
        }
        // consecutive problems reading the same activations keep them in registers
        if (i > 0 && (p.x != args.p[i - 1].x || p.k != args.p[i - 1].k || p.xdt != args.p[i - 1].xdt)) ++group;
        p.xgroup = group;
    }
    const dim3 g(grid), b(STREAM_THREADS);
    const bool pair = args.p[0].w2 != nullptr;
#define QMOE_STREAM(F)                                                                         \
    if (pair) hipLaunchKernelGGL((stream_kernel<F, true>), g, b, 0, s, args);                 \
    else hipLaunchKernelGGL((stream_kernel<F, false>), g, b, 0, s, args)
    switch (args.p[0].fmt) {
    case QMOE_FMT_Q8_0: QMOE_STREAM(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_STREAM(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_STREAM(QMOE_FMT_Q5_K); break;
    default: QMOE_STREAM(QMOE_FMT_BF16); break;
    }
#undef QMOE_STREAM
    return check_launch("stream kernel");
}

}  // namespace qmoe
