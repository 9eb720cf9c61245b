// Persistent single-token streaming kernel over a list of problems.
//
// One launch walks a list of independent problems (y = W x, or h = silu(G x) * (U x)) with a
// fixed grid of 2 workgroups per CU.  Inside a problem every wave keeps taking the next
// unprocessed row (or group of short rows) in round-robin order that continues across
// problem boundaries, so the HBM stream never drains between matrices; the activation
// slice of a new problem is fetched together with that problem's first rows.
#include "qmoe_span.hpp"
#include "qmoe_rowdot.hpp"

namespace qmoe {

// All problems of one launch share the packed format and are all plain rows or all gate/up
// pairs.  Two waves per SIMD (at most 256 VGPRs).
template <int FMT, bool PAIR>
__global__ __launch_bounds__(STREAM_THREADS, 2) void stream_kernel(const StreamArgs args) {
    __shared__ float partial[32 * 2 * 4];
    __shared__ StreamProblem probs[STREAM_MAX_PROBLEMS];
    __shared__ __attribute__((aligned(16))) float xs[STREAM_XS_FLOATS];
    if ((int)threadIdx.x < args.count) probs[threadIdx.x] = args.p[threadIdx.x];
    // Every activation row the flat stream will need is fetched at the start: a wave that moves
    // on to the next matrix finds its activations in LDS instead of waiting for them.  The
    // loads leave first; the wave then requests its first weight rows, and only then stores the
    // activations (which arrive first) and meets the other waves: the rows travel meanwhile.
    constexpr int STRIPE = STREAM_XS_FLOATS / STREAM_WAVES;
    float4 v[STREAM_WAVES][4];
    if (args.groups > 0) {
#pragma unroll
        for (int g = 0; g < STREAM_WAVES; ++g) {
            const StreamProblem& p = args.p[args.group_problem[g < args.groups ? g : 0]];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = 4 * threadIdx.x + 1024 * i;
                if (g < args.groups && col < p.k) v[g][i] = load_x4(p.x, p.xdt, col);
            }
        }
    }
    __syncthreads();   // the problem list is in LDS
    auto store_x = [&] {
        if (args.groups > 0) {
#pragma unroll
            for (int g = 0; g < STREAM_WAVES; ++g) {
                const int pk = args.p[args.group_problem[g < args.groups ? g : 0]].k;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int col = 4 * threadIdx.x + 1024 * i;
                    if (g < args.groups && col < pk) *(float4*)(xs + g * STRIPE + StagedX::at(col)) = v[g][i];
                }
            }
        }
        __syncthreads();
    };
    // (measured per format: Q6_K, whose rows are requested two steps ahead, is faster the plain way)
    if (FMT == QMOE_FMT_Q6_K) {
        store_x();
        stream_run<FMT, PAIR, true>(probs, args.count, 0, args.flat_items, false, partial, xs, args.groups > 0 ? xs : nullptr);
    } else {
        stream_run<FMT, PAIR, true>(probs, args.count, 0, args.flat_items, false, partial, xs, args.groups > 0 ? xs : nullptr,
                                    STREAM_XS_FLOATS / STREAM_WAVES, store_x);
    }
}

// ---- host side ---------------------------------------------------------------------------------
bool stream_supported(int fmt, const void* w, int n, int k, const void* x, int xdt) {
    if (!(fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q4_K || fmt == QMOE_FMT_BF16)) return false;
    if (k % 64 || k > 256 * 64 || n < 1) return false;
    if ((fmt == QMOE_FMT_Q6_K || fmt == QMOE_FMT_Q5_K || fmt == QMOE_FMT_Q4_K) && (k % 256)) return false;
    const int align = fmt == QMOE_FMT_Q8_0 ? 4 : fmt == QMOE_FMT_Q6_K ? 2 : 16;
    if ((uintptr_t)w % align || row_bytes(fmt, k) % align) return false;
    return x_fast(x, xdt, k);
}

int stream_grid() {
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
    if (span_supported(args)) return span_launch(args, s);
    const int grid = stream_grid();
    int flat = 0;   // global work items of the problems whose rows fit one wave
    int group = -1, wide_group = 1 << 20;
    const StreamProblem *last_narrow = nullptr, *last_wide = nullptr;
    bool fits = true;
    for (int i = 0; i < args.count; ++i) {
        StreamProblem& p = args.p[i];
        const int units = p.k >> 6;
        if (units > 64) {  // rows shared by the waves of a workgroup: workgroup-granular round robin
            p.first_item = flat % grid;
            p.flat_end = 0;
        } else {
            const int rpw = 64 / lanes_per_row(p.k);
            p.first_item = flat;
            flat += (p.n + rpw - 1) / rpw;
            p.flat_end = flat;
        }
        // consecutive problems reading the same activations keep them in registers; the groups
        // of the flat stream are numbered 0, 1, ... (their LDS stripes), the others apart
        if (units > 64) {
            if (last_wide && (p.x != last_wide->x || p.k != last_wide->k || p.xdt != last_wide->xdt)) ++wide_group;
            p.xgroup = wide_group;
            last_wide = &p;
        } else {
            if (!last_narrow || p.x != last_narrow->x || p.k != last_narrow->k || p.xdt != last_narrow->xdt) {
                ++group;
                if (group < STREAM_WAVES) args.group_problem[group] = i; else fits = false;
            }
            p.xgroup = group;
            last_narrow = &p;
        }
    }
    args.groups = fits ? group + 1 : 0;
    for (int g = args.groups > 0 ? args.groups : 0; g < STREAM_WAVES; ++g) args.group_problem[g] = 0;
    // the flat search skips problems with an empty range: give wide problems the running end
    int running = 0;
    for (int i = 0; i < args.count; ++i) {
        if ((args.p[i].k >> 6) > 64) args.p[i].flat_end = running; else running = args.p[i].flat_end;
    }
    args.flat_items = flat;
    const dim3 g(grid), b(STREAM_THREADS);
    const bool pair = args.p[0].w2 != nullptr;
#define QMOE_STREAM(F)                                                                         \
    if (pair) hipLaunchKernelGGL((stream_kernel<F, true>), g, b, 0, s, args);                 \
    else hipLaunchKernelGGL((stream_kernel<F, false>), g, b, 0, s, args)
    switch (args.p[0].fmt) {
    case QMOE_FMT_Q8_0: QMOE_STREAM(QMOE_FMT_Q8_0); break;
    case QMOE_FMT_Q6_K: QMOE_STREAM(QMOE_FMT_Q6_K); break;
    case QMOE_FMT_Q5_K: QMOE_STREAM(QMOE_FMT_Q5_K); break;
    case QMOE_FMT_Q4_K: QMOE_STREAM(QMOE_FMT_Q4_K); break;
    default: QMOE_STREAM(QMOE_FMT_BF16); break;
    }
#undef QMOE_STREAM
    return check_launch("stream kernel");
}

}  // namespace qmoe
