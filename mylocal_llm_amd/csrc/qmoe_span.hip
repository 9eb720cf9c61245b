// Persistent single-token streaming kernel, rows staged through LDS rings (see qmoe_span.hpp).
//
// One workgroup of eight waves per CU; every wave runs on its own, no barrier after the start.
// The launch's problems are cut into work items -- groups of 1..8 whole rows of up to 4096
// columns, or one wider row taken in parts of 4096 columns -- numbered through all problems, and
// wave w of the grid takes the items w, w + W, ...: at any moment the whole chip streams one
// window of neighbouring rows.  A wave's request side runs ahead of its multiplying side across
// problem boundaries, so its ring never drains between matrices.
//
// Activation rows live in LDS as fp32.  Two of them fit side by side (one from the front of the
// area, the next from its back, and so on in turn): while the waves multiply with one, the row
// of the next problems is already being fetched, each wave bringing an eighth of it and counting
// itself in; a wave enters the next problems when all eight have counted in, and overwrites a row
// only when all eight have left it.
#include "qmoe_span.hpp"
#include "qmoe_rowdot.hpp"

namespace qmoe {

#define QMOE_LDS __attribute__((address_space(3)))
typedef QMOE_LDS uint32_t* lds_counter;

// Rows of one work item and 4096-column parts of a row.
__host__ __device__ inline int span_parts(int k) { return ((k >> 6) + 63) >> 6; }
__host__ __device__ inline int span_rows_per_item(int k) { return (k >> 6) <= 64 ? 64 / lanes_per_row(k) : 1; }

template <int FMT, int PD> struct SpanLayout {   // dynamic LDS: rings | counters | dump | activations
    static constexpr int SLOT = SpanSlot<FMT>::BYTES;
    static constexpr int RING = (PD + 1) * SLOT;
    static constexpr int FLAGS = SPAN_WAVES * RING;          // ready[16], left[16], next item of the workgroup
    static constexpr int DUMP = FLAGS + (2 * SPAN_MAX_KEYS + 4) * 4;
    static constexpr int QUEUE = DUMP + SPAN_WAVES * 16;     // per wave: the items requested and not yet multiplied
    static constexpr int XS = QUEUE + SPAN_WAVES * 8 * 4;
    static constexpr int TOTAL = 160 * 1024;
    static constexpr int XS_BYTES = (TOTAL - XS) & ~1023;
};

template <int FMT, bool PAIR, int PD>
__global__ __launch_bounds__(SPAN_THREADS, 1) void span_kernel(const SpanArgs args) {
    using U = Unit64<FMT>;
    using S = SpanFmt<FMT>;
    using SL = SpanSlot<FMT>;
    using L = SpanLayout<FMT, PD>;
    constexpr int SLOT = L::SLOT, RING = L::RING;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = uniform((int)(threadIdx.x >> 6));
    const int W = gridDim.x * SPAN_WAVES, me = blockIdx.x * SPAN_WAVES + wave;
    // Round r of the item sequence is the items r W ... r W + W - 1, of which this workgroup takes
    // the eight at 8 blockIdx.x ...; its waves draw them from a counter in LDS as they get to them
    // (the two waves of a SIMD do not run at the same speed: the older one is served first).
    uint8_t* const ring = lds + wave * RING;
    const uint32_t ring0 = (uint32_t)(uintptr_t)ring;
    const lds_counter ready = (lds_counter)(lds + L::FLAGS);  // waves whose share of a row has arrived
    const lds_counter left = ready + SPAN_MAX_KEYS;           // waves that are through with a row
    const lds_counter drawn = left + SPAN_MAX_KEYS;           // items of this workgroup handed out so far
    const uint32_t dump = (uint32_t)(uintptr_t)(lds + L::DUMP + wave * 16);
    QMOE_LDS int* const queue = (QMOE_LDS int*)(lds + L::QUEUE) + wave * 8;
    uint8_t* const xs = lds + L::XS;
    // Every cache line of the arguments is requested now, in one go: the scalar loads further
    // down (problem after problem, each waiting for the one before) then hit the scalar cache.
    {
        const auto ka = __builtin_amdgcn_kernarg_segment_ptr();
        int t0, t1, t2, t3, t4, t5, t6, t7, t8, t9;
        asm volatile("s_load_dword %0, %10, 0x0\n\ts_load_dword %1, %10, 0x80\n\ts_load_dword %2, %10, 0x100\n\t"
                     "s_load_dword %3, %10, 0x180\n\ts_load_dword %4, %10, 0x200\n\ts_load_dword %5, %10, 0x280\n\t"
                     "s_load_dword %6, %10, 0x300\n\ts_load_dword %7, %10, 0x380\n\ts_load_dword %8, %10, 0x400\n\t"
                     "s_load_dword %9, %10, 0x480"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7), "=&s"(t8), "=&s"(t9)
                     : "s"(ka) : "memory");
        if (threadIdx.x <= 2 * SPAN_MAX_KEYS) ready[threadIdx.x] = threadIdx.x == 2 * SPAN_MAX_KEYS ? SPAN_WAVES : 0;
        asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(t0), "+s"(t1), "+s"(t2), "+s"(t3), "+s"(t4), "+s"(t5), "+s"(t6), "+s"(t7), "+s"(t8), "+s"(t9) :: "memory");
    }
    static_assert(sizeof(SpanArgs) <= 0x500, "argument lines requested at the start");
    const uint8_t* const any_w = args.p[0].w;   // a valid address for requests that carry nothing

    // ---- request side -----------------------------------------------------------------------
    int f_pi = -1, f_t = 0, f_items = 0, f_first = 0, f_g = 0, f_count = 0, f_e = 0, f_parts = 1, f_rpi = 1, f_n = 0, f_k = 256, f_m = 0;
    const uint8_t *f_w = nullptr, *f_w2 = nullptr;
    int64_t f_rb = 0;
    bool f_done = false;
    uint32_t f_slot = 0;
    const uint32_t voff0 = lane * 16, voff_last = S::src(lane + 64 * (SL::CHUNKS - 1));
    const uint64_t last_mask = SL::LAST_LANES >= 64 ? ~0ull : ((1ull << SL::LAST_LANES) - 1);

    // the next item of the workgroup, as an item of the launch
    // The next item of the workgroup, as an item of the launch: batch b of the workgroup is batch
    // b G + c of the launch (G workgroups), its eight items go to the waves in the order they ask.
    auto draw = [&] {
        int got = 0;
        if (lane == 0) got = (int)__atomic_fetch_add(drawn, 1u, __ATOMIC_RELAXED);   // (one lane: one item)
        const int idx = uniform(got);
        const int b = idx >> 3, pos = idx & 7;
        const long long item = ((long long)b * gridDim.x + blockIdx.x) * SPAN_WAVES + pos;
        f_g = item < args.items ? (int)item : args.items;
        if (f_g < args.items) queue[f_count++ & 7] = f_g;
    };
    auto next_problem = [&] {
        while (true) {
            ++f_pi;
            if (f_pi >= args.count || f_g >= args.items) { f_done = true; return; }
            const SpanProblem& p = args.p[f_pi];
            const int first = p.first_item, items = p.end_item - first;
            if (f_g >= p.end_item) continue;   // (f_g: my next item of the launch, always >= first here)
            f_first = first;
            f_k = p.k;
            f_n = p.n;
            f_w = p.w;
            if (PAIR) f_w2 = p.w2;
            f_parts = span_parts(f_k);
            f_rpi = span_rows_per_item(f_k);
            f_rb = row_bytes_dev(FMT, f_k);
            f_items = items;
            f_t = f_g - first;
            f_e = 0;
            return;
        }
    };
    // One span into the slot at f_slot -- always SL::CHUNKS load instructions, so that the wait
    // for a span is a constant: requests that carry nothing fetch 16 bytes into a dump.
    auto issue = [&] {
        const uint8_t* m = any_w;
        int quads = 0;
        if (!f_done) {
            const int row0 = f_t * f_rpi;
            if (f_parts == 1) {
                const int rows = f_n - row0 < f_rpi ? f_n - row0 : f_rpi;
                m = ((PAIR && f_m) ? f_w2 : f_w) + (int64_t)row0 * f_rb;
                quads = rows * (f_k >> 8);
            } else {
                const int mu = (f_k >> 6) - f_e * 64;
                m = f_w + (int64_t)row0 * f_rb + (int64_t)f_e * 16 * S::MEM4;
                quads = (mu > 64 ? 64 : mu) >> 2;
            }
        }
        const uint32_t at = ring0 + f_slot;
        if (quads == 16) {   // a whole slot: straight-line requests, the last one on LAST_LANES lanes
            if (S::LINEAR) {
                set_m0(at);
                QMOE_DMA16(m, voff0, 0);
                if (SL::CHUNKS > 2) QMOE_DMA16(m, voff0, 1024);
                if (SL::CHUNKS > 3) QMOE_DMA16(m, voff0, 2048);
                if (SL::CHUNKS > 4) QMOE_DMA16(m, voff0, 3072);
            } else {
#pragma unroll
                for (int j = 0; j + 1 < SL::CHUNKS; ++j) {
                    set_m0(at + 1024 * j);
                    const uint32_t o = S::src(lane + 64 * j);
                    QMOE_DMA16(m, o, 0);
                }
            }
            set_m0(at + (SL::CHUNKS - 1) * 1024);
            dma16_masked(m, voff_last, last_mask);
        } else {
            const int pieces = quads * S::PP4;
#pragma unroll
            for (int j = 0; j < SL::CHUNKS; ++j) {
                const int cnt = pieces - 64 * j;
                if (cnt > 0) {
                    set_m0(at + 1024 * j);
                    const uint32_t o = S::src(lane + 64 * j);
                    dma16_masked(m, o, cnt >= 64 ? ~0ull : ((1ull << cnt) - 1));
                } else {
                    set_m0(dump);
                    dma16_masked(any_w, 0u, 1ull);
                }
            }
        }
    };
    // ... and on to the span after it
    auto advance = [&] {
        if (f_done) return;
        f_slot = f_slot + SLOT == RING ? 0 : f_slot + SLOT;
        if (f_parts > 1) {
            if (++f_e < f_parts) return;
            f_e = 0;
        } else if (PAIR) {
            f_m ^= 1;
            if (f_m) return;
        }
        draw();
        f_t = f_g - f_first;
        if (f_t >= f_items) next_problem();
    };
    auto request = [&] {
        issue();
        advance();
    };

    // ---- activation rows ------------------------------------------------------------------------
    uint32_t sig_keys = 0;   // rows whose share this wave has requested but not yet counted in
    int sig_wait = 0;        // spans to wait for before those requests are certainly complete
    auto x_fetch = [&](int key) {
        const SpanKey& xk = args.key[key];
        const int chunks = xk.k >> 8;   // 1 KB of fp32 each
        uint8_t* const dst = xs + xk.offset;
        if (xk.xdt == QMOE_DT_F32) {
            const uint8_t* const src = (const uint8_t*)xk.x;
            for (int c = wave; c < chunks; c += SPAN_WAVES) {
                set_m0((uint32_t)(uintptr_t)dst + 1024 * c);
                const uint32_t o = 16 * swizzled_granule(lane + 64 * c);
                QMOE_DMA16(src, o, 0);
            }
            sig_keys |= 1u << key;
            sig_wait = PD + 1;
        } else {
            for (int c = wave; c < chunks; c += SPAN_WAVES) {
                const int g = lane + 64 * c;
                const float4 v = load_x4(xk.x, xk.xdt, 4 * g);
                *(float4*)(dst + 16 * swizzled_granule(g)) = v;
            }
            sig_keys |= 1u << key;   // (counted in at the next span, like the requests above)
            sig_wait = 1;
        }
    };
    auto count_in = [&] {
#pragma unroll 1
        for (uint32_t m = sig_keys; m; m &= m - 1)
            if (lane == 0) __atomic_fetch_add(&ready[__builtin_ctz(m)], 1u, __ATOMIC_RELAXED);
        sig_keys = 0;
    };
    // wait for the oldest outstanding span: everything but the requests of the PD newer ones
    auto arrive = [&] {
        wait_vmcnt<PD * SL::CHUNKS>();
        if (sig_keys && --sig_wait == 0) count_in();
    };
    // A wait for the other waves of the workgroup is bounded in wall-clock time (args.wait_ticks of
    // the 100 MHz counter; far longer than any launch streams).  A wave whose wait expires does not
    // hang and does not pretend: it raises the launch's status word with a vector store, stores no
    // more results, and runs on to its end so that every request it has made drains.  A negative
    // limit makes every wait expire at once (a host-forced run of this branch).
    bool failed = false;
    auto spin_until = [&](lds_counter counter) {
        bool ok = args.wait_ticks >= 0 && *(volatile QMOE_LDS uint32_t*)counter >= SPAN_WAVES;
        if (!ok && args.wait_ticks >= 0) {
            const uint64_t t0 = wall_clock64();
            do {
                __builtin_amdgcn_s_sleep(1);
                ok = *(volatile QMOE_LDS uint32_t*)counter >= SPAN_WAVES;
            } while (!ok && (int64_t)(wall_clock64() - t0) <= args.wait_ticks);
        }
        if (!uniform((int)ok) && !failed) {
            failed = true;
            if (lane == 0) stg<uint32_t>(args.status, QMOE_STATUS_WAIT_EXPIRED);
        }
    };

    // The first item of every wave is fixed (item `me`), so its request and the first activation
    // rows leave before the workgroup's waves meet; the barrier (which waits for this wave's own
    // requests, as the first multiplication has to anyway) publishes the counters, and only then
    // does anybody draw or count.
    f_g = me < args.items ? me : args.items;   // (batch c of the workgroup, position `wave`)
    if (f_g < args.items) queue[f_count++ & 7] = f_g;
    next_problem();
    issue();
    int fetched = -1;  // rows 0..fetched have been requested by this wave
    x_fetch(0);
    fetched = 0;
    if (args.keys > 1) { x_fetch(1); fetched = 1; }
    __syncthreads();
    advance();
#pragma unroll
    for (int j = 1; j < PD; ++j) request();

    // ---- multiplying side ---------------------------------------------------------------------
    uint32_t c_slot = 0;
    // my next item of the launch: the oldest of the queue (the request side is ahead by at
    // least one item whenever there is one)
    int c_count = 0, c_g = 0;
    auto c_next = [&] {
        c_g = c_count < f_count ? uniform(queue[c_count & 7]) : args.items;
        ++c_count;
    };
    c_next();
    int cur_key = -1, sliced_key = -1;
    const uint8_t* xrow = xs;
    float xr[64], aux[8];
    for (int pi = 0; pi < args.count; ++pi) {
        const SpanProblem& p = args.p[pi];
        const int key = p.key;
        if (key != cur_key) {
            if (cur_key >= 0 && lane == 0) __atomic_fetch_add(&left[cur_key], 1u, __ATOMIC_RELAXED);
            cur_key = key;
            while (fetched < key) {   // (normally fetched long ago, see below)
                ++fetched;
                if (fetched >= 2) spin_until(&left[fetched - 2]);
                x_fetch(fetched);
            }
            if (sig_keys) {
                wait_vmcnt<0>();
                                count_in();
            }
            spin_until(&ready[key]);
            xrow = xs + args.key[key].offset;
                    }
        const int first = p.first_item, end = p.end_item;
        if (c_g >= end) continue;
        const int k = p.k, n = p.n, units = k >> 6, ydt = p.ydt;
        void* const y = p.y;
        // the row after this one is fetched as soon as every wave has left the row before this one
        auto look_ahead = [&] {
            if (fetched == key && key + 1 < args.keys && (key < 1 || *(volatile QMOE_LDS uint32_t*)&left[key - 1] >= SPAN_WAVES)) {
                x_fetch(key + 1);
                fetched = key + 1;
            }
        };
        if (units <= 64) {
            const int lr = lanes_per_row(k), rpi = 64 / lr;
            const int u = lane & (lr - 1), sub = lane / lr;
            const bool active = u < units;
            if (sliced_key != key) {
                U::load_x(SwizzledX{xrow}, active ? u : 0, xr, aux);
                sliced_key = key;
                            }
            const uint32_t lane_off = sub * ((k >> 8) * S::PP4 * 16) + S::unit_offset(active ? u : 0);
            for (; c_g < end; c_next()) {
                const int t = c_g - first;
                if (fetched == key) look_ahead();
                request();
                arrive();
                uint32_t r[U::RAW];
                S::read(ring + c_slot + lane_off, u, r);
                float v = U::dot(r, xr, aux);
                v = group_sum_rt(active ? v : 0.f, lr);   // (a lane without a unit has read bytes of another one)
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot may be requested into again
                c_slot = c_slot + SLOT == RING ? 0 : c_slot + SLOT;
                if (PAIR) {
                    request();
                    arrive();
                    S::read(ring + c_slot + lane_off, u, r);
                    float up = U::dot(r, xr, aux);
                    up = group_sum_rt(active ? up : 0.f, lr);
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    c_slot = c_slot + SLOT == RING ? 0 : c_slot + SLOT;
                    v = silu_mul(v, up);
                }
                const int row = t * rpi + sub;
                if (u == lr - 1 && row < n && !failed) store_out(y, ydt, row, v);
            }
        } else {
            // a wider row: its parts of 4096 columns one after the other, the lane's slice of the
            // activations re-read for every part, one reduction per row
            const int parts = span_parts(k);
            const uint32_t lane_off = S::unit_offset(lane);
            sliced_key = -1;
            for (; c_g < end; c_next()) {
                const int t = c_g - first;
                float acc = 0.f;
                for (int e = 0; e < parts; ++e) {
                    if (fetched == key) look_ahead();
                    request();
                    const int u = e * 64 + lane;
                    const bool active = u < units;
                    U::load_x(SwizzledX{xrow}, active ? u : 0, xr, aux);
                    arrive();
                    uint32_t r[U::RAW];
                    S::read(ring + c_slot + lane_off, lane, r);
                    const float d = U::dot(r, xr, aux);
                    acc += active ? d : 0.f;
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    c_slot = c_slot + SLOT == RING ? 0 : c_slot + SLOT;
                }
                acc = group_sum<64>(acc);
                if (lane == 63 && !failed) store_out(y, ydt, t, acc);
            }
        }
    }
    if (cur_key >= 0 && lane == 0) __atomic_fetch_add(&left[cur_key], 1u, __ATOMIC_RELAXED);
    wait_vmcnt<0>();
}

// ---- host side ---------------------------------------------------------------------------------
// Items, activation rows and their places in LDS; false if the launch is not one the span kernel
// takes: Q8_0 and the K-quants, rows of whole 256-column groups that start 16-byte aligned (Q6_K:
// 2-byte aligned), gate/up pairs only with rows of up to 4096 columns, and every two consecutive
// activation rows fit the LDS area together.
template <int FMT, int PD>
static bool span_plan(const StreamArgs& in, SpanArgs* out) {
    constexpr int area = SpanLayout<FMT, PD>::XS_BYTES;
    SpanArgs a;
    a.count = in.count;
    a.pad = 0;
    // Order: the caller's first problems with rows of up to 4096 columns that share one activation
    // row (a small row to wait for at the start), then the problems with wider rows, widest first
    // (their items are the largest: taken last they would leave most waves idle while a few
    // finish), then the rest in the caller's order.
    int order[STREAM_MAX_PROBLEMS], placed = 0;
    bool taken[STREAM_MAX_PROBLEMS] = {};
    for (int i = 0; i < in.count && span_parts(in.p[i].k) == 1; ++i) {
        if (i > 0 && !(in.p[i].x == in.p[i - 1].x && in.p[i].k == in.p[i - 1].k && in.p[i].xdt == in.p[i - 1].xdt)) break;
        order[placed++] = i;
        taken[i] = true;
    }
    for (int parts = span_parts(STREAM_MAX_K); parts >= 1; --parts)
        for (int i = 0; i < in.count; ++i)
            if (!taken[i] && span_parts(in.p[i].k) == parts) order[placed++] = i;
    int items = 0, key = -1, prev_bytes = 0;
    for (int i = 0; i < in.count; ++i) {
        const StreamProblem& q = in.p[order[i]];
        SpanProblem& p = a.p[i];
        p.w = q.w; p.w2 = q.w2; p.y = q.y; p.n = q.n; p.k = q.k; p.ydt = q.ydt;
        const int rpi = span_rows_per_item(q.k);
        p.first_item = items;
        items += (q.n + rpi - 1) / rpi;
        p.end_item = items;
        const StreamProblem* const before = i > 0 ? &in.p[order[i - 1]] : nullptr;
        const bool same = before && q.x == before->x && q.k == before->k && q.xdt == before->xdt;
        if (!same) {
            ++key;
            const int bytes = q.k * 4;
            if (bytes + prev_bytes > area) return false;
            a.key[key] = SpanKey{q.x, q.k, q.xdt, (key & 1) ? area - bytes : 0, 0};
            prev_bytes = bytes;
        }
        p.key = key;
    }
    a.keys = key + 1;
    a.items = items;
    a.status = nullptr;      // (the launcher fills in the device's status word and the wait limit)
    a.wait_ticks = 0;
    if (out) *out = a;
    return true;
}

static bool span_basic(const StreamArgs& args) {
    for (int i = 0; i < args.count; ++i) {
        const StreamProblem& p = args.p[i];
        if (!(p.fmt == QMOE_FMT_Q8_0 || p.fmt == QMOE_FMT_Q6_K || p.fmt == QMOE_FMT_Q5_K || p.fmt == QMOE_FMT_Q4_K)) return false;
        if (p.fmt != args.p[0].fmt || (p.w2 != nullptr) != (args.p[0].w2 != nullptr)) return false;
        if (p.k % 256 || p.k > STREAM_MAX_K || p.n < 1) return false;
        const int align = p.fmt == QMOE_FMT_Q6_K ? 2 : 16;
        if ((uintptr_t)p.w % align || (p.w2 && (uintptr_t)p.w2 % align)) return false;
        if (p.w2 && p.k > 4096) return false;
        if (!x_fast(p.x, p.xdt, p.k)) return false;
    }
    return args.count > 0;
}

template <int FMT, bool PAIR, int PD>
static int span_launch_as(SpanArgs& args, hipStream_t s) {
    static bool configured = false;   // (benign if two threads both set it)
    constexpr int lds = SpanLayout<FMT, PD>::TOTAL;
    if (int rc = launch_status_word(&args.status)) return rc;
    args.wait_ticks = wait_limit_ticks();
    if (!configured) {
        if (hipFuncSetAttribute((const void*)span_kernel<FMT, PAIR, PD>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return fail(QMOE_ELAUNCH, "span kernel: cannot reserve %d bytes of LDS", lds);
        configured = true;
    }
    const int grid = stream_grid() / 2;   // one workgroup per CU
    hipLaunchKernelGGL((span_kernel<FMT, PAIR, PD>), dim3(grid), dim3(SPAN_THREADS), lds, s, args);
    return check_launch("span kernel");
}

template <int FMT, int PD0>
static int span_launch_fmt(const StreamArgs& in, bool pair, hipStream_t s) {
    SpanArgs a;
    if (span_plan<FMT, PD0>(in, &a)) return pair ? span_launch_as<FMT, true, PD0>(a, s) : span_launch_as<FMT, false, PD0>(a, s);
    if (PD0 > 1 && span_plan<FMT, (PD0 > 1 ? PD0 - 1 : 1)>(in, &a))
        return pair ? span_launch_as<FMT, true, (PD0 > 1 ? PD0 - 1 : 1)>(a, s) : span_launch_as<FMT, false, (PD0 > 1 ? PD0 - 1 : 1)>(a, s);
    return fail(QMOE_EUNSUPPORTED, "span kernel: activation rows do not fit");
}

// Depth of the ring tried first per format; one less if the activation rows then do not fit.
bool span_supported(const StreamArgs& args) {
    if (!span_basic(args)) return false;
    switch (args.p[0].fmt) {
    case QMOE_FMT_Q8_0: return span_plan<QMOE_FMT_Q8_0, 2>(args, nullptr) || span_plan<QMOE_FMT_Q8_0, 1>(args, nullptr);
    case QMOE_FMT_Q6_K: return span_plan<QMOE_FMT_Q6_K, 2>(args, nullptr) || span_plan<QMOE_FMT_Q6_K, 1>(args, nullptr);
    case QMOE_FMT_Q5_K: return span_plan<QMOE_FMT_Q5_K, 3>(args, nullptr) || span_plan<QMOE_FMT_Q5_K, 2>(args, nullptr);
    default: return span_plan<QMOE_FMT_Q4_K, 3>(args, nullptr) || span_plan<QMOE_FMT_Q4_K, 2>(args, nullptr);
    }
}

int span_launch(const StreamArgs& in, hipStream_t s) {
    const bool pair = in.p[0].w2 != nullptr;
    switch (in.p[0].fmt) {
    case QMOE_FMT_Q8_0: return span_launch_fmt<QMOE_FMT_Q8_0, 2>(in, pair, s);
    case QMOE_FMT_Q6_K: return span_launch_fmt<QMOE_FMT_Q6_K, 2>(in, pair, s);
    case QMOE_FMT_Q5_K: return span_launch_fmt<QMOE_FMT_Q5_K, 3>(in, pair, s);
    default: return span_launch_fmt<QMOE_FMT_Q4_K, 3>(in, pair, s);
    }
}

}  // namespace qmoe
