// Packed-expert MoE step: device-side token->expert plan, grouped gate/up + SwiGLU, grouped
// down projection scaled by the route, ordered combine, shared expert with sigmoid gate.
//
// Data in the workspace (all indices are positions in the expert-sorted assignment list):
//   offsets[E+1]      exclusive prefix of per-expert assignment counts
//   active[E]         ids of experts with at least one assignment, ascending; n_active
//   sorted_token[A]   token of each sorted assignment (ascending token inside an expert)
//   sorted_weight[A]  its routing weight
//   pos_of[T*k]       sorted position of assignment (t, slot)
//   hidden_act[A, F]  fp32 SwiGLU activations, terms[A, D] fp32 weighted expert outputs
// with A = T*k.  Nothing is read back by the host.
#include "qmoe_decode.hpp"
#include "qmoe_gemm.hpp"
#include "qmoe_rowdot.hpp"
#include <mutex>

#include "qmoe_stream.hpp"

namespace qmoe {

int linear_impl(const void* w, int fmt, int n, int k, const void* x, int xdt, int tokens, void* y, int ydt, hipStream_t s);
int swiglu_impl(const void* gate, int gf, const void* up, int uf, int f, int k, const void* x, int xdt, int tokens,
                void* h, int hdt, hipStream_t s);
int router_topk_impl(const float* logits, int tokens, int n, int k, float floor_value, int renorm, float* weights,
                     int64_t* ids, hipStream_t s);

static constexpr int PLAN_THREADS = 1024;
// Up to 16 tokens take the decode path where it applies (it is asked first); shapes outside it
// (an expert width that is no power-of-two multiple of 128, a shared expert in another format ...)
// take the token-tile GEMMs at any token count: at 16 tokens an order of magnitude faster than the
// general kernels.
static constexpr int GEMM_MIN_TOKENS = 1;
static constexpr size_t PLAN_LDS_LIMIT = 60 * 1024;

// Block-wide exclusive scan of one int per thread (PLAN_THREADS threads); returns the
// exclusive prefix and leaves the grand total in *total.
__device__ int block_exclusive_scan(int v, int* wave_sums, int* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        int o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
    }
    if (lane == 63) wave_sums[wave] = incl;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int i = 0; i < PLAN_THREADS / 64; ++i) { int c = wave_sums[i]; wave_sums[i] = run; run += c; }
        *total = run;
    }
    __syncthreads();
    int result = wave_sums[wave] + incl - v;
    __syncthreads();
    return result;
}

// One workgroup builds the whole plan.  selection[e * words + t/32] bit t%32 says token t
// chose expert e; counts, offsets and ranks all come from popcounts of that bitmap, so the
// result does not depend on the order in which lanes ran.
__global__ __launch_bounds__(PLAN_THREADS) void moe_plan_kernel(const int64_t* __restrict__ ids,
                                                                 const float* __restrict__ weights, int tokens,
                                                                 int k, int n_experts, int* __restrict__ offsets,
                                                                 int* __restrict__ active, int* __restrict__ n_active,
                                                                 int* __restrict__ sorted_token,
                                                                 float* __restrict__ sorted_weight,
                                                                 int* __restrict__ pos_of, int* __restrict__ status,
                                                                 int* __restrict__ status_out,
                                                                 float* __restrict__ out_weights, int64_t* __restrict__ out_ids,
                                                                 int* __restrict__ chunk_expert,
                                                                 int* __restrict__ chunk_start,
                                                                 int* __restrict__ chunk_count,
                                                                 int* __restrict__ n_chunks,
                                                                 int* __restrict__ order) {
    extern __shared__ uint32_t selection[];  // n_experts*words bitmap, then n_experts offsets
    __shared__ int wave_sums[PLAN_THREADS / 64];
    __shared__ int total;
    const int words = (tokens + 31) / 32;
    const int tid = threadIdx.x;
    const int assignments = tokens * k;
    int* expert_offset = (int*)(selection + (size_t)n_experts * words);
    for (int i = tid; i < n_experts * words; i += PLAN_THREADS) selection[i] = 0u;
    if (tid == 0) *status = 0;
    __syncthreads();
    // An expert id outside the bank, or the same expert named again by a token, contributes nothing
    // (of a repeated expert the first slot counts); both are reported.
    int bad = 0;
    for (int a = tid; a < assignments; a += PLAN_THREADS) {
        const int64_t e = ids[a];
        const int t = a / k;
        if (out_weights && out_weights != weights) out_weights[a] = weights[a];   // routing given by the caller: hand it back
        if (out_ids && out_ids != ids) out_ids[a] = e;
        if (e < 0 || e >= n_experts) { bad |= 1; continue; }
        atomicOr(&selection[(int)e * words + (t >> 5)], 1u << (t & 31));
    }
    __syncthreads();
    // Per-thread chunk of consecutive experts -> counts -> two scans (sizes, non-empty flags).
    const int chunk = (n_experts + PLAN_THREADS - 1) / PLAN_THREADS;
    const int first = tid * chunk;
    int my_count = 0, my_active = 0, my_chunks = 0;
    for (int e = first; e < first + chunk && e < n_experts; ++e) {
        int c = 0;
        for (int w = 0; w < words; ++w) c += __popc(selection[e * words + w]);
        my_count += c;
        my_active += c > 0;
        my_chunks += (c + GEMM_CHUNK - 1) / GEMM_CHUNK;
    }
    int count_prefix = block_exclusive_scan(my_count, wave_sums, &total);
    const int all = total;
    int active_prefix = block_exclusive_scan(my_active, wave_sums, &total);
    const int all_active = total;
    int chunk_prefix = block_exclusive_scan(my_chunks, wave_sums, &total);
    for (int e = first; e < first + chunk && e < n_experts; ++e) {
        int c = 0;
        for (int w = 0; w < words; ++w) c += __popc(selection[e * words + w]);
        offsets[e] = count_prefix;
        expert_offset[e] = count_prefix;
        // the expert's assignments in chunks of GEMM_CHUNK tokens, for the token-tile GEMM
        for (int at = 0; chunk_expert && at < c; at += GEMM_CHUNK) {
            chunk_expert[chunk_prefix] = e;
            chunk_start[chunk_prefix] = count_prefix + at;
            chunk_count[chunk_prefix] = c - at < GEMM_CHUNK ? c - at : GEMM_CHUNK;
            ++chunk_prefix;
        }
        count_prefix += c;
        if (c > 0) active[active_prefix++] = e;
    }
    if (tid == 0) {
        offsets[n_experts] = all;
        *n_active = all_active;
        if (n_chunks) *n_chunks = total;
    }
    __syncthreads();
    for (int a = tid; a < assignments; a += PLAN_THREADS) {
        const int64_t e64 = ids[a];
        if (e64 < 0 || e64 >= n_experts) { pos_of[a] = -1; continue; }
        const int e = (int)e64, t = a / k;
        bool again = false;
        for (int j = t * k; j < a; ++j) again |= ids[j] == e64;
        if (again) { pos_of[a] = -1; bad |= 2; continue; }
        int rank = 0;
        for (int w = 0; w < (t >> 5); ++w) rank += __popc(selection[e * words + w]);
        rank += __popc(selection[e * words + (t >> 5)] & ((1u << (t & 31)) - 1u));
        const int pos = expert_offset[e] + rank;
        sorted_token[pos] = t;
        sorted_weight[pos] = weights[a];
        pos_of[a] = pos;
        if (order) order[pos] = a;
    }
    if (bad) {
        atomicOr(status, bad);
        if (status_out) atomicOr(status_out, bad);
    }
}

// gate/up + SwiGLU of every active expert over its own token list.
template <int XDT, int MT>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const uint8_t* __restrict__ gate, int gf, int64_t gstride,
                                                          int64_t grb, bool gfast, const uint8_t* __restrict__ up,
                                                          int uf, int64_t ustride, int64_t urb, bool ufast, int f,
                                                          int d, const void* __restrict__ x,
                                                          const int* __restrict__ offsets,
                                                          const int* __restrict__ active,
                                                          const int* __restrict__ n_active,
                                                          const int* __restrict__ sorted_token,
                                                          float* __restrict__ hidden_act) {
    if ((int)blockIdx.y >= *n_active) return;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= f) return;
    const int e = active[blockIdx.y];
    const int lo = offsets[e], cnt = offsets[e + 1] - lo;
    const uint8_t* grow = gate + (int64_t)e * gstride + (int64_t)row * grb;
    const uint8_t* urow = up + (int64_t)e * ustride + (int64_t)row * urb;
    for (int j0 = 0; j0 < cnt; j0 += MT) {
        size_t xbase[MT];
        float ga[MT], ua[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            int j = j0 + m < cnt ? j0 + m : cnt - 1;
            xbase[m] = (size_t)sorted_token[lo + j] * d;
            ga[m] = ua[m] = 0.0f;
        }
        row_dot<XDT, MT>(gf, grow, d, gfast, x, xbase, lane, ga);
        row_dot<XDT, MT>(uf, urow, d, ufast, x, xbase, lane, ua);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float g = wave_sum(ga[m]), u = wave_sum(ua[m]);
            if (lane == m && j0 + m < cnt) hidden_act[(size_t)(lo + j0 + m) * f + row] = silu_mul(g, u);
        }
    }
}

// down projection of every active expert; each result is multiplied by its route and the
// product is stored (fp32) before any accumulation.
template <int MT>
__global__ __launch_bounds__(256) void moe_down_kernel(const uint8_t* __restrict__ down, int df, int64_t dstride,
                                                       int64_t drb, bool dfast, int d, int f,
                                                       const float* __restrict__ hidden_act,
                                                       const int* __restrict__ offsets,
                                                       const int* __restrict__ active,
                                                       const int* __restrict__ n_active,
                                                       const float* __restrict__ sorted_weight,
                                                       float* __restrict__ terms) {
    if ((int)blockIdx.y >= *n_active) return;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= d) return;
    const int e = active[blockIdx.y];
    const int lo = offsets[e], cnt = offsets[e + 1] - lo;
    const uint8_t* drow = down + (int64_t)e * dstride + (int64_t)row * drb;
    for (int j0 = 0; j0 < cnt; j0 += MT) {
        size_t xbase[MT];
        float acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            int j = j0 + m < cnt ? j0 + m : cnt - 1;
            xbase[m] = (size_t)(lo + j) * f;
            acc[m] = 0.0f;
        }
        row_dot<QMOE_DT_F32, MT>(df, drow, f, dfast, hidden_act, xbase, lane, acc);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float v = wave_sum(acc[m]);
            if (lane == m && j0 + m < cnt)
                terms[(size_t)(lo + j0 + m) * d + row] = mul_unfused(v, sorted_weight[lo + j0 + m]);
        }
    }
}

// out[t] = ((0 + term_e1) + term_e2) + ... in ascending expert id, then + shared * sigmoid.
template <int XDT>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ terms,
                                                          const int* __restrict__ pos_of, int k, int d,
                                                          const float* __restrict__ shared_out,
                                                          const float* __restrict__ shared_gate,
                                                          const void* __restrict__ x, void* __restrict__ out,
                                                          int odt, const float* __restrict__ residual) {
    __shared__ int order[32];
    __shared__ float partial[4];
    __shared__ float sigmoid;
    const int t = blockIdx.x, tid = threadIdx.x;
    if (tid < 64) {
        // ascending sorted position == ascending expert id; the first wave ranks the token's
        // valid assignments among themselves (positions are unique)
        const int p = tid < k ? pos_of[(size_t)t * k + tid] : -1;
        const bool valid = p >= 0;
        int rank = 0;
        for (int s = 0; s < k; ++s) {
            const int q = __builtin_amdgcn_readlane(p, s);
            rank += q >= 0 && q < p;
        }
        if (tid < 32) order[tid] = -1;   // (same wave: written before the ranked entries below)
        if (valid) order[rank] = p;
    }
    if (shared_out && shared_gate) {
        float a = 0.0f;
        if ((d & 3) == 0 && (((size_t)shared_gate | (size_t)x) & 15) == 0) {
            // up to four pieces a thread, loads first
            float4 h[4], g[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = 4 * tid + 1024 * j;
                const bool in = i < d;
                h[j] = Elem<XDT>::load4(x, (size_t)t * d + (in ? i : 0));
                g[j] = ldg<float4>(shared_gate + (in ? i : 0));
                if (!in) g[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) a += (h[j].x * g[j].x + h[j].y * g[j].y) + (h[j].z * g[j].z + h[j].w * g[j].w);
            for (int i = 4 * tid + 4096; i < d; i += 1024) {
                const float4 hh = Elem<XDT>::load4(x, (size_t)t * d + i), gg = ldg<float4>(shared_gate + i);
                a += (hh.x * gg.x + hh.y * gg.y) + (hh.z * gg.z + hh.w * gg.w);
            }
        } else {
            for (int i = tid; i < d; i += 256) a += Elem<XDT>::load(x, (size_t)t * d + i) * shared_gate[i];
        }
        a = wave_sum(a);
        if ((tid & 63) == 0) partial[tid >> 6] = a;
        __syncthreads();
        if (tid == 0) {
            float adm = (partial[0] + partial[1]) + (partial[2] + partial[3]);
            // exp(-logaddexp(0, -a)) == 1 / (1 + exp(-a)), evaluated without overflow
            sigmoid = adm >= 0.0f ? 1.0f / (1.0f + expf(-adm)) : expf(adm) / (1.0f + expf(adm));
        }
    }
    __syncthreads();
    const float sg = (shared_out && shared_gate) ? sigmoid : 1.0f;
    if ((d & 3) == 0) {
        // four columns per thread: the k loads of a column group travel together, the adds of
        // each column stay in ascending expert order
        for (int i = 4 * tid; i < d; i += 4 * 256) {
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
            // eight terms at a time: their loads leave together (an absent one reads row 0 and is
            // not added), the adds follow in order
            for (int s0 = 0; s0 < k; s0 += 8) {
                float4 v[8];
                bool live[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int p = s0 + j < k ? order[s0 + j] : -1;
                    live[j] = p >= 0;
                    v[j] = ldg<float4>(terms + (size_t)(live[j] ? p : 0) * d + i);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if (live[j]) {
                        acc.x = __fadd_rn(acc.x, v[j].x); acc.y = __fadd_rn(acc.y, v[j].y);
                        acc.z = __fadd_rn(acc.z, v[j].z); acc.w = __fadd_rn(acc.w, v[j].w);
                    }
                }
            }
            if (shared_out) {
                const float4 v = *(const float4*)(shared_out + (size_t)t * d + i);
                acc.x = add_product(acc.x, v.x, sg); acc.y = add_product(acc.y, v.y, sg);
                acc.z = add_product(acc.z, v.z, sg); acc.w = add_product(acc.w, v.w, sg);
            }
            if (residual) {
                const float4 r = *(const float4*)(residual + (size_t)t * d + i);
                acc.x = __fadd_rn(r.x, acc.x); acc.y = __fadd_rn(r.y, acc.y);
                acc.z = __fadd_rn(r.z, acc.z); acc.w = __fadd_rn(r.w, acc.w);
            }
            store_out(out, odt, (size_t)t * d + i, acc.x);
            store_out(out, odt, (size_t)t * d + i + 1, acc.y);
            store_out(out, odt, (size_t)t * d + i + 2, acc.z);
            store_out(out, odt, (size_t)t * d + i + 3, acc.w);
        }
        return;
    }
    for (int i = tid; i < d; i += 256) {
        float acc = 0.0f;
        for (int s = 0; s < k; ++s) {
            int p = order[s];
            if (p >= 0) acc = __fadd_rn(acc, terms[(size_t)p * d + i]);
        }
        if (shared_out) acc = add_product(acc, shared_out[(size_t)t * d + i], sg);
        if (residual) acc = __fadd_rn(residual[(size_t)t * d + i], acc);
        store_out(out, odt, (size_t)t * d + i, acc);
    }
}

// ---- single token, experts given by a device pointer table --------------------------------
__global__ __launch_bounds__(256) void grouped_gate_up_kernel(const void* const* __restrict__ table, int gf,
                                                              int64_t grb, int uf, int64_t urb, int f, int d,
                                                              bool fast_ok, const float* __restrict__ x,
                                                              float* __restrict__ hidden_act) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= f) return;
    const int e = blockIdx.y;
    const uint8_t* gate = (const uint8_t*)table[3 * e];
    const uint8_t* up = (const uint8_t*)table[3 * e + 1];
    // alignment of table entries is only known on the device
    const bool gfast = fast_ok && ((uintptr_t)gate % 4 == 0) && (grb % 4 == 0);
    const bool ufast = fast_ok && ((uintptr_t)up % 4 == 0) && (urb % 4 == 0);
    size_t xbase[1] = {0};
    float ga[1] = {0.0f}, ua[1] = {0.0f};
    row_dot<QMOE_DT_F32, 1>(gf, gate + (int64_t)row * grb, d, gfast, x, xbase, lane, ga);
    row_dot<QMOE_DT_F32, 1>(uf, up + (int64_t)row * urb, d, ufast, x, xbase, lane, ua);
    float g = wave_sum(ga[0]), u = wave_sum(ua[0]);
    if (lane == 0) hidden_act[(size_t)e * f + row] = silu_mul(g, u);
}

__global__ __launch_bounds__(256) void grouped_down_kernel(const void* const* __restrict__ table, int df,
                                                           int64_t drb, int d, int f, bool fast_ok,
                                                           const float* __restrict__ hidden_act,
                                                           const float* __restrict__ routes, int64_t route_stride,
                                                           const int32_t* __restrict__ slots,
                                                           float* __restrict__ terms) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= d) return;
    const int e = blockIdx.y;
    const uint8_t* down = (const uint8_t*)table[3 * e + 2];
    const bool dfast = fast_ok && ((uintptr_t)down % 4 == 0) && (drb % 4 == 0);
    size_t xbase[1] = {(size_t)e * f};
    float acc[1] = {0.0f};
    row_dot<QMOE_DT_F32, 1>(df, down + (int64_t)row * drb, f, dfast, hidden_act, xbase, lane, acc);
    float v = wave_sum(acc[0]);
    if (lane == 0) {
        const int slot = slots ? slots[e] : e;
        terms[(size_t)e * d + row] = mul_unfused(v, routes[(int64_t)slot * route_stride]);
    }
}

// Strictly sequential fp32 adds over the rows, starting at zero; no FMA, no tree.
__global__ __launch_bounds__(256) void ordered_reduce_kernel(const float* __restrict__ terms, int rows, int d,
                                                             float* __restrict__ out) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= d) return;
    float acc = 0.0f;
    for (int e = 0; e < rows; ++e) acc = __fadd_rn(acc, terms[(size_t)e * d + i]);
    out[i] = acc;
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct MoeWorkspace {
    size_t weights, ids, offsets, active, n_active, status, sorted_token, sorted_weight, pos_of, hidden_act, terms,
        shared_h, shared_out, sig, problems, chunk_expert, chunk_start, chunk_count, n_chunks, total;
    int max_chunks;
};

static MoeWorkspace moe_layout(int tokens, int k, int n_experts, int d_model, int d_ff, int d_ff_shared) {
    MoeWorkspace w;
    size_t at = 0;
    const size_t a = (size_t)tokens * k;
    auto take = [&](size_t bytes) { size_t here = at; at = align256(at + bytes); return here; };
    w.weights = take(a * 4);
    w.ids = take(a * 8);
    w.offsets = take(((size_t)n_experts + 1) * 4);
    w.active = take((size_t)n_experts * 4);
    w.n_active = take(4);
    w.status = take(4);
    w.sorted_token = take(a * 4);
    w.sorted_weight = take(a * 4);
    w.pos_of = take(a * 4);
    w.hidden_act = take(a * d_ff * 4);
    w.terms = take(a * d_model * 4);
    w.shared_h = take((size_t)tokens * d_ff_shared * 4);
    w.shared_out = take((size_t)tokens * d_model * 4);
    w.sig = take((size_t)tokens * 4);
    w.problems = take(a * 64 + (size_t)tokens * 64);  // device-side problem list of the decode path
    // every expert with assignments ends in one partly filled chunk at most
    w.max_chunks = (int)(a / GEMM_CHUNK + (a < (size_t)n_experts ? a : (size_t)n_experts));
    w.chunk_expert = take((size_t)w.max_chunks * 4);
    w.chunk_start = take((size_t)w.max_chunks * 4);
    w.chunk_count = take((size_t)w.max_chunks * 4);
    w.n_chunks = take(4);
    w.total = at;
    return w;
}


template <int XDT>
static void launch_gate_up(const qmoe_moe_args& a, const MoeWorkspace& L, char* ws, int max_active, bool xf,
                           hipStream_t s) {
    const qmoe_expert_bank& b = a.bank;
    const int64_t grb = row_bytes(b.gate_fmt, b.d_model), urb = row_bytes(b.up_fmt, b.d_model);
    const bool gfast = xf && rows_fast(b.gate_fmt, b.gate, grb, b.d_model) && b.gate_stride % 4 == 0;
    const bool ufast = xf && rows_fast(b.up_fmt, b.up, urb, b.d_model) && b.up_stride % 4 == 0;
    const dim3 grid((b.d_ff + 3) / 4, max_active), block(256);
#define QMOE_GU(MT)                                                                                                  \
    hipLaunchKernelGGL((moe_gate_up_kernel<XDT, MT>), grid, block, 0, s, (const uint8_t*)b.gate, b.gate_fmt,         \
                       b.gate_stride, grb, gfast, (const uint8_t*)b.up, b.up_fmt, b.up_stride, urb, ufast, b.d_ff,   \
                       b.d_model, a.hidden, (const int*)(ws + L.offsets), (const int*)(ws + L.active),               \
                       (const int*)(ws + L.n_active), (const int*)(ws + L.sorted_token), (float*)(ws + L.hidden_act))
    if (a.tokens == 1) QMOE_GU(1);
    else if (a.tokens <= 16) QMOE_GU(4);
    else QMOE_GU(8);
#undef QMOE_GU
}

// ---- token batches on MFMA ----------------------------------------------------------------------
// SwiGLU activations travel between the two GEMMs as bf16 hi / lo arrays; they take the place
// of the fp32 activations in the workspace (2 x 2 bytes per element).
static bool gemm_path(const qmoe_moe_args& a, const char* ws, const MoeWorkspace& L) {
    const qmoe_expert_bank& b = a.bank;
    if (a.tokens < GEMM_MIN_TOKENS) return false;
    if (b.gate_fmt != b.up_fmt) return false;
    if (!gemm_supported(b.gate_fmt, b.gate, b.gate_stride, b.d_ff, b.d_model, a.hidden, a.hidden_dtype, b.d_model)) return false;
    if (!gemm_supported(b.up_fmt, b.up, b.up_stride, b.d_ff, b.d_model, a.hidden, a.hidden_dtype, b.d_model)) return false;
    if (!gemm_supported(b.down_fmt, b.down, b.down_stride, b.d_model, b.d_ff, ws + L.hidden_act, GEMM_A_PAIR, b.d_ff)) return false;
    if ((size_t)a.tokens * a.top_k * b.d_ff * 2 % 16) return false;  // the lo array starts 16-byte aligned
    if (a.shared_gate_w) {
        if (a.shared_gate_fmt != a.shared_up_fmt) return false;
        if (!gemm_supported(a.shared_gate_fmt, a.shared_gate_w, 0, a.d_ff_shared, b.d_model, a.hidden, a.hidden_dtype, b.d_model)) return false;
        if (!gemm_supported(a.shared_up_fmt, a.shared_up_w, 0, a.d_ff_shared, b.d_model, a.hidden, a.hidden_dtype, b.d_model)) return false;
        if (!gemm_supported(a.shared_down_fmt, a.shared_down_w, 0, b.d_model, a.d_ff_shared, ws + L.shared_h, GEMM_A_PAIR, a.d_ff_shared)) return false;
        if ((size_t)a.tokens * a.d_ff_shared * 2 % 16) return false;
    }
    return true;
}

static int launch_combine(const qmoe_moe_args& a, char* ws, const MoeWorkspace& L, const float* shared_out, hipStream_t s);

// After the plan: grouped gate/up + SwiGLU, grouped down * route, the shared expert, combine.
static int gemm_forward(const qmoe_moe_args& a, char* ws, const MoeWorkspace& L, hipStream_t s) {
    const qmoe_expert_bank& b = a.bank;
    const size_t assignments = (size_t)a.tokens * a.top_k;
    int rc;
    GemmArgs g{};
    g.w = (const uint8_t*)b.gate;
    g.w2 = (const uint8_t*)b.up;
    g.stride = b.gate_stride;
    g.stride2 = b.up_stride;
    g.n = b.d_ff;
    g.k = b.d_model;
    g.a0 = a.hidden;
    g.a_stride = b.d_model;
    g.gather = (const int*)(ws + L.sorted_token);
    g.chunk_expert = (const int*)(ws + L.chunk_expert);
    g.chunk_start = (const int*)(ws + L.chunk_start);
    g.chunk_count = (const int*)(ws + L.chunk_count);
    g.n_chunks = (const int*)(ws + L.n_chunks);
    uint16_t* h_hi = (uint16_t*)(ws + L.hidden_act);
    uint16_t* h_lo = h_hi + assignments * b.d_ff;
    g.out0 = h_hi;
    g.out1 = h_lo;
    GemmArgs d = g;
    d.w = (const uint8_t*)b.down;
    d.w2 = nullptr;
    d.stride = b.down_stride;
    d.n = b.d_model;
    d.k = b.d_ff;
    d.a0 = h_hi;
    d.a1 = h_lo;
    d.a_stride = b.d_ff;
    d.gather = nullptr;
    d.out0 = ws + L.terms;
    d.out1 = nullptr;
    d.scale = (const float*)(ws + L.sorted_weight);
    const float* shared_out = nullptr;
    if (!a.shared_gate_w) {
        if ((rc = gemm_launch(b.gate_fmt, true, a.hidden_dtype, g, L.max_chunks, a.tokens, s))) return rc;
        if ((rc = gemm_launch(b.down_fmt, false, GEMM_A_PAIR, d, L.max_chunks, a.tokens, s))) return rc;
        return launch_combine(a, ws, L, shared_out, s);
    }
    const int chunks = (a.tokens + GEMM_CHUNK - 1) / GEMM_CHUNK;
    GemmArgs sg{};
    sg.w = (const uint8_t*)a.shared_gate_w;
    sg.w2 = (const uint8_t*)a.shared_up_w;
    sg.n = a.d_ff_shared;
    sg.k = b.d_model;
    sg.a0 = a.hidden;
    sg.a_stride = b.d_model;
    sg.dense_tokens = a.tokens;
    uint16_t* s_hi = (uint16_t*)(ws + L.shared_h);
    uint16_t* s_lo = s_hi + (size_t)a.tokens * a.d_ff_shared;
    sg.out0 = s_hi;
    sg.out1 = s_lo;
    GemmArgs sd{};
    sd.w = (const uint8_t*)a.shared_down_w;
    sd.n = b.d_model;
    sd.k = a.d_ff_shared;
    sd.a0 = s_hi;
    sd.a1 = s_lo;
    sd.a_stride = a.d_ff_shared;
    sd.dense_tokens = a.tokens;
    sd.out0 = ws + L.shared_out;
    // The shared expert's two GEMMs ride in the routed launches (its gate/up needs no routing, its
    // down needs only its own gate/up): on their own they are short launches of few, long
    // workgroups that leave most of the chip waiting.
    const bool together = a.shared_gate_fmt == b.gate_fmt && a.shared_down_fmt == b.down_fmt &&
                          gemm_side_fits(g, L.max_chunks, sg, chunks, a.tokens) && gemm_side_fits(d, L.max_chunks, sd, chunks, a.tokens);
    if (together) {
        if ((rc = gemm_launch(b.gate_fmt, true, a.hidden_dtype, g, L.max_chunks, a.tokens, s, &sg, chunks))) return rc;
        if ((rc = gemm_launch(b.down_fmt, false, GEMM_A_PAIR, d, L.max_chunks, a.tokens, s, &sd, chunks))) return rc;
    } else {
        if ((rc = gemm_launch(b.gate_fmt, true, a.hidden_dtype, g, L.max_chunks, a.tokens, s))) return rc;
        if ((rc = gemm_launch(b.down_fmt, false, GEMM_A_PAIR, d, L.max_chunks, a.tokens, s))) return rc;
        if ((rc = gemm_launch(a.shared_gate_fmt, true, a.hidden_dtype, sg, chunks, a.tokens, s))) return rc;
        if ((rc = gemm_launch(a.shared_down_fmt, false, GEMM_A_PAIR, sd, chunks, a.tokens, s))) return rc;
    }
    shared_out = (const float*)(ws + L.shared_out);
    return launch_combine(a, ws, L, shared_out, s);
}

int moe_forward_impl(const qmoe_moe_args& a, void* workspace, size_t workspace_bytes, hipStream_t s) {
    const qmoe_expert_bank& b = a.bank;
    const char* who = "qmoe_moe_forward";
    if (!a.hidden || !a.out) return fail(QMOE_EINVAL, "%s: null hidden or output pointer", who);
    if (a.tokens < 0) return fail(QMOE_EINVAL, "%s: negative token count", who);
    if (!dtype_size(a.hidden_dtype) || !dtype_size(a.out_dtype)) return fail(QMOE_EINVAL, "%s: bad element type", who);
    if (b.n_experts < 1 || b.n_experts > 4096) return fail(QMOE_EUNSUPPORTED, "%s: expert count %d outside 1..4096", who, b.n_experts);
    if (a.top_k < 1 || a.top_k > 32 || a.top_k > b.n_experts) return fail(QMOE_EUNSUPPORTED, "%s: top_k=%d outside 1..min(32, experts)", who, a.top_k);
    if (!b.gate || !b.up || !b.down) return fail(QMOE_EINVAL, "%s: null expert bank pointer", who);
    if (b.d_model < 1 || b.d_ff < 1) return fail(QMOE_EINVAL, "%s: bank dimensions must be positive", who);
    const int fmts[3] = {b.gate_fmt, b.up_fmt, b.down_fmt};
    const int ks[3] = {b.d_model, b.d_model, b.d_ff};
    const int ns[3] = {b.d_ff, b.d_ff, b.d_model};
    const int64_t strides[3] = {b.gate_stride, b.up_stride, b.down_stride};
    for (int i = 0; i < 3; ++i) {
        if (!block_elems(fmts[i])) return fail(QMOE_EINVAL, "%s: unknown packed format id %d", who, fmts[i]);
        if (!format_implemented(fmts[i])) return fail(QMOE_EUNSUPPORTED, "%s: packed format id %d has no kernel", who, fmts[i]);
        if (ks[i] % block_elems(fmts[i])) return fail(QMOE_EINVAL, "%s: projection K=%d is not a block multiple", who, ks[i]);
        if (strides[i] < row_bytes(fmts[i], ks[i]) * ns[i] || strides[i] % 2)
            return fail(QMOE_EINVAL, "%s: expert stride %lld smaller than one expert or odd", who, (long long)strides[i]);
    }
    const bool has_shared = a.shared_gate_w || a.shared_up_w || a.shared_down_w;
    if (has_shared && !(a.shared_gate_w && a.shared_up_w && a.shared_down_w && a.d_ff_shared > 0))
        return fail(QMOE_EINVAL, "%s: shared expert needs all three projections and d_ff_shared > 0", who);
    if (!a.logits && !(a.in_weights && a.in_ids)) return fail(QMOE_EINVAL, "%s: need router logits or weights+ids", who);
    if (a.tokens == 0) return QMOE_OK;
    const int words = (a.tokens + 31) / 32;
    const size_t plan_lds = ((size_t)b.n_experts * words + b.n_experts) * 4;
    if (plan_lds > PLAN_LDS_LIMIT)
        return fail(QMOE_EUNSUPPORTED, "%s: %d tokens x %d experts exceeds the plan kernel's LDS bitmap; split the tokens", who, a.tokens, b.n_experts);
    const MoeWorkspace L = moe_layout(a.tokens, a.top_k, b.n_experts, b.d_model, b.d_ff, has_shared ? a.d_ff_shared : 0);
    if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < L.total)
        return fail(QMOE_EWORKSPACE, "%s: workspace must be 256-byte aligned and hold %zu bytes (got %zu)", who, L.total, workspace_bytes);
    char* ws = (char*)workspace;
    int rc;
    static_assert(sizeof(StreamProblem) == 64, "problem list entries are 64 bytes");
    if (decode_supported(a, ws + L.hidden_act)) {
        DecodeBuffers db{(float*)(ws + L.weights), (int64_t*)(ws + L.ids), (int*)(ws + L.sorted_token),
                         (float*)(ws + L.sorted_weight), (float*)(ws + L.sig), (int*)(ws + L.status),
                         ws + L.problems, (int*)(ws + L.n_active), (float*)(ws + L.hidden_act), (float*)(ws + L.shared_h)};
        return decode_launch(a, db, s);
    }
    const float* weights = a.in_weights;
    const int64_t* ids = a.in_ids;
    if (a.logits) {
        float* wout = a.out_weights ? a.out_weights : (float*)(ws + L.weights);
        int64_t* iout = a.out_ids ? a.out_ids : (int64_t*)(ws + L.ids);
        rc = router_topk_impl(a.logits, a.tokens, b.n_experts, a.top_k, a.floor_value, a.renormalize, wout, iout, s);
        if (rc) return rc;
        weights = wout;
        ids = iout;
    }
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(PLAN_THREADS), plan_lds, s, ids, weights, a.tokens, a.top_k,
                       b.n_experts, (int*)(ws + L.offsets), (int*)(ws + L.active), (int*)(ws + L.n_active),
                       (int*)(ws + L.sorted_token), (float*)(ws + L.sorted_weight), (int*)(ws + L.pos_of),
                       (int*)(ws + L.status), a.status_out, a.logits ? nullptr : a.out_weights, a.logits ? nullptr : a.out_ids,
                       (int*)(ws + L.chunk_expert), (int*)(ws + L.chunk_start),
                       (int*)(ws + L.chunk_count), (int*)(ws + L.n_chunks), (int*)nullptr);
    if ((rc = check_launch("qmoe_moe_forward(plan)"))) return rc;
    const int assignments = a.tokens * a.top_k;
    const int max_active = assignments < b.n_experts ? assignments : b.n_experts;
    if (gemm_path(a, ws, L)) return gemm_forward(a, ws, L, s);
    const bool xf = x_fast(a.hidden, a.hidden_dtype, b.d_model);
    if (a.hidden_dtype == QMOE_DT_F32) launch_gate_up<QMOE_DT_F32>(a, L, ws, max_active, xf, s);
    else if (a.hidden_dtype == QMOE_DT_F16) launch_gate_up<QMOE_DT_F16>(a, L, ws, max_active, xf, s);
    else launch_gate_up<QMOE_DT_BF16>(a, L, ws, max_active, xf, s);
    if ((rc = check_launch("qmoe_moe_forward(gate_up)"))) return rc;
    {
        const int64_t drb = row_bytes(b.down_fmt, b.d_ff);
        const bool dfast = rows_fast(b.down_fmt, b.down, drb, b.d_ff) && b.down_stride % 4 == 0;
        const dim3 grid((b.d_model + 3) / 4, max_active), block(256);
#define QMOE_DOWN(MT)                                                                                                \
    hipLaunchKernelGGL((moe_down_kernel<MT>), grid, block, 0, s, (const uint8_t*)b.down, b.down_fmt, b.down_stride,  \
                       drb, dfast, b.d_model, b.d_ff, (const float*)(ws + L.hidden_act),                             \
                       (const int*)(ws + L.offsets), (const int*)(ws + L.active), (const int*)(ws + L.n_active),     \
                       (const float*)(ws + L.sorted_weight), (float*)(ws + L.terms))
        if (a.tokens == 1) QMOE_DOWN(1);
        else if (a.tokens <= 16) QMOE_DOWN(4);
        else QMOE_DOWN(8);
#undef QMOE_DOWN
        if ((rc = check_launch("qmoe_moe_forward(down)"))) return rc;
    }
    const float* shared_out = nullptr;
    if (has_shared) {
        rc = swiglu_impl(a.shared_gate_w, a.shared_gate_fmt, a.shared_up_w, a.shared_up_fmt, a.d_ff_shared, b.d_model,
                         a.hidden, a.hidden_dtype, a.tokens, ws + L.shared_h, QMOE_DT_F32, s);
        if (rc) return rc;
        rc = linear_impl(a.shared_down_w, a.shared_down_fmt, b.d_model, a.d_ff_shared, ws + L.shared_h, QMOE_DT_F32,
                         a.tokens, ws + L.shared_out, QMOE_DT_F32, s);
        if (rc) return rc;
        shared_out = (const float*)(ws + L.shared_out);
    }
    return launch_combine(a, ws, L, shared_out, s);
}

static int launch_combine(const qmoe_moe_args& a, char* ws, const MoeWorkspace& L, const float* shared_out, hipStream_t s) {
    const qmoe_expert_bank& b = a.bank;
    const dim3 cgrid(a.tokens), cblock(256);
#define QMOE_COMBINE(XDT)                                                                                            \
    hipLaunchKernelGGL((moe_combine_kernel<XDT>), cgrid, cblock, 0, s, (const float*)(ws + L.terms),                 \
                       (const int*)(ws + L.pos_of), a.top_k, b.d_model, shared_out, a.shared_gate, a.hidden, a.out,  \
                       a.out_dtype, a.residual)
    if (a.hidden_dtype == QMOE_DT_F32) QMOE_COMBINE(QMOE_DT_F32);
    else if (a.hidden_dtype == QMOE_DT_F16) QMOE_COMBINE(QMOE_DT_F16);
    else QMOE_COMBINE(QMOE_DT_BF16);
#undef QMOE_COMBINE
    return check_launch("qmoe_moe_forward(combine)");
}

}  // namespace qmoe

using namespace qmoe;

extern "C" {

size_t qmoe_moe_workspace_bytes(int tokens, int top_k, int n_experts, int d_model, int d_ff, int d_ff_shared) {
    if (tokens < 0 || top_k < 1 || n_experts < 1 || d_model < 1 || d_ff < 1 || d_ff_shared < 0) return 0;
    return moe_layout(tokens, top_k, n_experts, d_model, d_ff, d_ff_shared).total;
}

int qmoe_moe_forward(const qmoe_moe_args* args, void* workspace, size_t workspace_bytes, void* stream) {
    if (!args) return fail(QMOE_EINVAL, "qmoe_moe_forward: null argument struct");
    return moe_forward_impl(*args, workspace, workspace_bytes, (hipStream_t)stream);
}

// ---- the step without a caller's workspace ---------------------------------------------------------
// Scratch for callers that cannot allocate: a file-scope array in device memory, one copy per GPU
// the library runs on, kept until the process ends.  Its name is a host-side stand-in, not a device
// address: the address is asked for once per device (with that device current) and only that
// pointer is handed to the kernels.
static constexpr size_t MOE_STATIC_SCRATCH_BYTES = QMOE_MOE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[MOE_STATIC_SCRATCH_BYTES];

}  // extern "C"
int qmoe::static_scratch(void** out) {
    static constexpr int MAX_DEVICES = 64;
    static std::mutex lock;
    static void* per_device[MAX_DEVICES] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
        return fail(QMOE_ELAUNCH, "qmoe_moe_forward_static: no current HIP device");
    std::lock_guard<std::mutex> guard(lock);
    if (!per_device[dev]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(QMOE_ELAUNCH, "qmoe_moe_forward_static: scratch address: %s", hipGetErrorString(e));
        per_device[dev] = ptr;
    }
    *out = per_device[dev];
    return QMOE_OK;
}
extern "C" {

size_t qmoe_moe_static_scratch_bytes(void) { return MOE_STATIC_SCRATCH_BYTES; }

int qmoe_moe_forward_static(const qmoe_moe_args* args, void* stream) {
    if (!args) return fail(QMOE_EINVAL, "qmoe_moe_forward_static: null argument struct");
    const qmoe_expert_bank& b = args->bank;
    const bool has_shared = args->shared_gate_w || args->shared_up_w || args->shared_down_w;
    if (args->tokens > 0 && args->top_k >= 1 && b.n_experts >= 1 && b.d_model >= 1 && b.d_ff >= 1) {
        const size_t need = moe_layout(args->tokens, args->top_k, b.n_experts, b.d_model, b.d_ff,
                                       has_shared && args->d_ff_shared > 0 ? args->d_ff_shared : 0).total;
        if (need > MOE_STATIC_SCRATCH_BYTES)
            return fail(QMOE_EWORKSPACE, "qmoe_moe_forward_static: this step needs %zu bytes of scratch, the built-in area holds %zu; "
                        "use qmoe_moe_forward with a workspace", need, MOE_STATIC_SCRATCH_BYTES);
    }
    void* ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    return moe_forward_impl(*args, ptr, MOE_STATIC_SCRATCH_BYTES, (hipStream_t)stream);
}

int qmoe_grouped_decode(const float* x, const void* const* table, int n_rows, int gate_fmt, int up_fmt, int down_fmt,
                        int d_model, int d_ff, const float* routes, int64_t route_stride, const int32_t* slots,
                        float* out, float* workspace, void* stream) {
    const char* who = "qmoe_grouped_decode";
    if (!x || !table || !routes || !out) return fail(QMOE_EINVAL, "%s: null pointer", who);
    if (!workspace || (uintptr_t)workspace % 16) return fail(QMOE_EWORKSPACE, "%s: workspace of E*(d_ff+d_model) floats (16-byte aligned) required", who);
    if (n_rows < 1 || n_rows > 65535) return fail(QMOE_EINVAL, "%s: expert rows %d outside 1..65535", who, n_rows);
    if (d_model < 1 || d_ff < 1) return fail(QMOE_EINVAL, "%s: dimensions must be positive", who);
    const int fmts[3] = {gate_fmt, up_fmt, down_fmt};
    const int ks[3] = {d_model, d_model, d_ff};
    for (int i = 0; i < 3; ++i) {
        if (!block_elems(fmts[i])) return fail(QMOE_EINVAL, "%s: unknown packed format id %d", who, fmts[i]);
        if (!format_implemented(fmts[i])) return fail(QMOE_EUNSUPPORTED, "%s: packed format id %d has no kernel", who, fmts[i]);
        if (ks[i] % block_elems(fmts[i])) return fail(QMOE_EINVAL, "%s: projection K=%d is not a block multiple", who, ks[i]);
    }
    hipStream_t s = (hipStream_t)stream;
    float* hidden_act = workspace;
    float* terms = workspace + (size_t)n_rows * d_ff;
    const bool xf = x_fast(x, QMOE_DT_F32, d_model) && (d_model % 8 == 0);
    const bool hf = ((uintptr_t)hidden_act % 16 == 0) && (d_ff % 8 == 0);
    hipLaunchKernelGGL(grouped_gate_up_kernel, dim3((d_ff + 3) / 4, n_rows), dim3(256), 0, s, table, gate_fmt,
                       row_bytes(gate_fmt, d_model), up_fmt, row_bytes(up_fmt, d_model), d_ff, d_model, xf, x,
                       hidden_act);
    int rc = check_launch("qmoe_grouped_decode(gate_up)");
    if (rc) return rc;
    hipLaunchKernelGGL(grouped_down_kernel, dim3((d_model + 3) / 4, n_rows), dim3(256), 0, s, table, down_fmt,
                       row_bytes(down_fmt, d_ff), d_model, d_ff, hf, hidden_act, routes, route_stride, slots, terms);
    if ((rc = check_launch("qmoe_grouped_decode(down)"))) return rc;
    hipLaunchKernelGGL(ordered_reduce_kernel, dim3((d_model + 255) / 256), dim3(256), 0, s, terms, n_rows, d_model, out);
    return check_launch("qmoe_grouped_decode(reduce)");
}

}  // extern "C"

namespace qmoe {
// The listed experts' pointers and route positions from the kernel arguments into device memory
// (for the general kernels, which read a device table): no host-to-device copy is involved.
__global__ void listed_upload_kernel(const ListedExperts l, const void** table, int32_t* slots) {
    const int i = threadIdx.x;
    if (i < l.count) {
        table[3 * i] = l.gate[i];
        table[3 * i + 1] = l.up[i];
        table[3 * i + 2] = l.down[i];
        slots[i] = l.slot[i];
    }
}
}  // namespace qmoe

extern "C" int qmoe_grouped_decode_listed(const float* x, const void* const* experts, int n_rows, int gate_fmt, int up_fmt,
                                          int down_fmt, int d_model, int d_ff, const float* routes, int64_t route_stride,
                                          const int32_t* slots, float* out, float* workspace, void* stream) {
    const char* who = "qmoe_grouped_decode_listed";
    if (!x || !experts || !routes || !out) return fail(QMOE_EINVAL, "%s: null pointer", who);
    if (!workspace || (uintptr_t)workspace % 16) return fail(QMOE_EWORKSPACE, "%s: workspace of E*(d_ff+d_model+8) floats (16-byte aligned) required", who);
    if (n_rows < 1) return fail(QMOE_EINVAL, "%s: expert rows %d", who, n_rows);
    if (n_rows > LISTED_MAX) return fail(QMOE_EUNSUPPORTED, "%s: %d experts exceed the %d a host list carries; use qmoe_grouped_decode", who, n_rows, LISTED_MAX);
    if (d_model < 1 || d_ff < 1) return fail(QMOE_EINVAL, "%s: dimensions must be positive", who);
    const int fmts[3] = {gate_fmt, up_fmt, down_fmt};
    const int ks[3] = {d_model, d_model, d_ff};
    for (int i = 0; i < 3; ++i) {
        if (!block_elems(fmts[i])) return fail(QMOE_EINVAL, "%s: unknown packed format id %d", who, fmts[i]);
        if (!format_implemented(fmts[i])) return fail(QMOE_EUNSUPPORTED, "%s: packed format id %d has no kernel", who, fmts[i]);
        if (ks[i] % block_elems(fmts[i])) return fail(QMOE_EINVAL, "%s: projection K=%d is not a block multiple", who, ks[i]);
    }
    ListedExperts l{};
    for (int i = 0; i < n_rows; ++i) {
        l.gate[i] = (const uint8_t*)experts[3 * i];
        l.up[i] = (const uint8_t*)experts[3 * i + 1];
        l.down[i] = (const uint8_t*)experts[3 * i + 2];
        if (!l.gate[i] || !l.up[i] || !l.down[i]) return fail(QMOE_EINVAL, "%s: expert %d has a null projection", who, i);
        if ((uintptr_t)l.gate[i] % 2 || (uintptr_t)l.up[i] % 2 || (uintptr_t)l.down[i] % 2)
            return fail(QMOE_EINVAL, "%s: packed weights must be 2-byte aligned", who);
        l.slot[i] = slots ? slots[i] : i;
        if (l.slot[i] < 0) return fail(QMOE_EINVAL, "%s: negative route position", who);
    }
    l.routes = routes;
    l.route_stride = route_stride;
    l.count = n_rows;
    hipStream_t s = (hipStream_t)stream;
    if ((uintptr_t)x % 16 == 0) {
        const int rc = decode2_listed(x, l, gate_fmt, up_fmt, down_fmt, d_model, d_ff, out, workspace, s);
        if (rc != QMOE_EUNSUPPORTED) return rc;
    }
    // any other shape: the table goes to the end of the workspace, then the general kernels
    float* const tail = workspace + (size_t)n_rows * ((size_t)d_ff + d_model);
    const void** const table = (const void**)tail;
    int32_t* const dslots = (int32_t*)(tail + 6 * (size_t)n_rows);
    hipLaunchKernelGGL(listed_upload_kernel, dim3(1), dim3(64), 0, s, l, table, dslots);
    if (int rc = check_launch("qmoe_grouped_decode_listed(table)")) return rc;
    return qmoe_grouped_decode(x, (const void* const*)table, n_rows, gate_fmt, up_fmt, down_fmt, d_model, d_ff, routes, route_stride,
                               dslots, out, workspace, stream);
}

extern "C" int qmoe_routing_plan(const int64_t* ids, const float* weights, int tokens, int top_k, int n_experts,
                                 int* offsets, int* active, int* n_active, int* order, int* sorted_token,
                                 float* sorted_weight, int* pos_of, int* status, void* stream) {
    if (!ids || !weights || !offsets || !active || !n_active || !order || !sorted_token || !sorted_weight || !pos_of || !status)
        return fail(QMOE_EINVAL, "qmoe_routing_plan: null pointer");
    if (tokens < 1 || top_k < 1 || n_experts < 1 || top_k > n_experts || (int64_t)tokens * top_k > INT32_MAX)
        return fail(QMOE_EINVAL, "qmoe_routing_plan: tokens=%d top_k=%d n_experts=%d", tokens, top_k, n_experts);
    const int words = (tokens + 31) / 32;
    const size_t plan_lds = ((size_t)n_experts * words + n_experts) * 4;
    if (plan_lds > PLAN_LDS_LIMIT)
        return fail(QMOE_EUNSUPPORTED, "qmoe_routing_plan: %d tokens x %d experts exceed the plan's %zu-byte table; split the batch",
                    tokens, n_experts, PLAN_LDS_LIMIT);
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(PLAN_THREADS), plan_lds, (hipStream_t)stream, ids, weights, tokens, top_k,
                       n_experts, offsets, active, n_active, sorted_token, sorted_weight, pos_of, status, (int*)nullptr,
                       (float*)nullptr, (int64_t*)nullptr, (int*)nullptr, (int*)nullptr, (int*)nullptr, (int*)nullptr, order);
    return check_launch("qmoe_routing_plan");
}
