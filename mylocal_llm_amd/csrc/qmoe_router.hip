// Router: full softmax over all experts, exact top-k selection, optional renormalisation
// of the selected mass.  One wave per token row; the row lives in LDS, selection is k
// rounds of a wave-wide arg-best under the reference's order (descending value, NaN last,
// lower id on ties: mini_llm/ops/router_decode.py:19-26).
#include "qmoe_common.hpp"

namespace qmoe {

__device__ __forceinline__ bool selected_before(float a, int ia, float b, int ib, int n) {
    if (ia == n) return false;
    if (ib == n) return true;
    const bool an = isnan(a), bn = isnan(b);
    if (an) return bn && ia < ib;
    if (bn) return true;
    return a > b || (a == b && ia < ib);
}

__device__ __forceinline__ float nan_max(float a, float b) {
    return (isnan(a) || isnan(b)) ? __uint_as_float(0x7FC00000u) : fmaxf(a, b);
}

// n <= 4096 (64 values per lane at most), k <= 32.
__global__ __launch_bounds__(64) void router_topk_kernel(const float* __restrict__ logits, int n, int k,
                                                         float floor_value, int renorm,
                                                         float* __restrict__ weights, int64_t* __restrict__ ids) {
    extern __shared__ float values[];
    __shared__ float selected[32];
    const int lane = threadIdx.x;
    const float* z = logits + (size_t)blockIdx.x * n;
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) {
        float v = z[i];
        values[i] = v;
        m = nan_max(m, v);
    }
#pragma unroll
    for (int off = 32; off; off >>= 1) m = nan_max(m, __shfl_xor(m, off, 64));
    __syncthreads();
    double part = 0.0;
    for (int i = lane; i < n; i += 64) part += (double)expf(values[i] - m);
#pragma unroll
    for (int off = 32; off; off >>= 1) part += __shfl_xor(part, off, 64);
    const float denom = (float)part;
    unsigned long long used = 0ull;  // bit j: this lane's value at index lane + 64*j was taken
    for (int slot = 0; slot < k; ++slot) {
        float best = -INFINITY;
        int index = n;
        for (int i = lane, j = 0; i < n; i += 64, ++j) {
            if (!((used >> j) & 1ull) && selected_before(values[i], i, best, index, n)) {
                best = values[i];
                index = i;
            }
        }
#pragma unroll
        for (int off = 32; off; off >>= 1) {
            float ov = __shfl_xor(best, off, 64);
            int oi = __shfl_xor(index, off, 64);
            if (selected_before(ov, oi, best, index, n)) { best = ov; index = oi; }
        }
        // every lane now holds the same winner
        if ((index & 63) == lane && index < n) used |= 1ull << (index >> 6);
        if (lane == 0) {
            ids[(size_t)blockIdx.x * k + slot] = index;
            selected[slot] = expf(best - m) / denom;
        }
    }
    __syncthreads();
    if (lane == 0) {
        float mass = 0.0f;
        for (int slot = 0; slot < k; ++slot) mass += selected[slot];
        float norm = 1.0f;
        if (renorm) norm = isnan(mass) ? mass : fmaxf(mass, floor_value);
        for (int slot = 0; slot < k; ++slot)
            weights[(size_t)blockIdx.x * k + slot] = renorm ? selected[slot] / norm : selected[slot];
    }
}

int router_topk_impl(const float* logits, int tokens, int n, int k, float floor_value, int renorm, float* weights,
                     int64_t* ids, hipStream_t s) {
    if (!logits || !weights || !ids) return fail(QMOE_EINVAL, "qmoe_router_topk: null pointer");
    if (tokens < 0) return fail(QMOE_EINVAL, "qmoe_router_topk: negative token count");
    if (n < 1 || n > 4096) return fail(QMOE_EUNSUPPORTED, "qmoe_router_topk: expert count %d outside 1..4096", n);
    if (k < 1 || k > 32 || k > n) return fail(QMOE_EUNSUPPORTED, "qmoe_router_topk: k=%d outside 1..min(32, n)", k);
    if (renorm && !(floor_value >= 1.17549435e-38f && floor_value <= 3.40282347e38f))
        return fail(QMOE_EINVAL, "qmoe_router_topk: normalisation floor must be a finite positive normal float");
    if ((uintptr_t)logits % 4 || (uintptr_t)weights % 4 || (uintptr_t)ids % 8)
        return fail(QMOE_EINVAL, "qmoe_router_topk: misaligned pointer");
    if (tokens == 0) return QMOE_OK;
    hipLaunchKernelGGL(router_topk_kernel, dim3(tokens), dim3(64), (size_t)n * sizeof(float), s, logits, n, k,
                       floor_value, renorm, weights, ids);
    return check_launch("qmoe_router_topk");
}

}  // namespace qmoe

extern "C" int qmoe_router_topk(const float* logits, int tokens, int n, int k, float floor_value, int renormalize,
                                float* weights, int64_t* ids, void* stream) {
    return qmoe::router_topk_impl(logits, tokens, n, k, floor_value, renormalize, weights, ids, (hipStream_t)stream);
}
