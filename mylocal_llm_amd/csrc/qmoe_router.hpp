// Router row primitive shared by the stand-alone router kernel and the fused decode path.
#pragma once
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

// One wave routes one row: full softmax, k rounds of wave-wide arg-best, optional
// renormalisation.  `values` (n floats) and `selected` (32 floats) are LDS scratch of the
// calling wave; n <= 4096 (64 values per lane at most), k <= 32.  Results go to
// weights[0..k) / ids[0..k) (any address space) in selection order.
__device__ __forceinline__ void router_row(const float* __restrict__ z, int n, int k, float floor_value, int renorm,
                                           float* values, float* selected, float* __restrict__ weights,
                                           int64_t* __restrict__ ids) {
    const int lane = threadIdx.x & 63;
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
            ids[slot] = index;
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
            weights[slot] = renorm ? selected[slot] / norm : selected[slot];
    }
}


}  // namespace qmoe
