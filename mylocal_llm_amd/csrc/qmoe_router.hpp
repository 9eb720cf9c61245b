// Router row primitive shared by the stand-alone router kernel and the fused decode path.
#pragma once
#include "qmoe_common.hpp"

namespace qmoe {

// Monotone unsigned image of a float for selection: larger value -> larger key, -0 == +0,
// every NaN -> 0 (below -inf), so a 64-bit (key << 32 | ~index) maximum is "descending value,
// NaN last, lower id on ties" (mini_llm/ops/router_decode.py:19-26).
__device__ __forceinline__ uint32_t order_key(float v) {
    if (isnan(v)) return 0u;
    const uint32_t b = __float_as_uint(v == 0.0f ? 0.0f : v);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
    if (key == 0u) return __uint_as_float(0x7FC00000u);
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned long long dpp_max_u64(unsigned long long v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, CTRL, ROW_MASK, 0xf, false);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(v >> 32), CTRL, ROW_MASK, 0xf, false);
    const unsigned long long o = ((unsigned long long)hi << 32) | lo;
    return o > v ? o : v;
}
// Maximum over the wave, broadcast to every lane.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
    v = dpp_max_u64<0xB1, 0xf>(v);
    v = dpp_max_u64<0x4E, 0xf>(v);
    v = dpp_max_u64<0x141, 0xf>(v);
    v = dpp_max_u64<0x140, 0xf>(v);
    v = dpp_max_u64<0x142, 0xa>(v);
    v = dpp_max_u64<0x143, 0xc>(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 63);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), 63);
    return ((unsigned long long)hi << 32) | lo;
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_add_f64(double v) {
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)b, CTRL, ROW_MASK, 0xf, false);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(b >> 32), CTRL, ROW_MASK, 0xf, false);
    return v + __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    v = dpp_add_f64<0xB1, 0xf>(v);
    v = dpp_add_f64<0x4E, 0xf>(v);
    v = dpp_add_f64<0x141, 0xf>(v);
    v = dpp_add_f64<0x140, 0xf>(v);
    v = dpp_add_f64<0x142, 0xa>(v);
    v = dpp_add_f64<0x143, 0xc>(v);
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, 63);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), 63);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// One wave routes one row: full softmax, k rounds of wave-wide arg-best, optional
// renormalisation.  `keys` (n words) is LDS scratch of the calling wave; n <= 4096 (64 values
// per lane at most), k <= 32.  Results go to weights[0..k) / ids[0..k) (LDS or global) in
// selection order; every lane returns with the same view.
__device__ __forceinline__ void router_row(const float* __restrict__ z, int n, int k, float floor_value, int renorm,
                                           uint32_t* keys, float* __restrict__ weights, int64_t* __restrict__ ids) {
    const int lane = threadIdx.x & 63;
    unsigned long long best = 0ull;
    bool nan_seen = false;
    for (int i = lane; i < n; i += 64) {
        const float v = z[i];
        const uint32_t key = order_key(v);
        keys[i] = key;
        nan_seen |= isnan(v);
        const unsigned long long cand = ((unsigned long long)key << 32) | (uint32_t)~i;
        best = cand > best ? cand : best;
    }
    const bool any_nan = __any(nan_seen);
    const unsigned long long top = wave_max_u64(best);
    // maximum with NaN propagation, as the portable graph computes it
    const float m = any_nan ? __uint_as_float(0x7FC00000u) : key_value((uint32_t)(top >> 32));
    double part = 0.0;
    for (int i = lane; i < n; i += 64) part += (double)expf(z[i] - m);
    const float denom = (float)wave_sum_f64(part);
    unsigned long long used = 0ull;  // bit j: this lane's value at index lane + 64*j was taken
    float mass = 0.0f;
    float mine = 0.0f;               // lane s keeps the probability of selection s
    long long my_id = 0;
    for (int slot = 0; slot < k; ++slot) {
        unsigned long long cand = 0ull;
        for (int i = lane, j = 0; i < n; i += 64, ++j) {
            const unsigned long long c = ((unsigned long long)keys[i] << 32) | (uint32_t)~i;
            if (!((used >> j) & 1ull) && c > cand) cand = c;
        }
        // a removed or absent entry is 0, below every real candidate (~i is never 0 for i < 2^32-1)
        const unsigned long long win = wave_max_u64(cand);
        const int index = (int)~(uint32_t)win;
        if ((index & 63) == lane) used |= 1ull << (index >> 6);
        const float p = expf(key_value((uint32_t)(win >> 32)) - m) / denom;
        mass += p;
        if (lane == slot) { mine = p; my_id = index; }
    }
    if (lane < k) {
        float norm = 1.0f;
        if (renorm) norm = isnan(mass) ? mass : fmaxf(mass, floor_value);
        weights[lane] = renorm ? mine / norm : mine;
        ids[lane] = my_id;
    }
}

}  // namespace qmoe
