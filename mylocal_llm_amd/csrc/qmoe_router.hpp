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

// One wave routes one row with the row held in registers (NV values per lane, n <= 64*NV):
// full softmax, k rounds of wave-wide arg-best, optional renormalisation.  All loads of the
// row are issued together; nothing in the selection rounds touches memory.  Results go to
// weights[0..k) / ids[0..k) (LDS or global) in selection order.
template <int NV>
__device__ __forceinline__ void router_row_regs(const float* __restrict__ z, int n, int k, float floor_value,
                                                int renorm, float* __restrict__ weights, int64_t* __restrict__ ids) {
    const int lane = threadIdx.x & 63;
    float v[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = lane + 64 * j;
        v[j] = i < n ? z[i] : 0.0f;
    }
    unsigned long long cand[NV];
    unsigned long long best = 0ull;
    bool nan_seen = false;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = lane + 64 * j;
        const bool valid = i < n;
        cand[j] = valid ? (((unsigned long long)order_key(v[j]) << 32) | (uint32_t)~i) : 0ull;
        nan_seen |= valid && isnan(v[j]);
        best = cand[j] > best ? cand[j] : best;
    }
    const bool any_nan = __any(nan_seen);
    const unsigned long long top = wave_max_u64(best);
    // maximum with NaN propagation, as the portable graph computes it
    const float m = any_nan ? __uint_as_float(0x7FC00000u) : key_value((uint32_t)(top >> 32));
    double part = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j)
        if (lane + 64 * j < n) part += (double)expf(v[j] - m);
    const float denom = (float)wave_sum_f64(part);
    float mass = 0.0f;
    float mine = 0.0f;  // lane s keeps the probability of selection s
    long long my_id = 0;
    for (int slot = 0; slot < k; ++slot) {
        unsigned long long c = 0ull;
#pragma unroll
        for (int j = 0; j < NV; ++j) c = cand[j] > c ? cand[j] : c;
        // a removed or absent entry is 0, below every real candidate (~i is never 0)
        const unsigned long long win = wave_max_u64(c);
#pragma unroll
        for (int j = 0; j < NV; ++j) cand[j] = cand[j] == win ? 0ull : cand[j];  // ids are unique: only the owner matches
        const float p = expf(key_value((uint32_t)(win >> 32)) - m) / denom;
        mass += p;
        if (lane == slot) { mine = p; my_id = (int)~(uint32_t)win; }
    }
    if (lane < k) {
        float norm = 1.0f;
        if (renorm) norm = isnan(mass) ? mass : fmaxf(mass, floor_value);
        weights[lane] = renorm ? mine / norm : mine;
        ids[lane] = my_id;
    }
}

// One wave routes one row of any supported width (n <= 64 * MAXNV <= 4096, k <= 32); callers
// that are short of registers cap the width they accept.
template <int MAXNV = 64>
__device__ __forceinline__ void router_row(const float* __restrict__ z, int n, int k, float floor_value, int renorm,
                                           float* __restrict__ weights, int64_t* __restrict__ ids) {
    if (n <= 512) router_row_regs<8>(z, n, k, floor_value, renorm, weights, ids);
    else if (n <= 1024 || MAXNV <= 16) router_row_regs<16>(z, n, k, floor_value, renorm, weights, ids);
    else if (n <= 2048 || MAXNV <= 32) router_row_regs<32>(z, n, k, floor_value, renorm, weights, ids);
    else router_row_regs<64>(z, n, k, floor_value, renorm, weights, ids);
}

}  // namespace qmoe
