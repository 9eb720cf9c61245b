// Router row primitive shared by the stand-alone router kernel and the fused decode path.
#pragma once
#include "qmoe_common.hpp"

namespace qmoe {

// Monotone unsigned image of a float for selection: larger value -> larger key, -0 == +0,
// every NaN -> 0 (below -inf): the order "descending value, NaN last" of
// mini_llm/ops/router_decode.py:19-26; ties go to the lower id.
__device__ __forceinline__ uint32_t order_key(float v) {
    if (isnan(v)) return 0u;
    const uint32_t b = __float_as_uint(v == 0.0f ? 0.0f : v);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
    if (key <= 1u) return __uint_as_float(0x7FC00000u);
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
    return o > v ? o : v;
}
// Maximum over the wave, in a scalar register.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = dpp_max_u32<0xB1, 0xf>(v);
    v = dpp_max_u32<0x4E, 0xf>(v);
    v = dpp_max_u32<0x141, 0xf>(v);
    v = dpp_max_u32<0x140, 0xf>(v);
    v = dpp_max_u32<0x142, 0xa>(v);
    v = dpp_max_u32<0x143, 0xc>(v);
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
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

// One wave routes one row held in registers (NV values per lane, n <= 64*NV): full softmax,
// k rounds of wave-wide arg-best, optional renormalisation.  load() only issues the row's
// loads, so a caller can put further loads in flight before select() waits for the row;
// nothing in the selection rounds touches memory.  Lane s < k receives selection s.
//
// Selection keys are 32 bits: order_key, with every NaN raised to 1 (below -inf = 0x007FFFFF,
// above 0 = "taken or absent").  A round is one DPP maximum of the keys; the owner is the
// lowest index holding that key (lowest j first, then lowest lane, as index = lane + 64 j).
template <int NV> struct RouterRow {
    float v[NV];

    __device__ __forceinline__ void load(const float* __restrict__ z, int n) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = lane + 64 * j;
            v[j] = i < n ? z[i] : 0.0f;
        }
    }

    __device__ __forceinline__ void select(int n, int k, float floor_value, int renorm, float& weight, int64_t& id) {
        const int lane = threadIdx.x & 63;
        uint32_t key[NV];
        uint32_t best = 0u;
        bool nan_seen = false;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const bool valid = lane + 64 * j < n;
            const uint32_t ok = order_key(v[j]);
            key[j] = valid ? (ok ? ok : 1u) : 0u;
            nan_seen |= valid && ok == 0u;
            best = key[j] > best ? key[j] : best;
        }
        const bool any_nan = __any(nan_seen);
        // maximum with NaN propagation, as the portable graph computes it
        const float m = any_nan ? __uint_as_float(0x7FC00000u) : key_value(wave_max_u32(best));
        double part = 0.0;
#pragma unroll
        for (int j = 0; j < NV; ++j)
            if (lane + 64 * j < n) part += (double)expf(v[j] - m);
        const float denom = (float)wave_sum_f64(part);
        uint32_t my_key = 0u;
        int my_id = 0;
        for (int slot = 0; slot < k; ++slot) {
            uint32_t c = 0u;
#pragma unroll
            for (int j = 0; j < NV; ++j) c = key[j] > c ? key[j] : c;
            const uint32_t win = wave_max_u32(c);
            // owner: first j with a holder, then the lowest lane holding it there
            int wj = -1;
            unsigned long long holders = 0ull;
#pragma unroll
            for (int j = NV - 1; j >= 0; --j) {
                const unsigned long long b = __ballot(key[j] == win);
                if (b) { wj = j; holders = b; }
            }
            const int wl = __builtin_ctzll(holders);
#pragma unroll
            for (int j = 0; j < NV; ++j)
                if (j == wj) key[j] = lane == wl ? 0u : key[j];
            if (lane == slot) { my_key = win; my_id = wl + 64 * wj; }
        }
        // probabilities in parallel; their sum in selection order
        const float p = lane < k ? expf(key_value(my_key) - m) / denom : 0.0f;
        float mass = 0.0f;
        for (int slot = 0; slot < k; ++slot) mass += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), slot));
        float norm = 1.0f;
        if (renorm) norm = isnan(mass) ? mass : fmaxf(mass, floor_value);
        weight = renorm ? p / norm : p;
        id = my_id;
    }
};

// One wave routes one row of any supported width (n <= 64 * MAXNV <= 4096, k <= 32); callers
// that are short of registers cap the width they accept.  `between` runs after the row's
// loads are issued and before anything waits for them.
template <int MAXNV = 64, typename Between>
__device__ __forceinline__ void router_row(const float* __restrict__ z, int n, int k, float floor_value, int renorm,
                                           float& weight, int64_t& id, Between&& between) {
    if (n <= 512) { RouterRow<8> r; r.load(z, n); between(); r.select(n, k, floor_value, renorm, weight, id); }
    else if (n <= 1024 || MAXNV <= 16) { RouterRow<16> r; r.load(z, n); between(); r.select(n, k, floor_value, renorm, weight, id); }
    else if (n <= 2048 || MAXNV <= 32) { RouterRow<32> r; r.load(z, n); between(); r.select(n, k, floor_value, renorm, weight, id); }
    else { RouterRow<64> r; r.load(z, n); between(); r.select(n, k, floor_value, renorm, weight, id); }
}

}  // namespace qmoe
