// The step in front of the MoE block: RMSNorm of the residual stream and the router's logits,
// in one launch.
//
//   normalized[t] = (x[t] * inv_rms[t]) * gamma,  inv_rms = 1 / sqrt(mean(x[t]^2) + eps)
//                   (mini_llm/ops/rmsnorm_inference.py:109-118 and :517-520: divide, square root and
//                   reciprocal as separate correctly rounded operations, products not fused)
//   logits[t][e]  = normalized[t] . W[e] + b[e]      (mini_llm/ops/router_inference.py:40-46, fp32)
//
// Block b owns four experts (one wave each) and a slice of the columns of `normalized`; tokens are
// walked in groups of eight whose inverse RMS values the block computes itself (d_model floats per
// token from L2), so no grid-wide step separates the norm from the dot products.
#include "qmoe_common.hpp"

namespace qmoe {

static constexpr int FRONT_TOKENS = 8;

// One expert's logits for up to NT tokens: the expert's row and gamma are read once, the tokens'
// loads travel together.
template <int NT, bool NORM>
__device__ __forceinline__ void front_dots(const float* __restrict__ x, int d, int nt, const float* __restrict__ gamma,
                                           const float* __restrict__ wrow, const float* inv_rms, int lane, bool live,
                                           float bias, float* __restrict__ out, int out_stride) {
    float inv[NT], acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) { inv[j] = inv_rms[j < nt ? j : 0]; acc[j] = 0.f; }
    for (int i = 4 * lane; i < d; i += 256) {
        const float4 r = ldg<float4>(wrow + i);
        float4 v[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) v[j] = ldg<float4>(x + (size_t)(j < nt ? j : 0) * d + i);
        if (!NORM) {   // x is what the router multiplies
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[j] += (v[j].x * r.x + v[j].y * r.y) + (v[j].z * r.z + v[j].w * r.w);
            continue;
        }
        const float4 g = ldg<float4>(gamma + i);
#pragma unroll
        for (int j = 0; j < NT; ++j)
            acc[j] += (mul_unfused(mul_unfused(v[j].x, inv[j]), g.x) * r.x + mul_unfused(mul_unfused(v[j].y, inv[j]), g.y) * r.y) +
                      (mul_unfused(mul_unfused(v[j].z, inv[j]), g.z) * r.z + mul_unfused(mul_unfused(v[j].w, inv[j]), g.w) * r.w);
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const float sum = wave_sum(acc[j]);
        if (lane == 0 && j < nt && live) out[(size_t)j * out_stride] = sum + bias;
    }
}

template <bool NORM>
__global__ __launch_bounds__(256) void norm_router_kernel(const float* __restrict__ x, int tokens, int d,
                                                          const float* __restrict__ gamma, float eps,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          int n_experts, float* __restrict__ normalized,
                                                          float* __restrict__ logits) {
    __shared__ float inv_rms[FRONT_TOKENS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = blockIdx.x * 4 + wave;
    const float* wrow = w + (size_t)(e < n_experts ? e : 0) * d;
    // this block's share of the columns of `normalized`
    const int per_block = ((d / 4 + gridDim.x - 1) / gridDim.x) * 4;
    const int c0 = blockIdx.x * per_block, c1 = c0 + per_block < d ? c0 + per_block : d;
    for (int t0 = 0; t0 < tokens; t0 += FRONT_TOKENS) {
        const int nt = tokens - t0 < FRONT_TOKENS ? tokens - t0 : FRONT_TOKENS;
        __syncthreads();
        if (NORM) {
            // sums of squares: wave w takes tokens w and w + 4 of the group, both at once
            const int ja = wave, jb = wave + 4;
            const float* xa = x + (size_t)(t0 + (ja < nt ? ja : 0)) * d;
            const float* xb = x + (size_t)(t0 + (jb < nt ? jb : 0)) * d;
            float sa = 0.f, sb = 0.f;
            for (int i = 4 * lane; i < d; i += 256) {
                const float4 va = ldg<float4>(xa + i), vb = ldg<float4>(xb + i);
                sa += (va.x * va.x + va.y * va.y) + (va.z * va.z + va.w * va.w);
                sb += (vb.x * vb.x + vb.y * vb.y) + (vb.z * vb.z + vb.w * vb.w);
            }
            sa = wave_sum(sa);
            sb = wave_sum(sb);
            if (lane == 0) {
                if (ja < nt) inv_rms[ja] = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(sa, (float)d) + eps));
                if (jb < nt) inv_rms[jb] = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(sb, (float)d) + eps));
            }
        }
        __syncthreads();
        if (nt == 1) front_dots<1, NORM>(x + (size_t)t0 * d, d, nt, gamma, wrow, inv_rms, lane, e < n_experts, bias ? bias[e < n_experts ? e : 0] : 0.0f, logits + (size_t)t0 * n_experts + e, n_experts);
        else if (nt == 2) front_dots<2, NORM>(x + (size_t)t0 * d, d, nt, gamma, wrow, inv_rms, lane, e < n_experts, bias ? bias[e < n_experts ? e : 0] : 0.0f, logits + (size_t)t0 * n_experts + e, n_experts);
        else if (nt <= 4) front_dots<4, NORM>(x + (size_t)t0 * d, d, nt, gamma, wrow, inv_rms, lane, e < n_experts, bias ? bias[e < n_experts ? e : 0] : 0.0f, logits + (size_t)t0 * n_experts + e, n_experts);
        else front_dots<FRONT_TOKENS, NORM>(x + (size_t)t0 * d, d, nt, gamma, wrow, inv_rms, lane, e < n_experts, bias ? bias[e < n_experts ? e : 0] : 0.0f, logits + (size_t)t0 * n_experts + e, n_experts);
        if (!NORM) continue;
        for (int idx = threadIdx.x; idx < nt * (per_block / 4); idx += 256) {
            const int j = idx / (per_block / 4), i = c0 + 4 * (idx % (per_block / 4));
            if (i < c1) {
                const float4 v = ldg<float4>(x + (size_t)(t0 + j) * d + i), g = ldg<float4>(gamma + i);
                const float inv = inv_rms[j];
                stg<float4>(normalized + (size_t)(t0 + j) * d + i,
                            make_float4(mul_unfused(mul_unfused(v.x, inv), g.x), mul_unfused(mul_unfused(v.y, inv), g.y),
                                        mul_unfused(mul_unfused(v.z, inv), g.z), mul_unfused(mul_unfused(v.w, inv), g.w)));
            }
        }
    }
}

}  // namespace qmoe

using namespace qmoe;

extern "C" int qmoe_norm_router(const float* x, int tokens, int d_model, const float* gamma, float eps,
                                const float* router_w, const float* router_b, int n_experts, float* normalized,
                                float* logits, void* stream) {
    if (!x || !gamma || !router_w || !normalized || !logits)
        return fail(QMOE_EINVAL, "qmoe_norm_router: null pointer");
    if (tokens < 1 || d_model < 4 || n_experts < 1 || !(eps >= 0.0f))
        return fail(QMOE_EINVAL, "qmoe_norm_router: tokens=%d d_model=%d n_experts=%d eps=%g", tokens, d_model, n_experts, (double)eps);
    if (d_model % 4) return fail(QMOE_EUNSUPPORTED, "qmoe_norm_router: d_model=%d is not a multiple of 4", d_model);
    if (((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)router_w | (uintptr_t)normalized) % 16)
        return fail(QMOE_EUNSUPPORTED, "qmoe_norm_router: x, gamma, router_w and normalized must be 16-byte aligned");
    hipLaunchKernelGGL(norm_router_kernel<true>, dim3((n_experts + 3) / 4), dim3(256), 0, (hipStream_t)stream, x, tokens, d_model,
                       gamma, eps, router_w, router_b, n_experts, normalized, logits);
    return check_launch("qmoe_norm_router");
}

extern "C" int qmoe_router_logits(const float* x, int tokens, int d_model, const float* router_w,
                                  const float* router_b, int n_experts, float* logits, void* stream) {
    if (!x || !router_w || !logits) return fail(QMOE_EINVAL, "qmoe_router_logits: null pointer");
    if (tokens < 1 || d_model < 4 || n_experts < 1)
        return fail(QMOE_EINVAL, "qmoe_router_logits: tokens=%d d_model=%d n_experts=%d", tokens, d_model, n_experts);
    if (d_model % 4) return fail(QMOE_EUNSUPPORTED, "qmoe_router_logits: d_model=%d is not a multiple of 4", d_model);
    if (((uintptr_t)x | (uintptr_t)router_w) % 16)
        return fail(QMOE_EUNSUPPORTED, "qmoe_router_logits: x and router_w must be 16-byte aligned");
    hipLaunchKernelGGL(norm_router_kernel<false>, dim3((n_experts + 3) / 4), dim3(256), 0, (hipStream_t)stream, x, tokens,
                       d_model, (const float*)nullptr, 0.0f, router_w, router_b, n_experts, (float*)nullptr, logits);
    return check_launch("qmoe_router_logits");
}
