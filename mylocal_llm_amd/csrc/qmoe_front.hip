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

// The same for rows of up to 4096 columns, cut finer: a workgroup of eight waves owns two experts,
// four waves each, a wave one quarter of the row.  Everything a wave needs -- its quarter of the
// router row, of gamma and of up to four tokens -- is requested at once and kept in registers, so
// the launch is one round trip to memory (the router row comes from HBM) plus two meetings in LDS:
// the quarters' sums of squares, then the quarters' dot products, added in quarter order.
static constexpr int FRONT2_THREADS = 512, FRONT2_TOKENS = 4, FRONT2_ITERS = 4;

template <bool NORM>
__global__ __launch_bounds__(FRONT2_THREADS) void norm_router_quarters_kernel(const float* __restrict__ x, int tokens, int d,
                                                                             const float* __restrict__ gamma, float eps,
                                                                             const float* __restrict__ w, const float* __restrict__ bias,
                                                                             int n_experts, float* __restrict__ normalized,
                                                                             float* __restrict__ logits) {
    __shared__ float ss[8][FRONT2_TOKENS], dp[8][FRONT2_TOKENS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = wave >> 2, q = wave & 3;
    const int e = blockIdx.x * 2 + half;
    const bool live = e < n_experts;
    const float* const wrow = w + (size_t)(live ? e : 0) * d;
    const int qd = ((d / 4 + 3) / 4) * 4;                       // columns of a quarter (a multiple of four)
    const int c_lo = q * qd, c_hi = c_lo + qd < d ? c_lo + qd : d;
    // this block's share of the columns of `normalized`
    const int per_block = ((d / 4 + gridDim.x - 1) / gridDim.x) * 4;
    const int n0 = blockIdx.x * per_block, n1 = n0 + per_block < d ? n0 + per_block : d;
    float4 r[FRONT2_ITERS], g[FRONT2_ITERS];
#pragma unroll
    for (int it = 0; it < FRONT2_ITERS; ++it) {
        const int i = c_lo + 4 * lane + 256 * it;
        const bool in = i < c_hi;
        r[it] = in ? ldg<float4>(wrow + i) : make_float4(0, 0, 0, 0);
        g[it] = (NORM && in) ? ldg<float4>(gamma + i) : make_float4(1, 1, 1, 1);
    }
    for (int t0 = 0; t0 < tokens; t0 += FRONT2_TOKENS) {
        const int nt = tokens - t0 < FRONT2_TOKENS ? tokens - t0 : FRONT2_TOKENS;
        float4 v[FRONT2_TOKENS][FRONT2_ITERS];
#pragma unroll
        for (int j = 0; j < FRONT2_TOKENS; ++j)
#pragma unroll
            for (int it = 0; it < FRONT2_ITERS; ++it) {
                const int i = c_lo + 4 * lane + 256 * it;
                v[j][it] = (i < c_hi && j < nt) ? ldg<float4>(x + (size_t)(t0 + j) * d + i) : make_float4(0, 0, 0, 0);
            }
        float inv[FRONT2_TOKENS];
        if (NORM) {
#pragma unroll
            for (int j = 0; j < FRONT2_TOKENS; ++j) {
                float s = 0.f;
#pragma unroll
                for (int it = 0; it < FRONT2_ITERS; ++it)
                    s += (v[j][it].x * v[j][it].x + v[j][it].y * v[j][it].y) + (v[j][it].z * v[j][it].z + v[j][it].w * v[j][it].w);
                s = wave_sum(s);
                if (lane == 0) ss[wave][j] = s;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < FRONT2_TOKENS; ++j) {
                const float total = ((ss[4 * half][j] + ss[4 * half + 1][j]) + ss[4 * half + 2][j]) + ss[4 * half + 3][j];
                inv[j] = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(total, (float)d) + eps));
            }
        }
#pragma unroll
        for (int j = 0; j < FRONT2_TOKENS; ++j) {
            float acc = 0.f;
#pragma unroll
            for (int it = 0; it < FRONT2_ITERS; ++it) {
                const float4 a = v[j][it];
                if (NORM)
                    acc += (mul_unfused(mul_unfused(a.x, inv[j]), g[it].x) * r[it].x + mul_unfused(mul_unfused(a.y, inv[j]), g[it].y) * r[it].y) +
                           (mul_unfused(mul_unfused(a.z, inv[j]), g[it].z) * r[it].z + mul_unfused(mul_unfused(a.w, inv[j]), g[it].w) * r[it].w);
                else
                    acc += (a.x * r[it].x + a.y * r[it].y) + (a.z * r[it].z + a.w * r[it].w);
            }
            acc = wave_sum(acc);
            if (lane == 0) dp[wave][j] = acc;
        }
        __syncthreads();
        if (q == 0 && lane < nt && live) {
            const float sum = ((dp[4 * half][lane] + dp[4 * half + 1][lane]) + dp[4 * half + 2][lane]) + dp[4 * half + 3][lane];
            logits[(size_t)(t0 + lane) * n_experts + e] = sum + (bias ? bias[e] : 0.0f);
        }
        if (NORM) {
            // (the inverse RMS of a token is the same in every wave: any wave's copy will do)
            for (int idx = threadIdx.x; idx < nt * (per_block / 4); idx += FRONT2_THREADS) {
                const int j = idx / (per_block / 4), i = n0 + 4 * (idx % (per_block / 4));
                if (i < n1) {
                    const float4 xv = ldg<float4>(x + (size_t)(t0 + j) * d + i), gv = ldg<float4>(gamma + i);
                    const float total = ((ss[0][j] + ss[1][j]) + ss[2][j]) + ss[3][j];
                    const float iv = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(total, (float)d) + eps));
                    stg<float4>(normalized + (size_t)(t0 + j) * d + i,
                                make_float4(mul_unfused(mul_unfused(xv.x, iv), gv.x), mul_unfused(mul_unfused(xv.y, iv), gv.y),
                                            mul_unfused(mul_unfused(xv.z, iv), gv.z), mul_unfused(mul_unfused(xv.w, iv), gv.w)));
                }
            }
        }
        __syncthreads();   // the LDS cells are written again by the next group of tokens
    }
}

template <bool NORM>
static void launch_norm_router(const float* x, int tokens, int d, const float* gamma, float eps, const float* w, const float* bias,
                               int n_experts, float* normalized, float* logits, hipStream_t s) {
    if (d <= 4 * 256 * FRONT2_ITERS)
        hipLaunchKernelGGL(norm_router_quarters_kernel<NORM>, dim3((n_experts + 1) / 2), dim3(FRONT2_THREADS), 0, s, x, tokens, d, gamma,
                           eps, w, bias, n_experts, normalized, logits);
    else
        hipLaunchKernelGGL(norm_router_kernel<NORM>, dim3((n_experts + 3) / 4), dim3(256), 0, s, x, tokens, d, gamma, eps, w, bias,
                           n_experts, normalized, logits);
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
    launch_norm_router<true>(x, tokens, d_model, gamma, eps, router_w, router_b, n_experts, normalized, logits, (hipStream_t)stream);
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
    launch_norm_router<false>(x, tokens, d_model, (const float*)nullptr, 0.0f, router_w, router_b, n_experts, (float*)nullptr, logits,
                              (hipStream_t)stream);
    return check_launch("qmoe_router_logits");
}
