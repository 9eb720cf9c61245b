// Shared host/device helpers of libqmoe_hip.
#pragma once
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/qmoe.h"

namespace qmoe {

// ---- error reporting (thread-local message, int status) --------------------------------
char* error_buffer();
int fail(int status, const char* fmt, ...);
int check_launch(const char* what);

// ---- element types ---------------------------------------------------------------------
template <int DT> struct Elem;
template <> struct Elem<QMOE_DT_F32> {
    using T = float;
    __device__ static float load(const void* p, size_t i) { return ((const float*)p)[i]; }
    __device__ static float4 load4(const void* p, size_t i) { return *(const float4*)((const float*)p + i); }
};
template <> struct Elem<QMOE_DT_F16> {
    using T = __half;
    __device__ static float load(const void* p, size_t i) { return __half2float(((const __half*)p)[i]); }
    __device__ static float4 load4(const void* p, size_t i) {
        uint2 v = *(const uint2*)((const __half*)p + i);
        __half2 a = *(__half2*)&v.x, b = *(__half2*)&v.y;
        float2 fa = __half22float2(a), fb = __half22float2(b);
        return make_float4(fa.x, fa.y, fb.x, fb.y);
    }
};
template <> struct Elem<QMOE_DT_BF16> {
    using T = __hip_bfloat16;
    __device__ static float load(const void* p, size_t i) {
        return __uint_as_float((uint32_t)((const uint16_t*)p)[i] << 16);
    }
    __device__ static float4 load4(const void* p, size_t i) {
        uint2 v = *(const uint2*)((const uint16_t*)p + i);
        return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xFFFF0000u),
                           __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xFFFF0000u));
    }
};

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    uint32_t b = __float_as_uint(f);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x40u);
    return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}

// Store one fp32 result rounded once to the output element type.
__device__ __forceinline__ void store_out(void* y, int dtype, size_t i, float v) {
    if (dtype == QMOE_DT_F32) ((float*)y)[i] = v;
    else if (dtype == QMOE_DT_F16) ((__half*)y)[i] = __float2half_rn(v);
    else ((uint16_t*)y)[i] = float_to_bf16_bits(v);
}

inline int dtype_size(int dt) { return dt == QMOE_DT_F32 ? 4 : (dt == QMOE_DT_F16 || dt == QMOE_DT_BF16) ? 2 : 0; }

// ---- wave64 reductions -----------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// acc + round(a * b): the product is rounded to fp32 before the add, never fused into an FMA
// (the reference stores each routed product before accumulating it).
__device__ __forceinline__ float add_product(float acc, float a, float b) {
#pragma clang fp contract(off)
    const float prod = a * b;
    return acc + prod;
}
__device__ __forceinline__ float mul_unfused(float a, float b) {
#pragma clang fp contract(off)
    return a * b;
}

// g / (1 + exp(-g)) * u, the SwiGLU of mini_llm/ops/quantized_linear.py:367-370.
__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.0f + expf(-g))) * u; }

}  // namespace qmoe
