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

// ---- launch status ---------------------------------------------------------------------------
// One word per GPU inside the library's device image.  Kernels with bounded waits raise bits in
// it (vector stores) instead of hanging or returning wrong results silently; qmoe_check_status
// reads and clears it.  launch_status_word gives the word's address on the current device
// (resolved once per device), wait_limit_ticks the bound of such a wait in 100 MHz ticks.
static constexpr uint32_t QMOE_STATUS_WAIT_EXPIRED = 1u;
int launch_status_word(uint32_t** out);
int64_t wait_limit_ticks();
int static_scratch(void** out);

// ---- global memory access ----------------------------------------------------------------
// Pointers that reach a kernel inside an argument struct or through LDS carry no address
// space, and loads through them become FLAT instructions: those may complete out of order, so
// every wait behind one drains ALL outstanding loads and nothing stays in flight across a
// reduction.  Everything a caller hands over is device global memory: these accessors say so.
#define QMOE_GLOBAL __attribute__((address_space(1)))
// (scalar and built-in vector types only: copying a class type would bind its source to a
// reference without an address space again)
template <class T> __device__ __forceinline__ T ldg(const void* p) { return *(const QMOE_GLOBAL T*)p; }
template <class T> __device__ __forceinline__ void stg(void* p, T v) { *(QMOE_GLOBAL T*)p = v; }
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
// 16 / 8 bytes from an address aligned to ALIGN bytes
template <int ALIGN> struct AlignedVec;
#define QMOE_ALIGNED_VEC(A)                                                  \
    template <> struct AlignedVec<A> {                                       \
        typedef u32x4_t V4 __attribute__((aligned(A)));                      \
        typedef u32x2_t V2 __attribute__((aligned(A < 8 ? A : 8)));          \
    };
QMOE_ALIGNED_VEC(2) QMOE_ALIGNED_VEC(4) QMOE_ALIGNED_VEC(8) QMOE_ALIGNED_VEC(16)
#undef QMOE_ALIGNED_VEC
template <int ALIGN> __device__ __forceinline__ u32x4_t ldg_u32x4(const void* p) {
    return *(const QMOE_GLOBAL typename AlignedVec<ALIGN>::V4*)p;
}
template <int ALIGN> __device__ __forceinline__ u32x2_t ldg_u32x2(const void* p) {
    return *(const QMOE_GLOBAL typename AlignedVec<ALIGN>::V2*)p;
}
template <> __device__ __forceinline__ float4 ldg<float4>(const void* p) {
    const f32x4_t v = *(const QMOE_GLOBAL f32x4_t*)p;
    return make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ uint4 ldg<uint4>(const void* p) {
    const u32x4_t v = ldg_u32x4<16>(p);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ uint2 ldg<uint2>(const void* p) {
    const u32x2_t v = ldg_u32x2<8>(p);
    return make_uint2(v[0], v[1]);
}
template <> __device__ __forceinline__ void stg<float4>(void* p, float4 v) {
    *(QMOE_GLOBAL f32x4_t*)p = f32x4_t{v.x, v.y, v.z, v.w};
}

// ---- element types ---------------------------------------------------------------------
template <int DT> struct Elem;
template <> struct Elem<QMOE_DT_F32> {
    using T = float;
    __device__ static float load(const void* p, size_t i) { return ldg<float>((const float*)p + i); }
    __device__ static float4 load4(const void* p, size_t i) { return ldg<float4>((const float*)p + i); }
};
template <> struct Elem<QMOE_DT_F16> {
    using T = __half;
    __device__ static float load(const void* p, size_t i) { return __half2float(__ushort_as_half(ldg<unsigned short>((const __half*)p + i))); }
    __device__ static float4 load4(const void* p, size_t i) {
        uint2 v = ldg<uint2>((const __half*)p + i);
        __half2 a = *(__half2*)&v.x, b = *(__half2*)&v.y;
        float2 fa = __half22float2(a), fb = __half22float2(b);
        return make_float4(fa.x, fa.y, fb.x, fb.y);
    }
};
template <> struct Elem<QMOE_DT_BF16> {
    using T = __hip_bfloat16;
    __device__ static float load(const void* p, size_t i) {
        return __uint_as_float((uint32_t)ldg<uint16_t>((const uint16_t*)p + i) << 16);
    }
    __device__ static float4 load4(const void* p, size_t i) {
        uint2 v = ldg<uint2>((const uint16_t*)p + i);
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
    if (dtype == QMOE_DT_F32) stg<float>((float*)y + i, v);
    else if (dtype == QMOE_DT_F16) stg<unsigned short>((__half*)y + i, __half_as_ushort(__float2half_rn(v)));
    else stg<uint16_t>((uint16_t*)y + i, float_to_bf16_bits(v));
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
