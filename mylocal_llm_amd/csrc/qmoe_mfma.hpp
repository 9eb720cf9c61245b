// bf16 MFMA operand helpers of the token-tile GEMM.
#pragma once
#include "qmoe_common.hpp"

namespace qmoe {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

// bf16 pair from two floats that are exactly representable (upper halves of the fp32 words)
__device__ __forceinline__ uint32_t pack_exact_bf16(float a, float b) {
    return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xFFFF0000u);
}

union OperandBits {
    bf16x8 v;
    uint32_t u[4];
};

// Eight fp32 values -> two bf16 terms: hi = the value rounded to nearest bf16, lo = the exact
// remainder rounded to nearest bf16; hi + lo carries 16 significant bits of each value.
__device__ __forceinline__ void split_terms(const float* v, OperandBits& hi, OperandBits& lo) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float a = v[2 * i], b = v[2 * i + 1];
        hi.v[2 * i] = (__bf16)a;
        hi.v[2 * i + 1] = (__bf16)b;
        const float ra = a - __uint_as_float(hi.u[i] << 16);
        const float rb = b - __uint_as_float(hi.u[i] & 0xFFFF0000u);
        lo.v[2 * i] = (__bf16)ra;
        lo.v[2 * i + 1] = (__bf16)rb;
    }
}


template <int FMT> struct BTerms { static constexpr int N = FMT == QMOE_FMT_BF16 ? 1 : 2; };

}  // namespace qmoe
