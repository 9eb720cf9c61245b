// One wave, one packed row, MT activation rows: the dequant-fused dot product that the
// linear, SwiGLU and expert kernels are built from.
#pragma once
#include "qmoe_common.hpp"
#include "qmoe_formats.hpp"

namespace qmoe {

// Per-lane partial sums of  sum_i W[row, i] * x[m][i]  over the lane's units of the row.
// `fast` says the row is aligned for the format's unit loads; otherwise (and for the
// elements past the last whole unit) weights are decoded one element at a time.
template <int FMT, int XDT, int MT>
__device__ __forceinline__ void row_dot_fmt(const uint8_t* __restrict__ row, int k, bool fast,
                                            const void* __restrict__ x, const size_t* xbase, int lane,
                                            float* acc) {
    using F = Fmt<FMT>;
    const int units = fast ? F::units_per_row(k) : 0;
    for (int u = lane; u < units; u += 64) {
        float w[F::UNIT];
        F::decode(row, u, w);
#pragma unroll
        for (int g = 0; g < F::GROUPS; ++g) {
            const int xo = F::xoff(u, g);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float4 xv = Elem<XDT>::load4(x, xbase[m] + xo);
                acc[m] += w[4 * g] * xv.x + w[4 * g + 1] * xv.y + w[4 * g + 2] * xv.z + w[4 * g + 3] * xv.w;
            }
        }
    }
    for (int i = units * F::UNIT + lane; i < k; i += 64) {
        float wv = F::element(row + (size_t)(i / F::BLOCK_ELEMS) * F::BLOCK_BYTES, i % F::BLOCK_ELEMS);
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] += wv * Elem<XDT>::load(x, xbase[m] + i);
    }
}

// Format chosen at run time (uniform across the launch).
template <int XDT, int MT>
__device__ __forceinline__ void row_dot(int fmt, const uint8_t* __restrict__ row, int k, bool fast,
                                        const void* __restrict__ x, const size_t* xbase, int lane,
                                        float* acc) {
    switch (fmt) {
    case QMOE_FMT_Q8_0: row_dot_fmt<QMOE_FMT_Q8_0, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    case QMOE_FMT_Q4_0: row_dot_fmt<QMOE_FMT_Q4_0, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    case QMOE_FMT_Q3_K: row_dot_fmt<QMOE_FMT_Q3_K, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    case QMOE_FMT_Q4_K: row_dot_fmt<QMOE_FMT_Q4_K, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    case QMOE_FMT_Q5_K: row_dot_fmt<QMOE_FMT_Q5_K, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    case QMOE_FMT_Q6_K: row_dot_fmt<QMOE_FMT_Q6_K, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    default: row_dot_fmt<QMOE_FMT_BF16, XDT, MT>(row, k, fast, x, xbase, lane, acc); break;
    }
}

// Host: may rows of this matrix use the unit loads?  Needs the base and the row stride
// aligned to the widest load the format's decoder issues, and activations aligned for
// 128-bit (fp32) / 64-bit (16-bit types) loads.
inline bool rows_fast(int fmt, const void* w, int64_t row_stride_bytes, int64_t k) {
    int align = (fmt == QMOE_FMT_Q8_0 || fmt == QMOE_FMT_Q4_K || fmt == QMOE_FMT_Q5_K) ? 4 : 2;
    if (((uintptr_t)w % align) || (row_stride_bytes % align)) return false;
    if (fmt == QMOE_FMT_BF16 && (k % 8)) return false;
    return (k % 4) == 0;
}
inline bool x_fast(const void* x, int dtype, int64_t k) {
    return ((uintptr_t)x % 16) == 0 && ((k * dtype_size(dtype)) % 16) == 0;
}

}  // namespace qmoe
