// Interface of the token-tile MFMA GEMM (prefill-size token batches).
#pragma once
#include "qmoe_common.hpp"

namespace qmoe {

static constexpr int GEMM_CHUNK = 32;  // tokens of one expert handled by one workgroup

// kinds of A operand: 0..2 are the element types of the C ABI; PAIR = two bf16 arrays (hi, lo)
enum { GEMM_A_F32 = QMOE_DT_F32, GEMM_A_F16 = QMOE_DT_F16, GEMM_A_BF16 = QMOE_DT_BF16, GEMM_A_PAIR = 3 };

struct GemmArgs {
    const uint8_t* w;        // weights [n, k] of expert 0 (pair: gate)
    const uint8_t* w2;       // pair: up
    int64_t stride, stride2; // bytes between experts (0 for a dense matrix)
    int n, k;
    const void* a0;          // activations, rows of a_stride elements (PAIR: hi terms)
    const void* a1;          // PAIR: lo terms
    int64_t a_stride;
    const int* gather;       // activation row of sorted position p, or null: row p
    // chunk list built on the device (null chunk_expert: one dense matrix, chunk c = rows 32c..)
    const int* chunk_expert;
    const int* chunk_start;
    const int* chunk_count;
    const int* n_chunks;
    int dense_tokens;
    // pair: SwiGLU output as bf16 hi / lo [positions, n] (out1 given) or in out_dt (out1 null);
    // else [positions, n] in out_dt, or fp32 multiplied by scale[position] when scale is given
    void* out0;
    void* out1;
    const float* scale;
    int out_dt;              // element type of an unscaled plain output
};

static constexpr int GEMM_MAX_PROBLEMS = 16;

// Dense matrices sharing the packed format, the activation element type and the token count.
struct GemmDenseProblem {
    const uint8_t* w;
    const void* x;           // [tokens, k]
    void* y;                 // [tokens, n]
    int n, k, ydt;
    int ksplit;              // set by the launcher: the four waves of a workgroup split K
};
struct GemmDenseArgs {
    int count, tokens;
    int block_start[GEMM_MAX_PROBLEMS + 1];
    GemmDenseProblem p[GEMM_MAX_PROBLEMS];
};

bool gemm_supported(int fmt, const void* w, int64_t stride, int n, int k, const void* a0, int a_kind, int64_t a_stride);
// grid = (row blocks, chunks); `chunks` is an upper bound when the list lives on the device,
// `max_count` the most tokens a chunk can hold in this call
// `side`: a dense problem (null chunk_expert, `side_chunks` chunks of its dense_tokens) of the same
// format, pairing and activation kind that shares the launch; only where gemm_side_fits says so
int gemm_launch(int fmt, bool pair, int a_kind, const GemmArgs& a, int chunks, int max_count, hipStream_t s,
                const GemmArgs* side = nullptr, int side_chunks = 0);
bool gemm_side_fits(const GemmArgs& a, int chunks, const GemmArgs& side, int side_chunks, int max_count);
// fills block_start and launches
int gemm_dense_launch(int fmt, int a_kind, GemmDenseArgs& d, hipStream_t s);

}  // namespace qmoe
