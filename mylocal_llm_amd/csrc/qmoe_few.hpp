// Interface of the few-token (2..4) streaming kernel for Q8_0 rows of 1024..16384 columns.
#pragma once
#include "qmoe_common.hpp"

namespace qmoe {

static constexpr int FEW_MAX_PROBLEMS = 16;

struct FewProblem {
    const uint8_t* w;   // [n, k] Q8_0
    const void* x;      // [tokens, k]
    void* y;            // [tokens, n]
    int n, k, ydt;
};
// Problems of one launch share the token count and the activation element type, and are all
// wide (few_is_wide) or all not.
struct FewArgs {
    int count, tokens, xdt;
    int group_start[FEW_MAX_PROBLEMS + 1];   // filled by few_launch: first group of four rows of each problem
    FewProblem p[FEW_MAX_PROBLEMS];
};

bool few_supported(int fmt, const void* w, int n, int k, const void* x, int xdt, int tokens);
bool few_is_wide(int k);
int few_launch(FewArgs& a, hipStream_t s);

}  // namespace qmoe
