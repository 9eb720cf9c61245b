// Router: full softmax over all experts, exact top-k selection, optional renormalisation
// of the selected mass.  One wave per token row; the row lives in registers, selection is k
// rounds of a wave-wide arg-best under the reference's order (descending value, NaN last,
// lower id on ties: mini_llm/ops/router_decode.py:19-26).
#include "qmoe_router.hpp"

namespace qmoe {

__global__ __launch_bounds__(64) void router_topk_kernel(const float* __restrict__ logits, int n, int k,
                                                         float floor_value, int renorm,
                                                         float* __restrict__ weights, int64_t* __restrict__ ids) {
    float w;
    int64_t id;
    router_row(logits + (size_t)blockIdx.x * n, n, k, floor_value, renorm, w, id, [] {});
    if ((int)threadIdx.x < k) {
        weights[(size_t)blockIdx.x * k + threadIdx.x] = w;
        ids[(size_t)blockIdx.x * k + threadIdx.x] = id;
    }
}

int router_topk_impl(const float* logits, int tokens, int n, int k, float floor_value, int renorm, float* weights,
                     int64_t* ids, hipStream_t s) {
    if (!logits || !weights || !ids) return fail(QMOE_EINVAL, "qmoe_router_topk: null pointer");
    if (tokens < 0) return fail(QMOE_EINVAL, "qmoe_router_topk: negative token count");
    if (n < 1 || n > 4096) return fail(QMOE_EUNSUPPORTED, "qmoe_router_topk: expert count %d outside 1..4096", n);
    if (k < 1 || k > 32 || k > n) return fail(QMOE_EUNSUPPORTED, "qmoe_router_topk: k=%d outside 1..min(32, n)", k);
    if (renorm && !(floor_value >= 1.17549435e-38f && floor_value <= 3.40282347e38f))
        return fail(QMOE_EINVAL, "qmoe_router_topk: normalisation floor must be a finite positive normal float");
    if ((uintptr_t)logits % 4 || (uintptr_t)weights % 4 || (uintptr_t)ids % 8)
        return fail(QMOE_EINVAL, "qmoe_router_topk: misaligned pointer");
    if (tokens == 0) return QMOE_OK;
    hipLaunchKernelGGL(router_topk_kernel, dim3(tokens), dim3(64), 0, s, logits, n, k,
                       floor_value, renorm, weights, ids);
    return check_launch("qmoe_router_topk");
}

}  // namespace qmoe

extern "C" int qmoe_router_topk(const float* logits, int tokens, int n, int k, float floor_value, int renormalize,
                                float* weights, int64_t* ids, void* stream) {
    return qmoe::router_topk_impl(logits, tokens, n, k, floor_value, renormalize, weights, ids, (hipStream_t)stream);
}
