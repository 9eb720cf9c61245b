/* qmoe.h -- C ABI of libqmoe_hip.so: GGUF packed-weight linear and packed-expert
 * MoE step on one AMD Instinct MI355X (gfx950).
 *
 * Conventions (they follow the reference's existing native library,
 * mini_llm/ops/native_packed_cpu.cpp:206-246, loaded by
 * mini_llm/ops/native_packed_cpu.py:67-77):
 *   - every function is extern "C", takes plain pointers and sizes, and returns an
 *     int status: 0 = success, nonzero = error; on error no kernel has touched the
 *     output.  qmoe_last_error() returns a thread-local message for the last
 *     nonzero status on the calling thread.
 *   - every pointer named w/gate/up/down/x/y/out/logits/... is DEVICE memory on the
 *     current HIP device unless its comment says "host".  The caller owns all
 *     buffers; the library keeps no pointer after the call's work has drained from
 *     `stream`.  Weights and inputs are never written.
 *   - work is enqueued asynchronously on `stream` (a hipStream_t passed as void*;
 *     NULL = the null stream).  No call synchronises the device or allocates
 *     device memory; calls that need scratch take a caller-provided workspace.
 *   - packed matrices are row-major [N, K] GGUF blocks packed along K; expert banks
 *     are [E, N, K] with a byte stride between experts
 *     (mini_llm/ops/quantized_weight.py:85-99).
 */
#ifndef QMOE_H
#define QMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QMOE_ABI_VERSION 5

/* Packed formats.  Ids 0..5 are the reference's (_FORMAT_ID,
 * mini_llm/ops/quantized_linear.py:34 and native_packed_cpu.cpp:12).  BF16 has no
 * packed id in the reference (it is decoded as a dense tensor,
 * mini_llm/external/gguf_tensor.py:30-51); id 100 is this library's extension. */
enum {
    QMOE_FMT_Q8_0 = 0,
    QMOE_FMT_Q4_0 = 1,
    QMOE_FMT_Q4_K = 2,
    QMOE_FMT_Q3_K = 3,
    QMOE_FMT_Q5_K = 4,
    QMOE_FMT_Q6_K = 5,
    QMOE_FMT_BF16 = 100
};

/* Activation / output element types. */
enum { QMOE_DT_F32 = 0, QMOE_DT_F16 = 1, QMOE_DT_BF16 = 2 };

/* Status codes. */
enum {
    QMOE_OK = 0,
    QMOE_EINVAL = 1,       /* null pointer, bad shape, K not a block multiple, ... */
    QMOE_EUNSUPPORTED = 2, /* format / dtype / size outside what the kernels cover */
    QMOE_ELAUNCH = 3,      /* HIP reported a launch error */
    QMOE_EWORKSPACE = 4    /* workspace missing, misaligned or too small */
};

int qmoe_abi_version(void);
const char* qmoe_last_error(void);

/* Optional set-up of the current device ahead of the first compute call: resolves the addresses
 * of the library's per-GPU device variables (the launch status word and the scratch array of
 * qmoe_moe_forward_static), which the compute calls otherwise do on their first use on a device.
 * Call it once per device before recording a HIP graph: looking a device variable up is not
 * stream work and is not allowed while a stream captures.  No counterpart in the reference. */
int qmoe_init(void);

/* Waits inside the streaming kernels (a wave waiting for the other waves of its own workgroup)
 * are bounded in wall-clock time.  A wave whose wait expires raises the current device's launch
 * status word, stores no further results and runs to its end, so the launch ends normally and its
 * outputs are incomplete rather than wrong.  qmoe_check_status SYNCHRONISES `stream`, reads the
 * word and clears it: QMOE_OK if no launch on this device gave up since the last check, else
 * QMOE_ELAUNCH (the only call of this library that waits for the device).  No counterpart in
 * the reference, whose kernels have no waits. */
int qmoe_check_status(void* stream);

/* The bound of those waits in ticks of the 100 MHz device counter; 0 restores the default (one
 * second).  A negative value makes every wait expire at once: the host-forced way to exercise
 * the give-up path, every kernel still ends normally. */
void qmoe_set_wait_limit(long long ticks);

/* Elements and bytes per block of a format (BLOCK_FORMATS,
 * mini_llm/ops/quantized_weight.py:24-37). */
int qmoe_format_info(int fmt, int* block_elems, int* block_bytes);

/* out[n*k] fp32 = dequantised packed matrix; bit-identical to
 * PackedGGUFWeight.dequantize_reference (mini_llm/ops/quantized_weight.py:151-250)
 * and, for BF16, to decode_gguf_dense (mini_llm/external/gguf_tensor.py:48-51). */
int qmoe_dequantize(const void* w, int fmt, int64_t n, int64_t k, float* out, void* stream);

/* y[tokens, n] = x[tokens, k] @ W[n, k]^T with fp32 accumulation; replaces the
 * device branch of quantized_linear (mini_llm/ops/quantized_linear.py:306-335) and
 * has the argument order of mylocal_packed_gemv (native_packed_cpu.cpp:208-217)
 * with element types and a stream added.  x and y are contiguous. */
int qmoe_linear(const void* w, int fmt, int n, int k,
                const void* x, int x_dtype, int tokens,
                void* y, int y_dtype, void* stream);

/* One problem of a batched launch: y = x @ W^T.  Host struct. */
typedef struct qmoe_linear_problem {
    const void* w;
    const void* x;
    void* y;
    int fmt, n, k, tokens;
    int x_dtype, y_dtype;
} qmoe_linear_problem;

/* Several independent linears enqueued as one launch sequence (e.g. q/k/v of one
 * layer, which share x); `problems` is a HOST array read before the call returns.
 * No counterpart in the reference, which launches each projection separately
 * (mini_llm/external/gguf_projection.py:40-62). */
int qmoe_linear_batch(const qmoe_linear_problem* problems, int count, void* stream);

/* h[tokens, f] = silu(x @ G^T) * (x @ U^T); gate and up may differ in format.
 * Replaces the device branch of quantized_swiglu
 * (mini_llm/ops/quantized_linear.py:338-400). */
int qmoe_swiglu(const void* gate, int gate_fmt, const void* up, int up_fmt, int f, int k,
                const void* x, int x_dtype, int tokens,
                void* h, int h_dtype, void* stream);

/* out[tokens, d_model] = down(swiglu(x)): one packed SwiGLU expert.  Argument
 * order of mylocal_packed_expert (native_packed_cpu.cpp:219-245).  `workspace` holds
 * tokens*d_ff fp32 (the stored hidden activation). */
int qmoe_expert(const void* gate, int gate_fmt, const void* up, int up_fmt,
                const void* down, int down_fmt, int d_model, int d_ff,
                const void* x, int x_dtype, int tokens,
                void* out, int out_dtype, float* workspace, void* stream);

/* Rows of full softmax -> exact top-k (descending logit, lower id on ties, NaN
 * last) -> optional division by max(selected mass, floor).  weights fp32
 * [tokens,k], ids int64 [tokens,k].  Replaces expert_topk_forward +
 * RouterInference's renormalisation (mini_llm/ops/router.py:21-43,
 * mini_llm/ops/router_inference.py:47-61) and the single-row kernel
 * normalized_topk (mini_llm/ops/router_decode.py:27-95).  n <= 4096, k <= 32. */
int qmoe_router_topk(const float* logits, int tokens, int n, int k, float floor_value,
                     int renormalize, float* weights, int64_t* ids, void* stream);

/* A bank of E SwiGLU experts stored as three packed tensors [E,F,D], [E,F,D],
 * [E,D,F] (Qwen3NextGGUFIndex.expert_weights,
 * mini_llm/external/qwen3next_gguf.py:153-169).  A fused gate_up tensor [E,2F,D] is
 * described by up = gate + F rows and both strides = 2F rows.  Host struct. */
typedef struct qmoe_expert_bank {
    const void* gate;
    const void* up;
    const void* down;
    int64_t gate_stride, up_stride, down_stride; /* bytes between experts */
    int gate_fmt, up_fmt, down_fmt;
    int n_experts, d_model, d_ff;
} qmoe_expert_bank;

/* Single token, E selected experts given as a DEVICE table of E rows of three
 * device pointers (gate, up, down) in the order they are to be summed.
 * out[d] = sum over rows, sequentially from zero, of
 *          fp32(down_e(fp32 swiglu_e(x))[d] * routes[slot_e * route_stride])
 * with the product stored before each add (no FMA, no tree).  slots is a DEVICE
 * int32 array of E route positions or NULL for slot_e = e.  Replaces
 * grouped_quantized_experts_forward
 * (mini_llm/ops/grouped_quantized_experts.py:159-217).  workspace: fp32
 * E*d_ff + E*d_model elements. */
int qmoe_grouped_decode(const float* x, const void* const* table, int n_rows,
                        int gate_fmt, int up_fmt, int down_fmt, int d_model, int d_ff,
                        const float* routes, int64_t route_stride, const int32_t* slots,
                        float* out, float* workspace, void* stream);

/* qmoe_grouped_decode for a caller that holds the expert table on the HOST (as the reference's
 * wrapper does before it uploads it, mini_llm/ops/grouped_quantized_experts.py:180-186): `experts`
 * is a HOST array of n_rows x 3 device pointers (gate, up, down), `slots` a HOST array of n_rows
 * route positions or NULL; both are read before the call returns and travel in the kernel
 * arguments, so the call makes no host-to-device copy.  Up to 16 experts (more: QMOE_EUNSUPPORTED,
 * use the device-table form).  Same result as qmoe_grouped_decode: the same ordered sum of stored
 * products.  Shapes the streamed decode kernels take (all formats Q8_0 / Q4_K / Q5_K / Q6_K with
 * gate_fmt == up_fmt, d_model a multiple of 256 up to 2048, d_ff a power-of-two multiple of 256,
 * n_rows * d_ff / 128 <= 48) run on them in two launches; any other shape runs the general kernels.
 * workspace: fp32 n_rows * (d_ff + d_model + 8) elements, 16-byte aligned.  No counterpart in the
 * reference beyond the call it replaces. */
int qmoe_grouped_decode_listed(const float* x, const void* const* experts, int n_rows,
                               int gate_fmt, int up_fmt, int down_fmt, int d_model, int d_ff,
                               const float* routes, int64_t route_stride, const int32_t* slots,
                               float* out, float* workspace, void* stream);

/* Arguments of one MoE step over T tokens.  Host struct. */
typedef struct qmoe_moe_args {
    const void* hidden;     /* [T, d_model], hidden_dtype */
    int hidden_dtype;
    int tokens;
    int top_k;
    /* routing input: either logits (router runs on device) or precomputed
     * weights + ids (both device); logits wins when non-NULL. */
    const float* logits;    /* [T, n_experts] fp32 or NULL */
    float floor_value;      /* renormalisation floor, 2^-14 for Qwen3-Next */
    int renormalize;
    const float* in_weights;  /* [T, k] fp32, used when logits == NULL */
    const int64_t* in_ids;    /* [T, k] int64, used when logits == NULL */
    qmoe_expert_bank bank;
    /* shared expert (all NULL = none): gate/up [d_ff_shared, d_model], down
     * [d_model, d_ff_shared]; shared_gate fp32 [d_model] or NULL (= ungated). */
    const void* shared_gate_w;
    const void* shared_up_w;
    const void* shared_down_w;
    int shared_gate_fmt, shared_up_fmt, shared_down_fmt;
    int d_ff_shared;
    const float* shared_gate;
    void* out;              /* [T, d_model], out_dtype */
    int out_dtype;
    float* out_weights;     /* optional [T, k] fp32: routing weights used */
    int64_t* out_ids;       /* optional [T, k] int64: selected experts */
    /* optional fp32 [T, d_model]: out = residual + (routed + shared * sigmoid), the residual add
     * that follows the block (mini_llm/external/qwen3next_decoder.py:120) */
    const float* residual;
    /* optional device word that the CALLER has set to zero: bit 0 is set when an expert id of
     * in_ids lies outside [0, n_experts), bit 1 when one token names the same expert more than once.
     * Such assignments contribute nothing to the output (of a repeated expert only the first slot
     * counts); the reference's plan refuses them and leaves them to its general dispatcher
     * (mini_llm/ops/device_expert_plan.py:17-36, :183-186).  Ids selected by the router on the device
     * are always valid. */
    int* status_out;
} qmoe_moe_args;

/* Bytes of workspace qmoe_moe_forward needs for these sizes (256-byte aligned). */
size_t qmoe_moe_workspace_bytes(int tokens, int top_k, int n_experts, int d_model,
                                int d_ff, int d_ff_shared);

/* routed + shared * sigmoid(hidden . shared_gate): router (optional), device-side
 * token->expert compaction, packed experts, ordered weighted combine (ascending
 * expert id per token, product stored then added), shared expert.  Replaces
 * Qwen3NextMoEInference.forward (mini_llm/external/qwen3next_moe.py:129-147) with
 * ExpertsInference.forward's general path (mini_llm/ops/experts_inference.py:290-310)
 * and RoutingPlan.from_router_outputs (mini_llm/ops/routing_plan.py:52-118) inside;
 * there is no host round trip. */
int qmoe_moe_forward(const qmoe_moe_args* args, void* workspace, size_t workspace_bytes,
                     void* stream);

/* The token->expert plan alone, as qmoe_moe_forward builds it in its workspace
 * (RoutingPlan.from_router_outputs, mini_llm/ops/routing_plan.py:52-118): the T*k assignments
 * grouped by expert id, ascending token inside an expert.  All arrays are DEVICE memory;
 * A = tokens * top_k.
 *   offsets[n_experts + 1]  exclusive prefix of the per-expert assignment counts
 *   active[n_experts]       ids of the experts with assignments, ascending (first *n_active valid)
 *   order[A]                flat assignment index (token * top_k + slot) of each sorted position
 *   sorted_token[A]         order / top_k;  sorted_weight[A]  weights gathered in that order
 *   pos_of[A]               sorted position of assignment (token, slot), -1 for one that is dropped
 *   status                  bit 0: an id outside [0, n_experts); bit 1: an expert repeated in a token
 * Only the first offsets[n_experts] entries of the sorted arrays are written (dropped assignments
 * shorten the list).  One workgroup builds the plan in LDS: tokens x n_experts beyond its table is
 * QMOE_EUNSUPPORTED. */
int qmoe_routing_plan(const int64_t* ids, const float* weights, int tokens, int top_k, int n_experts,
                      int* offsets, int* active, int* n_active, int* order, int* sorted_token,
                      float* sorted_weight, int* pos_of, int* status, void* stream);

/* qmoe_moe_forward for callers that cannot allocate device memory or bring a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the scratch the
 * step needs lies in an array inside the library's device image (QMOE_MOE_STATIC_SCRATCH_BYTES,
 * one copy per GPU, held until the process ends).  No counterpart in the reference.  Same
 * arguments, results and errors as qmoe_moe_forward; steps that need more scratch than the
 * array holds return QMOE_EWORKSPACE and touch nothing (the 512-expert, top-10 layer of width
 * 2048 / 512 / 2048 fits up to 64 tokens).  The call allocates nothing, clears nothing and
 * does not synchronise.  All calls on one GPU share the one array, which keeps the last call's
 * contents: calls that overlap on one GPU (different streams, or threads) race and must be
 * serialised by the caller; calls on one stream are ordered by the stream.  The array's address on
 * a device is looked up once, by qmoe_init or by the first call on that device: callers that record
 * a HIP graph call qmoe_init first, because that look-up is not stream work. */
#define QMOE_MOE_STATIC_SCRATCH_BYTES ((size_t)8 << 20)
size_t qmoe_moe_static_scratch_bytes(void);
int qmoe_moe_forward_static(const qmoe_moe_args* args, void* stream);

/* RMSNorm of the residual stream followed by the router's logits, the step in front of the MoE
 * block, in one launch:  normalized = (x * inv_rms) * gamma  with  inv_rms = 1 / sqrt(mean(x^2) + eps)
 * (RMSNormInference.forward, mini_llm/ops/rmsnorm_inference.py:109-118, :517-520) and
 * logits = normalized @ router_w^T + router_b  (RouterInference.forward,
 * mini_llm/ops/router_inference.py:40-46; router_w is [n_experts, d_model] as stored in
 * ffn_gate_inp, router_b fp32 [n_experts] or NULL).  x [T, d_model], normalized [T, d_model] and
 * logits [T, n_experts] are fp32; d_model % 4 == 0. */
int qmoe_norm_router(const float* x, int tokens, int d_model, const float* gamma, float eps,
                     const float* router_w, const float* router_b, int n_experts, float* normalized,
                     float* logits, void* stream);

/* The router's logits alone, for a caller that holds the normalised hidden state already:
 * logits = x @ router_w^T + router_b  (RouterInference.forward, mini_llm/ops/router_inference.py:40-46),
 * fp32 throughout; x [T, d_model], router_w [n_experts, d_model] as stored in ffn_gate_inp,
 * router_b fp32 [n_experts] or NULL; d_model % 4 == 0.  Same kernel and summation order as
 * qmoe_norm_router's logits. */
int qmoe_router_logits(const float* x, int tokens, int d_model, const float* router_w,
                       const float* router_b, int n_experts, float* logits, void* stream);

/* Measurement aid, no counterpart in the reference: reads `bytes` (a multiple of 4096) of device
 * memory once with 16-byte loads, one workgroup of eight waves per CU, and writes nothing unless
 * the XOR of all dwords equals `match` (then that value goes to sink[0]).  Its duration is the
 * streaming-read ceiling of the device for a launch of that size. */
int qmoe_read_probe(const void* buffer, size_t bytes, uint32_t match, uint32_t* sink, void* stream);

/* ---- host twins -----------------------------------------------------------------------------
 * The same operators over HOST pointers, computed on the CPU by one thread of scalar C++ (no
 * stream, nothing touches the GPU).  They serve callers that hold NumPy activations and
 * host-packed weights -- the host branch of quantized_linear
 * (mini_llm/ops/quantized_linear.py:292-305) -- and have the argument order of the reference's
 * native CPU backend.  Activations and results are fp32; blocks are decoded exactly as on the
 * device, sums are fp32 in eight interleaved partials per row. */

/* out[n*k] fp32 = dequantised packed matrix on the host, the values of qmoe_dequantize bit for bit
 * (PackedGGUFWeight.dequantize_reference, mini_llm/ops/quantized_weight.py:151-250). */
int qmoe_dequantize_cpu(const void* w, int fmt, int64_t n, int64_t k, float* out);

/* y[tokens, n] = x[tokens, k] @ W[n, k]^T  (mylocal_packed_gemv, native_packed_cpu.cpp:206-217). */
int qmoe_linear_cpu(const void* w, int fmt, int n, int k, const float* x, int tokens, float* y);

/* h[tokens, f] = silu(x @ G^T) * (x @ U^T)  (host branch of quantized_swiglu,
 * mini_llm/ops/quantized_linear.py:361-368; sigmoid in the overflow-free form of
 * native_packed_cpu.cpp:236-238). */
int qmoe_swiglu_cpu(const void* gate, int gate_fmt, const void* up, int up_fmt, int f, int k,
                    const float* x, int tokens, float* h);

/* out[tokens, d_model] = down(swiglu(x))  (mylocal_packed_expert, native_packed_cpu.cpp:219-245). */
int qmoe_expert_cpu(const void* gate, int gate_fmt, const void* up, int up_fmt,
                    const void* down, int down_fmt, int d_model, int d_ff,
                    const float* x, int tokens, float* out);

/* qmoe_router_topk on the host: full softmax, exact top-k (descending logit, lower id on ties,
 * NaN last), optional division by max(selected mass, floor)  (mini_llm/ops/router.py:21-43,
 * mini_llm/ops/router_inference.py:47-61).  Any n, 1 <= k <= n. */
int qmoe_router_topk_cpu(const float* logits, int tokens, int n, int k, float floor_value,
                         int renormalize, float* weights, int64_t* ids);

#ifdef __cplusplus
}
#endif
#endif /* QMOE_H */
