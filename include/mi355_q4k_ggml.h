/*
 * mi355_q4k_ggml.h -- GGML_OP_CUSTOM adapters over the mi355_q4k C ABI.
 *
 * DenseCore replaces ggml_mul_mat / ggml_mul_mat_id by writing a
 * {ggml_custom_op_t fn, n_tasks, userdata} triple into dst->op_params with
 * dst->op = GGML_OP_CUSTOM (core/src/llm/matmul/graph_ops.cpp:212-227,297-308)
 * or through ggml_custom_4d (core/src/llm/moe/native.cpp:4872-4873,4907-4909).
 * The functions below have exactly that callback shape,
 *     void fn(struct ggml_tensor* dst, int ith, int nth, void* userdata),
 * read their operands from dst->src[] the way the callbacks they replace do,
 * run the whole node on the GPU when ith == 0, return at once for ith > 0
 * (the convention of cb_matmul_hal_custom, core/src/llm/matmul/exec.cpp:36),
 * and synchronise before returning because the next graph node reads dst->data
 * on the host.  Like the reference's callbacks they return void; an invalid
 * node leaves dst untouched (core/src/llm/matmul/gemv_exec.cpp:102-143) and
 * the reason is kept for mq_ggml_last_status() / mq_last_error().
 *
 * All tensor memory is host memory borrowed from the graph.  Weight tensors
 * are uploaded to HBM the first time their data pointer is seen and kept in a
 * process-wide cache keyed by (data, type, ne, nb, content fingerprint) -- the counterpart of
 * GetOrCreateQ4KRepackedGemvWeight's cache
 * (core/src/kernels/q4k_repacked_gemv.cpp:403-470) -- until
 * mq_ggml_weight_cache_clear().
 *
 * `struct ggml_tensor` is ggml's.  When no ggml header is on the include path
 * the implementation is compiled against a field-for-field mirror of the
 * members it reads (densecore_amd/host/ggml_tensor_mirror.h).
 */
#ifndef MI355_Q4K_GGML_H
#define MI355_Q4K_GGML_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct ggml_tensor;

/* Optional userdata of the matmul and expert adapters (NULL = defaults).  The graph owns it, as it owns
 * GemvUserData / Qwen35SharedQ8RowsUserData (core/src/llm/runtime/work_context.h:10-11,
 * core/src/llm/moe/native.cpp:1027-1038). */
typedef struct {
    int silu_mode;    /* MQ_SILU_*  (gate/up node); default MQ_SILU_EXACT for n <= 4, MQ_SILU_FAST above,
                         as core/src/llm/moe/native.cpp:3614-3616 and cpu_backend_moe_raw_batched.inl:1673 choose */
    int reserved;     /* not read (the down node always resolves its weights as
                         Qwen35NativeMoEComputeTopKWeightsFromLogits does, core/src/llm/moe/native.cpp:2305-2357) */
    int use_defaults; /* non-zero: ignore silu_mode */
    int last_status;  /* written by the adapter: MQ_OK or MQ_ERR_* */
    /* Opt-in hand-over between the two expert nodes of one graph (core/src/llm/moe/native.cpp:4871-4909): non-zero on
     * the gate/up node's userdata makes that node leave its result in HBM -- dst->data is NOT written and the node
     * does not synchronise -- and the down node that runs next on the same thread with that tensor as its `hidden`
     * operand reads it there (no download, no upload, one synchronisation for the pair).  Only for graphs in which
     * nothing but the down node reads the gate/up node's output (true of the native MoE graph); any other consumer
     * would read stale host memory. */
    int keep_hidden_on_device;
    /* The same flag on a dense node (mq_cb_gemv_custom, mq_cb_gemv_batched_custom) or on one of the two element-wise
     * nodes below: the node's result stays in HBM, dst->data is not written, nothing is waited for, and any later
     * dense or element-wise node of the graph that names the tensor (or a view of all of it) as an operand reads it
     * there -- gate -> up -> silu * up -> down -> scalar gate of a dense FFN or shared expert
     * (core/src/llm/graph/decoder.cpp:2426-2600) cost one synchronisation, at the node that does not set the flag.
     * Tensors are remembered by their ggml_tensor object for the calling thread until mq_ggml_graph_begin();
     * mq_ggml_tensor_to_host() brings one back for a consumer that is not one of these nodes. */
} mq_ggml_userdata;

/* dst F32 ne=[N_out, M]; src[0] = input F32 ne=[K_in, M] (column stride nb[1]); src[1] = weight
 * Q4_K ne=[K_in, N_out], nb[1] = row bytes.  cb_gemv_custom (core/src/llm/matmul/gemv_exec.cpp:99-143). */
void mq_cb_gemv_custom(struct ggml_tensor* dst, int ith, int nth, void* userdata);
/* Same operands with 2 <= M; cb_gemv_batched_custom (core/src/llm/matmul/batched_exec.cpp:55-74). */
void mq_cb_gemv_batched_custom(struct ggml_tensor* dst, int ith, int nth, void* userdata);
/* dst F32 ne=[n_ff, top_k, n_tokens]; src = {gate_exps Q4_K ne=[n_embd, n_ff, n_expert], up_exps,
 * input F32 ne=[n_embd, n_tokens], selected_experts I32 ne=[top_k, n_tokens]}.
 * cb_qwen35_native_moe_gateup_raw_qxk_swiglu (core/src/llm/moe/native.cpp:3929-4345, :4871-4874). */
void mq_cb_moe_gateup_swiglu(struct ggml_tensor* dst, int ith, int nth, void* userdata);
/* dst F32 ne=[n_embd, n_tokens]; src = {down_exps Q4_K / Q5_K / Q6_K / Q8_0 ne=[n_ff, n_embd, n_expert], hidden F32
 * ne=[n_ff, top_k, n_tokens], selected_experts I32 ne=[top_k, n_tokens], gate_logits F32
 * ne=[n_expert, n_tokens]}.  cb_qwen35_native_moe_down_q5k_weighted_logits
 * (core/src/llm/moe/native.cpp:3051-3295, :4906-4909). */
void mq_cb_moe_down_weighted_logits(struct ggml_tensor* dst, int ith, int nth, void* userdata);

/* The state block of the fused top-8 router node, laid out as the reference's QwenNativeMoEFusedRouterState
 * (core/src/llm/moe/native.cpp:602-608): the node's userdata. */
typedef struct {
    int64_t n_experts;
    int64_t n_tokens;
    int64_t top_k;
    float* normalized_weights; /* host, [n_tokens][top_k]: written by the node, read by the weights node */
    void* work_ctx;            /* the reference's InferenceWorkContext*; not touched here */
} mq_ggml_router_state;
/* dst I32 ne=[top_k, n_tokens] = the selected experts; src[0] = gate logits F32 ne=[n_experts, n_tokens]; userdata =
 * mq_ggml_router_state*, whose normalized_weights receive the softmax over the selection (uniform when a selected
 * logit is not finite).  cb_qwen_native_moe_fused_router (core/src/llm/moe/native.cpp:710-735, emitted at :4831-4834
 * for one token; ComputeQwenNativeMoEStableTopK :621-676).  A node that fails the reference's checks is left alone. */
void mq_cb_moe_fused_router(struct ggml_tensor* dst, int ith, int nth, void* userdata);
/* dst F32 ne=[1, top_k, n_tokens]; src = {logits F32 ne=[n_experts, n_tokens], selected I32 ne=[top_k, n_tokens]}:
 * softmax of the selected logits over the valid selection, denominator floored at 2^-14, uniform over the valid
 * entries when nothing finite is left, 0 for ids outside [0, n_experts).  cb_moe_topk_weights_from_logits
 * (core/src/llm/moe/native.cpp:800-868).  top_k <= 8. */
void mq_cb_moe_topk_weights_from_logits(struct ggml_tensor* dst, int ith, int nth, void* userdata);
/* A ggml_mul_mat_id node: dst F32 ne=[N, n_used, n_tokens]; src = {as Q4_K/Q5_K/Q6_K ne=[K, N, n_expert], b F32
 * ne=[K, n_used or 1, n_tokens], ids I32 ne=[n_used, n_tokens]}; dst[:, k, t] = as[ids[k, t]] . q8k(b[:, k or 0, t]).
 * The nodes emitted at core/src/llm/moe/native_gemma.cpp:1509-1559 (gate, up, gate_up and down of the routed
 * experts); rows whose id is outside [0, n_expert) come back as zeros. */
void mq_cb_mul_mat_id(struct ggml_tensor* dst, int ith, int nth, void* userdata);

/* The element-wise nodes between the products of a dense FFN / shared expert, with ggml_custom2_op_t's shape
 * (ggml_map_custom2): void fn(dst, a, b, ith, nth, userdata); userdata NULL or mq_ggml_userdata*.
 * dst = silu(a) * b, all F32 of one shape with unit element stride: cb_silu_mul_fused
 * (core/src/llm/graph/fused_ops.cpp:317-366; contiguous tensors take MQ_SILU_FAST_FMA as SiLUMulParallel does,
 * strided ones MQ_SILU_EXACT, unless userdata names a mode). */
void mq_cb_silu_mul_fused(struct ggml_tensor* dst, const struct ggml_tensor* a, const struct ggml_tensor* b, int ith, int nth,
                          void* userdata);
/* dst[:, t] = sigmoid(gate_logits_scalar[t]) * src[:, t], src / dst F32 ne=[hidden, tokens], one logit per token at
 * row stride nb[1]: cb_apply_shared_scalar_gate (core/src/llm/graph/fused_ops.cpp:437-475). */
void mq_cb_apply_shared_scalar_gate(struct ggml_tensor* dst, const struct ggml_tensor* src, const struct ggml_tensor* gate_logits_scalar,
                                    int ith, int nth, void* userdata);
/* Forgets every tensor the calling thread's nodes left on the device (call where a graph compute starts: a tensor
 * whose producer did not run through these adapters this time must not be answered from an old device copy). */
void mq_ggml_graph_begin(void);
/* Copies a tensor that a node left on the device into t->data (one synchronisation); 1 when it was there, else 0. */
int mq_ggml_tensor_to_host(struct ggml_tensor* t);

/* Status of the calling thread's last adapter call (MQ_OK / MQ_ERR_*). */
int mq_ggml_last_status(void);
/* Frees every cached device weight (call when the model is unloaded). */
int mq_ggml_weight_cache_clear(void);
int64_t mq_ggml_weight_cache_size(void);
/* The content key of the weight cache: a multiply-xor hash over the byte count, the first and last 4 KiB and 64
 * sixteen-byte samples in between (0 for an empty input).  A cached tensor is re-uploaded when its pointer, type, shape, strides or this
 * value changed -- FingerprintQ4KRepackedGemvWeight's role (core/src/kernels/q4k_repacked_gemv.cpp:353-393). */
uint64_t mq_ggml_weight_fingerprint(const void* data, size_t bytes);

/* Library-level boundary without a graph: C[M][N] = A[M][K] . W[N][K]^T with W raw ggml Q4_K rows.
 * CpuBackend::MatMulGgmlQuantizedTransB(const Tensor& A, const GgmlQuantizedMatrixView& W, Tensor* C, int)
 * (core/include/densecore/backend/cpu_backend.h:91-99,293-300) flattened to plain pointers: a/c are host
 * fp32 with row strides lda/ldc in elements (Tensor::stride[0]); w_type_id must be 12 (GGML_TYPE_Q4_K).
 * Returns 1 when the product was computed and 0 when the call is rejected, like the bool it replaces. */
int mq_matmul_ggml_quantized_transb(const float* a, int64_t m, int64_t k, int64_t lda, const void* w_data,
                                    int32_t w_type_id, int64_t w_rows, int64_t w_cols, size_t w_row_bytes, float* c,
                                    int64_t ldc);

#ifdef __cplusplus
}
#endif
#endif /* MI355_Q4K_GGML_H */
