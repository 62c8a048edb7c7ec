/*
 * mi355_q4k_debug.h -- verification hooks and measurement instruments of libmi355q4k.so.
 *
 * Exported by the same library as the entry points of mi355_q4k.h, kept apart from them: a DenseCore host binds
 * mi355_q4k.h; tests and benchmarks also include this file.  None of these calls changes what a product entry point
 * computes; mq_debug_set_dense_lds selects between kernels that return the same bits.
 */
#ifndef MI355_Q4K_DEBUG_H
#define MI355_Q4K_DEBUG_H

#include "mi355_q4k.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- verification hook -------------------------------------------------------------
 * Runs the production matmul kernel with its per-super-block integer sums
 * written out: dot_scaled_dev / min_dot_dev int32 [rows][n][cols/256], the two
 * integers every reference kernel forms before touching floating point
 * (core/src/llm/matmul/kquant_batched_kernels.h:285-297).  Mirrors the
 * reference's ...ForTest hooks (core/src/llm/moe/native.cpp:5107-5636). */
int mq_debug_block_sums(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, int32_t* dot_scaled_dev,
                        int32_t* min_dot_dev, float* y_dev, int64_t ldy, void* stream);

/* The expert-grouped work list ("gather tokens by expert") that the grouped kernels read, written out entry by
 * entry: triples_dev int32 [n * top_k][3] = (expert, token, k) in list order, count_dev int32 [1] = entries (pairs
 * whose id is outside [0, n_experts) are dropped).  The reference's list is sorted by (expert, token, k)
 * (Qwen35BuildMoEAssignments, core/src/llm/moe/native.cpp:1664-1733).  Pass ids_dev int32 [n][top_k] to group given
 * ids (the grouping launch of mq_mul_mat_id_q4k and of the two expert nodes) or logits_dev fp32 [n][n_experts] to
 * route and group in the one launch mq_moe_layer_q4k uses above eight tokens; the other pointer NULL. */
int mq_debug_moe_groups(const float* logits_dev, const int32_t* ids_dev, int64_t n_experts, int64_t n, int top_k,
                        int32_t* triples_dev, int32_t* count_dev, void* stream);

/* The fp32 intermediate the last mq_moe_layer_q4k / mq_ffn_swiglu_q4k call on this stream left in the library's
 * workspace, copied out: for the MoE layer the hidden rows silu(gate . x) * (up . x) as [n][top_k (+1 with a shared
 * expert)][inter], for the dense FFN [n][inter].  `count` floats.  A ...ForTest hook like mq_debug_block_sums. */
int mq_debug_moe_hidden(float* hidden_out_dev, size_t count, void* stream);
/* Device addresses of a decoder handle's exchange buffers after a step (the LAST layer's values): qkv [n][qkv_rows],
 * o [n][hidden], logits [n][n_experts], hidden rows [n][top_k (+1)][inter], MoE output y [n][hidden].  Any may be NULL. */
int mq_debug_decoder_buffers(mq_decoder* d, float** qkv_dev, float** o_dev, float** logits_dev, float** hidden_dev,
                             float** y_dev);

/* ---- launch census -------------------------------------------------------------------
 * When enabled, every matmul-kernel launch carries a start/stop HIP event pair that receives the
 * dispatch's own begin and end timestamps; mq_census_read synchronises and returns the kernel durations.  The GPU
 * counterpart of the reference's matmul dispatch census of (path, shape, wall ns)
 * (core/src/llm/matmul/gemv_exec.cpp:203-276).  Off by default. */
#define MQ_KIND_DENSE 0          /* one dense matrix                     */
#define MQ_KIND_DENSE_SWIGLU 1   /* gate + up fused, dense               */
#define MQ_KIND_GROUPED 2        /* expert-routed                        */
#define MQ_KIND_GROUPED_SWIGLU 3 /* expert-routed gate + up fused        */
#define MQ_KIND_COUNT 4
int mq_census_enable(int on);
int mq_census_reset(void);
int mq_census_read(int kind, double* avg_us, double* min_us, double* max_us, int64_t* count);

/* Debug switch: dense products of up to 16 rows normally run on the kernel that stages the quantized activations
 * in LDS once per workgroup (and, for up to four fp32 rows, quantizes them itself), and expert-grouped launches
 * with many groups on the kernel that gathers a group's rows into LDS once per eight wavefronts; on = 0 keeps
 * both on the kernel that reads its operand from global memory at every stage, on = 5 only the expert-grouped
 * ones; bit 3 (on = 9) makes Q4_K gate and up at prefill widths two GEMM launches and a SwiGLU pass instead of the
 * one launch that stores silu(gate) * up; bits 8..11 force the activation tiles per item of the expert-grouped GEMM (2,
 * 4 or 8; 0 = chosen by the rows per expert); bit 12 keeps dense Q4_K products of nine to 64 rows on the kernels
 * that multiply them as token tiles of eight (or on the GEMM) instead of the one that takes them as tiles of sixteen.  All
 * return the same bits (tests/test_gpu_dense_lds.py, tests/test_gpu_grouped_lds.py, tests/test_gpu_prefill.py); returns the
 * previous setting of bit 0.  No counterpart in the reference. */
int mq_debug_set_dense_lds(int on);

/* Measurement instrument: while on != 0 every compute and routing launch of the library is replaced by a kernel with
 * an empty body and the same grid, block and LDS size (weight set-up and launches that carry timing events are
 * not).  A graph captured in this state has the launches of the real one and none of their work: its replay time
 * is what the launches alone cost.  Outputs are not written while it is on.  Returns the previous setting.  No
 * counterpart in the reference. */
int mq_debug_set_skeleton(int on);

#ifdef __cplusplus
}
#endif
#endif
