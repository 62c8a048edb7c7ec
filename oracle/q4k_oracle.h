/*
 * q4k_oracle.h -- CPU restatement of DenseCore's Q4_K x Q8_K matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, its host
 * layer, the Python package) may include, link, import or call this code.
 * It exists so that tests, the smoke check and the bench's cpu_baseline leg
 * can compare the GPU path with an independent scalar implementation.
 *
 * The arithmetic follows these reference files (paths relative to the
 * DenseCore tree):
 *   core/src/kernels/hwy/hwy_moe_quant.cc:28-143    block layouts, fp16->fp32,
 *                                                    NearestInt, Q8_K quantizer
 *   core/src/kernels/hwy/hwy_moe_quant.cc:145-258   Highway-order dot
 *   core/src/llm/matmul/kquant_batched_kernels.h:37-129   scalar-order dot
 *   core/src/llm/matmul/kquant_batched_kernels.h:234-305  dotprod-order dot
 *   core/src/llm/matmul/kquant_batched_kernels.h:398-549  AVX2-order dot
 *   core/src/llm/moe/q4_rowpair.h:37-78             indexed scale/min formula
 *   core/src/backend/cpu_backend_internal.h:99-114  fast exp (plain)
 *   core/src/kernels/hwy/hwy_fastexp.h:50-84        fast exp (fused)
 *   core/src/llm/moe/native.cpp:610-676,800-868,1664-1733,2305-2357,3206-3286
 *                                                    router, assignments, down
 *   core/src/llm/graph/fused_ops.cpp:437-475        shared-expert sigmoid gate
 *
 * Pinning status (what fixes each function independently of this file):
 *   block layouts ........ static asserts below (144 / 292 bytes, offsets)
 *   orc_fp16_to_fp32 ..... exhaustive 65536-value check against F16C
 *   orc_nearest_int ...... equals lrintf under round-to-nearest-even
 *   orc_quantize_row_q8k . invariants (bsums, arg-max -> -127, sign symmetry,
 *                          reconstruction bound, first-max tie break)
 *   orc_q4k_scales ....... two independent formulas must agree + one-hot bytes
 *   orc_block_sums ....... brute-force int64 triple loop, closed-form extremes
 *   orc_dot_* ............ dequantize-then-double dot; all four fp32 orders
 *                          within 1e-4 of it
 *   orc_route_topk ....... stable sort + restricted softmax in double
 *   orc_build_assignments  qsort on the (expert, token, k) tuple
 *   orc_moe_layer ........ composition; tiny layer brute-forced in double
 *   orc_fast_exp* ........ closed form vs expf (cubic's known error class)
 * PARITY UNPINNED: the fp32 summation order of ggml's own
 * ggml_vec_dot_q4_K_q8_K / *_8x8 kernels and Highway's ReduceSum tree (both
 * third-party and absent from the reference tree); the orders here are the
 * ones DenseCore's own sources spell out.
 */
#ifndef Q4K_ORACLE_H
#define Q4K_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_QK_K 256
#define ORC_K_SCALE_SIZE 12

typedef struct {
    uint16_t d;                      /* fp16 super-block scale            */
    uint16_t dmin;                   /* fp16 super-block min scale        */
    uint8_t scales[ORC_K_SCALE_SIZE];/* 8 scales + 8 mins, 6 bits each    */
    uint8_t qs[ORC_QK_K / 2];        /* 256 x 4-bit quants                */
} orc_block_q4k;

typedef struct {
    float d;
    int8_t qs[ORC_QK_K];
    int16_t bsums[ORC_QK_K / 16];
} orc_block_q8k;

/* fp32 accumulation orders that exist in the reference. */
enum {
    ORC_ORDER_HWY = 0,     /* hwy_moe_quant.cc:248-253                    */
    ORC_ORDER_AVX2 = 1,    /* kquant_batched_kernels.h:540-541            */
    ORC_ORDER_SCALAR = 2,  /* kquant_batched_kernels.h:110-125            */
    ORC_ORDER_DOTPROD = 3, /* kquant_batched_kernels.h:299-301            */
    ORC_ORDER_COUNT = 4
};

/* SiLU-gate flavours (which one the reference runs depends on the branch). */
enum {
    ORC_SILU_EXACT = 0,     /* g/(1+expf(-g))*u   hwy_moe_quant.cc:377      */
    ORC_SILU_FAST = 1,      /* g/(1+FastExp(-g))*u raw_batched.inl:1673     */
    ORC_SILU_FAST_FMA = 2   /* g*(1/(1+FastExpHwy(-g)))*u hwy_activation.cc:163-166 */
};

/* ---- scalar building blocks ------------------------------------------ */
float orc_fp16_to_fp32(uint16_t h);
uint16_t orc_fp32_to_fp16(float f);        /* round-to-nearest-even, for generators */
int orc_nearest_int(float v);
void orc_q4k_scales_kmask(const uint8_t packed[12], uint8_t scales[8], uint8_t mins[8]);
void orc_q4k_scales_indexed(const uint8_t packed[12], uint8_t scales[8], uint8_t mins[8]);
float orc_fast_exp(float x);
float orc_fast_exp_fma(float x);
float orc_silu_mul(float gate, float up, int silu_mode);

/* ---- Q8_K quantizer ---------------------------------------------------- */
/* Returns 0 on success, -1 on bad arguments (null, cols <= 0, cols % 256). */
int orc_quantize_row_q8k(const float* x, void* q8_out, int64_t cols);
int orc_quantize_rows_q8k(const float* x, int64_t n, int64_t ldx, void* q8_out, int64_t cols);

/* ---- per-superblock integer sums --------------------------------------- */
void orc_block_sums(const orc_block_q4k* w, const orc_block_q8k* y, int32_t* dot_scaled, int32_t* min_dot);
/* [rows][n][nb] int32 arrays of both sums for a whole matrix. */
int orc_matrix_block_sums(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                          size_t q8_row_bytes, int32_t* dot_scaled, int32_t* min_dot);

/* ---- row dot, four fp32 orders ----------------------------------------- */
float orc_dot_q4k_q8k(const void* w_row, const void* q8_row, int64_t cols, int order);
double orc_dot_dequant_f64(const void* w_row, const void* q8_row, int64_t cols);
/* Sum over blocks of |d*yd*dot_scaled| + |dmin*yd*min_dot| in double: the
 * magnitude against which accumulation-order differences are judged. */
double orc_dot_magnitude_f64(const void* w_row, const void* q8_row, int64_t cols);

/* out[m*ldo + r] = W[r] . q8[m]   (token-major output, like RunMoEQ4KRawBatchedProjectionImpl) */
int orc_mul_mat_q4k_q8k(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                        size_t q8_row_bytes, float* out, int64_t ldo, int order);
/* fp32 activations in, quantized per row first (cb_gemv_custom / cb_gemv_batched_custom semantics). */
int orc_mul_mat_q4k_f32(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const float* x, int64_t n,
                        int64_t ldx, float* out, int64_t ldo, int order);

/* out[m][r] = silu(gate[r] . q8(x[m])) * (up[r] . q8(x[m])) */
int orc_swiglu_mul_mat_q4k_f32(const void* gate, const void* up, int64_t inter, int64_t hidden, const float* x,
                               int64_t n, float* out, int order, int silu_mode);

/* ---- dense SwiGLU FFN: y = down( silu(gate x) * (up x) ) --------------- */
int orc_ffn_swiglu_q4k(const void* gate, const void* up, const void* down, int64_t hidden, int64_t inter,
                       const float* x, int64_t n, float* y, int order, int silu_mode, float* inter_out);

/* ---- router ------------------------------------------------------------- */
/* Stable top-k (ties -> lower id, NaN last) + softmax over the selected
 * logits.  weights_mode 0 = single-token fused router (native.cpp:621-676),
 * 1 = multi-token variant with the 6.1035e-5 floor (native.cpp:2305-2357). */
int orc_route_topk(const float* logits, int64_t n_experts, int64_t n_tokens, int top_k, int weights_mode,
                   int32_t* ids, float* weights);
/* Weights of given ids from raw logits (core/src/llm/moe/native.cpp:2305-2357): softmax over the valid
 * selected logits, max replaced by 0 when not finite, denominator floored at 2^-14, invalid ids -> 0. */
int orc_route_weights_from_ids(const float* logits, int64_t n_experts, int64_t n_tokens, const int32_t* ids, int top_k,
                               float* weights);

typedef struct {
    int32_t expert;
    int32_t token;
    int32_t k;
} orc_assignment;
/* Sorted by (expert, token, k); returns the count (entries with invalid ids dropped). */
int64_t orc_build_assignments(const int32_t* ids, int64_t n_tokens, int top_k, int64_t n_experts, orc_assignment* out);

/* ---- MoE layer ------------------------------------------------------------ */
typedef struct {
    int64_t hidden;      /* model width (cols of gate/up, rows of down)     */
    int64_t inter;       /* expert intermediate width                       */
    int64_t n_experts;
    int top_k;
    const void* gate_exps; /* [n_experts][inter][hidden/256] blocks          */
    const void* up_exps;
    const void* down_exps; /* [n_experts][hidden][inter/256] blocks          */
    const void* sh_gate;   /* shared expert, may be NULL                     */
    const void* sh_up;
    const void* sh_down;
    const float* sh_gate_inp; /* [hidden] fp32 scalar-gate vector, may be NULL */
    /* ggml_type of the stacks: 12 = Q4_K, 13 = Q5_K, 14 = Q6_K; 0 reads as Q4_K.  The loader admits Q4_K / Q5_K gate and
     * up stacks and Q4_K / Q5_K / Q6_K / Q8_0 down stacks (core/src/llm/moe/native.cpp:4611-4620); one template multiplies
     * the first two (hwy_moe_quant.cc:145-258), ComputeQ6KQ8K the third (core/src/llm/matmul/q6_small_batch.h:13-92). */
    int gu_type, down_type, sh_gu_type, sh_down_type;
} orc_moe_weights;

/* Row product of a K-quant weight row of the given ggml_type (12, 13, 14; 0 = 12) with a Q8_K row, and the bytes of
 * such a weight row. */
float orc_dot_typed_q8k(int ggml_type, const void* w_row, const void* q8_row, int64_t cols, int order);
size_t orc_row_bytes_typed(int ggml_type, int64_t cols);
/* y = down(silu(gate x) * (up x)) with gate/up of gu_type and down of down_type. */
int orc_ffn_swiglu_typed(int gu_type, int down_type, const void* gate, const void* up, const void* down, int64_t hidden,
                         int64_t inter, const float* x, int64_t n, float* y, int order, int silu_mode, float* inter_out);

int orc_moe_gateup_swiglu(const orc_moe_weights* w, const float* x, const int32_t* ids, int64_t n_tokens, int order,
                          int silu_mode, float* hidden /* [n][top_k][inter] */);
int orc_moe_down_weighted(const orc_moe_weights* w, const float* hidden, const int32_t* ids, const float* weights,
                          int64_t n_tokens, int order, int accumulate_mode, float* y);
int orc_moe_add_shared(const orc_moe_weights* w, const float* x, int64_t n_tokens, int order, float* y);

/* accumulate_mode 0: per token, k = 0..top_k-1 in routing order (native.cpp:3233-3285)
 * accumulate_mode 1: expert-sorted assignment order (native.cpp:3152-3194) */
int orc_moe_layer(const orc_moe_weights* w, const float* x, const float* logits, int64_t n_tokens, float* y,
                  int order, int silu_mode, int weights_mode, int accumulate_mode, int32_t* ids_out,
                  float* weights_out, float* hidden_out /* [n][top_k][inter] or NULL */);

#ifdef __cplusplus
}
#endif
#endif
