/*
 * mi355_q4k.h -- C ABI of libmi355q4k.so: DenseCore's Q4_K-weight x
 * Q8_K-activation matmul path on one MI355X (gfx950).
 *
 * Every entry point is plain C: pointers, sizes, int status (0 = ok, negative
 * = error, text via mq_last_error()).  Pointers named *_dev are device
 * pointers (HBM), *_host are host pointers.  `stream` is a hipStream_t passed
 * as void* (NULL = the default stream).  All launches are stream-ordered and
 * return without synchronising unless the name ends in _host.
 *
 * Each declaration cites the DenseCore interface it stands in for
 * (paths relative to the DenseCore tree).
 */
#ifndef MI355_Q4K_H
#define MI355_Q4K_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MQ_OK 0
#define MQ_ERR_INVALID (-1)   /* bad argument (null, shape, alignment)          */
#define MQ_ERR_HIP (-2)       /* a HIP call failed                              */
#define MQ_ERR_STATE (-3)     /* library not initialised / no GPU               */
#define MQ_ERR_UNSUPPORTED (-4)

/* SiLU-gate flavours; which one the reference runs depends on the branch
 * (exact: core/src/kernels/hwy/hwy_moe_quant.cc:377; fast:
 * core/src/backend/cpu_backend_moe_raw_batched.inl:1673 with
 * cpu_backend_internal.h:99-114; fast_fma: core/src/kernels/hwy/hwy_activation.cc:153-167). */
#define MQ_SILU_EXACT 0
#define MQ_SILU_FAST 1
#define MQ_SILU_FAST_FMA 2

/* Router weight flavours (core/src/llm/moe/native.cpp:650-675, :2321-2355, :822-866). */
#define MQ_ROUTE_FUSED 0
#define MQ_ROUTE_FLOOR 1
#define MQ_ROUTE_FLOOR_FINITE 2

typedef struct mq_weight mq_weight; /* device-resident Q4_K matrix (or expert stack) */

/* ---- library state ---------------------------------------------------------
 * Mirrors the engine-level init/teardown and error string of the C API
 * (core/include/densecore.h:163 DenseCoreGetLastError, :296 InitEngine). */
int mq_init(int device);
int mq_shutdown(void);
const char* mq_last_error(void);
/* HIP runtime version, device name, CU count: what a host would log at load. */
int mq_device_info(char* name_out, size_t name_cap, int* cu_count, size_t* hbm_bytes);

/* ---- weights ----------------------------------------------------------------
 * Takes ggml-layout Q4_K bytes exactly as a GGUF tensor holds them: rows of
 * cols/256 block_q4_K (144 B each), `row_bytes` apart (ggml nb[1]); expert
 * matrices `expert_bytes` apart (ggml nb[2], core/src/llm/moe/native.cpp:4091-4094).
 * n_experts = 1 for a dense matrix.  The data is copied to HBM once and
 * re-tiled for the GPU (same 144 B per 256 weights); the host buffer is not
 * referenced afterwards.  Stands in for the weight side of
 * GgmlQuantizedMatrixView (core/include/densecore/backend/cpu_backend.h:91-99)
 * and for the repack cache GetOrCreateQ4KRepackedGemvWeight
 * (core/src/kernels/q4k_repacked_gemv.cpp:403). */
int mq_weight_upload(const void* q4k_host, int64_t rows, int64_t cols, int64_t n_experts, size_t row_bytes,
                     size_t expert_bytes, mq_weight** out);
/* The same for a tensor of another K-quant type.  ggml_type 12 = Q4_K (what mq_weight_upload takes),
 * 13 = Q5_K: block_q5_K is block_q4_K plus one high bit per weight (176 bytes: fp16 d, fp16 dmin, scales[12],
 * qh[32], qs[128]; core/src/kernels/hwy/hwy_moe_quant.cc:36-45), the type Q4_K_M files use for many down
 * projections (core/src/llm/moe/native.cpp:4611-4616) and DotKQ8KImpl<MoEQ5KBlock, true> multiplies
 * (core/src/kernels/hwy/hwy_moe_quant.cc:145-258); or 14 = Q6_K: 210 bytes, ql[128], qh[64], 16 signed
 * scales, fp16 d, weight = d * scale * (code - 32), multiplied as ComputeQ6KQ8KM4Native does
 * (core/src/llm/matmul/q6_small_batch.h:13-92): one integer sum_g scale_g * sum (code - 32) * q8 per
 * super-block (what mq_debug_block_sums returns as dot_scaled; min_dot is 0), one fused multiply-add per block.
 * Every product entry point accepts handles of any of the three types (gate and up of one call must share
 * theirs), the matrix-core GEMM (mq_gemm_q4k) and its expert-grouped form included -- the reference serves Q6_K at
 * every width through its batched machinery as well (core/src/llm/matmul/batched_exec.cpp:933,1280); the one-launch
 * decoder takes Q4_K only.
 * 8 = Q8_0 (fp16 d + 32 int8 codes, 34 bytes per 32 weights; core/src/llm/matmul/q8_small_batch.h:9-14): dense
 * matrices only (n_experts == 1, cols % 256 == 0, row_bytes >= cols / 32 * 34), taken by mq_mul_mat_q4k (and
 * mq_mul_mat_q4k_host, mq_debug_block_sums, the handle queries) and refused by every other entry point.  As in
 * the reference the activations of such a product are quantized to Q8_0 too (vec_dot_type of the type,
 * core/src/llm/matmul/batched_exec.cpp:630): d = amax / 127 per 32 values stored as fp16, codes =
 * round-half-even(x * (127 / amax)) -- ggml's x86 quantizer, which is not part of the reference tree, so its
 * parity is unpinned; y = sum over blocks of fp16(dx) * fp16(dy) * (integer dot), one fused multiply-add per block
 * (Q8SmallBatchDot4, core/src/llm/matmul/q8_small_batch.h:29-77).  x rows must be 16-byte aligned.
 * mq_debug_block_sums on such a handle writes dot_scaled as [rows][n][cols / 32], the integer dot of every block,
 * and leaves min_dot (may be NULL) alone.  Other types: MQ_ERR_UNSUPPORTED. */
int mq_weight_upload_typed(int ggml_type, const void* blocks_host, int64_t rows, int64_t cols, int64_t n_experts,
                           size_t row_bytes, size_t expert_bytes, mq_weight** out);
int mq_weight_synthetic_typed(int ggml_type, uint64_t seed, int64_t rows, int64_t cols, int64_t n_experts,
                              mq_weight** out);
int mq_weight_type(const mq_weight* w); /* 12, 13, 14, 8, or -1 for NULL */
/* Same tensor filled on the device from a 64-bit seed with the synthetic
 * recipe of densecore_amd/synth.py (byte-identical to uploading
 * synth.q4k_matrix(seed, rows*n_experts, cols)); for multi-GB benchmark sets. */
int mq_weight_synthetic(uint64_t seed, int64_t rows, int64_t cols, int64_t n_experts, mq_weight** out);
/* Copies the tensor back in ggml row layout (inverse of the re-tiling). */
int mq_weight_download(const mq_weight* w, void* q4k_host, size_t row_bytes, size_t expert_bytes);
int mq_weight_shape(const mq_weight* w, int64_t* rows, int64_t* cols, int64_t* n_experts, size_t* device_bytes);
int mq_weight_free(mq_weight* w);

/* ---- Q8_K activation quantizer ----------------------------------------------
 * x_dev fp32 [n][ldx] (first k of each row used) -> q8_dev [n][k/256] block_q8_K
 * (292 B: fp32 d, 256 int8, 16 int16 bsums), bit-exact with
 * QuantizeRowQ8K_Hwy (core/include/densecore/simd/hwy_ops.h:255,
 * core/src/kernels/hwy/hwy_moe_quant.cc:103-143) and ggml's from_float at
 * core/src/llm/matmul/gemv_exec.cpp:298-332. */
int mq_quantize_q8k(const float* x_dev, int64_t n, int64_t ldx, int64_t k, void* q8_dev, void* stream);

/* ---- dense matmul: ggml_mul_mat on GGML_TYPE_Q4_K ---------------------------
 * y[m][r] = W[r] . q8k(x[m]),  m < n, r < rows.  x_dev fp32 [n][ldx], y_dev
 * fp32 [n][ldy] (token-major, i.e. ggml dst ne = [rows, n]).  Replaces
 * cb_gemv_custom (core/src/llm/matmul/gemv_exec.cpp:99, n == 1),
 * cb_gemv_batched_custom (core/src/llm/matmul/batched_exec.cpp:55, 2 <= n <= 16)
 * and CpuBackend::MatMulGgmlQuantizedTransB
 * (core/include/densecore/backend/cpu_backend.h:293-300, any n). */
int mq_mul_mat_q4k(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                   void* stream);
/* Several products of ONE activation row in one launch: y_dev[i][r] = w[i][r] . q8k(x), i < count <= 8, all
 * weights dense with the same number of columns (x_dev fp32 [cols]; y_dev[i] fp32 [rows of w[i]]).  The graph
 * emits the q, k and v projections of a layer, and the gate and up projections of an FFN, as separate nodes on the
 * same input (core/src/llm/graph/decoder.cpp:1092-1099, :2662-2663; one fused tensor at :630); a caller that holds
 * them together hands them over together.  Q4_K matrices whose rows are short enough for the single-row kernel
 * with the quantizer inside share a launch -- the same bits as mq_mul_mat_q4k on each -- and pay the dispatch and
 * the first trip to memory once; any other weight in the list goes through mq_mul_mat_q4k.  An error leaves the
 * outputs of the list undefined. */
int mq_mul_mat_q4k_multi(const mq_weight* const* w, int count, const float* x_dev, float* const* y_dev, void* stream);
/* mq_mul_mat_q4k for callers that cannot allocate (code under HIP-graph capture, serving loops and harnesses that
 * forbid hipMalloc): the same product, bit for bit, for n <= 16 rows of cols <= 16384 (MQ_ERR_UNSUPPORTED beyond
 * that), Q4_K / Q5_K / Q6_K weights.  It calls no allocating routine: the quantized activations go to a fixed
 * 528,384-byte device array inside the library (one per GPU, held until the process ends) whose address mq_init
 * looks up.  It has no counterpart in the reference.  Every call on a GPU shares that GPU's array: calls that
 * overlap on one GPU (two streams, two threads' launches in flight together) race; order them on one stream. */
int mq_mul_mat_q4k_noalloc(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                           void* stream);
/* The same product computed by the matrix-core GEMM kernel whatever n is (mq_mul_mat_q4k switches to it
 * by itself from 48 rows up, from 17 for matrices of 24 MB and more; Q4_K products stay on the decode arithmetic up to
 * 32 rows, up to 64 where their rows pass through LDS in runs of super-blocks, Q5_K and Q6_K products likewise): weights are read once per 128 activation rows and the int8 MFMA
 * units do the arithmetic.  RunQ4KRawBatchedDenseGemm (core/src/backend/cpu_backend_q4k_dense.cpp:57-101),
 * the A.shape[0] >= 4 branch of MatMulGgmlQuantizedTransBWithPath
 * (core/src/backend/cpu_backend_quantized_matmul.cpp:164-170).  Same integers per super-block as
 * mq_mul_mat_q4k; the fp32 update uses fused multiply-adds, so results agree to rounding, not bitwise. */
int mq_gemm_q4k(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                void* stream);
/* Same with already-quantized activations: q8_dev [n][q8_row_bytes] block_q8_K rows
 * (RunMoEQ4KRawBatchedProjectionImpl, core/src/backend/cpu_backend_moe_raw_batched.inl:1352). */
int mq_mul_mat_q4k_q8k(const mq_weight* w, const void* q8_dev, int64_t n, size_t q8_row_bytes, float* y_dev,
                       int64_t ldy, void* stream);
/* Host-pointer convenience for a CPU graph executor: copies x in, y out, and
 * synchronises.  What a GGML_OP_CUSTOM callback calls when ith == 0. */
int mq_mul_mat_q4k_host(const mq_weight* w, const float* x_host, int64_t n, int64_t ldx, float* y_host, int64_t ldy);

/* ---- quantize once, multiply many times -----------------------------------------------------
 * A handle to Q8_K activation rows kept on the device in the layout the matmul kernels read, so that
 * several projections of one input (q/k/v, gate/up) pay for one quantization.  The reference does
 * the same with the Q8_K scratch that one thread fills and every row-partition thread reads
 * (core/src/llm/matmul/gemv_exec.cpp:298-341, MatmulWorkState core/src/llm/runtime/work_state.h:86-89)
 * and with Qwen35SharedQ8RowsUserData (core/src/llm/moe/native.cpp:1027-1038).
 * create/free allocate and must stay outside a HIP-graph capture; quantize and the two products
 * only launch kernels.  n of the products is the n of the handle's last mq_acts_quantize. */
typedef struct mq_acts mq_acts;
int mq_acts_create(int64_t max_rows, int64_t cols, mq_acts** out);
int mq_acts_free(mq_acts* a);
int mq_acts_quantize(mq_acts* a, const float* x_dev, int64_t n, int64_t ldx, void* stream);
int mq_mul_mat_q4k_acts(const mq_weight* w, const mq_acts* a, float* y_dev, int64_t ldy, void* stream);
int mq_swiglu_mul_mat_q4k_acts(const mq_weight* gate, const mq_weight* up, const mq_acts* a, float* h_dev,
                               int64_t ldh, int silu_mode, void* stream);

/* ---- fused gate/up + SwiGLU ----------------------------------------------------
 * h[m][r] = silu(gate[r] . q8k(x[m])) * (up[r] . q8k(x[m])), one pass over both matrices.
 * FusedSwiGLUQ4KQ8KRows_Hwy (core/include/densecore/simd/hwy_ops.h:275-281,
 * core/src/kernels/hwy/hwy_moe_quant.cc:359-380) and RunMoEQ4KRawBatchedFusedSwiGLUImpl
 * (core/src/backend/cpu_backend_moe_raw_batched.inl:1629-1698).  Wherever mq_mul_mat_q4k would take the
 * matrix-core GEMM (Q4_K, 48 rows and more, 17 for matrices of 24 MB and more; 16-byte aligned h rows) the two
 * products run on it and a third launch forms h. */
int mq_swiglu_mul_mat_q4k(const mq_weight* gate, const mq_weight* up, const float* x_dev, int64_t n, int64_t ldx,
                          float* h_dev, int64_t ldh, int silu_mode, void* stream);

/* ---- dense SwiGLU FFN --------------------------------------------------------
 * y = down( silu(gate x) * (up x) ), x_dev [n][hidden], y_dev [n][hidden].
 * gate/up: rows = inter, cols = hidden; down: rows = hidden, cols = inter.
 * The three smart_mul_mat calls plus cb_silu_mul_fused of a dense FFN block
 * (core/src/llm/graph/decoder.cpp:2662-2730, core/src/llm/graph/fused_ops.cpp:317-366).  Prefill widths (the
 * row counts from which mq_mul_mat_q4k takes the matrix-core GEMM for both shapes) run as three GEMMs, the SwiGLU
 * formed by the quantizer of the down product: 4096 -> 14336 -> 4096 at 512 / 2048 rows in 0.27 / 0.95 ms. */
int mq_ffn_swiglu_q4k(const mq_weight* gate, const mq_weight* up, const mq_weight* down, const float* x_dev,
                      int64_t n, float* y_dev, int silu_mode, void* stream);

/* ---- MoE router ---------------------------------------------------------------
 * logits_dev fp32 [n][n_experts] -> ids_dev int32 [n][top_k], weights_dev fp32
 * [n][top_k]: stable top-k (ties -> lower id, NaN last) and softmax over the
 * selected logits.  ComputeQwenNativeMoEStableTopK
 * (core/src/llm/moe/native.cpp:621-676) / cb_moe_topk_weights_from_logits (:800-868). */
int mq_moe_route_topk(const float* logits_dev, int64_t n_experts, int64_t n, int top_k, int weights_mode,
                      int32_t* ids_dev, float* weights_dev, void* stream);

/* Weights of ALREADY selected experts from the raw logits, as the down node resolves them itself:
 * softmax over the valid selected logits (a non-finite max counts as 0, denominator floored at 2^-14),
 * ids outside [0, n_experts) weigh 0.  Qwen35NativeMoEComputeTopKWeightsFromLogits
 * (core/src/llm/moe/native.cpp:2305-2357). */
int mq_moe_weights_from_logits(const float* logits_dev, int64_t n_experts, int64_t n, const int32_t* ids_dev,
                               int top_k, float* weights_dev, void* stream);

/* ---- expert-routed matmul: ggml_mul_mat_id on GGML_TYPE_Q4_K -----------------
 * y[t][k][r] = W[ids[t][k]][r] . q8k(x[t][k or 0]).  x_dev fp32 [n][x_slots][cols]
 * with x_slots == 1 (one row per token, broadcast over k: the gate/up case) or
 * x_slots == top_k (one row per (token, k): the down case).  ids_dev int32
 * [n][top_k]; entries outside [0, n_experts) produce zeros.  Tokens are grouped
 * by expert on the device; nothing returns to the host.  y_dev fp32
 * [n][top_k][rows].  (ggml_mul_mat_id as emitted at
 * core/src/llm/moe/native_gemma.cpp:1509-1559.)  Prefill widths (192 tokens
 * and more with six rows per expert on average) run on the int8 matrix-core
 * GEMM in its expert-grouped form, as do mq_moe_gateup_swiglu_q4k and
 * mq_moe_down_weighted_q4k below. */
int mq_mul_mat_id_q4k(const mq_weight* w_exps, const float* x_dev, int64_t n, int x_slots, const int32_t* ids_dev,
                      int top_k, float* y_dev, void* stream);

/* ---- the two expert nodes of the native MoE graph --------------------------------
 * gate/up node: hidden[t][k][r] = silu(gate_e[r] . q8k(x[t])) * (up_e[r] . q8k(x[t])), e = ids[t][k];
 * hidden_dev fp32 [n][top_k][inter].  cb_qwen35_native_moe_gateup_raw_qxk_swiglu
 * (core/src/llm/moe/native.cpp:3929-4345, built at :4871-4874).  Rows whose id is outside
 * [0, n_experts) are set to zero. */
int mq_moe_gateup_swiglu_q4k(const mq_weight* gate_exps, const mq_weight* up_exps, const float* x_dev, int64_t n,
                             const int32_t* ids_dev, int top_k, int silu_mode, float* hidden_dev, void* stream);
/* down node: y[t][r] = sum_k weights[t][k] * (down_e[r] . q8k(hidden[t][k])), k in routing order,
 * zero weights and invalid ids skipped.  cb_qwen35_native_moe_down_q5k_weighted_logits
 * (core/src/llm/moe/native.cpp:3051-3295, built at :4906-4911) with the weights already resolved
 * by mq_moe_route_topk; also RunMoEQ4KRawBatchedWeightedScatterProjectionImpl
 * (core/src/backend/cpu_backend_moe_raw_batched.inl:1437-1492). */
int mq_moe_down_weighted_q4k(const mq_weight* down_exps, const float* hidden_dev, int64_t n, const int32_t* ids_dev,
                             const float* weights_dev, int top_k, float* y_dev, void* stream);

/* ---- fused MoE layer -------------------------------------------------------------
 * The four custom nodes of TryBuildQwen35NativeMoEGraph
 * (core/src/llm/moe/native.cpp:4691, :4831-4911) plus the shared-expert branch
 * (core/src/llm/graph/decoder.cpp:2426-2600):
 *   route top_k -> gate/up + SwiGLU per (token, k) -> Q8_K -> down ->
 *   y[t] = sum_k w[t][k] * down_k (k in routing order) + sigmoid(sh_gate_inp . x[t]) * shared_ffn(x[t]).
 * shared_* may all be NULL (no shared expert); sh_gate_inp_dev fp32 [hidden] or NULL (gate = 1).
 * Up to eight tokens (and 512 experts) two launches: gate/up + SwiGLU with the router and the Q8_K of x inside,
 * down with the Q8_K of the hidden rows and the weighted combine inside.  Above: router + expert grouping + Q8_K
 * of x, expert-grouped gate/up leaving its rows in Q8_K, expert-grouped down, combine.  Same bits either way.
 * Prefill widths (192 tokens and more with six routed rows per expert on average): the expert products run on the
 * int8 matrix-core GEMM in an expert-grouped form (entries in 16-row tiles per expert), the shared expert as one more
 * group of all tokens; a Q8_0 down stack takes the fp32 hidden rows of that gate/up through its own launches; same routing, results within the fp32 tolerance of the other form (the
 * summation order differs), and mq_debug_moe_hidden does not apply. */
typedef struct {
    const mq_weight* gate_exps; /* n_experts x [inter][hidden]  */
    const mq_weight* up_exps;
    const mq_weight* down_exps; /* n_experts x [hidden][inter]  */
    const mq_weight* shared_gate;
    const mq_weight* shared_up;
    const mq_weight* shared_down;
    const float* sh_gate_inp_dev;
    int top_k;
    int silu_mode;        /* routed experts; the shared expert always uses MQ_SILU_FAST_FMA */
    int route_mode;
} mq_moe_layer_desc;
int mq_moe_layer_q4k(const mq_moe_layer_desc* layer, const float* x_dev, const float* logits_dev, int64_t n,
                     float* y_dev, int32_t* ids_out_dev /* may be NULL */, float* weights_out_dev /* may be NULL */,
                     void* stream);

/* ---- a run of decoder layers in one launch --------------------------------------------
 * Per layer, for n <= 8 tokens (x is the residual stream, fp32 [n][hidden]):
 *   h   = rmsnorm(x) * attn_norm          qkv = wqkv . q8k(h)          o = wo . q8k(qkv[:, :n_q])
 *   x  += o          h2 = rmsnorm(x) * ffn_norm          logits = router . h2 (fp32)
 *   x  += moe(h2, logits)                 (mq_moe_layer_q4k's arithmetic, shared expert included)
 * i.e. the node sequence the reference's graph builder emits for a Qwen3.5-MoE-class layer
 * (core/src/llm/graph/decoder.cpp:2265, :2426-2600; core/src/llm/moe/native.cpp:4831-4911) with the attention
 * core left out (the first n_q columns of qkv stand in for its output).  The reference runs those nodes on CPU
 * threads that meet at a barrier after each one; here one persistent kernel does, with device-wide barriers
 * between the phases, and returns bit for bit what the node-by-node entry points above return
 * (mq_add_rmsnorm_q8k, mq_mul_mat_q4k_acts, mq_mul_mat_q4k, mq_add_rmsnorm_f32, mq_router_logits_f32,
 * mq_moe_layer_q4k).  All weights Q4_K; every layer has layer 0's shapes; n_experts <= 512; top_k <= 8.
 * The kernel needs every compute unit of the device free for this process: a barrier that is not met within
 * 200 ms is abandoned, the launch drains, and mq_decoder_status reports it.  Steps of one handle, and steps of
 * different handles, must not overlap on the device (one stream, or streams ordered by events). */
typedef struct mq_decoder mq_decoder;
typedef struct {
    const mq_weight* wqkv;            /* [n_q + 2 n_kv][hidden], wq / wk / wv stacked row-wise */
    const mq_weight* wo;              /* [hidden][n_q] */
    const float* attn_norm_dev;       /* fp32 [hidden] or NULL (ones) */
    const float* ffn_norm_dev;
    const float* router_dev;          /* fp32 [n_experts][hidden] */
    const float* fixed_logits_dev;    /* NULL, or fp32 [n][n_experts]: route on these, not on router . h2 */
    mq_moe_layer_desc moe;            /* silu_mode is taken from mq_decoder_step, not from here */
} mq_decoder_layer_desc;
/* Copies the layer table to the device and allocates the exchange buffers; the weights stay the caller's. */
int mq_decoder_create(const mq_decoder_layer_desc* layers, int n_layers, int64_t max_tokens, float eps, mq_decoder** out);
/* out = x after the last layer, fp32 [n][hidden].  silu_mode: MQ_SILU_* for the routed experts, or -1 for the
 * reference's rule (exact for n <= 4, polynomial above; core/src/llm/moe/native.cpp:3614-3616).
 * ids_out_dev int32 / weights_out_dev fp32 [n_layers][n][top_k], or NULL.  Allocates nothing (capturable). */
int mq_decoder_step(mq_decoder* d, const float* x_dev, int64_t n, int silu_mode, float* out_dev, int32_t* ids_out_dev,
                    float* weights_out_dev, void* stream);
/* Synchronises the device; MQ_OK, or MQ_ERR_STATE when a step since the last call abandoned a barrier (its
 * outputs are void; the handle is usable again afterwards). */
int mq_decoder_status(mq_decoder* d);
/* How long a workgroup waits at a device-wide barrier before it abandons the step (default 200 ms).  0 makes
 * every waiter give up at once: the error path can be exercised without hanging anything. */
int mq_decoder_set_patience(mq_decoder* d, int64_t microseconds);
void mq_decoder_free(mq_decoder* d);

/* ---- the fp32 operators either side of the path --------------------------------------------
 * sum = x + delta (delta_dev may be NULL: sum = x), normed = sum * (weight / sqrt(mean(sum^2) + eps));
 * x/delta/sum/normed fp32 [n][cols] dense, weight_dev fp32 [cols] or NULL (ones), sum_out_dev may be NULL
 * or alias x_dev.  AddRMSNorm (core/src/kernels/hwy/hwy_normalization.cc:102-153) as wired by
 * cb_add_rms_norm (core/src/llm/graph/fused_ops.cpp:138-169); the input of every projection above. */
int mq_add_rmsnorm_f32(const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n, int64_t cols,
                       float eps, float* sum_out_dev, float* normed_out_dev, void* stream);
/* The same with the normalised rows also (or only: normed_out_dev may be NULL) leaving as Q8_K in an
 * activation handle, ready for mq_mul_mat_q4k_acts: the quantizer that every projection would otherwise
 * launch first, folded into the operator that produces its input.  cols % 256 == 0, cols = the handle's.
 * The Q8_K rows are bit-identical to mq_acts_quantize of the fp32 rows this call writes. */
int mq_add_rmsnorm_q8k(const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n, int64_t cols,
                       float eps, float* sum_out_dev, float* normed_out_dev, mq_acts* acts, void* stream);
/* mq_add_rmsnorm_q8k followed by mq_mul_mat_q4k_acts: sum = x + delta (delta_dev may be NULL), h = rmsnorm(sum) *
 * weight (weight_dev may be NULL), y[t] = W . q8k(h[t]); x/delta/sum fp32 [n][cols] dense, y fp32 [n][ldy].  Up to
 * four rows of input against Q4_K weights with short rows run as ONE launch (norm and quantizer inside the GEMV),
 * otherwise two; the same bits either way.  sum_out_dev (may be NULL) must be neither x_dev nor delta_dev.  At the
 * widths where mq_mul_mat_q4k takes the matrix-core GEMM the normalised rows are written as fp32 and go through it, and
 * likewise, from seventeen rows, where it takes the rows as tiles of sixteen. */
int mq_rmsnorm_mul_mat_q4k(const mq_weight* w, const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n,
                           float eps, float* sum_out_dev, float* y_dev, int64_t ldy, void* stream);
/* logits[t][e] = w[e] . x[t] in fp32: the ffn_gate_inp router projection
 * (core/src/llm/graph/decoder.cpp:2265) whose output mq_moe_layer_q4k consumes.  w_dev fp32
 * [n_experts][cols], x_dev fp32 [n][ldx], logits_dev fp32 [n][n_experts]; cols % 256 == 0. */
int mq_router_logits_f32(const float* w_dev, int64_t n_experts, int64_t cols, const float* x_dev, int64_t n,
                         int64_t ldx, float* logits_dev, void* stream);
/* mq_add_rmsnorm_f32 followed by mq_router_logits_f32 on its normalised rows, in one launch and with the same
 * bits: sum = x + delta, normed = rmsnorm(sum) * weight, logits[t][e] = router[e] . normed[t].  cols a multiple
 * of 256 up to 4096; sum_out_dev (may be NULL, as normed_out_dev) must be neither x_dev nor delta_dev. */
int mq_add_rmsnorm_router_f32(const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n, int64_t cols,
                              float eps, float* sum_out_dev, float* normed_out_dev, const float* router_dev, int64_t n_experts,
                              float* logits_dev, void* stream);

/* ---- the two element-wise nodes of a dense FFN / shared expert as the graph emits them ---------------
 * out[t][c] = silu(gate[t][c]) * up[t][c] over [n][cols] fp32 with row strides in floats: cb_silu_mul_fused
 * (core/src/llm/graph/fused_ops.cpp:317-366).  The reference runs MQ_SILU_FAST_FMA on contiguous tensors
 * (SiLUMulParallel, core/src/kernels/hwy/hwy_activation.cc:153-167) and MQ_SILU_EXACT on strided ones (:364). */
int mq_silu_mul_f32(const float* gate_dev, const float* up_dev, int64_t n, int64_t cols, int64_t ld_gate, int64_t ld_up, float* out_dev,
                    int64_t ld_out, int silu_mode, void* stream);
/* out[t][c] = sigmoid(logit[t * ld_logit]) * src[t][c], the sigmoid two-sided (1 / (1 + e^-x) for x >= 0, e^x / (1 + e^x)
 * below): cb_apply_shared_scalar_gate (core/src/llm/graph/fused_ops.cpp:437-475), the scalar gate on the shared expert's
 * output. */
int mq_scale_rows_sigmoid_f32(const float* src_dev, int64_t n, int64_t cols, int64_t ld_src, const float* logit_dev, int64_t ld_logit,
                              float* out_dev, int64_t ld_out, void* stream);

/* Verification hooks (per-super-block integer sums, work lists, intermediates), the launch census and the kernel
 * selection switch are declared in mi355_q4k_debug.h: test and measurement instruments, not part of what a host binds. */

/* ---- device memory helpers (so a C host needs no HIP headers) -------------------- */
int mq_device_malloc(void** ptr, size_t bytes);
int mq_device_free(void* ptr);
int mq_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes);
int mq_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes);
/* Page-locked host memory (allocated, not registered) and copies that are asynchronous on a stream when the host
 * side is such memory: what the ggml adapters stage graph tensors through, so that a node costs one
 * synchronisation instead of one per copy. */
int mq_host_malloc(void** ptr, size_t bytes);
int mq_host_free(void* ptr);
int mq_memcpy_h2d_async(void* dst_dev, const void* src_pinned, size_t bytes, void* stream);
int mq_memcpy_d2h_async(void* dst_pinned, const void* src_dev, size_t bytes, void* stream);
int mq_stream_synchronize(void* stream);

#ifdef __cplusplus
}
#endif
#endif
