// Host-callable launchers of the gfx950 kernels (internal to libmi355q4k.so).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mq {

// ---- quantize.hip ----------------------------------------------------------------------------
// fp32 rows -> Q8_K.  q8_std (block_q8_K rows, may be null) and/or the A-major pair (aq, ad; may be
// null) are written from the same registers.
hipError_t launch_quantize_q8k(const float* x, int64_t n, int64_t ldx, int64_t k, void* q8_std, size_t q8_row_bytes,
                               uint8_t* aq, float* ad, hipStream_t stream);
// block_q8_K rows -> A-major layout.
hipError_t launch_q8k_to_amajor(const void* q8_std, int64_t n, size_t q8_row_bytes, int64_t k, uint8_t* aq, float* ad,
                                hipStream_t stream);

// ---- weights.hip -----------------------------------------------------------------------------
// ggml row layout (rows x nb blocks, row_bytes apart) -> tiled layout, one expert per grid.y.
// type: kTypeQ4K or kTypeQ5K (ggml_type values).
hipError_t launch_tile_weights(const uint8_t* raw, int64_t rows, int64_t nb, int type, size_t row_bytes,
                               size_t expert_bytes, int64_t n_experts, uint8_t* tiled, size_t tiled_expert_bytes,
                               hipStream_t stream);
hipError_t launch_untile_weights(const uint8_t* tiled, int64_t rows, int64_t nb, int type, size_t row_bytes,
                                 size_t expert_bytes, int64_t n_experts, uint8_t* raw, size_t tiled_expert_bytes,
                                 hipStream_t stream);
hipError_t launch_synth_weights(uint64_t seed, int64_t rows, int64_t nb, int type, int64_t n_experts, uint8_t* tiled,
                                size_t tiled_expert_bytes, hipStream_t stream);

// ---- matmul.hip ------------------------------------------------------------------------------
struct MatmulArgs {
    const uint8_t* w0 = nullptr;   // tiled weights (expert 0); gate when swiglu
    const uint8_t* w1 = nullptr;   // up weights when swiglu, else unused
    int64_t rows = 0;              // output rows of one matrix
    int64_t nb = 0;                // super-blocks per row (cols / 256)
    size_t expert_bytes = 0;       // tiled bytes per expert (grouped mode)
    const uint8_t* aq = nullptr;   // A-major activations
    const float* ad = nullptr;
    // dense mode, nine to sixteen rows of a Q4_K matrix: the rows as one P-major tile per super-block instead (skinny16_kernel)
    const uint8_t* ap = nullptr;
    // dense mode, n == 1: the activation row as fp32 instead; every wavefront quantizes the super-blocks it
    // multiplies (same codes and scales as the stand-alone quantizer, so the same result)
    const float* xf = nullptr;
    int64_t ldx = 0;               // xf with n > 1 (taken by the LDS-staged dense kernel only): floats between rows
    int64_t n = 0;                 // activation rows (dense mode)
    float* y = nullptr;            // dense: [n][ldy]; grouped: [entry][ldy]
    int64_t ldy = 0;
    int wtype = 12;                // ggml_type of the weights: 12 (Q4_K) or 13 (Q5_K); gate and up share it
    int rt_per_wg = 1;             // row tiles per workgroup (set by launch_matmul)
    int swiglu = 0;                // 1: y = silu(w0 x) * (w1 x)
    int silu_mode = 0;
    int32_t* dbg_dot = nullptr;    // optional [rows][n][nb]
    int32_t* dbg_min = nullptr;
    // optional fused re-quantization of the output: the workgroup that completes a 256-row block of
    // y (the last of its 16 row tiles to finish) quantizes that block of every live activation row
    // to Q8_K in the A-major layout, ready to be the next matmul's input.  rows % 256 == 0.
    uint8_t* out_aq = nullptr;
    float* out_ad = nullptr;
    uint32_t* out_counters = nullptr;  // [groups][rows/256], zero before the launch, zero again after it
    // grouped (expert-routed) mode: work list built on the device
    int grouped = 0;
    const int32_t* group_expert = nullptr;  // [max_groups] expert id per group
    const int32_t* group_begin = nullptr;   // [max_groups + 1] offsets into entries
    const int32_t* n_groups = nullptr;      // [1]
    const int32_t* entry_token = nullptr;   // [n_entries] token of each entry, sorted by (expert, token, k)
    const int32_t* entry_k = nullptr;       // [n_entries] routing slot of each entry
    int a_tok_stride = 1, a_k_stride = 0;   // activation row of an entry = token * a_tok_stride + k * a_k_stride
    int y_tok_stride = 1, y_k_stride = 0;   // output row of an entry
    int max_groups = 0;
    // few tokens: group g is the pair (token g / direct_top_k, slot g % direct_top_k) with expert direct_ids[g];
    // no lists are read (grouping by expert shares nothing when nearly every pair has an expert of its own)
    const int32_t* direct_ids = nullptr;
    int direct_top_k = 0;
    int n_experts = 0;             // for range-checking direct_ids
    // optional second family of groups with their own weights (the shared expert): group ids >= n_groups
    const uint8_t* sh_w0 = nullptr;
    const uint8_t* sh_w1 = nullptr;
    int sh_tokens = 0;             // number of activation rows the shared expert sees (0 = none)
    int sh_arow_stride = 1;        // activation row of token t = t * sh_arow_stride + sh_arow_offset
    int sh_arow_offset = 0;
    int sh_yrow_stride = 1;        // output row of token t
    int sh_yrow_offset = 0;
    int sh_silu_mode = 2;
};
// Waves per workgroup that launch_matmul gives `workgroups` workgroups of rows with nb super-blocks.
int pick_waves(int64_t nb, int64_t workgroups);
// Compute units the launch heuristics size their grids for (mq_init sets the device's count; a partitioned device has fewer).
void set_compute_units(int count);
int compute_units();
// start/stop (both or neither): events that receive the kernel dispatch's own begin and end timestamps.
hipError_t launch_matmul(const MatmulArgs& a, hipStream_t stream, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);

// ---- grouped_lds.hip -------------------------------------------------------------------------
// Expert-grouped launches with many groups: a group's activation rows gathered into LDS once per workgroup of eight
// wavefronts (the same bits as matmul_kernel's one-wave workgroups).
bool grouped_lds_applies(const MatmulArgs& a);
hipError_t launch_grouped_lds(const MatmulArgs& a, int rt_per_wave, int groups, hipStream_t stream, hipEvent_t start = nullptr,
                              hipEvent_t stop = nullptr);
void set_grouped_lds(bool on);  // debug switch: off keeps these launches on matmul_kernel

// ---- dense_lds.hip ---------------------------------------------------------------------------
// Dense product for 1..16 rows with the quantized activations staged once per workgroup in LDS (same bits as
// launch_matmul on the same operands).  Either (aq, ad) -- the A-major workspace -- or xf: fp32 rows (n <= 8,
// 16-byte aligned, ldx % 4 == 0) that the kernel quantizes itself.
struct DenseLdsArgs {
    const uint8_t* w0 = nullptr;   // tiled weights; gate when w1 is set
    const uint8_t* w1 = nullptr;   // up weights: y = silu(w0 x) * (w1 x)
    int64_t rows = 0, nb = 0;
    const uint8_t* aq = nullptr;
    const float* ad = nullptr;
    const float* xf = nullptr;
    int64_t ldx = 0;
    int64_t n = 0;
    float* y = nullptr;
    int64_t ldy = 0;
    int wtype = 12;
    int silu_mode = 0;
};
// true when the shape fits the kernel (LDS capacity, wavefront split)
bool dense_lds_applies(int64_t nb, int64_t rowtiles, int64_t n, bool swiglu, int wtype);
hipError_t launch_dense_lds(const DenseLdsArgs& a, hipStream_t stream, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);

// Wavefronts per row tile of the LDS-staged dense kernels for a matrix (pick_waves, as a divisor of eight; 0: none)
int dense_lds_wpr(int64_t nb, int64_t rowtiles);

// ---- prefill.hip: nine to sixteen rows as ONE activation tile against a streamed Q4_K matrix (skinny16_kernel) ----
struct Skinny16Args {
    const uint8_t* w0 = nullptr;   // tiled Q4_K weights; gate when w1 is set
    const uint8_t* w1 = nullptr;   // up weights: y = silu(w0 x) * (w1 x)
    int64_t rows = 0, nb = 0;
    const uint8_t* ap = nullptr;   // the rows' P-major tiles: [nb][tiles][4688], tiles = ceil(n / 16) (launch_quantize_q8k_pmajor)
    int64_t n = 0;                 // live rows, 1..64
    float* y = nullptr;
    int64_t ldy = 0;
    int silu_mode = 0;
    int wtype = kTypeQ4K;          // kTypeQ4K, or kTypeQ5K / kTypeQ6K (one and two tiles)
    int ranges = 1;                // set by the launcher: runs of super-blocks the tiles pass through LDS in
};
bool skinny16_applies(int64_t nb, int64_t rowtiles, bool swiglu, int64_t n, int wtype = kTypeQ4K);
hipError_t launch_skinny16(const Skinny16Args& a, hipStream_t stream, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);

// ---- q8_0.hip --------------------------------------------------------------------------------
// Q8_0 weights (16-row tiles of common.h) x Q8_0 activations, dense, any n (passes of eight rows).
struct Q80MatmulArgs {
    const uint8_t* w = nullptr;    // tiled weights
    int64_t rows = 0;
    int64_t nb = 0;                // 256-weight groups per row (cols / 256)
    const uint8_t* aq = nullptr;   // A-major codes (the layout of the Q8_K codes)
    const uint16_t* ah = nullptr;  // fp16 d: eight per (row, group), at ad_index(row, group, nb) * 8
    int64_t n = 0;
    float* y = nullptr;            // [n][ldy]
    int64_t ldy = 0;
    int32_t* dbg_sum = nullptr;    // optional [rows][n][cols / 32] integer block sums
    // expert-routed mode (the MoE down node with Q8_0 experts): activation / output row g = token * slots + slot is
    // multiplied by expert pair_ids[token * top_k + slot] (slot < top_k) or by the shared expert sh_w (slot >= top_k);
    // n = tokens * slots rows; pairs with an id outside [0, n_experts) are skipped
    const int32_t* pair_ids = nullptr;
    int top_k = 0, slots = 0, n_experts = 0;
    size_t expert_bytes = 0;
    const uint8_t* sh_w = nullptr;
    // expert-grouped mode (the same node above eight tokens, where the pairs were sorted by expert): workgroup column g
    // is group g of the work list -- its expert's weights against the group's rows in passes of eight, so an expert is
    // streamed once per eight of its rows instead of once per row; columns past the groups are passes of the shared
    // expert (sh_w) over all tokens.  Rows as above: token * slots + slot.  pair_ids stays null.
    const int32_t* group_expert = nullptr;
    const int32_t* group_begin = nullptr;
    const int32_t* n_groups = nullptr;
    const int32_t* entry_token = nullptr;
    const int32_t* entry_k = nullptr;
    int max_groups = 0;
    int sh_tokens = 0;
};
size_t q80_scale_bytes(int64_t n, int64_t nb);
// x rows 16-byte aligned (ldx % 4 == 0), cols % 256 == 0
hipError_t launch_quantize_q80(const float* x, int64_t n, int64_t ldx, int64_t cols, uint8_t* aq, uint16_t* ah, hipStream_t stream);
hipError_t launch_q80_matmul(const Q80MatmulArgs& a, hipStream_t stream);

// ---- gemv1.hip -------------------------------------------------------------------------------
// One activation row, quantizer inside the kernel; applies when a wave sees at most two super-blocks.
bool gemv1_fused_applies(int64_t nb, int waves);
// Up to eight rows with the quantizer inside, optionally with the residual add and the RMSNorm of the rows as well
// (norm: delta, weight, eps, sum_out as in launch_add_rmsnorm; x rows then dense, ldx == cols).
hipError_t launch_gemvn_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, int64_t ldx, const float* delta,
                              const float* weight, float eps, float* sum_out, float* y, int64_t ldy, int n, bool norm, int waves,
                              hipStream_t stream);
// The same with the residual add and the RMSNorm of the row inside (sum_out apart from x and delta).
hipError_t launch_gemv1_norm_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, const float* delta,
                                   const float* weight, float eps, float* sum_out, float* y, int waves, hipStream_t stream);
// Several single-row GEMVs of one activation row in one launch (gemv1.hip): matrices of one column count, each
// with the wave split a launch of its own would take.
constexpr int kGemvMultiMax = 8;
struct Gemv1MultiArgs {
    const uint8_t* w[kGemvMultiMax] = {};
    float* y[kGemvMultiMax] = {};
    int64_t rows[kGemvMultiMax] = {};
    int rt_begin[kGemvMultiMax + 1] = {};  // filled by the launcher: first workgroup of matrix i
    int count = 0;
    int64_t nb = 0;
    const float* x = nullptr;
};
hipError_t launch_gemv1_multi(const Gemv1MultiArgs& a, int waves, hipStream_t stream);
hipError_t launch_gemv1_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, float* y, int waves,
                              hipStream_t stream);

// ---- prefill.hip -----------------------------------------------------------------------------
// fp32 rows -> Q8_K in the P-major layout of the prefill GEMM (pmajor_bytes(n, nb) bytes).
size_t pmajor_bytes(int64_t n, int64_t nb);
// plan (optional): the rows are an expert-grouped GEMM's tiles in the plan's order; tiles past the plan's count are skipped
hipError_t launch_quantize_q8k_pmajor(const float* x, int64_t n, int64_t ldx, int64_t k, uint8_t* ap,
                                      hipStream_t stream, const int32_t* plan = nullptr);
// The same for the rows silu(gate) * up (both [n][ldx]); h_out (may be null) receives them as fp32 [n][ldh] as well.
hipError_t launch_swiglu_quantize_q8k_pmajor(const float* gate, const float* up, int64_t n, int64_t ldx, int64_t k,
                                             int silu_mode, float* h_out, int64_t ldh, uint8_t* ap, hipStream_t stream);
// y[n][ldy] = P-major activations . tiled weights^T on the int8 matrix cores.  A launch that would leave workgroup
// slots empty splits K into runs of super-blocks whose sums go to planes of `part` (prefill_part_bytes() bytes, 0 when
// nothing is split) and are added in order by a second launch.
// wtype: kTypeQ4K, or kTypeQ5K (a third MFMA chain for the fifth code bits; 64-row workgroups).
size_t prefill_part_bytes(int64_t rows, int64_t nb, int64_t n, int wtype);
// silu(gate . x) * (up . x) from ONE launch (prefill.hip: the pair form of the GEMM kernel), dense and expert-grouped
bool prefill_pair_applies(int wtype, int64_t rows, int64_t nb, int64_t n);
hipError_t launch_prefill_gemm_pair(const uint8_t* gate, const uint8_t* up, int wtype, int64_t rows, int64_t nb, const uint8_t* ap,
                                    int64_t n, int silu_mode, float* h, int64_t ldh, hipStream_t stream);
hipError_t launch_prefill_gemm_grouped_pair(const uint8_t* gate, const uint8_t* up, int wtype, int64_t expert_bytes,
                                            const uint8_t* gate_shared, const uint8_t* up_shared, int64_t rows, int64_t nb,
                                            const uint8_t* ap, int64_t entries, int64_t groups_max, const int32_t* plan, bool scatter,
                                            int silu_mode, float* h, int64_t ldh, hipStream_t stream, int mt = 8);
hipError_t launch_prefill_gemm(const uint8_t* w, int wtype, int64_t rows, int64_t nb, const uint8_t* ap, int64_t n, float* y,
                               int64_t ldy, float* part, hipStream_t stream);

// Expert-grouped form of the GEMM (a MoE block at prefill widths): a plan lays the routed entries out in 16-row tiles
// per expert (moe_gemm_plan_ints() int32 of workspace; sizes from the upper bounds entries = n * top_k and groups_max),
// the quantizer gathers or forms the rows of those tiles, the GEMM multiplies every item by its expert's weights.
// sh_tokens > 0 appends the shared expert as one more group of all tokens (weights w_shared, output slot slots - 1);
// `entries` and `groups_max` then count its rows and its group as well.
int64_t moe_gemm_tiles_max(int64_t entries, int64_t groups_max);
int64_t moe_gemm_items_max(int64_t entries, int64_t groups_max);
size_t moe_gemm_plan_ints(int64_t entries, int64_t groups_max);
// activation tiles per item (2 or 8) of an expert-grouped launch over `entries` rows in `groups` groups: the plan and
// every launch that reads it take the same value
int moe_gemm_item_tiles(int64_t entries, int64_t groups);
hipError_t launch_moe_gemm_plan(const int32_t* n_groups, const int32_t* group_expert, const int32_t* group_begin,
                                const int32_t* entry_token, const int32_t* entry_k, int slots, bool src_per_slot, int64_t entries,
                                int64_t groups_max, int64_t sh_tokens, int sh_silu_mode, int32_t* plan, hipStream_t stream, int mt = 8);
hipError_t launch_quantize_q8k_pmajor_grouped(const float* x, const float* x2, bool swiglu, int silu_mode, int64_t ldx, int64_t k,
                                              int64_t entries, int64_t groups_max, const int32_t* plan, uint8_t* ap, float* h_out,
                                              int64_t ldh, hipStream_t stream, int64_t distinct_rows = 0,
                                              uint8_t* ap_rows = nullptr);
hipError_t launch_prefill_gemm_grouped(const uint8_t* w, int wtype, int64_t expert_bytes, const uint8_t* w_shared, int64_t rows,
                                       int64_t nb, const uint8_t* ap, int64_t entries, int64_t groups_max, const int32_t* plan,
                                       bool scatter, float* y, int64_t ldy, hipStream_t stream, int mt = 8);

// ---- elementwise.hip -------------------------------------------------------------------------
hipError_t launch_add_rmsnorm(const float* x, const float* delta, const float* weight, int64_t n, int64_t cols,
                              float eps, float* sum_out, float* normed_out, uint8_t* q_aq, float* q_ad,
                              hipStream_t stream);
// Residual add + RMSNorm + router projection in one launch (cols % 256 == 0, cols <= 4096; sum_out apart from x and delta).
hipError_t launch_add_rmsnorm_router(const float* x, const float* delta, const float* weight, int64_t n, int64_t cols, float eps,
                                     float* sum_out, float* normed_out, const float* w_router, int64_t n_experts, float* logits,
                                     hipStream_t stream);
hipError_t launch_router_logits(const float* w, int64_t n_experts, int64_t cols, const float* x, int64_t n, int64_t ldx,
                                float* logits, hipStream_t stream);
// out = silu(gate) * up over [n][cols] (mode: MQ_SILU_*), and out[t] = sigmoid(logit[t * ld_logit]) * src[t]
hipError_t launch_silu_mul(const float* gate, const float* up, int64_t n, int64_t cols, int64_t ld_gate, int64_t ld_up, float* out,
                           int64_t ld_out, int mode, hipStream_t stream);
hipError_t launch_scale_rows_sigmoid(const float* src, int64_t n, int64_t cols, int64_t ld_src, const float* logit, int64_t ld_logit,
                                     float* out, int64_t ld_out, hipStream_t stream);

// ---- router.hip ------------------------------------------------------------------------------
hipError_t launch_route_topk(const float* logits, int64_t n_experts, int64_t n, int top_k, int mode, int32_t* ids,
                             float* weights, hipStream_t stream);
// Expert-grouped work list from ids [n][top_k]: entries sorted by (expert, token, k).
//   group_expert[g], group_begin[g..g+1], n_groups[0], entry_token[e], entry_k[e]
hipError_t launch_weights_from_ids(const float* logits, int64_t n_experts, int64_t n, const int32_t* ids, int top_k,
                                   float* weights, hipStream_t stream);
hipError_t launch_build_groups(const int32_t* ids, int64_t n, int top_k, int64_t n_experts, int32_t* group_expert,
                               int32_t* group_begin, int32_t* n_groups, int32_t* entry_token, int32_t* entry_k,
                               hipStream_t stream);
// Router and grouping in one launch at decode widths (falls back to the two kernels above for n > 256).
hipError_t launch_route_and_group(const float* logits, int64_t n_experts, int64_t n, int top_k, int mode, int32_t* ids,
                                  float* weights, uint32_t* arrivals, int32_t* group_expert, int32_t* group_begin,
                                  int32_t* n_groups, int32_t* entry_token, int32_t* entry_k, bool build_groups, const float* qx,
                                  int64_t q_ldx, int64_t q_cols, uint8_t* q_aq, float* q_ad, hipStream_t stream);
// y[t][r] = sum_k w[t][k] * part[t*slots + k][r]  (k in order) + gate[t] * part[t*slots + top_k][r]
hipError_t launch_moe_combine(const float* part, int64_t n, int top_k, int slots, int64_t rows, const float* weights,
                              const int32_t* ids, int64_t n_experts, int has_shared, const float* sh_gate_inp,
                              const float* x, float* y, hipStream_t stream);
hipError_t launch_fill_zero(float* p, size_t count, hipStream_t stream);
// A measurement instrument (mq_debug_set_skeleton): while it is on, every launch of the compute and routing kernels
// is replaced by a kernel with an empty body and the same grid, block and LDS size -- a captured graph then has the
// dependent launches of the real one and none of their work, which is what the launches alone cost.  Weight set-up
// and launches that carry timing events are not replaced.
extern int g_skeleton;
hipError_t launch_skeleton(dim3 grid, dim3 block, size_t lds, hipStream_t stream);
#define MQ_LAUNCH(kernel, grid, block, lds, stream, ...)                            \
    do {                                                                            \
        if (::mq::g_skeleton) (void)::mq::launch_skeleton(grid, block, lds, stream); \
        else hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);     \
    } while (0)

// The work list written out as (expert, token, k) triples in list order, and the number of entries.
hipError_t launch_flatten_groups(const int32_t* group_expert, const int32_t* group_begin, const int32_t* n_groups,
                                 const int32_t* entry_token, const int32_t* entry_k, int max_entries, int32_t* triples,
                                 int32_t* count, hipStream_t stream);

// ---- moe_down.hip ----------------------------------------------------------------------------
// Down projection + weighted combine, one workgroup per (token, 16 output rows): for decode widths, where
// grouping by expert shares nothing.  Hidden rows (row = token * slots + slot) are Q8_K in the A-major layout or fp32.
struct MoeDownTokenArgs {
    const uint8_t* w = nullptr;        // tiled down experts [n_experts][rows x nb]
    size_t expert_bytes = 0;
    const uint8_t* sh_w = nullptr;     // shared expert's down matrix or null; its hidden row is slot top_k
    int wtype = 12;
    int64_t rows = 0, nb = 0;          // output rows (hidden), super-blocks per row (inter / 256)
    int64_t n = 0;
    int top_k = 0, n_experts = 0;
    uint32_t inv_nb = 0;               // ceil(2^32 / nb) for nb > 1, filled in by the launcher: i / nb == umulhi(i, inv_nb) for i, nb < 2^16
    uint32_t inv_items = 0;            // the same for slots * nb (> 1)
    int rt_per_wg = 1;                 // row tiles of one token per workgroup (launcher)
    const uint8_t* aq = nullptr;       // A-major hidden rows, or
    const float* ad = nullptr;
    const float* hidden = nullptr;     // fp32 hidden rows [n * slots][nb * 256] (quantized inside the kernel)
    const int32_t* ids = nullptr;      // [n][top_k]
    const float* weights = nullptr;    // [n][top_k]
    const float* sh_gate_inp = nullptr;  // [rows] or null (gate = 1)
    const float* x = nullptr;          // [n][rows]: the MoE block's input, for the gate
    float* y = nullptr;                // [n][rows]
};
hipError_t launch_moe_down_token(const MoeDownTokenArgs& a, hipStream_t stream);
// LDS that launch takes for `slots` hidden rows per token of nb super-blocks, and the most it may take: the one
// predicate of the launcher and of the callers that choose between it and the expert-grouped launches.
size_t moe_down_token_lds_bytes(int slots, int64_t nb);
constexpr size_t kMoeDownTokenMaxLds = 48 * 1024;

// ---- moe_gateup.hip --------------------------------------------------------------------------
// Gate/up + SwiGLU with the router and the Q8_K of the layer input inside, one workgroup per (token, slot,
// 16 hidden rows): decode widths, where neither grouping by expert nor separate routing / quantizing launches pay.
struct MoeGateupTokenArgs {
    const uint8_t* gate = nullptr;     // tiled experts [n_experts][rows x nb]
    const uint8_t* up = nullptr;
    size_t expert_bytes = 0;
    const uint8_t* sh_gate = nullptr;  // shared expert (both or neither); its hidden row is slot top_k
    const uint8_t* sh_up = nullptr;
    int wtype = 12;
    int64_t rows = 0, nb = 0;          // hidden rows per expert (inter), super-blocks per row (hidden / 256)
    int64_t n = 0;
    int top_k = 0, n_experts = 0;      // n_experts <= 512
    int route_mode = 0, silu_mode = 0, sh_silu_mode = 2;
    int waves = 1;                     // wavefronts per workgroup: moe_gateup_token_waves(); nb % waves == 0
    int stages = 0;                    // nb / waves, filled in by the launcher (the kernel makes no division)
    int slots_per_wg = 0;              // moe_gateup_slots_kernel: slots (wavefronts) of one workgroup, filled in by the launcher
    const float* x = nullptr;          // [n][nb * 256]
    const float* logits = nullptr;     // [n][n_experts]
    float* hidden = nullptr;           // [n * slots][rows]
    int32_t* ids_out = nullptr;        // [n][top_k]
    float* weights_out = nullptr;      // [n][top_k]
};
hipError_t launch_moe_gateup_token(const MoeGateupTokenArgs& a, hipStream_t stream);
// Wavefronts per workgroup for that launch (rows = hidden rows per expert), and the wavefronts the chip holds of it.
int moe_gateup_token_waves(int64_t nb, int64_t rows, int64_t n, int slots, int wtype);
int moe_gateup_token_capacity(int wtype);
int moe_gateup_slots_capacity(int wtype);

// ---- decoder_layers.hip ----------------------------------------------------------------------
// A run of MoE decoder layers at decode width as one persistent launch (one workgroup per compute unit,
// device-wide barriers between the phases of a layer).  All weights are Q4_K in the tiled layout.
constexpr int kDecoderMaxExperts = 512;
constexpr int kTokenMajorDownMaxTokens = 8;  // widest MoE block whose down projection runs token-major (measured: 16 loses)
constexpr int kDirectPairsMaxTokens = 8;  // widest MoE block whose (token, slot) pairs are not grouped by expert (measured: 16 loses)
struct DecoderLayerDev {               // one per layer, in device memory
    const uint8_t* wqkv = nullptr;     // [qkv_rows x hidden]
    const uint8_t* wo = nullptr;       // [hidden x n_q]; its input is qkv[:, :n_q]
    int64_t qkv_rows = 0;
    const float* attn_norm = nullptr;  // [hidden] or null (ones)
    const float* ffn_norm = nullptr;
    const float* router = nullptr;     // fp32 [n_experts x hidden]
    const float* fixed_logits = nullptr;  // fp32 [n x n_experts] or null: route on these instead of router . h2
    const uint8_t* gate_exps = nullptr;
    const uint8_t* up_exps = nullptr;
    const uint8_t* down_exps = nullptr;
    size_t gu_expert_bytes = 0, down_expert_bytes = 0;
    const uint8_t* sh_gate = nullptr;  // shared expert (all three or none, as DecoderArgs::has_shared says)
    const uint8_t* sh_up = nullptr;
    const uint8_t* sh_down = nullptr;
    const float* sh_gate_inp = nullptr;  // fp32 [hidden] or null (gate = 1)
};
struct DecoderArgs {
    const DecoderLayerDev* layers = nullptr;  // device table
    int n_layers = 0;
    int n = 0;                         // tokens, 1..8
    int hidden = 0, inter = 0, n_q = 0, n_experts = 0, top_k = 0;
    int has_shared = 0;
    int silu_mode = 0, route_mode = 0;
    int gateup_order = 8;              // wavefronts per row tile of the one-node expert gate/up launch at this width (pick_waves)
    float eps = 0.0f;
    long long spin_ticks = 0;          // barrier patience in wall_clock64 ticks
    const float* x_in = nullptr;       // [n x hidden]
    float* out = nullptr;              // [n x hidden]
    float* qkv = nullptr;              // exchange buffers: [n x qkv_rows]
    float* o = nullptr;                // [n x hidden]
    float* logits = nullptr;           // [n x n_experts]
    float* mid = nullptr;              // [n x (top_k + has_shared) x inter]
    float* y = nullptr;                // [n x hidden]
    int32_t* ids_out = nullptr;        // optional [n_layers x n x top_k]
    float* wts_out = nullptr;
    uint32_t* sync = nullptr;          // decoder_sync_bytes(), zero before the first launch
};
size_t decoder_layers_lds_bytes(const DecoderArgs& a);
size_t decoder_sync_bytes(int n_workgroups);
hipError_t prepare_decoder_layers(size_t lds_bytes);
hipError_t launch_decoder_layers(const DecoderArgs& a, int n_workgroups, hipStream_t stream);

}  // namespace mq
