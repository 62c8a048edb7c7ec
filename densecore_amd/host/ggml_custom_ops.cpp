// GGML_OP_CUSTOM adapters and the library-level quantized matmul over the mi355_q4k C ABI.
// Host-only C++ (no HIP headers): every GPU action goes through libmi355q4k.so.
//
// Each adapter mirrors the operand conventions and the rejection behaviour of the DenseCore
// callback it replaces (cited at each function); none of them owns or frees graph memory.
#include "mi355_q4k_ggml.h"

#include <cstdio>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "ggml_tensor_mirror.h"
#include "mi355_q4k.h"

namespace {

constexpr int64_t kSuperBlock = 256;
constexpr size_t kQ4KBlockBytes = 144;
constexpr size_t kQ5KBlockBytes = 176;
constexpr size_t kQ6KBlockBytes = 210;
// block bytes of a weight type this library multiplies, 0 for any other
constexpr size_t kquant_block_bytes(int type) {
    return type == (int)GGML_TYPE_Q4_K   ? kQ4KBlockBytes
           : type == (int)GGML_TYPE_Q5_K ? kQ5KBlockBytes
           : type == (int)GGML_TYPE_Q6_K ? kQ6KBlockBytes
                                         : 0;
}

thread_local int t_status = MQ_OK;

int note(int rc) {
    t_status = rc;
    return rc;
}

// ---- device weight cache ---------------------------------------------------------------------
// Keyed by the host data pointer; shape and strides are compared on every hit so that a graph
// arena which reuses an address for another tensor is re-uploaded rather than mis-read.
struct CachedWeight {
    mq_weight* handle = nullptr;
    int type = -1;
    int64_t ne[3] = {0, 0, 0};
    size_t nb[3] = {0, 0, 0};
};
std::mutex g_cache_mu;
std::unordered_map<const void*, CachedWeight> g_cache;

// A dense Q8_0 matrix (34-byte blocks of 32 weights, core/src/llm/matmul/q8_small_batch.h:9-14) whose rows hold
// whole groups of 256 weights: the dense callback and the library entry take it, the MoE callbacks do not.
constexpr size_t kQ80BlockBytes = 34;
bool is_q80_matrix(const ggml_tensor* w) {
    return w && w->data && (int)w->type == (int)GGML_TYPE_Q8_0 && w->ne[0] > 0 && w->ne[0] % kSuperBlock == 0 && w->ne[1] > 0 &&
           w->ne[2] == 1 && w->ne[3] == 1 && w->nb[0] == kQ80BlockBytes && w->nb[1] >= (size_t)(w->ne[0] / 32) * kQ80BlockBytes;
}

// Q4_K, Q5_K or Q6_K rows of whole super-blocks (the K-quant weight types of the callbacks replaced:
// core/src/llm/moe/native.cpp:2745-2752, core/src/backend/cpu_backend_moe_raw_batched.inl:1552)
bool is_kquant_matrix(const ggml_tensor* w) {
    if (!w || !w->data) return false;
    const size_t bb = kquant_block_bytes((int)w->type);
    return bb != 0 && w->ne[0] > 0 && w->ne[0] % kSuperBlock == 0 && w->ne[1] > 0 && w->ne[2] > 0 && w->ne[3] == 1 &&
           w->nb[0] == bb && w->nb[1] >= (size_t)(w->ne[0] / kSuperBlock) * bb;
}

const mq_weight* device_weight(const void* data, int type, int64_t cols, int64_t rows, int64_t n_experts,
                               size_t row_bytes, size_t expert_bytes) {
    std::lock_guard<std::mutex> lock(g_cache_mu);
    CachedWeight& slot = g_cache[data];
    const bool same = slot.handle && slot.type == type && slot.ne[0] == cols && slot.ne[1] == rows && slot.ne[2] == n_experts &&
                      slot.nb[1] == row_bytes && slot.nb[2] == expert_bytes;
    if (same) return slot.handle;
    if (slot.handle) mq_weight_free(slot.handle);
    slot = CachedWeight{};
    mq_weight* h = nullptr;
    if (note(mq_weight_upload_typed(type, data, rows, cols, n_experts, row_bytes, expert_bytes, &h)) != MQ_OK) {
        g_cache.erase(data);
        return nullptr;
    }
    slot.handle = h;
    slot.type = type;
    slot.ne[0] = cols, slot.ne[1] = rows, slot.ne[2] = n_experts;
    slot.nb[1] = row_bytes, slot.nb[2] = expert_bytes;
    return h;
}

const mq_weight* device_weight(const ggml_tensor* w) {
    return device_weight(w->data, (int)w->type, w->ne[0], w->ne[1], w->ne[2], w->nb[1],
                         w->ne[2] > 1 ? w->nb[2] : w->nb[1] * w->ne[1]);
}

// ---- per-thread staging in HBM -------------------------------------------------------------------
// Grow-only device buffers for the host<->device hops of one node; a thread's buffers are reused
// by its next call (callbacks of one graph run one node at a time per ggml thread 0).
struct Staging {
    void* ptr = nullptr;
    size_t cap = 0;
    void* get(size_t bytes) {
        if (bytes <= cap) return ptr;
        if (ptr) mq_device_free(ptr);
        ptr = nullptr, cap = 0;
        const size_t want = bytes + bytes / 2 + 4096;
        if (note(mq_device_malloc(&ptr, want)) != MQ_OK) return nullptr;
        cap = want;
        return ptr;
    }
    ~Staging() {
        if (ptr) mq_device_free(ptr);
    }
};
struct ThreadStage {
    Staging in, aux, ids, wts, out;
};
thread_local ThreadStage t_stage;

// Copies a strided host matrix [rows][cols] of 4-byte elements (row stride in bytes) into a dense
// device matrix.  Dense sources go in one copy.
int upload_rows(void* dst_dev, const void* src_host, int64_t rows, int64_t cols, size_t row_stride_bytes) {
    const size_t row_bytes = (size_t)cols * 4;
    if (row_stride_bytes == row_bytes || rows == 1) return mq_memcpy_h2d(dst_dev, src_host, row_bytes * (size_t)rows);
    for (int64_t r = 0; r < rows; ++r) {
        const int rc = mq_memcpy_h2d((char*)dst_dev + (size_t)r * row_bytes,
                                     (const char*)src_host + (size_t)r * row_stride_bytes, row_bytes);
        if (rc != MQ_OK) return rc;
    }
    return MQ_OK;
}

int download_rows(void* dst_host, const void* src_dev, int64_t rows, int64_t cols, size_t row_stride_bytes) {
    const size_t row_bytes = (size_t)cols * 4;
    if (row_stride_bytes == row_bytes || rows == 1) return mq_memcpy_d2h(dst_host, src_dev, row_bytes * (size_t)rows);
    for (int64_t r = 0; r < rows; ++r) {
        const int rc = mq_memcpy_d2h((char*)dst_host + (size_t)r * row_stride_bytes,
                                     (const char*)src_dev + (size_t)r * row_bytes, row_bytes);
        if (rc != MQ_OK) return rc;
    }
    return MQ_OK;
}

struct Options {
    int silu_mode;
    int route_mode;
    mq_ggml_userdata* ud;
};

Options options_for(void* userdata, int64_t n_tokens) {
    auto* ud = static_cast<mq_ggml_userdata*>(userdata);
    Options o;
    // decode widths use the exact exponential, wider batches the polynomial one
    // (core/src/llm/moe/native.cpp:3614-3616, core/src/backend/cpu_backend_moe_raw_batched.inl:1673)
    o.silu_mode = n_tokens <= 4 ? MQ_SILU_EXACT : MQ_SILU_FAST;
    o.route_mode = MQ_ROUTE_FLOOR;
    o.ud = ud;
    if (ud && !ud->use_defaults) {
        o.silu_mode = ud->silu_mode;
        o.route_mode = ud->route_mode;
    }
    return o;
}

void finish(const Options& o, int rc) {
    note(rc);
    if (o.ud) o.ud->last_status = rc;
    if (rc != MQ_OK) std::fprintf(stderr, "mi355_q4k adapter: %s\n", mq_last_error());
}

// Dense node: y[M][N_out] = W . q8k(x[M]).
void dense_node(ggml_tensor* dst, int ith, void* userdata) {
    if (ith != 0 || !dst) return;
    const ggml_tensor* src = dst->src[0];
    const ggml_tensor* weight = dst->src[1];
    Options o = options_for(userdata, 1);
    if (!src || !weight || !src->data || !dst->data) return finish(o, MQ_ERR_INVALID);
    if ((!is_kquant_matrix(weight) && !is_q80_matrix(weight)) || weight->ne[2] != 1) return finish(o, MQ_ERR_UNSUPPORTED);
    const int64_t k_in = weight->ne[0], n_out = weight->ne[1];
    const int64_t m = src->ne[1] * src->ne[2] * src->ne[3];
    // the reference leaves dst untouched on a shape mismatch (core/src/llm/matmul/gemv_exec.cpp:131-143)
    if (src->type != GGML_TYPE_F32 || dst->type != GGML_TYPE_F32 || src->ne[0] != k_in || dst->ne[0] != n_out ||
        dst->ne[1] * dst->ne[2] * dst->ne[3] != m || src->nb[0] != 4 || dst->nb[0] != 4 || m <= 0)
        return finish(o, MQ_ERR_INVALID);
    if ((src->ne[2] > 1 && src->nb[2] != src->nb[1] * (size_t)src->ne[1]) ||
        (dst->ne[2] > 1 && dst->nb[2] != dst->nb[1] * (size_t)dst->ne[1]))
        return finish(o, MQ_ERR_UNSUPPORTED);
    const mq_weight* w = device_weight(weight);
    if (!w) return finish(o, t_status);
    float* x_dev = (float*)t_stage.in.get((size_t)m * k_in * 4);
    float* y_dev = (float*)t_stage.out.get((size_t)m * n_out * 4);
    if (!x_dev || !y_dev) return finish(o, t_status);
    int rc = upload_rows(x_dev, src->data, m, k_in, src->nb[1]);
    if (rc == MQ_OK) rc = mq_mul_mat_q4k(w, x_dev, m, k_in, y_dev, n_out, nullptr);
    if (rc == MQ_OK) rc = download_rows(dst->data, y_dev, m, n_out, dst->nb[1]);  // blocking copy = synchronisation
    finish(o, rc);
}

// selected_experts I32 ne=[top_k, n_tokens] -> dense device [n_tokens][top_k]
int upload_ids(const ggml_tensor* sel, int32_t** ids_dev) {
    const int64_t top_k = sel->ne[0], n = sel->ne[1];
    *ids_dev = (int32_t*)t_stage.ids.get((size_t)n * top_k * 4);
    if (!*ids_dev) return t_status;
    if (sel->nb[0] == 4) return upload_rows(*ids_dev, sel->data, n, top_k, sel->nb[1]);
    std::vector<int32_t> dense((size_t)n * top_k);  // element stride other than 4 bytes: gather on the host
    for (int64_t t = 0; t < n; ++t)
        for (int64_t k = 0; k < top_k; ++k)
            std::memcpy(&dense[(size_t)(t * top_k + k)], (const char*)sel->data + t * sel->nb[1] + k * sel->nb[0], 4);
    return mq_memcpy_h2d(*ids_dev, dense.data(), dense.size() * 4);
}

}  // namespace

extern "C" {

void mq_cb_gemv_custom(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) { dense_node(dst, ith, userdata); }

void mq_cb_gemv_batched_custom(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) {
    dense_node(dst, ith, userdata);
}

void mq_cb_moe_gateup_swiglu(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) {
    if (ith != 0 || !dst) return;
    const ggml_tensor* gate = dst->src[0];
    const ggml_tensor* up = dst->src[1];
    const ggml_tensor* input = dst->src[2];
    const ggml_tensor* sel = dst->src[3];
    Options o = options_for(userdata, sel ? sel->ne[1] : 1);
    if (!gate || !up || !input || !sel || !input->data || !sel->data || !dst->data) return finish(o, MQ_ERR_INVALID);
    if (!is_kquant_matrix(gate) || !is_kquant_matrix(up) || gate->type != up->type) return finish(o, MQ_ERR_UNSUPPORTED);
    const int64_t n_embd = gate->ne[0], n_ff = gate->ne[1], n_expert = gate->ne[2];
    const int64_t top_k = sel->ne[0], n = sel->ne[1];
    // operand checks of core/src/llm/moe/native.cpp:3935-3990
    if (up->ne[0] != n_embd || up->ne[1] != n_ff || up->ne[2] != n_expert || input->type != GGML_TYPE_F32 ||
        input->ne[0] != n_embd || input->ne[1] * input->ne[2] != n || sel->type != GGML_TYPE_I32 ||
        dst->type != GGML_TYPE_F32 || dst->ne[0] != n_ff || dst->ne[1] != top_k || dst->ne[2] != n || top_k <= 0 ||
        top_k > 8 || n <= 0 || input->nb[0] != 4 || dst->nb[0] != 4)
        return finish(o, MQ_ERR_INVALID);
    const mq_weight* wg = device_weight(gate);
    const mq_weight* wu = wg ? device_weight(up) : nullptr;
    if (!wg || !wu) return finish(o, t_status);
    float* x_dev = (float*)t_stage.in.get((size_t)n * n_embd * 4);
    float* h_dev = (float*)t_stage.out.get((size_t)n * top_k * n_ff * 4);
    int32_t* ids_dev = nullptr;
    if (!x_dev || !h_dev) return finish(o, t_status);
    const size_t x_stride = input->ne[1] == n ? input->nb[1] : input->nb[2];
    int rc = upload_rows(x_dev, input->data, n, n_embd, x_stride);
    if (rc == MQ_OK) rc = upload_ids(sel, &ids_dev);
    if (rc == MQ_OK) rc = mq_moe_gateup_swiglu_q4k(wg, wu, x_dev, n, ids_dev, (int)top_k, o.silu_mode, h_dev, nullptr);
    if (rc == MQ_OK) {
        // dst may be a strided view (core/src/llm/moe/native.cpp:4201-4209): rows are (token, k) pairs
        if (dst->nb[2] == dst->nb[1] * (size_t)top_k) {
            rc = download_rows(dst->data, h_dev, n * top_k, n_ff, dst->nb[1]);
        } else {
            for (int64_t t = 0; t < n && rc == MQ_OK; ++t)
                rc = download_rows((char*)dst->data + t * dst->nb[2], h_dev + (size_t)t * top_k * n_ff, top_k, n_ff,
                                   dst->nb[1]);
        }
    }
    finish(o, rc);
}

void mq_cb_moe_down_weighted_logits(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) {
    if (ith != 0 || !dst) return;
    const ggml_tensor* down = dst->src[0];
    const ggml_tensor* hidden = dst->src[1];
    const ggml_tensor* sel = dst->src[2];
    const ggml_tensor* logits = dst->src[3];
    Options o = options_for(userdata, sel ? sel->ne[1] : 1);
    if (!down || !hidden || !sel || !logits || !hidden->data || !sel->data || !logits->data || !dst->data)
        return finish(o, MQ_ERR_INVALID);
    if (!is_kquant_matrix(down)) return finish(o, MQ_ERR_UNSUPPORTED);
    const int64_t n_ff = down->ne[0], n_embd = down->ne[1], n_expert = down->ne[2];
    const int64_t top_k = sel->ne[0], n = sel->ne[1];
    // operand checks of core/src/llm/moe/native.cpp:3060-3120 and :2309-2317
    if (hidden->type != GGML_TYPE_F32 || hidden->ne[0] != n_ff || hidden->ne[1] != top_k || hidden->ne[2] != n ||
        sel->type != GGML_TYPE_I32 || logits->type != GGML_TYPE_F32 || logits->ne[0] != n_expert ||
        logits->ne[1] != n || dst->type != GGML_TYPE_F32 || dst->ne[0] != n_embd || dst->ne[1] != n || top_k <= 0 ||
        top_k > 8 || n <= 0 || hidden->nb[0] != 4 || logits->nb[0] != 4 || dst->nb[0] != 4)
        return finish(o, MQ_ERR_INVALID);
    const mq_weight* wd = device_weight(down);
    if (!wd) return finish(o, t_status);
    float* h_dev = (float*)t_stage.in.get((size_t)n * top_k * n_ff * 4);
    float* l_dev = (float*)t_stage.aux.get((size_t)n * n_expert * 4);
    float* w_dev = (float*)t_stage.wts.get((size_t)n * top_k * 4);
    float* y_dev = (float*)t_stage.out.get((size_t)n * n_embd * 4);
    int32_t* ids_dev = nullptr;
    if (!h_dev || !l_dev || !w_dev || !y_dev) return finish(o, t_status);
    int rc = MQ_OK;
    if (hidden->nb[2] == hidden->nb[1] * (size_t)top_k) {
        rc = upload_rows(h_dev, hidden->data, n * top_k, n_ff, hidden->nb[1]);
    } else {
        for (int64_t t = 0; t < n && rc == MQ_OK; ++t)
            rc = upload_rows(h_dev + (size_t)t * top_k * n_ff, (const char*)hidden->data + t * hidden->nb[2], top_k,
                             n_ff, hidden->nb[1]);
    }
    if (rc == MQ_OK) rc = upload_rows(l_dev, logits->data, n, n_expert, logits->nb[1]);
    if (rc == MQ_OK) rc = upload_ids(sel, &ids_dev);
    if (rc == MQ_OK) rc = mq_moe_weights_from_logits(l_dev, n_expert, n, ids_dev, (int)top_k, w_dev, nullptr);
    if (rc == MQ_OK) rc = mq_moe_down_weighted_q4k(wd, h_dev, n, ids_dev, w_dev, (int)top_k, y_dev, nullptr);
    if (rc == MQ_OK) rc = download_rows(dst->data, y_dev, n, n_embd, dst->nb[1]);
    finish(o, rc);
}

int mq_ggml_last_status(void) { return t_status; }

int mq_ggml_weight_cache_clear(void) {
    std::lock_guard<std::mutex> lock(g_cache_mu);
    int rc = MQ_OK;
    for (auto& kv : g_cache)
        if (kv.second.handle) {
            const int r = mq_weight_free(kv.second.handle);
            if (r != MQ_OK) rc = r;
        }
    g_cache.clear();
    return rc;
}

int64_t mq_ggml_weight_cache_size(void) {
    std::lock_guard<std::mutex> lock(g_cache_mu);
    return (int64_t)g_cache.size();
}

int mq_matmul_ggml_quantized_transb(const float* a, int64_t m, int64_t k, int64_t lda, const void* w_data,
                                    int32_t w_type_id, int64_t w_rows, int64_t w_cols, size_t w_row_bytes, float* c,
                                    int64_t ldc) {
    // rejection rules of MatMulGgmlQuantizedTransBWithPath
    // (core/src/backend/cpu_backend_quantized_matmul.cpp:150-163), narrowed to Q4_K, Q5_K, Q6_K and Q8_0
    const size_t group_bytes = w_type_id == (int)GGML_TYPE_Q8_0 ? 8 * kQ80BlockBytes : kquant_block_bytes(w_type_id);
    if (!a || !w_data || !c || m <= 0 || w_rows <= 0 || w_cols <= 0 || k != w_cols || lda < k || ldc < w_rows ||
        group_bytes == 0 || w_cols % kSuperBlock != 0 || w_row_bytes != (size_t)(w_cols / kSuperBlock) * group_bytes) {
        note(MQ_ERR_INVALID);
        return 0;
    }
    const mq_weight* w = device_weight(w_data, w_type_id, w_cols, w_rows, 1, w_row_bytes, w_row_bytes * (size_t)w_rows);
    if (!w) return 0;
    return note(mq_mul_mat_q4k_host(w, a, m, lda, c, ldc)) == MQ_OK ? 1 : 0;
}

}  // extern "C"
