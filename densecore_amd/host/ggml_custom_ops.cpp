// GGML_OP_CUSTOM adapters and the library-level quantized matmul over the mi355_q4k C ABI.
// Host-only C++ (no HIP headers): every GPU action goes through libmi355q4k.so.
//
// Each adapter mirrors the operand conventions and the rejection behaviour of the DenseCore
// callback it replaces (cited at each function); none of them owns or frees graph memory.
#include "mi355_q4k_ggml.h"

#include <cstdio>
#include <cstring>
#include <memory>
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
// Keyed by the host data pointer; type, shape, strides AND a fingerprint of the bytes are compared on every hit, so
// that an address which now holds other weights (a reloaded model, an mmap reused for another file, a graph arena
// that recycled the slot) is re-uploaded rather than answered from stale HBM tiles.
struct CachedWeight {
    mq_weight* handle = nullptr;
    int type = -1;
    int64_t ne[3] = {0, 0, 0};
    size_t nb[3] = {0, 0, 0};
    uint64_t fingerprint = 0;
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
// core/src/llm/moe/native.cpp:4611-4620, core/src/backend/cpu_backend_moe_raw_batched.inl:1552)
bool is_kquant_matrix(const ggml_tensor* w) {
    if (!w || !w->data) return false;
    const size_t bb = kquant_block_bytes((int)w->type);
    return bb != 0 && w->ne[0] > 0 && w->ne[0] % kSuperBlock == 0 && w->ne[1] > 0 && w->ne[2] > 0 && w->ne[3] == 1 &&
           w->nb[0] == bb && w->nb[1] >= (size_t)(w->ne[0] / kSuperBlock) * bb;
}

// Content key of a tensor: the byte count, the first and the last 4 KiB and 64 sixteen-byte samples spread evenly
// between them, mixed eight bytes at a time through four independent multiply-xor streams (a byte-serial hash of
// these 9 KB would cost more than the node's kernel) -- cheap enough for every node, and any reload that changes the
// header blocks, the tail or one of the samples changes the key.  The reference keys its prepared weights the same
// way, by content (FingerprintQ4KRepackedGemvWeight, core/src/kernels/q4k_repacked_gemv.cpp:353-393: length + first
// and last window; core/tests/runtime/test_q4k_fingerprint.cpp).  0 only for an empty input.
uint64_t fingerprint_bytes(const void* data, size_t bytes) {
    if (!data || bytes == 0) return 0;
    const auto* p = static_cast<const uint8_t*>(data);
    constexpr uint64_t kMul[4] = {0x9E3779B97F4A7C15ull, 0xC2B2AE3D27D4EB4Full, 0x165667B19E3779F9ull, 0xD6E8FEB86659FD93ull};
    uint64_t lane[4] = {bytes, ~(uint64_t)bytes, bytes * kMul[0], bytes ^ kMul[1]};
    uint64_t position = 0;  // words mixed so far: equal words at different places give different keys
    auto mix = [&](const uint8_t* q, size_t n) {
        size_t i = 0;
        for (; i + 8 <= n; i += 8, ++position) {
            uint64_t w;
            std::memcpy(&w, q + i, 8);  // any alignment
            uint64_t& l = lane[position & 3];
            l = (l ^ w ^ position) * kMul[position & 3];
            l ^= l >> 29;
        }
        if (i < n) {
            uint64_t w = 0;
            std::memcpy(&w, q + i, n - i);
            w |= (uint64_t)(n - i) << 56;
            uint64_t& l = lane[position & 3];
            l = (l ^ w ^ position) * kMul[position & 3];
            l ^= l >> 29;
            ++position;
        }
    };
    constexpr size_t kWindow = 4096, kSamples = 64, kSampleBytes = 16;
    if (bytes <= 2 * kWindow) {
        mix(p, bytes);
    } else {
        mix(p, kWindow);
        const size_t inner = bytes - 2 * kWindow;
        if (inner >= kSamples * kSampleBytes) {
            const size_t step = inner / kSamples;
            for (size_t i = 0; i < kSamples; ++i) mix(p + kWindow + i * step, kSampleBytes);
        } else {
            mix(p + kWindow, inner);
        }
        mix(p + bytes - kWindow, kWindow);
    }
    uint64_t h = 0;
    for (int i = 0; i < 4; ++i) {
        h = (h ^ lane[i]) * kMul[(i + 1) & 3];
        h ^= h >> 32;
    }
    return h ? h : 1;
}

const mq_weight* device_weight(const void* data, int type, int64_t cols, int64_t rows, int64_t n_experts,
                               size_t row_bytes, size_t expert_bytes) {
    // bytes the tensor spans in host memory (strided rows and experts included)
    const size_t span = (size_t)(n_experts - 1) * expert_bytes + (size_t)(rows - 1) * row_bytes +
                        (size_t)(cols / (type == (int)GGML_TYPE_Q8_0 ? 32 : kSuperBlock)) *
                            (type == (int)GGML_TYPE_Q8_0 ? 34 : kquant_block_bytes(type));
    const uint64_t fp = fingerprint_bytes(data, span);
    std::lock_guard<std::mutex> lock(g_cache_mu);
    CachedWeight& slot = g_cache[data];
    const bool same = slot.handle && slot.type == type && slot.ne[0] == cols && slot.ne[1] == rows && slot.ne[2] == n_experts &&
                      slot.nb[1] == row_bytes && slot.nb[2] == expert_bytes && slot.fingerprint == fp;
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
    slot.fingerprint = fp;
    return h;
}

const mq_weight* device_weight(const ggml_tensor* w) {
    return device_weight(w->data, (int)w->type, w->ne[0], w->ne[1], w->ne[2], w->nb[1],
                         w->ne[2] > 1 ? w->nb[2] : w->nb[1] * w->ne[1]);
}

// ---- per-thread staging ---------------------------------------------------------------------------
// Grow-only device buffers for the operands of one node, each with a page-locked host twin: graph tensors live in
// pageable memory, so a row is first copied into the pinned twin (a strided tensor is gathered on the way), then
// all copies and kernels of the node are queued asynchronously on the null stream and the node synchronises ONCE,
// before it scatters its result into dst.  A thread's buffers are reused by its next call (callbacks of one graph
// run one node at a time on ggml thread 0).
struct Staging {
    void* dev = nullptr;
    void* pin = nullptr;
    size_t cap = 0;
    bool get(size_t bytes) {
        if (bytes <= cap) return true;
        release();
        const size_t want = bytes + bytes / 2 + 4096;
        if (note(mq_device_malloc(&dev, want)) != MQ_OK) return false;
        if (note(mq_host_malloc(&pin, want)) != MQ_OK) {
            mq_device_free(dev);
            dev = nullptr;
            return false;
        }
        cap = want;
        return true;
    }
    void release() {
        if (dev) mq_device_free(dev);
        if (pin) mq_host_free(pin);
        dev = pin = nullptr;
        cap = 0;
    }
    ~Staging() { release(); }
};
struct ThreadStage {
    Staging in, aux, ids, wts, out, keep;
    // the down node's own buffers for what it uploads: with the hand-over the gate/up node returns while the copies
    // out of its pinned twins (in, ids) are still queued, so the node after it must not write those twins
    Staging in2, ids2;
};
thread_local ThreadStage t_stage;

// The gate/up node's result left on the device for the down node of the same graph (mq_ggml_userdata::
// keep_hidden_on_device): which host tensor it stands for, and its shape.
struct Resident {
    const void* host = nullptr;
    int64_t n_ff = 0, top_k = 0, n = 0;
};
thread_local Resident t_resident;
// True between a gate/up node that handed its rows over (and returned without waiting) and the next synchronisation
// of this thread: the pinned twins of `in` and `ids` may still be read by queued copies.
thread_local bool t_unsettled = false;

// Every node but the down node of a hand-over starts here: if the previous node left copies queued, wait for them
// before this node writes the same pinned twins (a graph whose gate/up node is not followed by its down node).
// Dense nodes and the element-wise nodes upload through a ring of four pinned twins, so that a short run of nodes that
// leave their results on the device (gate, up, silu * up, down of a dense FFN) queues its uploads without waiting for
// one another; a twin is written again only after a synchronisation has passed since its last upload.
constexpr int kInRing = 4;
struct InRing {
    Staging slot[kInRing];
    bool dirty[kInRing] = {false, false, false, false};
    int next = 0;
};
thread_local InRing t_ring;

void settle() {
    bool any = t_unsettled;
    for (int i = 0; i < kInRing; ++i) any = any || t_ring.dirty[i];
    if (!any) return;
    (void)mq_stream_synchronize(nullptr);
    t_unsettled = false;
    for (int i = 0; i < kInRing; ++i) t_ring.dirty[i] = false;
}
void settled_by_sync() {  // the caller has just synchronised the null stream
    t_unsettled = false;
    for (int i = 0; i < kInRing; ++i) t_ring.dirty[i] = false;
}
// the next twin of the ring, free to be written (waits for the queued copies only when the ring has gone round)
Staging* ring_slot(size_t bytes) {
    const int i = t_ring.next;
    t_ring.next = (i + 1) % kInRing;
    if (t_ring.dirty[i] || bytes > t_ring.slot[i].cap) settle();  // growing a twin frees it: nothing may still read it
    if (!t_ring.slot[i].get(bytes)) return nullptr;
    t_ring.dirty[i] = true;
    return &t_ring.slot[i];
}

// ---- tensors left on the device between the nodes of one graph -----------------------------------------------
// A node whose userdata asks for it (mq_ggml_userdata::keep_hidden_on_device) leaves its result in HBM and does not
// write dst->data; a later node of the same graph that names that tensor as an operand (the same ggml_tensor, or a
// view of all of it) reads it there.  Keyed by the tensor object, not by its data pointer: graph allocators give the
// memory of a dead tensor to a later one, tensor objects are one per node.  mq_ggml_graph_begin() forgets everything.
struct KeptTensor {
    const ggml_tensor* tensor = nullptr;
    int64_t rows = 0, cols = 0;  // dense fp32 [rows][cols]
    Staging buf;
};
thread_local std::vector<KeptTensor*> t_kept;

const ggml_tensor* whole_view_base(const ggml_tensor* t) {
    // a reshape / view of a whole contiguous tensor stands for the same rows
    while (t && t->view_src && t->view_offs == 0) t = t->view_src;
    return t;
}
KeptTensor* kept_find(const ggml_tensor* t, int64_t rows, int64_t cols) {
    const ggml_tensor* base = whole_view_base(t);
    for (KeptTensor* k : t_kept)
        if (k->tensor && (k->tensor == t || k->tensor == base) && k->rows * k->cols == rows * cols) return k;
    return nullptr;
}
void kept_forget(const ggml_tensor* t) {
    for (KeptTensor* k : t_kept)
        if (k->tensor == t) k->tensor = nullptr;
}
KeptTensor* kept_slot(const ggml_tensor* t, int64_t rows, int64_t cols) {
    KeptTensor* pick = nullptr;
    for (KeptTensor* k : t_kept)
        if (k->tensor == t) pick = k;
    if (!pick)
        for (KeptTensor* k : t_kept)
            if (!k->tensor) pick = k;
    if (!pick) {
        pick = new KeptTensor;
        t_kept.push_back(pick);
    }
    const size_t bytes = (size_t)rows * (size_t)cols * 4;
    if (bytes > pick->buf.cap) settle();  // growing frees the old buffer: queued work may still use it
    if (!pick->buf.get(bytes)) {
        pick->tensor = nullptr;
        return nullptr;
    }
    pick->tensor = t;
    pick->rows = rows, pick->cols = cols;
    return pick;
}

// Gathers a strided host matrix [rows][cols] of 4-byte elements (row stride in bytes) into the pinned twin and queues
// its copy to the device buffer.
int upload_rows(Staging& st, size_t offset_bytes, const void* src_host, int64_t rows, int64_t cols, size_t row_stride_bytes) {
    const size_t row_bytes = (size_t)cols * 4;
    char* pin = (char*)st.pin + offset_bytes;
    if (row_stride_bytes == row_bytes || rows == 1) {
        std::memcpy(pin, src_host, row_bytes * (size_t)rows);
    } else {
        for (int64_t r = 0; r < rows; ++r) std::memcpy(pin + (size_t)r * row_bytes, (const char*)src_host + (size_t)r * row_stride_bytes, row_bytes);
    }
    return mq_memcpy_h2d_async((char*)st.dev + offset_bytes, pin, row_bytes * (size_t)rows, nullptr);
}

// Queues the copy of a dense device matrix into its pinned twin; scatter_rows() moves it on after the synchronisation.
int download_rows(Staging& st, size_t bytes) { return mq_memcpy_d2h_async(st.pin, st.dev, bytes, nullptr); }
void scatter_rows(void* dst_host, const Staging& st, size_t offset_bytes, int64_t rows, int64_t cols, size_t row_stride_bytes) {
    const size_t row_bytes = (size_t)cols * 4;
    const char* pin = (const char*)st.pin + offset_bytes;
    if (row_stride_bytes == row_bytes || rows == 1) {
        std::memcpy(dst_host, pin, row_bytes * (size_t)rows);
    } else {
        for (int64_t r = 0; r < rows; ++r) std::memcpy((char*)dst_host + (size_t)r * row_stride_bytes, pin + (size_t)r * row_bytes, row_bytes);
    }
}

struct Options {
    int silu_mode;
    bool keep_hidden;
    mq_ggml_userdata* ud;
};

Options options_for(void* userdata, int64_t n_tokens) {
    auto* ud = static_cast<mq_ggml_userdata*>(userdata);
    Options o;
    // decode widths use the exact exponential, wider batches the polynomial one
    // (core/src/llm/moe/native.cpp:3614-3616, core/src/backend/cpu_backend_moe_raw_batched.inl:1673)
    o.silu_mode = n_tokens <= 4 ? MQ_SILU_EXACT : MQ_SILU_FAST;
    o.keep_hidden = ud && ud->keep_hidden_on_device != 0;
    o.ud = ud;
    if (ud && !ud->use_defaults) o.silu_mode = ud->silu_mode;
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
    t_resident = Resident{};  // (no wait here: this node uploads through the ring, whose twins wait for themselves)
    if (!src || !weight || !src->data || !dst->data) return finish(o, MQ_ERR_INVALID);
    if ((!is_kquant_matrix(weight) && !is_q80_matrix(weight)) || weight->ne[2] != 1) return finish(o, MQ_ERR_UNSUPPORTED);
    const int64_t k_in = weight->ne[0], n_out = weight->ne[1];
    const int64_t m = src->ne[1] * src->ne[2] * src->ne[3];
    // the reference leaves dst untouched on a shape mismatch (core/src/llm/matmul/gemv_exec.cpp:131-143)
    if (src->type != GGML_TYPE_F32 || dst->type != GGML_TYPE_F32 || src->ne[0] != k_in || dst->ne[0] != n_out ||
        dst->ne[1] * dst->ne[2] * dst->ne[3] != m || src->nb[0] != 4 || dst->nb[0] != 4 || m <= 0)
        return finish(o, MQ_ERR_INVALID);
    if ((src->ne[2] > 1 && src->nb[2] != src->nb[1] * (size_t)src->ne[1]) ||
        (dst->ne[2] > 1 && dst->nb[2] != dst->nb[1] * (size_t)dst->ne[1]) ||
        (src->ne[3] > 1 && src->nb[3] != src->nb[2] * (size_t)src->ne[2]) ||
        (dst->ne[3] > 1 && dst->nb[3] != dst->nb[2] * (size_t)dst->ne[2]))
        return finish(o, MQ_ERR_UNSUPPORTED);
    const mq_weight* w = device_weight(weight);
    if (!w) return finish(o, t_status);
    // the input: left on the device by an earlier node of this graph, or uploaded through the ring of pinned twins
    const float* x_dev = nullptr;
    int64_t ldx = k_in;
    if (KeptTensor* kin = kept_find(src, m, k_in)) {
        x_dev = (const float*)kin->buf.dev;
    } else {
        Staging* in = ring_slot((size_t)m * k_in * 4);
        if (!in) return finish(o, t_status);
        if (int rc = upload_rows(*in, 0, src->data, m, k_in, src->nb[1])) return finish(o, rc);
        x_dev = (const float*)in->dev;
    }
    if (o.keep_hidden) {  // the result stays in HBM for the nodes that read this tensor; nothing is waited for
        KeptTensor* kout = kept_slot(dst, m, n_out);
        if (!kout) return finish(o, t_status);
        return finish(o, mq_mul_mat_q4k(w, x_dev, m, ldx, (float*)kout->buf.dev, n_out, nullptr));
    }
    kept_forget(dst);
    Staging& out = t_stage.out;
    if (!out.get((size_t)m * n_out * 4)) return finish(o, t_status);
    int rc = mq_mul_mat_q4k(w, x_dev, m, ldx, (float*)out.dev, n_out, nullptr);
    if (rc == MQ_OK) rc = download_rows(out, (size_t)m * n_out * 4);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);  // the node's one synchronisation
    if (rc == MQ_OK) settled_by_sync();
    if (rc == MQ_OK) scatter_rows(dst->data, out, 0, m, n_out, dst->nb[1]);
    finish(o, rc);
}

// An fp32 operand [rows][cols] of an element-wise node: on the device already, or uploaded through the ring.
const float* operand_rows(const ggml_tensor* t, int64_t rows, int64_t cols, int* rc) {
    if (KeptTensor* k = kept_find(t, rows, cols)) return (const float*)k->buf.dev;
    Staging* in = ring_slot((size_t)rows * cols * 4);
    if (!in) {
        *rc = t_status;
        return nullptr;
    }
    *rc = upload_rows(*in, 0, t->data, rows, cols, t->nb[1]);
    return *rc == MQ_OK ? (const float*)in->dev : nullptr;
}

// Ends an element-wise node: the rows stay on the device (kept) or travel to dst->data after one synchronisation.
void deliver_rows(const Options& o, ggml_tensor* dst, KeptTensor* kout, const Staging* out, int64_t rows, int64_t cols, int rc) {
    if (rc != MQ_OK || kout) return finish(o, rc);
    rc = mq_memcpy_d2h_async(out->pin, out->dev, (size_t)rows * cols * 4, nullptr);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    if (rc == MQ_OK) settled_by_sync();
    if (rc == MQ_OK) scatter_rows(dst->data, *out, 0, rows, cols, dst->nb[1]);
    finish(o, rc);
}

bool rows_layout(const ggml_tensor* t, int64_t* rows, int64_t* cols) {
    // fp32, unit element stride, rows evenly spaced over the outer dimensions (what upload_rows / scatter_rows walk)
    if (!t || !t->data || t->type != GGML_TYPE_F32 || t->nb[0] != 4 || t->ne[0] <= 0) return false;
    *cols = t->ne[0];
    *rows = t->ne[1] * t->ne[2] * t->ne[3];
    if (*rows <= 0) return false;
    return (t->ne[2] <= 1 || t->nb[2] == t->nb[1] * (size_t)t->ne[1]) && (t->ne[3] <= 1 || t->nb[3] == t->nb[2] * (size_t)t->ne[2]);
}

// selected_experts I32 ne=[top_k, n_tokens] -> dense device [n_tokens][top_k] (queued, not synchronised)
int upload_ids(const ggml_tensor* sel, Staging& st) {
    const int64_t top_k = sel->ne[0], n = sel->ne[1];
    if (!st.get((size_t)n * top_k * 4)) return t_status;
    if (sel->nb[0] == 4) return upload_rows(st, 0, sel->data, n, top_k, sel->nb[1]);
    auto* dense = (int32_t*)st.pin;  // element stride other than 4 bytes: gather element by element
    for (int64_t t = 0; t < n; ++t)
        for (int64_t k = 0; k < top_k; ++k)
            std::memcpy(&dense[(size_t)(t * top_k + k)], (const char*)sel->data + t * sel->nb[1] + k * sel->nb[0], 4);
    return mq_memcpy_h2d_async(st.dev, st.pin, (size_t)n * top_k * 4, nullptr);
}

// rows (token, k) of an F32 tensor ne=[cols, top_k, n] whose token stride may differ from top_k * nb[1]
int upload_pairs(Staging& st, const ggml_tensor* t, int64_t cols, int64_t top_k, int64_t n) {
    if (t->nb[2] == t->nb[1] * (size_t)top_k) return upload_rows(st, 0, t->data, n * top_k, cols, t->nb[1]);
    int rc = MQ_OK;
    for (int64_t tok = 0; tok < n && rc == MQ_OK; ++tok)
        rc = upload_rows(st, (size_t)tok * top_k * cols * 4, (const char*)t->data + tok * t->nb[2], top_k, cols, t->nb[1]);
    return rc;
}
void scatter_pairs(const ggml_tensor* t, const Staging& st, int64_t cols, int64_t top_k, int64_t n) {
    if (t->nb[2] == t->nb[1] * (size_t)top_k) return scatter_rows(t->data, st, 0, n * top_k, cols, t->nb[1]);
    for (int64_t tok = 0; tok < n; ++tok)
        scatter_rows((char*)t->data + tok * t->nb[2], st, (size_t)tok * top_k * cols * 4, top_k, cols, t->nb[1]);
}

// A Q8_0 expert stack (34-byte blocks, rows of whole 256-weight groups): the MoE down node takes it
// (core/src/llm/moe/native.cpp:4611-4616), no other expert node does.
bool is_q80_stack(const ggml_tensor* w) {
    return w && w->data && (int)w->type == (int)GGML_TYPE_Q8_0 && w->ne[0] > 0 && w->ne[0] % kSuperBlock == 0 && w->ne[1] > 0 &&
           w->ne[2] > 0 && w->ne[3] == 1 && w->nb[0] == kQ80BlockBytes && w->nb[1] >= (size_t)(w->ne[0] / 32) * kQ80BlockBytes;
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
    settle();
    t_resident = Resident{};
    if (!gate || !up || !input || !sel || !input->data || !sel->data || !dst->data) return finish(o, MQ_ERR_INVALID);
    if (!is_kquant_matrix(gate) || !is_kquant_matrix(up) || gate->type != up->type) return finish(o, MQ_ERR_UNSUPPORTED);
    const int64_t n_embd = gate->ne[0], n_ff = gate->ne[1], n_expert = gate->ne[2];
    const int64_t top_k = sel->ne[0], n = sel->ne[1];
    // operand checks of core/src/llm/moe/native.cpp:3935-3990
    if (up->ne[0] != n_embd || up->ne[1] != n_ff || up->ne[2] != n_expert || input->type != GGML_TYPE_F32 ||
        input->ne[0] != n_embd || input->ne[1] * input->ne[2] != n || (input->ne[1] != n && input->ne[1] != 1) ||
        sel->type != GGML_TYPE_I32 ||
        dst->type != GGML_TYPE_F32 || dst->ne[0] != n_ff || dst->ne[1] != top_k || dst->ne[2] != n || top_k <= 0 ||
        top_k > 8 || n <= 0 || input->nb[0] != 4 || dst->nb[0] != 4)
        return finish(o, MQ_ERR_INVALID);
    const mq_weight* wg = device_weight(gate);
    const mq_weight* wu = wg ? device_weight(up) : nullptr;
    if (!wg || !wu) return finish(o, t_status);
    // with keep_hidden_on_device the result stays in a buffer of its own (the down node's output uses `out`)
    Staging &in = t_stage.in, &out = o.keep_hidden ? t_stage.keep : t_stage.out;
    const size_t out_bytes = (size_t)n * top_k * n_ff * 4;
    if (!in.get((size_t)n * n_embd * 4) || !out.get(out_bytes)) return finish(o, t_status);
    const size_t x_stride = input->ne[1] == n ? input->nb[1] : input->nb[2];
    int rc = upload_rows(in, 0, input->data, n, n_embd, x_stride);
    if (rc == MQ_OK) rc = upload_ids(sel, t_stage.ids);
    if (rc == MQ_OK)
        rc = mq_moe_gateup_swiglu_q4k(wg, wu, (const float*)in.dev, n, (const int32_t*)t_stage.ids.dev, (int)top_k, o.silu_mode,
                                      (float*)out.dev, nullptr);
    if (rc == MQ_OK && o.keep_hidden) {
        // The rows stay in HBM for the down node of this graph; dst->data is NOT written and nothing is waited for
        // (the null stream keeps the order).  The pinned twins of `in` and `ids` are still being read by the queued
        // copies; the down node uploads through buffers of its own (in2, ids2), and this node writes them again only
        // after that node's synchronisation.
        t_resident.host = dst->data;
        t_resident.n_ff = n_ff, t_resident.top_k = top_k, t_resident.n = n;
        t_unsettled = true;
        return finish(o, rc);
    }
    if (rc == MQ_OK) rc = download_rows(out, out_bytes);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    // dst may be a strided view (core/src/llm/moe/native.cpp:4201-4209): rows are (token, k) pairs
    if (rc == MQ_OK) scatter_pairs(dst, out, n_ff, top_k, n);
    finish(o, rc);
}

void mq_cb_moe_down_weighted_logits(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) {
    if (ith != 0 || !dst) return;
    const ggml_tensor* down = dst->src[0];
    const ggml_tensor* hidden = dst->src[1];
    const ggml_tensor* sel = dst->src[2];
    const ggml_tensor* logits = dst->src[3];
    Options o = options_for(userdata, sel ? sel->ne[1] : 1);
    const Resident resident = t_resident;  // valid for the node that follows the gate/up node only
    t_resident = Resident{};
    if (!down || !hidden || !sel || !logits || !hidden->data || !sel->data || !logits->data || !dst->data)
        return finish(o, MQ_ERR_INVALID);
    if (!is_kquant_matrix(down) && !is_q80_stack(down)) return finish(o, MQ_ERR_UNSUPPORTED);
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
    const bool on_device = resident.host == hidden->data && resident.n_ff == n_ff && resident.top_k == top_k && resident.n == n;
    if (!on_device) settle();
    Staging &hin = t_stage.aux, &lg = t_stage.in2, &wts = t_stage.wts, &out = t_stage.out;
    if ((!on_device && !hin.get((size_t)n * top_k * n_ff * 4)) || !lg.get((size_t)n * n_expert * 4) || !wts.get((size_t)n * top_k * 4) ||
        !out.get((size_t)n * n_embd * 4))
        return finish(o, t_status);
    int rc = MQ_OK;
    if (!on_device) rc = upload_pairs(hin, hidden, n_ff, top_k, n);
    const float* h_dev = (const float*)(on_device ? t_stage.keep.dev : hin.dev);
    if (rc == MQ_OK) rc = upload_rows(lg, 0, logits->data, n, n_expert, logits->nb[1]);
    if (rc == MQ_OK) rc = upload_ids(sel, t_stage.ids2);
    const int32_t* ids_dev = (const int32_t*)t_stage.ids2.dev;
    if (rc == MQ_OK) rc = mq_moe_weights_from_logits((const float*)lg.dev, n_expert, n, ids_dev, (int)top_k, (float*)wts.dev, nullptr);
    if (rc == MQ_OK) rc = mq_moe_down_weighted_q4k(wd, h_dev, n, ids_dev, (const float*)wts.dev, (int)top_k, (float*)out.dev, nullptr);
    if (rc == MQ_OK) rc = download_rows(out, (size_t)n * n_embd * 4);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    if (rc == MQ_OK) t_unsettled = false;
    if (rc == MQ_OK) scatter_rows(dst->data, out, 0, n, n_embd, dst->nb[1]);
    finish(o, rc);
}

void mq_cb_moe_fused_router(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) {
    auto* state = static_cast<mq_ggml_router_state*>(userdata);
    const ggml_tensor* logits = dst ? dst->src[0] : nullptr;
    if (ith != 0) return;
    settle();
    t_resident = Resident{};
    // the checks of cb_qwen_native_moe_fused_router (core/src/llm/moe/native.cpp:710-718): a node that fails them is left alone
    if (!dst || !state || !logits || !dst->data || !logits->data || dst->type != GGML_TYPE_I32 || logits->type != GGML_TYPE_F32 ||
        logits->ne[0] != state->n_experts || logits->ne[1] != state->n_tokens || dst->ne[0] != state->top_k ||
        dst->ne[1] != state->n_tokens || !state->normalized_weights || logits->nb[0] != 4 || dst->nb[0] != 4 ||
        state->top_k <= 0 || state->top_k > 8 || state->top_k > state->n_experts || state->n_experts > 2048 || state->n_tokens <= 0) {
        note(MQ_ERR_INVALID);
        return;
    }
    const int64_t E = state->n_experts, n = state->n_tokens, K = state->top_k;
    Staging &lg = t_stage.in, &ids = t_stage.ids, &wts = t_stage.wts;
    if (!lg.get((size_t)n * E * 4) || !ids.get((size_t)n * K * 4) || !wts.get((size_t)n * K * 4)) return;
    int rc = upload_rows(lg, 0, logits->data, n, E, logits->nb[1]);
    if (rc == MQ_OK) rc = mq_moe_route_topk((const float*)lg.dev, E, n, (int)K, MQ_ROUTE_FUSED, (int32_t*)ids.dev, (float*)wts.dev, nullptr);
    if (rc == MQ_OK) rc = download_rows(ids, (size_t)n * K * 4);
    if (rc == MQ_OK) rc = download_rows(wts, (size_t)n * K * 4);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    if (rc == MQ_OK) {
        scatter_rows(dst->data, ids, 0, n, K, dst->nb[1]);
        std::memcpy(state->normalized_weights, wts.pin, (size_t)n * K * 4);  // dense [n_tokens][top_k], as the reference keeps them
    }
    note(rc);
    if (rc != MQ_OK) std::fprintf(stderr, "mi355_q4k adapter: %s\n", mq_last_error());
}

void mq_cb_moe_topk_weights_from_logits(struct ggml_tensor* dst, int ith, int /*nth*/, void* /*userdata*/) {
    if (ith != 0) return;
    settle();
    t_resident = Resident{};
    // the checks of cb_moe_topk_weights_from_logits (core/src/llm/moe/native.cpp:800-813)
    if (!dst || !dst->src[0] || !dst->src[1] || !dst->data || !dst->src[0]->data || !dst->src[1]->data) return;
    const ggml_tensor* logits = dst->src[0];
    const ggml_tensor* sel = dst->src[1];
    if (dst->type != GGML_TYPE_F32 || logits->type != GGML_TYPE_F32 || sel->type != GGML_TYPE_I32 || logits->ne[0] <= 0 ||
        logits->ne[1] <= 0 || sel->ne[0] <= 0 || sel->ne[1] != logits->ne[1] || dst->ne[0] != 1 || dst->ne[1] != sel->ne[0] ||
        dst->ne[2] != logits->ne[1] || logits->nb[0] != 4 || sel->ne[0] > 8) {
        note(MQ_ERR_INVALID);
        return;
    }
    const int64_t E = logits->ne[0], n = logits->ne[1], K = sel->ne[0];
    Staging &lg = t_stage.in, &wts = t_stage.wts;
    if (!lg.get((size_t)n * E * 4) || !wts.get((size_t)n * K * 4)) return;
    int rc = upload_rows(lg, 0, logits->data, n, E, logits->nb[1]);
    if (rc == MQ_OK) rc = upload_ids(sel, t_stage.ids);
    if (rc == MQ_OK) rc = mq_moe_weights_from_logits((const float*)lg.dev, E, n, (const int32_t*)t_stage.ids.dev, (int)K, (float*)wts.dev, nullptr);
    if (rc == MQ_OK) rc = download_rows(wts, (size_t)n * K * 4);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    if (rc == MQ_OK) {  // dst ne = [1, top_k, n_tokens]: element (k, token) at k * nb[1] + token * nb[2]
        const float* w = (const float*)wts.pin;
        for (int64_t t = 0; t < n; ++t)
            for (int64_t k = 0; k < K; ++k) std::memcpy((char*)dst->data + k * dst->nb[1] + t * dst->nb[2], &w[t * K + k], 4);
    }
    note(rc);
    if (rc != MQ_OK) std::fprintf(stderr, "mi355_q4k adapter: %s\n", mq_last_error());
}

void mq_cb_mul_mat_id(struct ggml_tensor* dst, int ith, int /*nth*/, void* userdata) {
    if (ith != 0 || !dst) return;
    const ggml_tensor* as = dst->src[0];
    const ggml_tensor* b = dst->src[1];
    const ggml_tensor* sel = dst->src[2];
    Options o = options_for(userdata, sel ? sel->ne[1] : 1);
    settle();
    t_resident = Resident{};
    if (!as || !b || !sel || !b->data || !sel->data || !dst->data) return finish(o, MQ_ERR_INVALID);
    if (!is_kquant_matrix(as)) return finish(o, MQ_ERR_UNSUPPORTED);
    // ggml_mul_mat_id: as [K, N, n_expert], b F32 [K, n_used or 1, n_tokens], ids I32 [n_used, n_tokens],
    // dst F32 [N, n_used, n_tokens]
    const int64_t k_in = as->ne[0], n_out = as->ne[1];
    const int64_t top_k = sel->ne[0], n = sel->ne[1];
    const int64_t x_slots = b->ne[1];
    if (b->type != GGML_TYPE_F32 || sel->type != GGML_TYPE_I32 || dst->type != GGML_TYPE_F32 || b->ne[0] != k_in || b->ne[2] != n ||
        (x_slots != 1 && x_slots != top_k) || dst->ne[0] != n_out || dst->ne[1] != top_k || dst->ne[2] != n || top_k <= 0 || top_k > 8 ||
        top_k > as->ne[2] || n <= 0 || b->nb[0] != 4 || dst->nb[0] != 4)
        return finish(o, MQ_ERR_INVALID);
    const mq_weight* w = device_weight(as);
    if (!w) return finish(o, t_status);
    Staging &in = t_stage.in, &out = t_stage.out;
    const size_t out_bytes = (size_t)n * top_k * n_out * 4;
    if (!in.get((size_t)n * x_slots * k_in * 4) || !out.get(out_bytes)) return finish(o, t_status);
    int rc = upload_pairs(in, b, k_in, x_slots, n);
    if (rc == MQ_OK) rc = upload_ids(sel, t_stage.ids);
    if (rc == MQ_OK)
        rc = mq_mul_mat_id_q4k(w, (const float*)in.dev, n, (int)x_slots, (const int32_t*)t_stage.ids.dev, (int)top_k, (float*)out.dev, nullptr);
    if (rc == MQ_OK) rc = download_rows(out, out_bytes);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    if (rc == MQ_OK) scatter_pairs(dst, out, n_out, top_k, n);
    finish(o, rc);
}

void mq_cb_silu_mul_fused(struct ggml_tensor* dst, const struct ggml_tensor* a, const struct ggml_tensor* b, int ith, int /*nth*/,
                          void* userdata) {
    if (ith != 0) return;
    Options o = options_for(userdata, 1);
    t_resident = Resident{};
    // the checks of cb_silu_mul_fused (core/src/llm/graph/fused_ops.cpp:317-340): anything else leaves dst untouched
    int64_t rows = 0, cols = 0, rb = 0, cb = 0, rd = 0, cd = 0;
    if (!dst || !rows_layout(a, &rows, &cols) || !rows_layout(b, &rb, &cb) || !rows_layout(dst, &rd, &cd) || rows != rb || cols != cb ||
        rows != rd || cols != cd)
        return finish(o, MQ_ERR_INVALID);
    // contiguous tensors take the reference's SIMD routine (fused-multiply-add polynomial), strided ones its scalar
    // loop with the exact exponential (fused_ops.cpp:342-365)
    const bool contiguous = a->nb[1] == (size_t)cols * 4 && b->nb[1] == (size_t)cols * 4 && dst->nb[1] == (size_t)cols * 4;
    const int mode = (o.ud && !o.ud->use_defaults) ? o.silu_mode : (contiguous ? MQ_SILU_FAST_FMA : MQ_SILU_EXACT);
    int rc = MQ_OK;
    const float* g_dev = operand_rows(a, rows, cols, &rc);
    const float* u_dev = g_dev ? operand_rows(b, rows, cols, &rc) : nullptr;
    if (!g_dev || !u_dev) return finish(o, rc);
    KeptTensor* kout = nullptr;
    Staging* out = &t_stage.out;
    if (o.keep_hidden) {
        kout = kept_slot(dst, rows, cols);
        if (!kout) return finish(o, t_status);
        out = &kout->buf;
    } else {
        kept_forget(dst);
        if (!out->get((size_t)rows * cols * 4)) return finish(o, t_status);
    }
    rc = mq_silu_mul_f32(g_dev, u_dev, rows, cols, cols, cols, (float*)out->dev, cols, mode, nullptr);
    deliver_rows(o, dst, kout, out, rows, cols, rc);
}

void mq_cb_apply_shared_scalar_gate(struct ggml_tensor* dst, const struct ggml_tensor* src, const struct ggml_tensor* gate_logits_scalar,
                                    int ith, int /*nth*/, void* userdata) {
    if (ith != 0) return;
    Options o = options_for(userdata, 1);
    t_resident = Resident{};
    // the checks of cb_apply_shared_scalar_gate (core/src/llm/graph/fused_ops.cpp:437-449): hidden = src->ne[0], tokens =
    // max(1, src->ne[1]), one logit per token at gate_logits_scalar row stride nb[1]
    int64_t rows = 0, cols = 0, rd = 0, cd = 0;
    if (!dst || !gate_logits_scalar || !gate_logits_scalar->data || gate_logits_scalar->type != GGML_TYPE_F32 ||
        !rows_layout(src, &rows, &cols) || !rows_layout(dst, &rd, &cd) || rows != rd || cols != cd || src->ne[2] * src->ne[3] != 1)
        return finish(o, MQ_ERR_INVALID);
    const int64_t scalar_elems = gate_logits_scalar->ne[0] * gate_logits_scalar->ne[1] * gate_logits_scalar->ne[2] * gate_logits_scalar->ne[3];
    if (scalar_elems < rows) return finish(o, MQ_ERR_INVALID);
    int rc = MQ_OK;
    const float* s_dev = operand_rows(src, rows, cols, &rc);
    if (!s_dev) return finish(o, rc);
    // the logits: one per token, gate_logits_scalar->nb[1] apart
    const float* l_dev = nullptr;
    if (KeptTensor* kl = kept_find(gate_logits_scalar, rows, gate_logits_scalar->ne[0])) {
        l_dev = (const float*)kl->buf.dev;
    } else {
        Staging* lg = ring_slot((size_t)rows * 4);
        if (!lg) return finish(o, t_status);
        for (int64_t t = 0; t < rows; ++t) std::memcpy((char*)lg->pin + t * 4, (const char*)gate_logits_scalar->data + t * gate_logits_scalar->nb[1], 4);
        rc = mq_memcpy_h2d_async(lg->dev, lg->pin, (size_t)rows * 4, nullptr);
        if (rc != MQ_OK) return finish(o, rc);
        l_dev = (const float*)lg->dev;
    }
    const int64_t ld_logit = kept_find(gate_logits_scalar, rows, gate_logits_scalar->ne[0]) ? gate_logits_scalar->ne[0] : 1;
    KeptTensor* kout = nullptr;
    Staging* out = &t_stage.out;
    if (o.keep_hidden) {
        kout = kept_slot(dst, rows, cols);
        if (!kout) return finish(o, t_status);
        out = &kout->buf;
    } else {
        kept_forget(dst);
        if (!out->get((size_t)rows * cols * 4)) return finish(o, t_status);
    }
    rc = mq_scale_rows_sigmoid_f32(s_dev, rows, cols, cols, l_dev, ld_logit, (float*)out->dev, cols, nullptr);
    deliver_rows(o, dst, kout, out, rows, cols, rc);
}

void mq_ggml_graph_begin(void) {
    settle();
    for (KeptTensor* k : t_kept) k->tensor = nullptr;
    t_resident = Resident{};
}

int mq_ggml_tensor_to_host(struct ggml_tensor* t) {
    int64_t rows = 0, cols = 0;
    if (!rows_layout(t, &rows, &cols)) return 0;
    KeptTensor* k = kept_find(t, rows, cols);
    if (!k) return 0;
    int rc = mq_memcpy_d2h_async(k->buf.pin, k->buf.dev, (size_t)rows * cols * 4, nullptr);
    if (rc == MQ_OK) rc = mq_stream_synchronize(nullptr);
    if (note(rc) != MQ_OK) return 0;
    settled_by_sync();
    scatter_rows(t->data, k->buf, 0, rows, cols, t->nb[1]);
    return 1;
}

int mq_ggml_last_status(void) { return t_status; }

uint64_t mq_ggml_weight_fingerprint(const void* data, size_t bytes) { return fingerprint_bytes(data, bytes); }

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
