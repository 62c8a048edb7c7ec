// C ABI of libmi355q4k.so (declared in include/mi355_q4k.h): argument checks, weight handles,
// a grow-only device workspace and the sequencing of kernel launches.  No arithmetic lives here.
#include "../../include/mi355_q4k.h"
#include "../../include/mi355_q4k_debug.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "kernels.h"

using namespace mq;

struct mq_weight {
    uint8_t* data = nullptr;     // tiled layout, experts back to back
    int64_t rows = 0, cols = 0, n_experts = 0;
    int64_t nb = 0, rowtiles = 0;
    int type = kTypeQ4K;         // ggml_type: 12 (Q4_K) or 13 (Q5_K)
    size_t expert_bytes = 0;     // tiled bytes per expert
    size_t total_bytes = 0;
};

struct mq_acts {
    void* aq = nullptr;   // A-major codes
    void* ad = nullptr;   // A-major scales
    void* ap = nullptr;   // handles of more than eight rows: the rows as P-major tiles of sixteen as well (written for 9..64 rows)
    int64_t max_rows = 0, cols = 0, nb = 0;
    int64_t n = 0;        // rows quantized by the last mq_acts_quantize
    bool tile16 = false;  // ap holds those rows (set by the quantizer that wrote both layouts, cleared by one that did not)
};

// Scratch of mq_mul_mat_q4k_noalloc: the quantized activations (A-major codes, then the scales) of at most
// kNoAllocMaxRows rows of kNoAllocMaxCols columns.  One copy per GPU, held until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; the device address is looked up once per device in mq_init.
// (File scope, not the unnamed namespace below: there the device-side symbol is local to the code object and the
// runtime cannot find it.)
constexpr int64_t kNoAllocMaxRows = 16, kNoAllocMaxCols = 16384;
constexpr size_t kNoAllocAqBytes = (size_t)((kNoAllocMaxRows + 7) / 8) * (kNoAllocMaxCols / mq::kQK) * 4096;
constexpr size_t kNoAllocAdBytes = (size_t)((kNoAllocMaxRows + 7) / 8) * (kNoAllocMaxCols / mq::kQK) * 8 * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kNoAllocAqBytes + kNoAllocAdBytes];

namespace {

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

// Set once any entry point has been called on a stream under HIP-graph capture: from then on a graph may hold the
// address of a workspace buffer, so a buffer that has to grow is retired (kept allocated until mq_shutdown) instead
// of freed -- the graph's replays keep working on the addresses they captured.
bool g_graph_seen = false;
std::vector<void*> g_retired;

int hip_fail(hipError_t e, const char* what) {
    return fail(MQ_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define MQ_HIP(call)                                     \
    do {                                                 \
        hipError_t e_ = (call);                          \
        if (e_ != hipSuccess) return hip_fail(e_, #call); \
    } while (0)

// A device buffer that only grows.  Growing frees the old allocation, which synchronises the device, so kernels
// already queued on any stream have finished with it -- unless a HIP-graph capture has been seen: a captured graph
// would keep launching kernels on the freed address, so the old allocation is retired instead (and the new one is at
// least twice as large, which bounds what retirement can hold to the size of the live buffer).
struct Buffer {
    void* ptr = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes) {
        if (bytes <= cap) return hipSuccess;
        if (ptr && g_graph_seen) {
            g_retired.push_back(ptr);
            if (bytes < 2 * cap) bytes = 2 * cap;
            ptr = nullptr;
            cap = 0;
        }
        if (ptr) {
            hipError_t e = hipFree(ptr);
            ptr = nullptr;
            cap = 0;
            if (e != hipSuccess) return e;
        }
        const size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        hipError_t e = hipMalloc(&ptr, want);
        if (e == hipSuccess) cap = want;
        return e;
    }
    void release() {
        if (ptr) (void)hipFree(ptr);
        ptr = nullptr;
        cap = 0;
    }
};

// Page-locked host memory for the host-pointer entry points (allocated, never registered).
struct PinnedBuffer {
    void* ptr = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes) {
        if (bytes <= cap) return hipSuccess;
        if (ptr) {
            hipError_t e = hipHostFree(ptr);
            ptr = nullptr;
            cap = 0;
            if (e != hipSuccess) return e;
        }
        const size_t want = (bytes + (size_t(1) << 16) - 1) & ~((size_t(1) << 16) - 1);
        hipError_t e = hipHostMalloc(&ptr, want, hipHostMallocDefault);
        if (e == hipSuccess) cap = want;
        return e;
    }
    void release() {
        if (ptr) (void)hipHostFree(ptr);
        ptr = nullptr;
        cap = 0;
    }
};

struct State {
    bool ready = false;
    int device = -1;
    std::recursive_mutex mu;  // recursive: the host-pointer entry points call the device-pointer ones while holding it
    Buffer aq, ad;        // A-major activations of the op input
    Buffer ap, ap2;       // P-major activations of the prefill GEMM (input; FFN intermediate)
    Buffer ap_rows;       // the distinct rows of an expert-grouped GEMM's input, quantized once, before they are copied to their groups
    Buffer mid2;          // gate and up products of a wide FFN, fp32
    Buffer kpart;         // planes of partial sums of a prefill GEMM whose K is split
    Buffer plan;          // tile plan of the expert-grouped GEMM
    Buffer mid;           // fp32 intermediate (FFN hidden, MoE per-(token,k) hidden)
    Buffer aq2, ad2;      // A-major activations of the intermediate
    Buffer part;          // MoE per-(token,k) down results
    Buffer counters;      // arrival counters of the fused output quantization (kept zero between launches)
    Buffer route;         // ids / weights / groups / entries
    Buffer stage_in, stage_out;  // host-pointer entry points
    PinnedBuffer pin_in, pin_out;
    // the stream of the last call that used the workspaces above, and an event to order the next stream behind it
    bool have_last_stream = false;
    hipStream_t last_stream = nullptr;
    hipEvent_t order_event = nullptr;
} g;

constexpr int kMaxDevices = 64;
unsigned char* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each GPU that mq_init has seen

// Launch census: a start/stop event pair bound to each dispatch of the decode matmul kernels (see mq_census_* in
// include/mi355_q4k_debug.h).  Purely an observer: no entry point chooses its kernels by whether it is on; launches of
// other kernels are simply not recorded.
struct Census {
    bool on = false;
    struct Rec {
        hipEvent_t start, stop;
        int kind;
    };
    std::vector<Rec> pool;   // created once, reused after reset
    size_t used = 0;
    static constexpr size_t kMax = 8192;
} census;

// Dense products of up to 16 rows go to the kernel that stages the activations in LDS where the shape fits it (the
// same bits as matmul_kernel on the same operands); mq_debug_set_dense_lds(0) keeps them on matmul_kernel.
int g_dense_lds = 1;
int g_moe_item_tiles = 0;  // 0: chosen per launch (moe_gemm_item_tiles); 2, 4 or 8: forced (mq_debug_set_dense_lds bits 8..11)
int g_gemm_pair = 1;  // prefill widths: Q4_K gate and up in ONE GEMM launch that stores silu(gate) * up (mq_debug_set_dense_lds bit 3 turns it off)
// Widest product whose fp32 rows the LDS-staged kernel quantizes itself (no quantizer launch).
constexpr int64_t kDenseXfRowsDefault = 2;
int64_t g_dense_xf_rows = kDenseXfRowsDefault;  // measured on the 4096 -> 14336 gate/up pair: two rows 15.4 against 16.5 us with the quantizer launch, four rows 16.9 against 16.4

bool dense_lds_takes(const MatmulArgs& a) {
    return g_dense_lds && !a.grouped && !a.dbg_dot && !a.out_aq && a.n >= 1 && a.n <= 16 &&
           dense_lds_applies(a.nb, (a.rows + 15) / 16, a.n, a.swiglu != 0, a.wtype);
}
// fp32 rows straight into the product (n rows, ldx apart): true when the call may skip its quantizer launch
bool dense_lds_quantizes(const mq_weight* w, const float* x, int64_t n, int64_t ldx, bool swiglu) {
    return g_dense_lds && n >= 1 && n <= g_dense_xf_rows && n <= 4 && n * w->nb <= 64 && !(reinterpret_cast<uintptr_t>(x) & 15u) && !(ldx & 3) &&
           dense_lds_applies(w->nb, w->rowtiles, n, swiglu, w->type);
}

// Nine to 64 rows of a Q4_K matrix: one to four activation tiles of sixteen rows per weight tile
// (skinny16_kernel, the same bits as the token tiles of eight of the other decode kernels); mq_debug_set_dense_lds
// bit 12 turns it off.  kSkinnyMaxRows: beyond it the matrix-core GEMM (large matrices) or the 16-row passes of the
// decode kernels take over.
int g_skinny16 = 1;
constexpr int64_t kSkinnyMaxRows = 64;
bool skinny16_takes(const mq_weight* w, int64_t n, bool swiglu) {
    return g_skinny16 && g_dense_lds && n > 8 && n <= kSkinnyMaxRows && skinny16_applies(w->nb, w->rowtiles, swiglu, n, w->type);
}

hipError_t dense_launch(const MatmulArgs& a, hipStream_t s, hipEvent_t start = nullptr, hipEvent_t stop = nullptr) {
    if (a.ap) {  // callers ask skinny16_takes first
        if (a.grouped || a.dbg_dot || a.out_aq) return hipErrorInvalidValue;
        Skinny16Args k;
        k.w0 = a.w0;
        k.w1 = a.swiglu ? a.w1 : nullptr;
        k.rows = a.rows;
        k.nb = a.nb;
        k.ap = a.ap;
        k.n = a.n;
        k.y = a.y;
        k.ldy = a.ldy;
        k.silu_mode = a.silu_mode;
        k.wtype = a.wtype;
        return launch_skinny16(k, s, start, stop);
    }
    if (!dense_lds_takes(a)) {
        if (a.xf && a.n != 1) return hipErrorInvalidValue;  // callers ask dense_lds_quantizes first
        return launch_matmul(a, s, start, stop);
    }
    DenseLdsArgs d;
    d.w0 = a.w0;
    d.w1 = a.swiglu ? a.w1 : nullptr;
    d.rows = a.rows;
    d.nb = a.nb;
    d.aq = a.aq;
    d.ad = a.ad;
    d.xf = a.xf;
    d.ldx = a.xf ? (a.n == 1 ? a.nb * kQK : a.ldx) : 0;
    d.n = a.n;
    d.y = a.y;
    d.ldy = a.ldy;
    d.wtype = a.wtype;
    d.silu_mode = a.silu_mode;
    return launch_dense_lds(d, s, start, stop);
}

hipError_t census_launch(const MatmulArgs& a, hipStream_t s) {
    if (!census.on || census.used >= Census::kMax) return dense_launch(a, s);
    if (census.used == census.pool.size()) {
        Census::Rec r;
        hipError_t e = hipEventCreate(&r.start);
        if (e != hipSuccess) return e;
        e = hipEventCreate(&r.stop);
        if (e != hipSuccess) return e;
        census.pool.push_back(r);
    }
    Census::Rec& r = census.pool[census.used++];
    r.kind = (a.grouped ? 2 : 0) + (a.swiglu ? 1 : 0);
    return dense_launch(a, s, r.start, r.stop);
}

// Every entry point that touches the shared workspaces goes through this: it serialises host-side callers and orders
// the device work of callers on DIFFERENT streams -- the workspaces (quantized activations, routing lists, arrival
// counters) are one set per process, so a call on stream B must not start on the device before the previous call on
// stream A has finished with them.  A stream under graph capture is left alone (an event recorded outside the capture
// cannot be waited on inside it): a graph's replays are ordered by whoever launches them.
int order_stream(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        st = hipStreamCaptureStatusNone;
    }
    if (st != hipStreamCaptureStatusNone) {
        g_graph_seen = true;
        return MQ_OK;
    }
    if (g.have_last_stream && g.last_stream != s) {
        hipError_t e = hipSuccess;
        // the event exists since mq_init: no entry point creates anything here (one of them must not allocate)
        if (!g.order_event) e = hipErrorNotReady;
        if (e == hipSuccess) e = hipEventRecord(g.order_event, g.last_stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(s, g.order_event, 0);
        if (e != hipSuccess) {  // e.g. the previous stream no longer exists: wait for everything instead
            (void)hipGetLastError();
            e = hipDeviceSynchronize();
            if (e != hipSuccess) return hip_fail(e, "ordering a new stream behind the previous one");
        }
    }
    g.last_stream = s;
    g.have_last_stream = true;
    return MQ_OK;
}
struct Entry {
    std::lock_guard<std::recursive_mutex> lock;
    int rc;
    explicit Entry(hipStream_t s) : lock(g.mu), rc(order_stream(s)) {}
};

int check_ready() {
    if (!g.ready) return fail(MQ_ERR_STATE, "mq_init has not been called (or no GPU is present)");
    return MQ_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Q8_0 weights: dense projections through mq_mul_mat_q4k, expert stacks as the down experts of the MoE down node and
// of the MoE layer (their activations are Q8_0 too); nothing else takes them.
int check_weight(const mq_weight* w, const char* name, bool q80_ok = false) {
    if (!w || !w->data) return fail(MQ_ERR_INVALID, "%s: null weight handle", name);
    if (w->type == kTypeQ80 && !q80_ok) return fail(MQ_ERR_UNSUPPORTED, "%s: Q8_0 weights are taken by mq_mul_mat_q4k and as MoE down experts only", name);
    return MQ_OK;
}

int check_x(const float* x, int64_t n, int64_t ldx, int64_t cols, const char* name) {
    if (n < 0) return fail(MQ_ERR_INVALID, "%s: negative row count", name);
    if (n == 0) return MQ_OK;  // an empty matrix may come with null pointers; every caller returns before using them
    if (!x) return fail(MQ_ERR_INVALID, "%s: null activation pointer", name);
    if (ldx < cols) return fail(MQ_ERR_INVALID, "%s: ldx %lld < cols %lld", name, (long long)ldx, (long long)cols);
    if (!aligned16(x) || (ldx & 3)) return fail(MQ_ERR_INVALID, "%s: activations must be 16-byte aligned with ldx %% 4 == 0", name);
    return MQ_OK;
}

// Quantize x into the A-major workspace pair (aq, ad).
int quantize_into(Buffer& aq, Buffer& ad, const float* x, int64_t n, int64_t ldx, int64_t cols, hipStream_t s) {
    const int64_t nb = cols / kQK;
    MQ_HIP(aq.reserve(aq_bytes(n, nb)));
    MQ_HIP(ad.reserve(ad_count(n, nb) * sizeof(float)));
    MQ_HIP(launch_quantize_q8k(x, n, ldx, cols, nullptr, 0, (uint8_t*)aq.ptr, (float*)ad.ptr, s));
    return MQ_OK;
}

// Quantize up to 64 rows of x into one to four P-major tiles per super-block (g.ap), the operand of skinny16_kernel.
int quantize_into_tile16(const float* x, int64_t n, int64_t ldx, int64_t cols, hipStream_t s) {
    MQ_HIP(g.ap.reserve(pmajor_bytes(n, cols / kQK)));
    MQ_HIP(launch_quantize_q8k_pmajor(x, n, ldx, cols, (uint8_t*)g.ap.ptr, s));
    return MQ_OK;
}

// Arrival counters for the fused output quantization: zeroed when (re)allocated, and every launch
// leaves them zero again.
int reserve_counters(size_t count) {
    const size_t before = g.counters.cap;
    MQ_HIP(g.counters.reserve(count * sizeof(uint32_t)));
    if (g.counters.cap != before) MQ_HIP(hipMemset(g.counters.ptr, 0, g.counters.cap));
    return MQ_OK;
}

int alloc_weight(int type, int64_t rows, int64_t cols, int64_t n_experts, mq_weight** out) {
    if (!out) return fail(MQ_ERR_INVALID, "null output handle");
    *out = nullptr;
    if (type != kTypeQ4K && type != kTypeQ5K && type != kTypeQ6K && type != kTypeQ80)
        return fail(MQ_ERR_UNSUPPORTED, "ggml type %d: only Q4_K (12), Q5_K (13), Q6_K (14) and Q8_0 (8) weights are supported", type);
    if (rows <= 0 || cols <= 0 || n_experts <= 0) return fail(MQ_ERR_INVALID, "rows, cols and n_experts must be positive");
    if (cols % kQK) return fail(MQ_ERR_INVALID, "cols %lld is not a multiple of 256", (long long)cols);
    mq_weight* w = new mq_weight;
    w->type = type;
    w->rows = rows;
    w->cols = cols;
    w->n_experts = n_experts;
    w->nb = cols / kQK;
    w->rowtiles = (rows + 15) / 16;
    // shapes may come from an untrusted file header: no product may wrap
    size_t eb = 0, tb = 0;
    if (__builtin_mul_overflow((size_t)w->rowtiles, (size_t)w->nb, &eb) || __builtin_mul_overflow(eb, (size_t)tile_bytes_of(type), &eb) ||
        __builtin_mul_overflow(eb, (size_t)n_experts, &tb) || tb > (size_t(1) << 46)) {
        delete w;
        return fail(MQ_ERR_INVALID, "a weight tensor of %lld x %lld x %lld does not fit a device allocation", (long long)rows, (long long)cols,
                    (long long)n_experts);
    }
    w->expert_bytes = eb;
    w->total_bytes = tb;
    hipError_t e = hipMalloc((void**)&w->data, w->total_bytes);
    if (e != hipSuccess) {
        delete w;
        return hip_fail(e, "hipMalloc(weights)");
    }
    if (rows % 16) {  // padding rows of the last tile must read as zero blocks
        e = hipMemset(w->data, 0, w->total_bytes);
        if (e != hipSuccess) {
            (void)hipFree(w->data);
            delete w;
            return hip_fail(e, "hipMemset(weights)");
        }
    }
    *out = w;
    return MQ_OK;
}

}  // namespace

extern "C" {

const char* mq_last_error(void) { return g_error.c_str(); }

int mq_init(int device) {
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) return fail(MQ_ERR_STATE, "no HIP device available (%s)", hipGetErrorString(e));
    if (device < 0 || device >= count) return fail(MQ_ERR_INVALID, "device %d out of range [0, %d)", device, count);
    MQ_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    MQ_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(MQ_ERR_UNSUPPORTED, "built for gfx950, device is %s", prop.gcnArchName);
    if (device < kMaxDevices && !g_scratch_ptr[device]) {  // this GPU's copy of the allocation-free entry point's scratch
        void* ptr = nullptr;
        MQ_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        g_scratch_ptr[device] = static_cast<unsigned char*>(ptr);
    }
    set_compute_units(prop.multiProcessorCount);
    if (!g.order_event) MQ_HIP(hipEventCreateWithFlags(&g.order_event, hipEventDisableTiming));  // orders calls on different streams
    g.device = device;
    g.ready = true;
    return MQ_OK;
}

int mq_shutdown(void) {
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    if (!g.ready) return MQ_OK;
    (void)hipDeviceSynchronize();
    for (Buffer* b : {&g.aq, &g.ad, &g.ap, &g.ap2, &g.ap_rows, &g.mid, &g.mid2, &g.kpart, &g.plan, &g.aq2, &g.ad2, &g.part, &g.counters, &g.route, &g.stage_in, &g.stage_out}) b->release();
    g.pin_in.release();
    g.pin_out.release();
    if (g.order_event) (void)hipEventDestroy(g.order_event);
    g.order_event = nullptr;
    g.have_last_stream = false;
    for (void* p : g_retired) (void)hipFree(p);
    g_retired.clear();
    g_graph_seen = false;
    g.ready = false;
    return MQ_OK;
}

int mq_device_info(char* name_out, size_t name_cap, int* cu_count, size_t* hbm_bytes) {
    if (int rc = check_ready()) return rc;
    hipDeviceProp_t prop;
    MQ_HIP(hipGetDeviceProperties(&prop, g.device));
    if (name_out && name_cap) snprintf(name_out, name_cap, "%s (%s)", prop.name, prop.gcnArchName);
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
    return MQ_OK;
}

// ---------------------------------------------------------------------------------- weights
int mq_weight_upload(const void* q4k_host, int64_t rows, int64_t cols, int64_t n_experts, size_t row_bytes,
                     size_t expert_bytes, mq_weight** out) {
    return mq_weight_upload_typed(kTypeQ4K, q4k_host, rows, cols, n_experts, row_bytes, expert_bytes, out);
}

int mq_weight_upload_typed(int ggml_type, const void* q4k_host, int64_t rows, int64_t cols, int64_t n_experts,
                           size_t row_bytes, size_t expert_bytes, mq_weight** out) {
    if (int rc = check_ready()) return rc;
    if (ggml_type != kTypeQ4K && ggml_type != kTypeQ5K && ggml_type != kTypeQ6K && ggml_type != kTypeQ80)
        return fail(MQ_ERR_UNSUPPORTED, "mq_weight_upload: ggml type %d (only 12 = Q4_K, 13 = Q5_K, 14 = Q6_K and 8 = Q8_0)", ggml_type);
    if (!q4k_host) return fail(MQ_ERR_INVALID, "mq_weight_upload: null host pointer");
    if (cols <= 0 || cols % kQK) return fail(MQ_ERR_INVALID, "mq_weight_upload: cols %lld is not a positive multiple of 256", (long long)cols);
    const size_t min_row = (size_t)(cols / kQK) * (size_t)block_bytes_of(ggml_type);
    if (row_bytes < min_row || (row_bytes & 1)) return fail(MQ_ERR_INVALID, "mq_weight_upload: row_bytes %zu < %zu or odd", row_bytes, min_row);
    if (rows <= 0 || n_experts <= 0) return fail(MQ_ERR_INVALID, "mq_weight_upload: rows and n_experts must be positive");
    // bytes read from the host: checked products (the shape may come from a file header)
    size_t one = 0, raw_total = 0;
    bool overflow = __builtin_mul_overflow(row_bytes, (size_t)rows, &one);
    if (n_experts > 1) {
        if (!overflow && expert_bytes < one) return fail(MQ_ERR_INVALID, "mq_weight_upload: expert_bytes too small");
        overflow = overflow || __builtin_mul_overflow(expert_bytes, (size_t)(n_experts - 1), &raw_total) ||
                   __builtin_add_overflow(raw_total, one, &raw_total);
    } else {
        raw_total = one - row_bytes + min_row;
    }
    if (overflow || raw_total > (size_t(1) << 46)) return fail(MQ_ERR_INVALID, "mq_weight_upload: tensor size overflows");
    mq_weight* w = nullptr;
    if (int rc = alloc_weight(ggml_type, rows, cols, n_experts, &w)) return rc;
    void* raw = nullptr;
    hipError_t e = hipMalloc(&raw, raw_total);
    if (e == hipSuccess) e = hipMemcpy(raw, q4k_host, raw_total, hipMemcpyHostToDevice);
    if (e == hipSuccess)
        e = launch_tile_weights((const uint8_t*)raw, rows, w->nb, ggml_type, row_bytes, expert_bytes, n_experts, w->data,
                                w->expert_bytes, nullptr);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (raw) (void)hipFree(raw);
    if (e != hipSuccess) {
        mq_weight_free(w);
        return hip_fail(e, "mq_weight_upload");
    }
    *out = w;
    return MQ_OK;
}

int mq_weight_synthetic(uint64_t seed, int64_t rows, int64_t cols, int64_t n_experts, mq_weight** out) {
    return mq_weight_synthetic_typed(kTypeQ4K, seed, rows, cols, n_experts, out);
}

int mq_weight_synthetic_typed(int ggml_type, uint64_t seed, int64_t rows, int64_t cols, int64_t n_experts,
                              mq_weight** out) {
    if (int rc = check_ready()) return rc;
    mq_weight* w = nullptr;
    if (int rc = alloc_weight(ggml_type, rows, cols, n_experts, &w)) return rc;
    hipError_t e = launch_synth_weights(seed, rows, w->nb, ggml_type, n_experts, w->data, w->expert_bytes, nullptr);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        mq_weight_free(w);
        return hip_fail(e, "mq_weight_synthetic");
    }
    *out = w;
    return MQ_OK;
}

int mq_weight_download(const mq_weight* w, void* q4k_host, size_t row_bytes, size_t expert_bytes) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_weight_download", true)) return rc;
    if (!q4k_host) return fail(MQ_ERR_INVALID, "mq_weight_download: null host pointer");
    const size_t min_row = (size_t)w->nb * (size_t)block_bytes_of(w->type);
    if (row_bytes < min_row || (row_bytes & 1)) return fail(MQ_ERR_INVALID, "mq_weight_download: bad row_bytes");
    if (w->n_experts > 1 && expert_bytes < row_bytes * (size_t)w->rows) return fail(MQ_ERR_INVALID, "mq_weight_download: bad expert_bytes");
    const size_t raw_total = w->n_experts > 1 ? expert_bytes * (size_t)(w->n_experts - 1) + row_bytes * (size_t)w->rows
                                              : row_bytes * (size_t)(w->rows - 1) + min_row;
    void* raw = nullptr;
    hipError_t e = hipMalloc(&raw, raw_total);
    if (e == hipSuccess) e = hipMemcpy(raw, q4k_host, raw_total, hipMemcpyHostToDevice);  // keep caller's padding bytes
    if (e == hipSuccess)
        e = launch_untile_weights(w->data, w->rows, w->nb, w->type, row_bytes, expert_bytes, w->n_experts, (uint8_t*)raw,
                                  w->expert_bytes, nullptr);
    if (e == hipSuccess) e = hipMemcpy(q4k_host, raw, raw_total, hipMemcpyDeviceToHost);
    if (raw) (void)hipFree(raw);
    if (e != hipSuccess) return hip_fail(e, "mq_weight_download");
    return MQ_OK;
}

int mq_weight_shape(const mq_weight* w, int64_t* rows, int64_t* cols, int64_t* n_experts, size_t* device_bytes) {
    if (int rc = check_weight(w, "mq_weight_shape", true)) return rc;
    if (rows) *rows = w->rows;
    if (cols) *cols = w->cols;
    if (n_experts) *n_experts = w->n_experts;
    if (device_bytes) *device_bytes = w->total_bytes;
    return MQ_OK;
}

int mq_weight_type(const mq_weight* w) { return w ? w->type : -1; }

int mq_weight_free(mq_weight* w) {
    if (!w) return MQ_OK;
    if (w->data) (void)hipFree(w->data);
    delete w;
    return MQ_OK;
}

// ---------------------------------------------------------------------------------- quantizer
int mq_quantize_q8k(const float* x_dev, int64_t n, int64_t ldx, int64_t k, void* q8_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (k <= 0 || k % kQK) return fail(MQ_ERR_INVALID, "mq_quantize_q8k: k %lld is not a positive multiple of 256", (long long)k);
    if (int rc = check_x(x_dev, n, ldx, k, "mq_quantize_q8k")) return rc;
    if (n == 0) return MQ_OK;
    if (!q8_dev || (reinterpret_cast<uintptr_t>(q8_dev) & 3u)) return fail(MQ_ERR_INVALID, "mq_quantize_q8k: output must be non-null and 4-byte aligned");
    MQ_HIP(launch_quantize_q8k(x_dev, n, ldx, k, q8_dev, (size_t)(k / kQK) * kQ8Block, nullptr, nullptr, (hipStream_t)stream));
    return MQ_OK;
}

// ---------------------------------------------------------------------------------- dense matmul
static int matmul_from_ws(const mq_weight* w, int64_t n, float* y, int64_t ldy, int32_t* dbg_dot, int32_t* dbg_min,
                          hipStream_t s) {
    if (n == 0) return MQ_OK;
    MatmulArgs a;
    a.w0 = w->data;
    a.wtype = w->type;
    a.rows = w->rows;
    a.nb = w->nb;
    a.aq = (const uint8_t*)g.aq.ptr;
    a.ad = (const float*)g.ad.ptr;
    a.n = n;
    a.y = y;
    a.ldy = ldy;
    a.dbg_dot = dbg_dot;
    a.dbg_min = dbg_min;
    MQ_HIP(census_launch(a, s));
    return MQ_OK;
}

// Activation rows from which the matrix-core GEMM beats re-streaming the weights per 16-row chunk: 48 in general,
// 17 for matrices of 24 MB and more (14336 x 4096 and 4096 x 14336: 19 against 24 us at 17 rows, 21 against 35-38 us
// at 47; 4096 x 4096: 17.4 against 14.1 us at 17 rows, 17.9 against 14.6 at 47).  Q4_K products of up to 32 rows go to
// skinny16_kernel ahead of both (skinny16_takes: gate/up of a 4096 -> 14336 FFN 41 -> 22 us at 17 to 32 rows,
// 4096 x 4096 11.5 -> 9.5 us).  The 17-row rule holds for Q5_K and Q6_K matrices of that many weights as well (4096 x
// 14336: Q5_K 28.7 / 30.7 / 42.5 us in 16-row passes against 22.3 / 22.6 / 25.3 on the GEMM at 17 / 32 / 47 rows, Q6_K 30.7 /
// 33.2 / 46.3 against 28.2 / 28.5 / 32.3; 4096 x 4096 stays: 12.1 against 14.1 us at 17 rows, 16.8 against 15.9 at 47).
constexpr int64_t kPrefillMinRows = 48;
constexpr int64_t kPrefillMinRowsLarge = 17;
constexpr int64_t kPrefillLargeBytes = 24ll << 20;
static bool prefill_applies(const mq_weight* w, int64_t n) {
    if (w->type != kTypeQ4K && w->type != kTypeQ5K && w->type != kTypeQ6K) return false;
    return n >= kPrefillMinRows || (n >= kPrefillMinRowsLarge && w->rows * w->nb * (int64_t)kQ4Block >= kPrefillLargeBytes);
}
constexpr int64_t kGemvFusedMaxRows = 4;  // widest product whose quantizer runs inside the GEMV kernel (measured: 8 loses)
// At three and four rows the quantizer inside pays only for a small matrix with short rows: 2048x2048 and 2560x2048 take
// 5.3 / 5.6 us against 5.8 for a quantizer launch and the LDS-staged product; 1024x4096 6.6 / 7.3 against 6.6,
// 4096x4096 7.5 / 8.3 against 7.2, 8192x2048 7.5 / 8.2 against 7.0.
static bool gemvn_fused_pays(const mq_weight* w, int64_t n) {
    return n <= 2 || (w->nb <= 8 && w->rowtiles * w->nb <= 1536);
}
// Widest product that also runs the residual add and the RMSNorm inside the GEMV kernel: every workgroup repeats the
// rows' norm, about 1.25 us per row.  Decoder layer (2048 hidden, 64 experts) with the norm inside / as a launch of
// its own that emits Q8_K for the LDS-staged product: 36.0 / 36.2 us at two rows, 43.9 / 42.4 at three, 48.6 / 45.7 at four.
constexpr int64_t kNormFusedMaxRows = 2;

static int gemm_locked(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                       hipStream_t s) {
    if (n == 0) return MQ_OK;
    MQ_HIP(g.ap.reserve(pmajor_bytes(n, w->nb)));
    MQ_HIP(launch_quantize_q8k_pmajor(x_dev, n, ldx, w->cols, (uint8_t*)g.ap.ptr, s));
    const size_t part_bytes = prefill_part_bytes(w->rows, w->nb, n, w->type);
    if (part_bytes) MQ_HIP(g.kpart.reserve(part_bytes));
    MQ_HIP(launch_prefill_gemm(w->data, w->type, w->rows, w->nb, (const uint8_t*)g.ap.ptr, n, y_dev, ldy,
                               part_bytes ? (float*)g.kpart.ptr : nullptr, s));
    return MQ_OK;
}

// Wide FFN on the matrix-core GEMM: gate and up products into the two halves of g.mid2, their SwiGLU formed by the
// quantizer of the down product (and written to h_dev / g.mid as fp32 as well), then the down product if asked for.
static int ffn_wide_locked(const mq_weight* gate, const mq_weight* up, const mq_weight* down, const float* x_dev, int64_t n,
                           int64_t ldx, int silu_mode, float* h_dev, int64_t ldh, float* y_dev, int64_t ldy, hipStream_t s) {
    const int64_t inter = gate->rows;
    MQ_HIP(g.ap.reserve(pmajor_bytes(n, gate->nb)));
    MQ_HIP(launch_quantize_q8k_pmajor(x_dev, n, ldx, gate->cols, (uint8_t*)g.ap.ptr, s));
    if (g_gemm_pair && gate->type == kTypeQ4K && up->type == kTypeQ4K && prefill_pair_applies(gate->type, inter, gate->nb, n)) {
        // gate and up in one launch that stores silu(gate) * up: no fp32 planes, no pass that reads them back
        MQ_HIP(launch_prefill_gemm_pair(gate->data, up->data, gate->type, inter, gate->nb, (const uint8_t*)g.ap.ptr, n, silu_mode, h_dev, ldh, s));
        if (!down) return MQ_OK;
        MQ_HIP(g.ap2.reserve(pmajor_bytes(n, down->nb)));
        MQ_HIP(launch_quantize_q8k_pmajor(h_dev, n, ldh, inter, (uint8_t*)g.ap2.ptr, s));
        const size_t part2 = prefill_part_bytes(down->rows, down->nb, n, down->type);
        if (part2) MQ_HIP(g.kpart.reserve(part2));
        MQ_HIP(launch_prefill_gemm(down->data, down->type, down->rows, down->nb, (const uint8_t*)g.ap2.ptr, n, y_dev, ldy,
                                   part2 ? (float*)g.kpart.ptr : nullptr, s));
        return MQ_OK;
    }
    MQ_HIP(g.mid2.reserve(2 * (size_t)n * (size_t)inter * sizeof(float)));
    float* gbuf = (float*)g.mid2.ptr;
    float* ubuf = gbuf + (size_t)n * (size_t)inter;
    const size_t part_bytes = prefill_part_bytes(inter, gate->nb, n, gate->type);
    if (part_bytes) MQ_HIP(g.kpart.reserve(part_bytes));
    float* part = part_bytes ? (float*)g.kpart.ptr : nullptr;
    MQ_HIP(launch_prefill_gemm(gate->data, gate->type, inter, gate->nb, (const uint8_t*)g.ap.ptr, n, gbuf, inter, part, s));
    MQ_HIP(launch_prefill_gemm(up->data, up->type, inter, up->nb, (const uint8_t*)g.ap.ptr, n, ubuf, inter, part, s));
    if (!down && inter % kQK) {  // SwiGLU rows that do not divide into super-blocks: nothing to quantize them for
        MQ_HIP(launch_silu_mul(gbuf, ubuf, n, inter, inter, inter, h_dev, ldh, silu_mode, s));
        return MQ_OK;
    }
    if (!down) {  // SwiGLU rows only: the quantizer's fp32 side output is the result
        MQ_HIP(g.ap2.reserve(pmajor_bytes(n, inter / kQK)));
        MQ_HIP(launch_swiglu_quantize_q8k_pmajor(gbuf, ubuf, n, inter, inter, silu_mode, h_dev, ldh, (uint8_t*)g.ap2.ptr, s));
        return MQ_OK;
    }
    MQ_HIP(g.ap2.reserve(pmajor_bytes(n, down->nb)));
    MQ_HIP(launch_swiglu_quantize_q8k_pmajor(gbuf, ubuf, n, inter, inter, silu_mode, h_dev, ldh, (uint8_t*)g.ap2.ptr, s));
    const size_t part2 = prefill_part_bytes(down->rows, down->nb, n, down->type);
    if (part2) MQ_HIP(g.kpart.reserve(part2));
    MQ_HIP(launch_prefill_gemm(down->data, down->type, down->rows, down->nb, (const uint8_t*)g.ap2.ptr, n, y_dev, ldy,
                               part2 ? (float*)g.kpart.ptr : nullptr, s));
    return MQ_OK;
}

// Q8_0 weights: the activations are quantized to Q8_0 as well (codes into g.aq in the A-major order, fp16 scales
// into g.ad), then one launch.
static int mul_mat_q80_locked(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                              int32_t* dbg_sum, hipStream_t s) {
    if ((ldx & 3) || (reinterpret_cast<uintptr_t>(x_dev) & 15u))
        return fail(MQ_ERR_INVALID, "Q8_0 product: activation rows must be 16-byte aligned (ldx %% 4 == 0)");
    MQ_HIP(g.aq.reserve(aq_bytes(n, w->nb)));
    MQ_HIP(g.ad.reserve(q80_scale_bytes(n, w->nb)));
    MQ_HIP(launch_quantize_q80(x_dev, n, ldx, w->cols, (uint8_t*)g.aq.ptr, (uint16_t*)g.ad.ptr, s));
    Q80MatmulArgs a;
    a.w = w->data;
    a.rows = w->rows;
    a.nb = w->nb;
    a.aq = (const uint8_t*)g.aq.ptr;
    a.ah = (const uint16_t*)g.ad.ptr;
    a.n = n;
    a.y = y_dev;
    a.ldy = ldy;
    a.dbg_sum = dbg_sum;
    MQ_HIP(launch_q80_matmul(a, s));
    return MQ_OK;
}

int mq_gemm_q4k(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_gemm_q4k")) return rc;
    if (w->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_gemm_q4k: weight is an expert stack");
    if (w->type != kTypeQ4K && w->type != kTypeQ5K && w->type != kTypeQ6K)
        return fail(MQ_ERR_UNSUPPORTED, "mq_gemm_q4k: the matrix-core GEMM takes Q4_K, Q5_K and Q6_K weights only");
    if (int rc = check_x(x_dev, n, ldx, w->cols, "mq_gemm_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!y_dev || ldy < w->rows) return fail(MQ_ERR_INVALID, "mq_gemm_q4k: null output or ldy < rows");
    Entry entry((hipStream_t)stream);
    if (entry.rc) return entry.rc;
    return gemm_locked(w, x_dev, n, ldx, y_dev, ldy, (hipStream_t)stream);
}

int mq_mul_mat_q4k(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                   void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_mul_mat_q4k", true)) return rc;
    if (w->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k: weight is an expert stack; use mq_mul_mat_id_q4k");
    if (int rc = check_x(x_dev, n, ldx, w->cols, "mq_mul_mat_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!y_dev || ldy < w->rows) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k: null output or ldy < rows");
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    if (w->type == kTypeQ80) return mul_mat_q80_locked(w, x_dev, n, ldx, y_dev, ldy, nullptr, s);
    if (prefill_applies(w, n) && !skinny16_takes(w, n, false)) return gemm_locked(w, x_dev, n, ldx, y_dev, ldy, s);
    if (n == 1 && w->type == kTypeQ4K) {  // single row, short K per wave: the quantizer runs inside the GEMV kernel
        const int waves = pick_waves(w->nb, w->rowtiles);
        if (gemv1_fused_applies(w->nb, waves)) {
            MQ_HIP(launch_gemv1_fused(w->data, w->rows, w->nb, x_dev, y_dev, waves, s));
            return MQ_OK;
        }
    }
    if (n <= kGemvFusedMaxRows && w->type == kTypeQ4K && gemvn_fused_pays(w, n)) {  // a few rows, short K per wave: the same with the rows' codes going through LDS
        const int waves = pick_waves(w->nb, w->rowtiles);
        if (gemv1_fused_applies(w->nb, waves)) {
            MQ_HIP(launch_gemvn_fused(w->data, w->rows, w->nb, x_dev, ldx, nullptr, nullptr, 0.0f, nullptr, y_dev, ldy, (int)n, false, waves, s));
            return MQ_OK;
        }
    }
    // single row (long K per wave), or a few rows where the LDS-staged kernel applies: the quantizer runs inside the product
    if ((n == 1 && !(reinterpret_cast<uintptr_t>(x_dev) & 15u)) || dense_lds_quantizes(w, x_dev, n, ldx, false)) {
        MatmulArgs a;
        a.w0 = w->data;
        a.wtype = w->type;
        a.rows = w->rows;
        a.nb = w->nb;
        a.xf = x_dev;
        a.ldx = ldx;
        a.n = n;
        a.y = y_dev;
        a.ldy = ldy;
        MQ_HIP(census_launch(a, s));
        return MQ_OK;
    }
    if (skinny16_takes(w, n, false)) {  // nine to 64 rows as one to four tiles of sixteen
        if (int rc = quantize_into_tile16(x_dev, n, ldx, w->cols, s)) return rc;
        MatmulArgs a;
        a.w0 = w->data;
        a.wtype = w->type;
        a.rows = w->rows;
        a.nb = w->nb;
        a.ap = (const uint8_t*)g.ap.ptr;
        a.n = n;
        a.y = y_dev;
        a.ldy = ldy;
        MQ_HIP(census_launch(a, s));
        return MQ_OK;
    }
    if (int rc = quantize_into(g.aq, g.ad, x_dev, n, ldx, w->cols, s)) return rc;
    return matmul_from_ws(w, n, y_dev, ldy, nullptr, nullptr, s);
}

int mq_mul_mat_q4k_multi(const mq_weight* const* w, int count, const float* x_dev, float* const* y_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (count < 0 || count > kGemvMultiMax) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_multi: count %d is outside [0, %d]", count, kGemvMultiMax);
    if (count == 0) return MQ_OK;
    if (!w || !y_dev) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_multi: null weight or output list");
    for (int i = 0; i < count; ++i) {
        if (int rc = check_weight(w[i], "mq_mul_mat_q4k_multi", true)) return rc;
        if (w[i]->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_multi: weight %d is an expert stack", i);
        if (w[i]->cols != w[0]->cols) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_multi: weight %d has %lld columns, weight 0 has %lld", i, (long long)w[i]->cols, (long long)w[0]->cols);
        if (!y_dev[i]) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_multi: output %d is null", i);
    }
    if (int rc = check_x(x_dev, 1, w[0]->cols, w[0]->cols, "mq_mul_mat_q4k_multi")) return rc;
    hipStream_t s = (hipStream_t)stream;
    // Matrices that take the single-row kernel with the quantizer inside share launches, one per wave split (a launch
    // has one workgroup shape, and every matrix keeps the split -- so the bits -- of a launch of its own); the others
    // (another type, long rows, a misaligned x) go through mq_mul_mat_q4k one by one.
    bool taken[kGemvMultiMax] = {};
    for (int i = 0; i < count; ++i) {
        if (taken[i]) continue;
        const int waves = pick_waves(w[i]->nb, w[i]->rowtiles);
        const bool fused = w[i]->type == kTypeQ4K && gemv1_fused_applies(w[i]->nb, waves);
        if (!fused) {
            taken[i] = true;
            if (int rc = mq_mul_mat_q4k(w[i], x_dev, 1, w[i]->cols, y_dev[i], w[i]->rows, stream)) return rc;
            continue;
        }
        Gemv1MultiArgs a;
        a.nb = w[i]->nb;
        a.x = x_dev;
        for (int j = i; j < count; ++j) {
            if (taken[j] || w[j]->type != kTypeQ4K || pick_waves(w[j]->nb, w[j]->rowtiles) != waves) continue;
            taken[j] = true;
            a.w[a.count] = w[j]->data, a.y[a.count] = y_dev[j], a.rows[a.count] = w[j]->rows;
            ++a.count;
        }
        Entry entry(s);
        if (entry.rc) return entry.rc;
        MQ_HIP(launch_gemv1_multi(a, waves, s));
    }
    return MQ_OK;
}

int mq_mul_mat_q4k_noalloc(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, float* y_dev, int64_t ldy,
                           void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_mul_mat_q4k_noalloc")) return rc;
    if (w->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_noalloc: weight is an expert stack");
    if (int rc = check_x(x_dev, n, ldx, w->cols, "mq_mul_mat_q4k_noalloc")) return rc;
    if (n > kNoAllocMaxRows || w->cols > kNoAllocMaxCols)
        return fail(MQ_ERR_UNSUPPORTED, "mq_mul_mat_q4k_noalloc: %lld rows of %lld columns exceed the fixed scratch (at most %lld rows of %lld columns)",
                    (long long)n, (long long)w->cols, (long long)kNoAllocMaxRows, (long long)kNoAllocMaxCols);
    if (n == 0) return MQ_OK;
    if (!y_dev || ldy < w->rows) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_noalloc: null output or ldy < rows");
    unsigned char* ws = g.device >= 0 && g.device < kMaxDevices ? g_scratch_ptr[g.device] : nullptr;
    if (!ws) return fail(MQ_ERR_STATE, "mq_mul_mat_q4k_noalloc: no scratch address for device %d (mq_init looks it up)", g.device);
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    uint8_t* aq = ws;
    float* ad = reinterpret_cast<float*>(ws + kNoAllocAqBytes);
    MatmulArgs a;
    a.w0 = w->data;
    a.wtype = w->type;
    a.rows = w->rows;
    a.nb = w->nb;
    // Every byte of the scratch that the product reads is written by this call's quantizer (slots past row n read
    // row n - 1; rows past n of a tile of sixteen are written as zeros), so nothing of an earlier call is seen and
    // nothing needs clearing.
    static_assert((kNoAllocMaxCols / mq::kQK) * 4688 <= kNoAllocAqBytes + kNoAllocAdBytes, "the rows' tiles of sixteen fit the scratch as well");
    if (skinny16_takes(w, n, false)) {  // nine to sixteen rows: one P-major tile per super-block, in the same scratch
        MQ_HIP(launch_quantize_q8k_pmajor(x_dev, n, ldx, w->cols, ws, s));
        a.ap = ws;
    } else {
        MQ_HIP(launch_quantize_q8k(x_dev, n, ldx, w->cols, nullptr, 0, aq, ad, s));
        a.aq = aq;
        a.ad = ad;
    }
    a.n = n;
    a.y = y_dev;
    a.ldy = ldy;
    MQ_HIP(dense_launch(a, s));
    return MQ_OK;
}

int mq_rmsnorm_mul_mat_q4k(const mq_weight* w, const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n,
                           float eps, float* sum_out_dev, float* y_dev, int64_t ldy, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_rmsnorm_mul_mat_q4k")) return rc;
    if (w->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_rmsnorm_mul_mat_q4k: weight is an expert stack");
    if (int rc = check_x(x_dev, n, w->cols, w->cols, "mq_rmsnorm_mul_mat_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!y_dev || ldy < w->rows) return fail(MQ_ERR_INVALID, "mq_rmsnorm_mul_mat_q4k: null output or ldy < rows");
    if (sum_out_dev && (sum_out_dev == x_dev || sum_out_dev == delta_dev))
        return fail(MQ_ERR_INVALID, "mq_rmsnorm_mul_mat_q4k: the sum must not overwrite x or delta (every workgroup reads them)");
    if ((reinterpret_cast<uintptr_t>(delta_dev) | reinterpret_cast<uintptr_t>(weight_dev) | reinterpret_cast<uintptr_t>(sum_out_dev)) & 15u)
        return fail(MQ_ERR_INVALID, "mq_rmsnorm_mul_mat_q4k: rows must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    if (n == 1 && w->type == kTypeQ4K) {  // one row, short K per wave: norm and quantizer run inside the GEMV kernel
        const int waves = pick_waves(w->nb, w->rowtiles);
        if (gemv1_fused_applies(w->nb, waves)) {
            MQ_HIP(launch_gemv1_norm_fused(w->data, w->rows, w->nb, x_dev, delta_dev, weight_dev, eps, sum_out_dev, y_dev, waves, s));
            return MQ_OK;
        }
    }
    if (n <= kNormFusedMaxRows && w->type == kTypeQ4K) {
        const int waves = pick_waves(w->nb, w->rowtiles);
        if (gemv1_fused_applies(w->nb, waves)) {
            MQ_HIP(launch_gemvn_fused(w->data, w->rows, w->nb, x_dev, w->cols, delta_dev, weight_dev, eps, sum_out_dev, y_dev, ldy, (int)n, true,
                                      waves, s));
            return MQ_OK;
        }
    }
    // Seventeen to 64 rows where mq_mul_mat_q4k takes them as tiles of sixteen: the normalised rows as fp32, their
    // quantizer, the same launch (up to sixteen rows the norm's own Q8_K output and the kernels with token tiles of
    // eight below cost a launch less; the bits are the same)
    const bool tiles16 = n > 16 && skinny16_takes(w, n, false);
    if (tiles16 || prefill_applies(w, n)) {
        // ... and prefill widths: the normalised rows as fp32, then the matrix-core GEMM (its quantizer reads them)
        MQ_HIP(g.mid.reserve((size_t)n * (size_t)w->cols * sizeof(float)));
        MQ_HIP(launch_add_rmsnorm(x_dev, delta_dev, weight_dev, n, w->cols, eps, sum_out_dev, (float*)g.mid.ptr, nullptr, nullptr, s));
        if (!tiles16) return gemm_locked(w, (const float*)g.mid.ptr, n, w->cols, y_dev, ldy, s);
        if (int rc = quantize_into_tile16((const float*)g.mid.ptr, n, w->cols, w->cols, s)) return rc;
        MatmulArgs a;
        a.w0 = w->data;
        a.wtype = w->type;
        a.rows = w->rows;
        a.nb = w->nb;
        a.ap = (const uint8_t*)g.ap.ptr;
        a.n = n;
        a.y = y_dev;
        a.ldy = ldy;
        MQ_HIP(census_launch(a, s));
        return MQ_OK;
    }
    const int64_t nb = w->cols / kQK;
    MQ_HIP(g.aq.reserve(aq_bytes(n, nb)));
    MQ_HIP(g.ad.reserve(ad_count(n, nb) * sizeof(float)));
    MQ_HIP(launch_add_rmsnorm(x_dev, delta_dev, weight_dev, n, w->cols, eps, sum_out_dev, nullptr, (uint8_t*)g.aq.ptr, (float*)g.ad.ptr, s));
    return matmul_from_ws(w, n, y_dev, ldy, nullptr, nullptr, s);
}

int mq_mul_mat_q4k_q8k(const mq_weight* w, const void* q8_dev, int64_t n, size_t q8_row_bytes, float* y_dev,
                       int64_t ldy, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_mul_mat_q4k_q8k")) return rc;
    if (w->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_q8k: weight is an expert stack");
    if (n == 0) return MQ_OK;
    if (!q8_dev || !y_dev || n < 0 || ldy < w->rows) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_q8k: bad arguments");
    if (q8_row_bytes < (size_t)w->nb * kQ8Block || (q8_row_bytes & 3) || (reinterpret_cast<uintptr_t>(q8_dev) & 3u))
        return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_q8k: q8 rows too short or not 4-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    MQ_HIP(g.aq.reserve(aq_bytes(n, w->nb)));
    MQ_HIP(g.ad.reserve(ad_count(n, w->nb) * sizeof(float)));
    MQ_HIP(launch_q8k_to_amajor(q8_dev, n, q8_row_bytes, w->cols, (uint8_t*)g.aq.ptr, (float*)g.ad.ptr, s));
    return matmul_from_ws(w, n, y_dev, ldy, nullptr, nullptr, s);
}

int mq_mul_mat_q4k_host(const mq_weight* w, const float* x_host, int64_t n, int64_t ldx, float* y_host, int64_t ldy) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_mul_mat_q4k_host", true)) return rc;
    if (!x_host || !y_host || n < 0 || ldx < w->cols || ldy < w->rows) return fail(MQ_ERR_INVALID, "mq_mul_mat_q4k_host: bad arguments");
    if (n == 0) return MQ_OK;
    // The lock is held from the first staging copy to the last: a second thread's copy must not land between this
    // call's copy and its launch.  Host rows go through page-locked staging buffers, so that both copies are
    // asynchronous on the stream and the call synchronises once, at its end.
    Entry entry(nullptr);
    if (entry.rc) return entry.rc;
    const size_t in_bytes = (size_t)n * (size_t)w->cols * sizeof(float), out_bytes = (size_t)n * (size_t)w->rows * sizeof(float);
    MQ_HIP(g.stage_in.reserve(in_bytes));
    MQ_HIP(g.stage_out.reserve(out_bytes));
    MQ_HIP(g.pin_in.reserve(in_bytes));
    MQ_HIP(g.pin_out.reserve(out_bytes));
    float* xin = (float*)g.stage_in.ptr;
    float* yout = (float*)g.stage_out.ptr;
    for (int64_t m = 0; m < n; ++m) memcpy((float*)g.pin_in.ptr + m * w->cols, x_host + m * ldx, (size_t)w->cols * sizeof(float));
    MQ_HIP(hipMemcpyAsync(xin, g.pin_in.ptr, in_bytes, hipMemcpyHostToDevice, nullptr));
    if (int rc = mq_mul_mat_q4k(w, xin, n, w->cols, yout, w->rows, nullptr)) return rc;
    MQ_HIP(hipMemcpyAsync(g.pin_out.ptr, yout, out_bytes, hipMemcpyDeviceToHost, nullptr));
    MQ_HIP(hipStreamSynchronize(nullptr));
    for (int64_t m = 0; m < n; ++m) memcpy(y_host + m * ldy, (const float*)g.pin_out.ptr + m * w->rows, (size_t)w->rows * sizeof(float));
    return MQ_OK;
}

int mq_debug_block_sums(const mq_weight* w, const float* x_dev, int64_t n, int64_t ldx, int32_t* dot_scaled_dev,
                        int32_t* min_dot_dev, float* y_dev, int64_t ldy, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_debug_block_sums", true)) return rc;
    if (w->n_experts != 1) return fail(MQ_ERR_INVALID, "mq_debug_block_sums: dense weights only");
    if (int rc = check_x(x_dev, n, ldx, w->cols, "mq_debug_block_sums")) return rc;
    if (n == 0) return MQ_OK;
    if (!dot_scaled_dev || (!min_dot_dev && w->type != kTypeQ80) || !y_dev || ldy < w->rows)
        return fail(MQ_ERR_INVALID, "mq_debug_block_sums: null output");
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    if (w->type == kTypeQ80) return mul_mat_q80_locked(w, x_dev, n, ldx, y_dev, ldy, dot_scaled_dev, s);
    if (int rc = quantize_into(g.aq, g.ad, x_dev, n, ldx, w->cols, s)) return rc;
    return matmul_from_ws(w, n, y_dev, ldy, dot_scaled_dev, min_dot_dev, s);
}

// ---------------------------------------------------------------------------------- dense FFN
int mq_ffn_swiglu_q4k(const mq_weight* gate, const mq_weight* up, const mq_weight* down, const float* x_dev,
                      int64_t n, float* y_dev, int silu_mode, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(gate, "mq_ffn_swiglu_q4k(gate)")) return rc;
    if (int rc = check_weight(up, "mq_ffn_swiglu_q4k(up)")) return rc;
    if (int rc = check_weight(down, "mq_ffn_swiglu_q4k(down)")) return rc;
    const int64_t hidden = gate->cols, inter = gate->rows;
    if (up->cols != hidden || up->rows != inter || down->cols != inter || down->rows != hidden || gate->n_experts != 1 ||
        up->n_experts != 1 || down->n_experts != 1)
        return fail(MQ_ERR_INVALID, "mq_ffn_swiglu_q4k: gate/up must be [inter][hidden] and down [hidden][inter]");
    if (up->type != gate->type) return fail(MQ_ERR_INVALID, "mq_ffn_swiglu_q4k: gate and up must have one quantization type");
    if (inter % kQK) return fail(MQ_ERR_INVALID, "mq_ffn_swiglu_q4k: inter %lld is not a multiple of 256", (long long)inter);
    if (silu_mode < 0 || silu_mode > 2) return fail(MQ_ERR_INVALID, "mq_ffn_swiglu_q4k: silu_mode %d", silu_mode);
    if (int rc = check_x(x_dev, n, hidden, hidden, "mq_ffn_swiglu_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!y_dev) return fail(MQ_ERR_INVALID, "mq_ffn_swiglu_q4k: null output");
    if (n == 0) return MQ_OK;
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    const bool gateup16 = skinny16_takes(gate, n, true);  // up to 64 rows: gate/up on the decode arithmetic below
    if (!gateup16 && prefill_applies(gate, n) && prefill_applies(down, n)) {  // wide: the matrix-core GEMM, three times
        MQ_HIP(g.mid.reserve((size_t)n * (size_t)inter * sizeof(float)));
        return ffn_wide_locked(gate, up, down, x_dev, n, hidden, silu_mode, (float*)g.mid.ptr, inter, y_dev, hidden, s);
    }
    // One row: both quantizers run inside the products (two launches instead of four, the same bits).
    const bool one_row = n == 1 && !(reinterpret_cast<uintptr_t>(x_dev) & 15u);
    const bool inline_quant = one_row || dense_lds_quantizes(gate, x_dev, n, hidden, true);
    const bool tile16 = !inline_quant && skinny16_takes(gate, n, true);
    if (tile16) {
        if (int rc = quantize_into_tile16(x_dev, n, hidden, hidden, s)) return rc;
    } else if (!inline_quant) {
        if (int rc = quantize_into(g.aq, g.ad, x_dev, n, hidden, hidden, s)) return rc;
    }
    MQ_HIP(g.mid.reserve((size_t)n * (size_t)inter * sizeof(float)));
    MatmulArgs a;
    a.w0 = gate->data;
    a.wtype = gate->type;
    a.w1 = up->data;
    a.rows = inter;
    a.nb = gate->nb;
    if (inline_quant) {
        a.xf = x_dev;
        a.ldx = hidden;
    } else if (tile16) {
        a.ap = (const uint8_t*)g.ap.ptr;
    } else {
        a.aq = (const uint8_t*)g.aq.ptr;
        a.ad = (const float*)g.ad.ptr;
    }
    a.n = n;
    a.y = (float*)g.mid.ptr;
    a.ldy = inter;
    a.swiglu = 1;
    a.silu_mode = silu_mode;
    MQ_HIP(census_launch(a, s));
    // The SwiGLU output is re-quantized by a launch of its own: the kernel's fused re-quantization (last
    // workgroup per 256-row block) serialises n rows per block at the kernel's tail and measures slower here.
    const bool inline_quant_down = one_row || dense_lds_quantizes(down, (const float*)g.mid.ptr, n, inter, false);
    const bool tile16_down = !inline_quant_down && skinny16_takes(down, n, false);  // (g.ap again: the gate/up launch ahead on the stream has read it)
    // beyond the rows the decode kernels take for this matrix (its rows are too long to pass through LDS): the GEMM on the SwiGLU rows
    if (!tile16_down && prefill_applies(down, n)) return gemm_locked(down, (const float*)g.mid.ptr, n, inter, y_dev, hidden, s);
    if (tile16_down) {
        if (int rc = quantize_into_tile16((const float*)g.mid.ptr, n, inter, inter, s)) return rc;
    } else if (!inline_quant_down) {
        if (int rc = quantize_into(g.aq2, g.ad2, (const float*)g.mid.ptr, n, inter, inter, s)) return rc;
    }
    MatmulArgs d;
    d.w0 = down->data;
    d.wtype = down->type;
    d.rows = hidden;
    d.nb = down->nb;
    if (inline_quant_down) {
        d.xf = (const float*)g.mid.ptr;
        d.ldx = inter;
    } else if (tile16_down) {
        d.ap = (const uint8_t*)g.ap.ptr;
    } else {
        d.aq = (const uint8_t*)g.aq2.ptr;
        d.ad = (const float*)g.ad2.ptr;
    }
    d.n = n;
    d.y = y_dev;
    d.ldy = hidden;
    MQ_HIP(census_launch(d, s));
    return MQ_OK;
}

// ---------------------------------------------------------------------------------- router / MoE
namespace {
struct RouteWs {  // carved out of g.route
    int32_t* ids;
    float* weights;
    int32_t* group_expert;
    int32_t* group_begin;
    int32_t* n_groups;
    int32_t* entry_token;
    int32_t* entry_k;
    const int32_t* direct_ids = nullptr;  // one token: the grouped kernels read the ids themselves, no lists
};
int carve_route(int64_t n, int top_k, int64_t n_experts, RouteWs& r) {
    const size_t entries = (size_t)n * (size_t)top_k;
    const size_t groups = (size_t)n_experts + 2;
    const size_t ints = entries * 4 + groups * 2 + 16;
    MQ_HIP(g.route.reserve(ints * 4));
    int32_t* p = (int32_t*)g.route.ptr;
    r.ids = p;
    p += entries;
    r.weights = (float*)p;
    p += entries;
    r.entry_token = p;
    p += entries;
    r.entry_k = p;
    p += entries;
    r.group_expert = p;
    p += groups;
    r.group_begin = p;
    p += groups;
    r.n_groups = p;
    return MQ_OK;
}
}  // namespace

int mq_moe_route_topk(const float* logits_dev, int64_t n_experts, int64_t n, int top_k, int weights_mode,
                      int32_t* ids_dev, float* weights_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (n == 0) return MQ_OK;
    if (!logits_dev || !ids_dev || !weights_dev) return fail(MQ_ERR_INVALID, "mq_moe_route_topk: null pointer");
    if (n < 0 || n_experts <= 0 || n_experts > 2048 || top_k <= 0 || top_k > n_experts || top_k > 8)
        return fail(MQ_ERR_INVALID, "mq_moe_route_topk: need 0 < top_k <= min(8, n_experts) and n_experts <= 2048");
    if (weights_mode < 0 || weights_mode > 2) return fail(MQ_ERR_INVALID, "mq_moe_route_topk: weights_mode %d", weights_mode);
    if (n == 0) return MQ_OK;
    MQ_HIP(launch_route_topk(logits_dev, n_experts, n, top_k, weights_mode, ids_dev, weights_dev, (hipStream_t)stream));
    return MQ_OK;
}

int mq_add_rmsnorm_f32(const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n, int64_t cols,
                       float eps, float* sum_out_dev, float* normed_out_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (n == 0) return MQ_OK;
    if (!x_dev || !normed_out_dev || n < 0 || cols <= 0) return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_f32: bad arguments");
    MQ_HIP(launch_add_rmsnorm(x_dev, delta_dev, weight_dev, n, cols, eps, sum_out_dev, normed_out_dev, nullptr, nullptr,
                              (hipStream_t)stream));
    return MQ_OK;
}

int mq_add_rmsnorm_q8k(const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n, int64_t cols,
                       float eps, float* sum_out_dev, float* normed_out_dev, mq_acts* acts, void* stream) {
    if (int rc = check_ready()) return rc;
    if (!x_dev || !acts || n < 0 || cols <= 0) return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_q8k: bad arguments");
    if (acts->cols != cols || n > acts->max_rows) return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_q8k: the handle holds %lld x %lld, asked for %lld x %lld", (long long)acts->max_rows, (long long)acts->cols, (long long)n, (long long)cols);
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15u) || (normed_out_dev && (reinterpret_cast<uintptr_t>(normed_out_dev) & 15u)))
        return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_q8k: rows must be 16-byte aligned");
    acts->n = n;
    acts->tile16 = false;  // this producer writes the A-major rows only
    MQ_HIP(launch_add_rmsnorm(x_dev, delta_dev, weight_dev, n, cols, eps, sum_out_dev, normed_out_dev, (uint8_t*)acts->aq,
                              (float*)acts->ad, (hipStream_t)stream));
    return MQ_OK;
}

int mq_router_logits_f32(const float* w_dev, int64_t n_experts, int64_t cols, const float* x_dev, int64_t n, int64_t ldx,
                         float* logits_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (!w_dev || !x_dev || !logits_dev || n < 0 || n > 65535 || n_experts <= 0 || cols <= 0 || (cols & 255) || ldx < cols ||
        (ldx & 3) || (reinterpret_cast<uintptr_t>(x_dev) & 15u) || (reinterpret_cast<uintptr_t>(w_dev) & 15u))
        return fail(MQ_ERR_INVALID, "mq_router_logits_f32: need cols %% 256 == 0, 16-byte aligned rows, n <= 65535");
    MQ_HIP(launch_router_logits(w_dev, n_experts, cols, x_dev, n, ldx, logits_dev, (hipStream_t)stream));
    return MQ_OK;
}

int mq_add_rmsnorm_router_f32(const float* x_dev, const float* delta_dev, const float* weight_dev, int64_t n, int64_t cols,
                              float eps, float* sum_out_dev, float* normed_out_dev, const float* router_dev, int64_t n_experts,
                              float* logits_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (n == 0) return MQ_OK;
    if (!x_dev || !router_dev || !logits_dev || n < 0 || n > 65535 || n_experts <= 0 || cols <= 0)
        return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_router_f32: bad arguments");
    if ((cols & 255) || cols > 4096) return fail(MQ_ERR_UNSUPPORTED, "mq_add_rmsnorm_router_f32: cols %lld (a multiple of 256 up to 4096)", (long long)cols);
    if (sum_out_dev && (sum_out_dev == x_dev || sum_out_dev == delta_dev))
        return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_router_f32: the sum must not overwrite x or delta (every workgroup of a row reads them)");
    if ((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(delta_dev) | reinterpret_cast<uintptr_t>(weight_dev) |
         reinterpret_cast<uintptr_t>(sum_out_dev) | reinterpret_cast<uintptr_t>(normed_out_dev) | reinterpret_cast<uintptr_t>(router_dev)) & 15u)
        return fail(MQ_ERR_INVALID, "mq_add_rmsnorm_router_f32: rows must be 16-byte aligned");
    MQ_HIP(launch_add_rmsnorm_router(x_dev, delta_dev, weight_dev, n, cols, eps, sum_out_dev, normed_out_dev, router_dev, n_experts,
                                     logits_dev, (hipStream_t)stream));
    return MQ_OK;
}

int mq_silu_mul_f32(const float* gate_dev, const float* up_dev, int64_t n, int64_t cols, int64_t ld_gate, int64_t ld_up, float* out_dev,
                    int64_t ld_out, int silu_mode, void* stream) {
    if (int rc = check_ready()) return rc;
    if (n == 0 || cols == 0) return MQ_OK;
    if (!gate_dev || !up_dev || !out_dev || n < 0 || cols < 0 || ld_gate < cols || ld_up < cols || ld_out < cols)
        return fail(MQ_ERR_INVALID, "mq_silu_mul_f32: null pointer, negative size or a row stride below cols");
    if (silu_mode < 0 || silu_mode > 2) return fail(MQ_ERR_INVALID, "mq_silu_mul_f32: silu_mode %d", silu_mode);
    MQ_HIP(launch_silu_mul(gate_dev, up_dev, n, cols, ld_gate, ld_up, out_dev, ld_out, silu_mode, (hipStream_t)stream));
    return MQ_OK;
}

int mq_scale_rows_sigmoid_f32(const float* src_dev, int64_t n, int64_t cols, int64_t ld_src, const float* logit_dev, int64_t ld_logit,
                              float* out_dev, int64_t ld_out, void* stream) {
    if (int rc = check_ready()) return rc;
    if (n == 0 || cols == 0) return MQ_OK;
    if (!src_dev || !logit_dev || !out_dev || n < 0 || cols < 0 || ld_src < cols || ld_out < cols || ld_logit < 1)
        return fail(MQ_ERR_INVALID, "mq_scale_rows_sigmoid_f32: null pointer, negative size or a row stride too small");
    MQ_HIP(launch_scale_rows_sigmoid(src_dev, n, cols, ld_src, logit_dev, ld_logit, out_dev, ld_out, (hipStream_t)stream));
    return MQ_OK;
}

int mq_moe_weights_from_logits(const float* logits_dev, int64_t n_experts, int64_t n, const int32_t* ids_dev, int top_k,
                               float* weights_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (n == 0) return MQ_OK;
    if (!logits_dev || !ids_dev || !weights_dev) return fail(MQ_ERR_INVALID, "mq_moe_weights_from_logits: null pointer");
    if (n < 0 || n_experts <= 0 || top_k <= 0 || top_k > 8)
        return fail(MQ_ERR_INVALID, "mq_moe_weights_from_logits: need n_experts > 0 and 0 < top_k <= 8");
    if (n == 0) return MQ_OK;
    MQ_HIP(launch_weights_from_ids(logits_dev, n_experts, n, ids_dev, top_k, weights_dev, (hipStream_t)stream));
    return MQ_OK;
}

// Widths at which an expert product runs on the matrix-core GEMM in its expert-grouped form (see moe_gemm_applies).
static bool moe_gemm_width(const mq_weight* w, int64_t n, int top_k) {
    return (w->type == kTypeQ4K || w->type == kTypeQ5K || w->type == kTypeQ6K) && n >= 192 && n * top_k >= 6 * w->n_experts && w->n_experts <= 4096 && !(w->rows & 3) &&
           !(w->cols & 3);
}

int mq_mul_mat_id_q4k(const mq_weight* w, const float* x_dev, int64_t n, int x_slots, const int32_t* ids_dev,
                      int top_k, float* y_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w, "mq_mul_mat_id_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!ids_dev || !y_dev || top_k <= 0) return fail(MQ_ERR_INVALID, "mq_mul_mat_id_q4k: null pointer or top_k <= 0");
    if (x_slots != 1 && x_slots != top_k) return fail(MQ_ERR_INVALID, "mq_mul_mat_id_q4k: x_slots must be 1 or top_k");
    if (int rc = check_x(x_dev, n * x_slots, w->cols, w->cols, "mq_mul_mat_id_q4k")) return rc;
    if (n == 0) return MQ_OK;
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    // prefill widths: the matrix-core GEMM in its expert-grouped form (see mq_moe_layer_q4k)
    const bool use_gemm = moe_gemm_width(w, n, top_k);
    if (!use_gemm)
        if (int rc = quantize_into(g.aq, g.ad, x_dev, n * x_slots, w->cols, w->cols, s)) return rc;
    RouteWs r;
    if (int rc = carve_route(n, top_k, w->n_experts, r)) return rc;
    // entries with ids outside [0, n_experts) are dropped by the grouping, so clear y first
    MQ_HIP(launch_fill_zero(y_dev, (size_t)n * top_k * (size_t)w->rows, s));
    MQ_HIP(launch_build_groups(ids_dev, n, top_k, w->n_experts, r.group_expert, r.group_begin, r.n_groups,
                               r.entry_token, r.entry_k, s));
    if (use_gemm) {
        const int64_t entries = n * top_k, E = w->n_experts;
        MQ_HIP(g.plan.reserve(moe_gemm_plan_ints(entries, E) * sizeof(int32_t)));
        const int mt = g_moe_item_tiles ? g_moe_item_tiles : moe_gemm_item_tiles(entries, E);  // tiles per item: the plan and every launch reading it
        MQ_HIP(launch_moe_gemm_plan(r.n_groups, r.group_expert, r.group_begin, r.entry_token, r.entry_k, top_k, x_slots != 1, entries, E,
                                    0, 0, (int32_t*)g.plan.ptr, s, mt));
        MQ_HIP(g.ap.reserve(pmajor_bytes(moe_gemm_tiles_max(entries, E) * 16, w->nb)));
        // one row per token (b broadcast over the slots): the rows repeat top_k times -- quantize each once
        if (x_slots == 1) MQ_HIP(g.ap_rows.reserve(pmajor_bytes(n, w->nb)));
        MQ_HIP(launch_quantize_q8k_pmajor_grouped(x_dev, nullptr, false, 0, w->cols, w->cols, entries, E, (const int32_t*)g.plan.ptr,
                                                  (uint8_t*)g.ap.ptr, nullptr, 0, s, x_slots == 1 ? n : 0,
                                                  x_slots == 1 ? (uint8_t*)g.ap_rows.ptr : nullptr));
        MQ_HIP(launch_prefill_gemm_grouped(w->data, w->type, w->expert_bytes, nullptr, w->rows, w->nb, (const uint8_t*)g.ap.ptr, entries, E,
                                           (const int32_t*)g.plan.ptr, true, y_dev, w->rows, s, mt));
        return MQ_OK;
    }
    MatmulArgs a;
    a.w0 = w->data;
    a.wtype = w->type;
    a.rows = w->rows;
    a.nb = w->nb;
    a.expert_bytes = w->expert_bytes;
    a.aq = (const uint8_t*)g.aq.ptr;
    a.ad = (const float*)g.ad.ptr;
    a.n = n;  // widest possible group
    a.y = y_dev;
    a.ldy = w->rows;
    a.grouped = 1;
    a.group_expert = r.group_expert;
    a.group_begin = r.group_begin;
    a.n_groups = r.n_groups;
    a.entry_token = r.entry_token;
    a.entry_k = r.entry_k;
    a.a_tok_stride = x_slots == 1 ? 1 : top_k;  // activation row: token, or token*top_k + k
    a.a_k_stride = x_slots == 1 ? 0 : 1;
    a.y_tok_stride = top_k;                     // output row: token*top_k + k
    a.y_k_stride = 1;
    const int64_t pairs = n * (int64_t)top_k;
    a.max_groups = (int)(pairs < w->n_experts ? pairs : w->n_experts);
    MQ_HIP(census_launch(a, s));
    return MQ_OK;
}

int mq_debug_moe_groups(const float* logits_dev, const int32_t* ids_dev, int64_t n_experts, int64_t n, int top_k,
                        int32_t* triples_dev, int32_t* count_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if ((logits_dev == nullptr) == (ids_dev == nullptr)) return fail(MQ_ERR_INVALID, "mq_debug_moe_groups: pass logits or ids, not both");
    if (!triples_dev || !count_dev) return fail(MQ_ERR_INVALID, "mq_debug_moe_groups: null output");
    if (n <= 0 || top_k <= 0 || top_k > 8 || n_experts <= 0 || n_experts > 2048 || (logits_dev && top_k > n_experts))
        return fail(MQ_ERR_INVALID, "mq_debug_moe_groups: need n > 0, 0 < top_k <= 8, 0 < n_experts <= 2048");
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    RouteWs r;
    if (int rc = carve_route(n, top_k, n_experts, r)) return rc;
    if (ids_dev) {
        MQ_HIP(launch_build_groups(ids_dev, n, top_k, n_experts, r.group_expert, r.group_begin, r.n_groups, r.entry_token, r.entry_k, s));
    } else {
        if (int rc = reserve_counters(4096)) return rc;
        MQ_HIP(launch_route_and_group(logits_dev, n_experts, n, top_k, MQ_ROUTE_FUSED, r.ids, r.weights, (uint32_t*)g.counters.ptr + 4095,
                                      r.group_expert, r.group_begin, r.n_groups, r.entry_token, r.entry_k, true, nullptr, 0, 0,
                                      nullptr, nullptr, s));
    }
    MQ_HIP(launch_flatten_groups(r.group_expert, r.group_begin, r.n_groups, r.entry_token, r.entry_k, (int)(n * top_k), triples_dev,
                                 count_dev, s));
    return MQ_OK;
}

namespace {

struct SharedExpert {
    const mq_weight* gate = nullptr;
    const mq_weight* up = nullptr;
    const mq_weight* down = nullptr;
};

// gate/up + SwiGLU for every routed (token, k) pair (and the shared expert as slot top_k):
// hidden row = token * slots + k.  Caller holds g.mu; groups are already built in r.
int run_moe_gateup(const mq_weight* gate, const mq_weight* up, const SharedExpert& sh, int64_t n, int top_k, int slots,
                   int silu_mode, const RouteWs& r, float* hidden, bool quantize_hidden, hipStream_t s) {
    const int64_t pairs = n * (int64_t)top_k;
    MatmulArgs a;
    if (quantize_hidden) {  // hidden rows leave the kernel already in Q8_K (A-major), ready for the down projection
        const int64_t out_nb = gate->rows / kQK;
        const int64_t groups = (r.direct_ids || pairs < gate->n_experts ? pairs : gate->n_experts) + (n + 7) / 8;  // + shared-expert passes
        MQ_HIP(g.aq2.reserve(aq_bytes(n * slots, out_nb)));
        MQ_HIP(g.ad2.reserve(ad_count(n * slots, out_nb) * sizeof(float)));
        if (int rc = reserve_counters((size_t)(groups * out_nb))) return rc;
        a.out_aq = (uint8_t*)g.aq2.ptr;
        a.out_ad = (float*)g.ad2.ptr;
        a.out_counters = (uint32_t*)g.counters.ptr;
    }
    a.w0 = gate->data;
    a.wtype = gate->type;
    a.w1 = up->data;
    a.rows = gate->rows;
    a.nb = gate->nb;
    a.expert_bytes = gate->expert_bytes;
    a.aq = (const uint8_t*)g.aq.ptr;
    a.ad = (const float*)g.ad.ptr;
    a.n = n;
    a.y = hidden;
    a.ldy = gate->rows;
    a.swiglu = 1;
    a.silu_mode = silu_mode;
    a.grouped = 1;
    a.group_expert = r.group_expert;
    a.group_begin = r.group_begin;
    a.n_groups = r.n_groups;
    a.entry_token = r.entry_token;
    a.entry_k = r.entry_k;
    a.a_tok_stride = 1;
    a.a_k_stride = 0;
    a.y_tok_stride = slots;
    a.y_k_stride = 1;
    a.max_groups = (int)(r.direct_ids || pairs < gate->n_experts ? pairs : gate->n_experts);
    a.direct_ids = r.direct_ids;
    a.direct_top_k = top_k;
    a.n_experts = (int)gate->n_experts;
    if (sh.gate) {
        a.sh_w0 = sh.gate->data;
        a.sh_w1 = sh.up->data;
        a.sh_tokens = (int)n;
        a.sh_arow_stride = 1;
        a.sh_arow_offset = 0;
        a.sh_yrow_stride = slots;
        a.sh_yrow_offset = top_k;
        a.sh_silu_mode = MQ_SILU_FAST_FMA;
    }
    MQ_HIP(census_launch(a, s));
    return MQ_OK;
}

// Does the down projection of this MoE block run token-major (moe_down.hip)?
bool token_major_down(const mq_weight* down, int64_t n, int slots) {
    return down->type != kTypeQ80 && n <= kTokenMajorDownMaxTokens && (down->rows & 15) == 0 &&
           moe_down_token_lds_bytes(slots, down->nb) <= kMoeDownTokenMaxLds;
}

// Q8_K of the hidden rows, down projection per (token, k) into g.part, then the weighted combine.
int run_moe_down(const mq_weight* down, const SharedExpert& sh, const float* hidden, bool hidden_is_quantized, int64_t n,
                 int top_k, int slots, const RouteWs& r, const int32_t* ids, const float* weights,
                 const float* sh_gate_inp, const float* x, float* y, hipStream_t s) {
    const int64_t pairs = n * (int64_t)top_k;
    const int64_t mid_rows = n * slots;
    const int64_t inter = down->cols, hidden_dim = down->rows;
    // rows of dropped entries may hold anything; they are never read
    const bool token_major = token_major_down(down, n, slots);
    if (!hidden_is_quantized && !token_major && down->type != kTypeQ80) {
        if (int rc = quantize_into(g.aq2, g.ad2, hidden, mid_rows, inter, inter, s)) return rc;
    }
    if (token_major) {
        // few tokens: a workgroup per (token, 16 output rows) multiplies and combines in one launch, and
        // quantizes the hidden rows it reads when they come as fp32
        MoeDownTokenArgs a;
        a.w = down->data;
        a.expert_bytes = down->expert_bytes;
        a.sh_w = sh.down ? sh.down->data : nullptr;
        a.wtype = down->type;
        a.rows = hidden_dim, a.nb = down->nb, a.n = n;
        a.top_k = top_k, a.n_experts = (int)down->n_experts;
        if (hidden_is_quantized) a.aq = (const uint8_t*)g.aq2.ptr, a.ad = (const float*)g.ad2.ptr;
        else a.hidden = hidden;
        a.ids = ids, a.weights = weights;
        a.sh_gate_inp = sh_gate_inp, a.x = x, a.y = y;
        MQ_HIP(launch_moe_down_token(a, s));
        return MQ_OK;
    }
    MQ_HIP(g.part.reserve((size_t)mid_rows * (size_t)hidden_dim * sizeof(float)));
    if (down->type == kTypeQ80) {
        // Q8_0 experts take Q8_0 hidden rows (core/src/llm/moe/native.cpp:3239-3245: the row is quantized for the
        // weight's type), one (token, slot) pair per workgroup column, then the same k-ordered combine
        if (hidden_is_quantized) return fail(MQ_ERR_STATE, "Q8_0 down experts need their hidden rows as fp32");
        MQ_HIP(g.aq2.reserve(aq_bytes(mid_rows, down->nb)));
        MQ_HIP(g.ad2.reserve(q80_scale_bytes(mid_rows, down->nb)));
        MQ_HIP(launch_quantize_q80(hidden, mid_rows, inter, inter, (uint8_t*)g.aq2.ptr, (uint16_t*)g.ad2.ptr, s));
        Q80MatmulArgs q;
        q.w = down->data;
        q.rows = hidden_dim;
        q.nb = down->nb;
        q.aq = (const uint8_t*)g.aq2.ptr;
        q.ah = (const uint16_t*)g.ad2.ptr;
        q.n = mid_rows;
        q.y = (float*)g.part.ptr;
        q.ldy = hidden_dim;
        q.top_k = top_k;
        q.slots = slots;
        q.n_experts = (int)down->n_experts;
        q.expert_bytes = down->expert_bytes;
        q.sh_w = sh.down ? sh.down->data : nullptr;
        if (r.direct_ids) {  // few tokens: nothing was grouped, every pair is a column of its own
            q.pair_ids = ids;
        } else {             // an expert's rows together, eight to a pass
            q.group_expert = r.group_expert, q.group_begin = r.group_begin, q.n_groups = r.n_groups;
            q.entry_token = r.entry_token, q.entry_k = r.entry_k;
            q.max_groups = (int)(pairs < down->n_experts ? pairs : down->n_experts);
            q.sh_tokens = sh.down ? (int)n : 0;
        }
        MQ_HIP(launch_q80_matmul(q, s));
        MQ_HIP(launch_moe_combine((const float*)g.part.ptr, n, top_k, slots, hidden_dim, weights, ids, down->n_experts,
                                  sh.down ? 1 : 0, sh_gate_inp, x, y, s));
        return MQ_OK;
    }
    MatmulArgs d;
    d.w0 = down->data;
    d.wtype = down->type;
    d.rows = hidden_dim;
    d.nb = down->nb;
    d.expert_bytes = down->expert_bytes;
    d.aq = (const uint8_t*)g.aq2.ptr;
    d.ad = (const float*)g.ad2.ptr;
    d.n = n;
    d.y = (float*)g.part.ptr;
    d.ldy = hidden_dim;
    d.grouped = 1;
    d.group_expert = r.group_expert;
    d.group_begin = r.group_begin;
    d.n_groups = r.n_groups;
    d.entry_token = r.entry_token;
    d.entry_k = r.entry_k;
    d.a_tok_stride = slots;
    d.a_k_stride = 1;
    d.y_tok_stride = slots;
    d.y_k_stride = 1;
    d.max_groups = (int)(r.direct_ids || pairs < down->n_experts ? pairs : down->n_experts);
    d.direct_ids = r.direct_ids;
    d.direct_top_k = top_k;
    d.n_experts = (int)down->n_experts;
    if (sh.down) {
        d.sh_w0 = sh.down->data;
        d.sh_tokens = (int)n;
        d.sh_arow_stride = slots;
        d.sh_arow_offset = top_k;
        d.sh_yrow_stride = slots;
        d.sh_yrow_offset = top_k;
    }
    MQ_HIP(census_launch(d, s));
    MQ_HIP(launch_moe_combine((const float*)g.part.ptr, n, top_k, slots, hidden_dim, weights, ids, down->n_experts,
                              sh.down ? 1 : 0, sh_gate_inp, x, y, s));
    return MQ_OK;
}

int check_experts(const mq_weight* gate, const mq_weight* up, const mq_weight* down, int top_k, const char* name) {
    if (gate && up) {
        if (up->cols != gate->cols || up->rows != gate->rows || up->n_experts != gate->n_experts || up->type != gate->type)
            return fail(MQ_ERR_INVALID, "%s: gate and up expert tensors disagree", name);
        if (gate->rows % kQK) return fail(MQ_ERR_INVALID, "%s: inter must be a multiple of 256", name);
    }
    if (gate && down) {
        if (down->cols != gate->rows || down->rows != gate->cols || down->n_experts != gate->n_experts)
            return fail(MQ_ERR_INVALID, "%s: down expert tensor does not match gate/up", name);
    }
    const mq_weight* any = gate ? gate : down;
    if (top_k <= 0 || top_k > 8 || top_k > any->n_experts)
        return fail(MQ_ERR_INVALID, "%s: need 0 < top_k <= min(8, n_experts)", name);
    return MQ_OK;
}

}  // namespace

int mq_swiglu_mul_mat_q4k(const mq_weight* gate, const mq_weight* up, const float* x_dev, int64_t n, int64_t ldx,
                          float* h_dev, int64_t ldh, int silu_mode, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(gate, "mq_swiglu_mul_mat_q4k(gate)")) return rc;
    if (int rc = check_weight(up, "mq_swiglu_mul_mat_q4k(up)")) return rc;
    if (up->cols != gate->cols || up->rows != gate->rows || gate->n_experts != 1 || up->n_experts != 1 || up->type != gate->type)
        return fail(MQ_ERR_INVALID, "mq_swiglu_mul_mat_q4k: gate and up must be dense matrices of one shape and type");
    if (silu_mode < 0 || silu_mode > 2) return fail(MQ_ERR_INVALID, "mq_swiglu_mul_mat_q4k: silu_mode %d", silu_mode);
    if (int rc = check_x(x_dev, n, ldx, gate->cols, "mq_swiglu_mul_mat_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!h_dev || ldh < gate->rows) return fail(MQ_ERR_INVALID, "mq_swiglu_mul_mat_q4k: null output or ldh < rows");
    if (n == 0) return MQ_OK;
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    if (prefill_applies(gate, n) && !skinny16_takes(gate, n, true) && !(ldh & 3) && !(reinterpret_cast<uintptr_t>(h_dev) & 15u))
        return ffn_wide_locked(gate, up, nullptr, x_dev, n, ldx, silu_mode, h_dev, ldh, nullptr, 0, s);
    // one row, or a few where the LDS-staged kernel applies: the quantizer runs inside the product
    const bool inline_quant = (n == 1 && !(reinterpret_cast<uintptr_t>(x_dev) & 15u)) || dense_lds_quantizes(gate, x_dev, n, ldx, true);
    const bool tile16 = !inline_quant && skinny16_takes(gate, n, true);
    if (tile16) {
        if (int rc = quantize_into_tile16(x_dev, n, ldx, gate->cols, s)) return rc;
    } else if (!inline_quant) {
        if (int rc = quantize_into(g.aq, g.ad, x_dev, n, ldx, gate->cols, s)) return rc;
    }
    MatmulArgs a;
    a.w0 = gate->data;
    a.wtype = gate->type;
    a.w1 = up->data;
    a.rows = gate->rows;
    a.nb = gate->nb;
    if (inline_quant) {
        a.xf = x_dev;
        a.ldx = ldx;
    } else if (tile16) {
        a.ap = (const uint8_t*)g.ap.ptr;
    } else {
        a.aq = (const uint8_t*)g.aq.ptr;
        a.ad = (const float*)g.ad.ptr;
    }
    a.n = n;
    a.y = h_dev;
    a.ldy = ldh;
    a.swiglu = 1;
    a.silu_mode = silu_mode;
    MQ_HIP(census_launch(a, s));
    return MQ_OK;
}

// ---------------------------------------------------------------------------------- shared Q8_K rows
int mq_acts_create(int64_t max_rows, int64_t cols, mq_acts** out) {
    if (int rc = check_ready()) return rc;
    if (!out || max_rows <= 0 || cols <= 0 || cols % kQK) return fail(MQ_ERR_INVALID, "mq_acts_create: need max_rows > 0 and cols a positive multiple of 256");
    mq_acts* a = new mq_acts;
    a->max_rows = max_rows, a->cols = cols, a->nb = cols / kQK;
    hipError_t e = hipMalloc(&a->aq, aq_bytes(max_rows, a->nb));
    if (e == hipSuccess) e = hipMalloc(&a->ad, ad_count(max_rows, a->nb) * sizeof(float));
    if (e == hipSuccess && max_rows > 8) e = hipMalloc(&a->ap, pmajor_bytes(max_rows < kSkinnyMaxRows ? max_rows : kSkinnyMaxRows, a->nb));
    if (e != hipSuccess) {
        if (a->aq) (void)hipFree(a->aq);
        if (a->ad) (void)hipFree(a->ad);
        delete a;
        return fail(MQ_ERR_HIP, "mq_acts_create: %s", hipGetErrorString(e));
    }
    *out = a;
    return MQ_OK;
}

int mq_acts_free(mq_acts* a) {
    if (!a) return MQ_OK;
    if (a->aq) (void)hipFree(a->aq);
    if (a->ad) (void)hipFree(a->ad);
    if (a->ap) (void)hipFree(a->ap);
    delete a;
    return MQ_OK;
}

int mq_acts_quantize(mq_acts* a, const float* x_dev, int64_t n, int64_t ldx, void* stream) {
    if (int rc = check_ready()) return rc;
    if (!a) return fail(MQ_ERR_INVALID, "mq_acts_quantize: null handle");
    if (n > a->max_rows) return fail(MQ_ERR_INVALID, "mq_acts_quantize: %lld rows exceed the handle's %lld", (long long)n, (long long)a->max_rows);
    if (int rc = check_x(x_dev, n, ldx, a->cols, "mq_acts_quantize")) return rc;
    a->n = n;
    a->tile16 = false;
    if (n == 0) return MQ_OK;
    MQ_HIP(launch_quantize_q8k(x_dev, n, ldx, a->cols, nullptr, 0, (uint8_t*)a->aq, (float*)a->ad, (hipStream_t)stream));
    // nine to 64 rows: their tiles of sixteen as well, for the Q4_K products that take them (skinny16_takes)
    a->tile16 = n > 8 && n <= kSkinnyMaxRows && a->ap;
    if (a->tile16) MQ_HIP(launch_quantize_q8k_pmajor(x_dev, n, ldx, a->cols, (uint8_t*)a->ap, (hipStream_t)stream));
    return MQ_OK;
}

static int acts_matmul(const mq_weight* w0, const mq_weight* w1, const mq_acts* a, float* y_dev, int64_t ldy, int swiglu,
                       int silu_mode, void* stream, const char* who) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(w0, who)) return rc;
    if (w1) {
        if (int rc = check_weight(w1, who)) return rc;
        if (w1->cols != w0->cols || w1->rows != w0->rows || w1->n_experts != 1 || w1->type != w0->type) return fail(MQ_ERR_INVALID, "%s: gate and up must be dense matrices of one shape", who);
    }
    if (!a || !y_dev || w0->n_experts != 1 || a->cols != w0->cols || ldy < w0->rows) return fail(MQ_ERR_INVALID, "%s: null argument, expert stack, column mismatch or ldy < rows", who);
    if (silu_mode < 0 || silu_mode > 2) return fail(MQ_ERR_INVALID, "%s: silu_mode %d", who, silu_mode);
    if (a->n == 0) return MQ_OK;
    MatmulArgs m;
    m.w0 = w0->data;
    m.wtype = w0->type;
    m.w1 = w1 ? w1->data : nullptr;
    m.rows = w0->rows;
    m.nb = w0->nb;
    if (a->tile16 && skinny16_takes(w0, a->n, swiglu != 0)) {
        m.ap = (const uint8_t*)a->ap;
    } else {
        m.aq = (const uint8_t*)a->aq;
        m.ad = (const float*)a->ad;
    }
    m.n = a->n;
    m.y = y_dev;
    m.ldy = ldy;
    m.swiglu = swiglu;
    m.silu_mode = silu_mode;
    Entry entry((hipStream_t)stream);  // the handle's rows are the caller's; the launch itself shares nothing, but stays ordered
    if (entry.rc) return entry.rc;
    MQ_HIP(census_launch(m, (hipStream_t)stream));
    return MQ_OK;
}

int mq_mul_mat_q4k_acts(const mq_weight* w, const mq_acts* a, float* y_dev, int64_t ldy, void* stream) {
    return acts_matmul(w, nullptr, a, y_dev, ldy, 0, 0, stream, "mq_mul_mat_q4k_acts");
}

int mq_swiglu_mul_mat_q4k_acts(const mq_weight* gate, const mq_weight* up, const mq_acts* a, float* h_dev, int64_t ldh,
                               int silu_mode, void* stream) {
    if (!up) return fail(MQ_ERR_INVALID, "mq_swiglu_mul_mat_q4k_acts: null up matrix");
    return acts_matmul(gate, up, a, h_dev, ldh, 1, silu_mode, stream, "mq_swiglu_mul_mat_q4k_acts");
}

int mq_moe_gateup_swiglu_q4k(const mq_weight* gate_exps, const mq_weight* up_exps, const float* x_dev, int64_t n,
                             const int32_t* ids_dev, int top_k, int silu_mode, float* hidden_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(gate_exps, "mq_moe_gateup_swiglu_q4k(gate_exps)")) return rc;
    if (int rc = check_weight(up_exps, "mq_moe_gateup_swiglu_q4k(up_exps)")) return rc;
    if (int rc = check_experts(gate_exps, up_exps, nullptr, top_k, "mq_moe_gateup_swiglu_q4k")) return rc;
    if (silu_mode < 0 || silu_mode > 2) return fail(MQ_ERR_INVALID, "mq_moe_gateup_swiglu_q4k: silu_mode %d", silu_mode);
    if (int rc = check_x(x_dev, n, gate_exps->cols, gate_exps->cols, "mq_moe_gateup_swiglu_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!ids_dev || !hidden_dev) return fail(MQ_ERR_INVALID, "mq_moe_gateup_swiglu_q4k: null ids or output");
    if (n == 0) return MQ_OK;
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    RouteWs r;
    if (int rc = carve_route(n, top_k, gate_exps->n_experts, r)) return rc;
    MQ_HIP(launch_fill_zero(hidden_dev, (size_t)n * top_k * (size_t)gate_exps->rows, s));
    MQ_HIP(launch_build_groups(ids_dev, n, top_k, gate_exps->n_experts, r.group_expert, r.group_begin, r.n_groups,
                               r.entry_token, r.entry_k, s));
    if (moe_gemm_width(gate_exps, n, top_k)) {  // gate and up share their type
        // prefill widths: both products on the expert-grouped GEMM, SwiGLU rows scattered to their (token, slot) places
        const int64_t entries = n * top_k, E = gate_exps->n_experts, inter = gate_exps->rows, hidden = gate_exps->cols;
        MQ_HIP(g.plan.reserve(moe_gemm_plan_ints(entries, E) * sizeof(int32_t)));
        const int mt = g_moe_item_tiles ? g_moe_item_tiles : moe_gemm_item_tiles(entries, E);  // tiles per item: the plan and every launch reading it
        const int32_t* plan = (const int32_t*)g.plan.ptr;
        MQ_HIP(launch_moe_gemm_plan(r.n_groups, r.group_expert, r.group_begin, r.entry_token, r.entry_k, top_k, false, entries, E,
                                    0, 0, (int32_t*)g.plan.ptr, s, mt));
        const int64_t rows_max = moe_gemm_tiles_max(entries, E) * 16;
        MQ_HIP(g.ap.reserve(pmajor_bytes(rows_max, hidden / kQK)));
        MQ_HIP(g.ap_rows.reserve(pmajor_bytes(n, hidden / kQK)));  // every token is a row of top_k experts: quantized once
        MQ_HIP(launch_quantize_q8k_pmajor_grouped(x_dev, nullptr, false, 0, hidden, hidden, entries, E, plan, (uint8_t*)g.ap.ptr, nullptr, 0, s,
                                                  n, (uint8_t*)g.ap_rows.ptr));
        if (g_gemm_pair && gate_exps->type == kTypeQ4K && up_exps->type == kTypeQ4K) {
            // one launch for gate and up, silu(gate) * up scattered to its (token, slot) place by the epilogue
            MQ_HIP(launch_prefill_gemm_grouped_pair(gate_exps->data, up_exps->data, gate_exps->type, gate_exps->expert_bytes, nullptr, nullptr,
                                                    inter, gate_exps->nb, (const uint8_t*)g.ap.ptr, entries, E, plan, true, silu_mode, hidden_dev,
                                                    inter, s, mt));
            return MQ_OK;
        }
        MQ_HIP(g.mid2.reserve(2 * (size_t)rows_max * (size_t)inter * sizeof(float)));
        float* gbuf = (float*)g.mid2.ptr;
        float* ubuf = gbuf + (size_t)rows_max * (size_t)inter;
        MQ_HIP(launch_prefill_gemm_grouped(gate_exps->data, gate_exps->type, gate_exps->expert_bytes, nullptr, inter, gate_exps->nb,
                                           (const uint8_t*)g.ap.ptr, entries, E, plan, false, gbuf, inter, s, mt));
        MQ_HIP(launch_prefill_gemm_grouped(up_exps->data, up_exps->type, up_exps->expert_bytes, nullptr, inter, up_exps->nb,
                                           (const uint8_t*)g.ap.ptr, entries, E, plan, false, ubuf, inter, s, mt));
        MQ_HIP(g.ap2.reserve(pmajor_bytes(rows_max, inter / kQK)));
        MQ_HIP(launch_quantize_q8k_pmajor_grouped(gbuf, ubuf, true, silu_mode, inter, inter, entries, E, plan, (uint8_t*)g.ap2.ptr,
                                                  hidden_dev, inter, s));
        return MQ_OK;
    }
    if (int rc = quantize_into(g.aq, g.ad, x_dev, n, gate_exps->cols, gate_exps->cols, s)) return rc;
    return run_moe_gateup(gate_exps, up_exps, SharedExpert{}, n, top_k, top_k, silu_mode, r, hidden_dev, false, s);
}

int mq_moe_down_weighted_q4k(const mq_weight* down_exps, const float* hidden_dev, int64_t n, const int32_t* ids_dev,
                             const float* weights_dev, int top_k, float* y_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (int rc = check_weight(down_exps, "mq_moe_down_weighted_q4k(down_exps)", true)) return rc;
    if (int rc = check_experts(nullptr, nullptr, down_exps, top_k, "mq_moe_down_weighted_q4k")) return rc;
    if (int rc = check_x(hidden_dev, n * top_k, down_exps->cols, down_exps->cols, "mq_moe_down_weighted_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!ids_dev || !weights_dev || !y_dev) return fail(MQ_ERR_INVALID, "mq_moe_down_weighted_q4k: null pointer");
    if (n == 0) return MQ_OK;
    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    RouteWs r;
    if (int rc = carve_route(n, top_k, down_exps->n_experts, r)) return rc;
    MQ_HIP(launch_build_groups(ids_dev, n, top_k, down_exps->n_experts, r.group_expert, r.group_begin, r.n_groups,
                               r.entry_token, r.entry_k, s));
    if (moe_gemm_width(down_exps, n, top_k)) {
        // prefill widths: the product on the expert-grouped GEMM into the per-(token, slot) rows, then the combine
        const int64_t entries = n * top_k, E = down_exps->n_experts, hidden = down_exps->rows, inter = down_exps->cols;
        MQ_HIP(g.plan.reserve(moe_gemm_plan_ints(entries, E) * sizeof(int32_t)));
        const int mt = g_moe_item_tiles ? g_moe_item_tiles : moe_gemm_item_tiles(entries, E);  // tiles per item: the plan and every launch reading it
        const int32_t* plan = (const int32_t*)g.plan.ptr;
        MQ_HIP(launch_moe_gemm_plan(r.n_groups, r.group_expert, r.group_begin, r.entry_token, r.entry_k, top_k, true, entries, E,
                                    0, 0, (int32_t*)g.plan.ptr, s, mt));
        MQ_HIP(g.ap2.reserve(pmajor_bytes(moe_gemm_tiles_max(entries, E) * 16, inter / kQK)));
        MQ_HIP(launch_quantize_q8k_pmajor_grouped(hidden_dev, nullptr, false, 0, inter, inter, entries, E, plan, (uint8_t*)g.ap2.ptr,
                                                  nullptr, 0, s));
        MQ_HIP(g.part.reserve((size_t)n * top_k * (size_t)hidden * sizeof(float)));
        MQ_HIP(launch_prefill_gemm_grouped(down_exps->data, down_exps->type, down_exps->expert_bytes, nullptr, hidden, down_exps->nb,
                                           (const uint8_t*)g.ap2.ptr, entries, E, plan, true, (float*)g.part.ptr, hidden, s, mt));
        MQ_HIP(launch_moe_combine((const float*)g.part.ptr, n, top_k, top_k, hidden, weights_dev, ids_dev, E, 0, nullptr, nullptr, y_dev, s));
        return MQ_OK;
    }
    return run_moe_down(down_exps, SharedExpert{}, hidden_dev, false, n, top_k, top_k, r, ids_dev, weights_dev, nullptr,
                        nullptr, y_dev, s);
}

namespace {

// Workgroups of the persistent decoder kernel (decoder_layers.hip): one per compute unit, all resident at once.
int decoder_grid(size_t lds_bytes, int* n_workgroups, long long* spin_ticks) {
    hipDeviceProp_t prop;
    MQ_HIP(hipGetDeviceProperties(&prop, g.device));
    if (lds_bytes > (size_t)prop.maxSharedMemoryPerMultiProcessor)
        return fail(MQ_ERR_UNSUPPORTED, "fused decoder layers need %zu bytes of LDS per workgroup, the device has %zu", lds_bytes,
                    (size_t)prop.maxSharedMemoryPerMultiProcessor);
    static size_t prepared = 0;  // the kernel attribute only ever grows (caller holds g.mu)
    if (lds_bytes > prepared) {
        MQ_HIP(prepare_decoder_layers(lds_bytes));
        prepared = lds_bytes;
    }
    int rate_khz = 0;
    if (hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, g.device) != hipSuccess || rate_khz <= 0) rate_khz = 100000;
    *spin_ticks = (long long)rate_khz * 200;  // 200 ms: a phase takes microseconds
    *n_workgroups = prop.multiProcessorCount;
    return MQ_OK;
}

}  // namespace

// The expert-grouped GEMM pays from six routed rows per expert on average (its workgroups multiply 16-row tiles, two,
// four or eight of an expert at a time): 256 experts, top-8, 2048 x 512: 152 against 153 us per block at 192 tokens, 158
// against 186 at 256, 164 against 217 at 320 -- and 141 against 119 at 128, where the decode kernels' 8-row groups stay.
// Decided per product: gate / up (one type) and down each run on it when their type is one it takes; a layer with
// a Q8_0 down stack (core/src/llm/moe/native.cpp:4611-4620; its activations are Q8_0 as well) keeps its two large
// products on the matrix cores and sends the fp32 hidden rows through the Q8_0 launches.
static bool moe_gemm_takes(const mq_weight* w) { return w->type == kTypeQ4K || w->type == kTypeQ5K || w->type == kTypeQ6K; }
static bool moe_gemm_applies(const mq_moe_layer_desc* L, int64_t n) {
    const mq_weight* ge = L->gate_exps;
    if (!moe_gemm_takes(ge) || !moe_gemm_takes(L->up_exps)) return false;  // the shared expert has the stacks' types
    if (ge->n_experts > 4096 || (ge->rows & 3) || (ge->cols & 3)) return false;
    // (256 + 1 experts, top-8, 2048 x 512, the expert-grouped decode launches against the GEMM with items of two tiles:
    // 106 / 135 us at 96 tokens, 119 / 141 at 128, 153 / 152 at 192, 186 / 158 at 256, 217 / 164 at 320)
    return n >= 192 && n * L->top_k >= 6 * ge->n_experts;
}

int mq_moe_layer_q4k(const mq_moe_layer_desc* L, const float* x_dev, const float* logits_dev, int64_t n, float* y_dev,
                     int32_t* ids_out_dev, float* weights_out_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (!L) return fail(MQ_ERR_INVALID, "mq_moe_layer_q4k: null layer");
    if (int rc = check_weight(L->gate_exps, "mq_moe_layer_q4k(gate_exps)")) return rc;
    if (int rc = check_weight(L->up_exps, "mq_moe_layer_q4k(up_exps)")) return rc;
    if (int rc = check_weight(L->down_exps, "mq_moe_layer_q4k(down_exps)", true)) return rc;
    if (int rc = check_experts(L->gate_exps, L->up_exps, L->down_exps, L->top_k, "mq_moe_layer_q4k")) return rc;
    const int64_t hidden = L->gate_exps->cols, inter = L->gate_exps->rows, E = L->gate_exps->n_experts;
    const int K = L->top_k;
    if (L->silu_mode < 0 || L->silu_mode > 2 || L->route_mode < 0 || L->route_mode > 2)
        return fail(MQ_ERR_INVALID, "mq_moe_layer_q4k: bad silu_mode or route_mode");
    SharedExpert sh;
    if (L->shared_gate || L->shared_up || L->shared_down) {
        if (int rc = check_weight(L->shared_gate, "mq_moe_layer_q4k(shared_gate)")) return rc;
        if (int rc = check_weight(L->shared_up, "mq_moe_layer_q4k(shared_up)")) return rc;
        if (int rc = check_weight(L->shared_down, "mq_moe_layer_q4k(shared_down)", true)) return rc;
        if (L->shared_gate->cols != hidden || L->shared_gate->rows != inter || L->shared_up->cols != hidden ||
            L->shared_up->rows != inter || L->shared_down->cols != inter || L->shared_down->rows != hidden ||
            L->shared_gate->n_experts != 1 || L->shared_up->n_experts != 1 || L->shared_down->n_experts != 1 ||
            L->shared_gate->type != L->gate_exps->type || L->shared_up->type != L->gate_exps->type ||
            L->shared_down->type != L->down_exps->type)
            return fail(MQ_ERR_INVALID, "mq_moe_layer_q4k: shared expert must have the routed experts' shape and types");
        sh.gate = L->shared_gate;
        sh.up = L->shared_up;
        sh.down = L->shared_down;
    }
    if (int rc = check_x(x_dev, n, hidden, hidden, "mq_moe_layer_q4k")) return rc;
    if (n == 0) return MQ_OK;
    if (!logits_dev || !y_dev) return fail(MQ_ERR_INVALID, "mq_moe_layer_q4k: null logits or output");
    if (n == 0) return MQ_OK;

    hipStream_t s = (hipStream_t)stream;
    Entry entry(s);
    if (entry.rc) return entry.rc;
    const int slots = K + (sh.gate ? 1 : 0);  // hidden / partial rows per token
    RouteWs r;
    if (int rc = carve_route(n, K, E, r)) return rc;
    // ids and weights go straight to the caller's buffers when it wants them
    int32_t* ids = ids_out_dev ? ids_out_dev : r.ids;
    float* wts = weights_out_dev ? weights_out_dev : r.weights;
    if (n <= kDirectPairsMaxTokens && E <= kDecoderMaxExperts && token_major_down(L->down_exps, n, slots)) {
        // few tokens: two launches -- gate/up with the router and the input quantizer inside (moe_gateup.hip), down
        // with the hidden-row quantizer and the combine inside (moe_down.hip)
        MQ_HIP(g.mid.reserve((size_t)n * slots * (size_t)inter * sizeof(float)));
        MoeGateupTokenArgs a;
        a.gate = L->gate_exps->data, a.up = L->up_exps->data, a.expert_bytes = L->gate_exps->expert_bytes;
        if (sh.gate) a.sh_gate = sh.gate->data, a.sh_up = sh.up->data;
        a.wtype = L->gate_exps->type;
        a.rows = inter, a.nb = L->gate_exps->nb, a.n = n;
        a.top_k = K, a.n_experts = (int)E;
        a.route_mode = L->route_mode, a.silu_mode = L->silu_mode, a.sh_silu_mode = MQ_SILU_FAST_FMA;
        a.waves = moe_gateup_token_waves(L->gate_exps->nb, inter, n, slots, L->gate_exps->type);
        a.x = x_dev, a.logits = logits_dev, a.hidden = (float*)g.mid.ptr, a.ids_out = ids, a.weights_out = wts;
        MQ_HIP(launch_moe_gateup_token(a, s));
        return run_moe_down(L->down_exps, sh, (const float*)g.mid.ptr, false, n, K, slots, r, ids, wts, L->sh_gate_inp_dev,
                            x_dev, y_dev, s);
    }
    // one arrival counter, kept apart from the quantization counters (last slot of that buffer)
    if (int rc = reserve_counters(4096)) return rc;
    if (moe_gemm_applies(L, n)) {
        // Prefill widths: the three expert products on the matrix-core GEMM in its expert-grouped form, the shared
        // expert as a dense FFN on it; per-(token, slot) rows and the combine as at the other widths.
        // The shared expert rides along as one more group of all tokens (its own weights, its own SiLU form, output slot K).
        const int64_t entries = n * K + (sh.gate ? n : 0), G = E + (sh.gate ? 1 : 0);
        MQ_HIP(g.part.reserve((size_t)n * slots * (size_t)hidden * sizeof(float)));
        float* part = (float*)g.part.ptr;
        MQ_HIP(launch_route_and_group(logits_dev, E, n, K, L->route_mode, ids, wts, (uint32_t*)g.counters.ptr + 4095,
                                      r.group_expert, r.group_begin, r.n_groups, r.entry_token, r.entry_k, true, nullptr, 0, 0,
                                      nullptr, nullptr, s));
        MQ_HIP(g.plan.reserve(moe_gemm_plan_ints(entries, G) * sizeof(int32_t)));
        const int mt = g_moe_item_tiles ? g_moe_item_tiles : moe_gemm_item_tiles(entries, G);  // tiles per item: the plan and every launch reading it
        const int32_t* plan = (const int32_t*)g.plan.ptr;
        MQ_HIP(launch_moe_gemm_plan(r.n_groups, r.group_expert, r.group_begin, r.entry_token, r.entry_k, slots, false, entries, G,
                                    sh.gate ? n : 0, MQ_SILU_FAST_FMA, (int32_t*)g.plan.ptr, s, mt));
        const int64_t rows_max = moe_gemm_tiles_max(entries, G) * 16;
        MQ_HIP(g.ap.reserve(pmajor_bytes(rows_max, hidden / kQK)));
        MQ_HIP(g.ap_rows.reserve(pmajor_bytes(n, hidden / kQK)));  // every token is a row of top_k (+ the shared) experts: quantized once
        MQ_HIP(launch_quantize_q8k_pmajor_grouped(x_dev, nullptr, false, 0, hidden, hidden, entries, G, plan, (uint8_t*)g.ap.ptr, nullptr, 0, s,
                                                  n, (uint8_t*)g.ap_rows.ptr));
        MQ_HIP(g.mid2.reserve(2 * (size_t)rows_max * (size_t)inter * sizeof(float)));
        float* gbuf = (float*)g.mid2.ptr;
        float* ubuf = gbuf + (size_t)rows_max * (size_t)inter;
        const uint8_t* shg = sh.gate ? sh.gate->data : nullptr;
        const uint8_t* shu = sh.gate ? sh.up->data : nullptr;
        const uint8_t* shd = sh.gate ? sh.down->data : nullptr;
        if (g_gemm_pair && L->gate_exps->type == kTypeQ4K && L->up_exps->type == kTypeQ4K) {
            // gate and up in ONE launch whose epilogue stores silu(gate) * up (the shared expert's rows with its own SiLU form)
            if (!moe_gemm_takes(L->down_exps)) {  // fp32 rows at their (token, slot) places for the down stack's own kernel
                MQ_HIP(g.mid.reserve((size_t)n * slots * (size_t)inter * sizeof(float)));
                MQ_HIP(launch_prefill_gemm_grouped_pair(L->gate_exps->data, L->up_exps->data, kTypeQ4K, L->gate_exps->expert_bytes, shg, shu, inter,
                                                        L->gate_exps->nb, (const uint8_t*)g.ap.ptr, entries, G, plan, true, L->silu_mode,
                                                        (float*)g.mid.ptr, inter, s, mt));
                return run_moe_down(L->down_exps, sh, (const float*)g.mid.ptr, false, n, K, slots, r, ids, wts, L->sh_gate_inp_dev, x_dev, y_dev, s);
            }
            MQ_HIP(launch_prefill_gemm_grouped_pair(L->gate_exps->data, L->up_exps->data, kTypeQ4K, L->gate_exps->expert_bytes, shg, shu, inter,
                                                    L->gate_exps->nb, (const uint8_t*)g.ap.ptr, entries, G, plan, false, L->silu_mode, gbuf, inter, s, mt));
            MQ_HIP(g.ap2.reserve(pmajor_bytes(rows_max, inter / kQK)));
            MQ_HIP(launch_quantize_q8k_pmajor(gbuf, rows_max, inter, inter, (uint8_t*)g.ap2.ptr, s, plan));  // rows in the plan's order already
            MQ_HIP(launch_prefill_gemm_grouped(L->down_exps->data, L->down_exps->type, L->down_exps->expert_bytes, shd, hidden, L->down_exps->nb,
                                               (const uint8_t*)g.ap2.ptr, entries, G, plan, true, part, hidden, s, mt));
            MQ_HIP(launch_moe_combine(part, n, K, slots, hidden, wts, ids, E, sh.gate ? 1 : 0, L->sh_gate_inp_dev, x_dev, y_dev, s));
            return MQ_OK;
        }
        MQ_HIP(launch_prefill_gemm_grouped(L->gate_exps->data, L->gate_exps->type, L->gate_exps->expert_bytes, shg, inter, L->gate_exps->nb,
                                           (const uint8_t*)g.ap.ptr, entries, G, plan, false, gbuf, inter, s, mt));
        MQ_HIP(launch_prefill_gemm_grouped(L->up_exps->data, L->up_exps->type, L->up_exps->expert_bytes, shu, inter, L->up_exps->nb,
                                           (const uint8_t*)g.ap.ptr, entries, G, plan, false, ubuf, inter, s, mt));
        MQ_HIP(g.ap2.reserve(pmajor_bytes(rows_max, inter / kQK)));
        if (!moe_gemm_takes(L->down_exps)) {
            // a down stack of a type the GEMM does not take: the SwiGLU rows leave the quantizer as fp32 at their
            // (token, slot) places as well, and the expert-grouped decode launches take them from there (their own
            // quantizer -- Q8_K, or Q8_0 for Q8_0 experts -- and the same combine)
            MQ_HIP(g.mid.reserve((size_t)n * slots * (size_t)inter * sizeof(float)));
            MQ_HIP(launch_quantize_q8k_pmajor_grouped(gbuf, ubuf, true, L->silu_mode, inter, inter, entries, G, plan, (uint8_t*)g.ap2.ptr,
                                                      (float*)g.mid.ptr, inter, s));
            return run_moe_down(L->down_exps, sh, (const float*)g.mid.ptr, false, n, K, slots, r, ids, wts, L->sh_gate_inp_dev, x_dev, y_dev, s);
        }
        MQ_HIP(launch_quantize_q8k_pmajor_grouped(gbuf, ubuf, true, L->silu_mode, inter, inter, entries, G, plan, (uint8_t*)g.ap2.ptr, nullptr, 0, s));
        MQ_HIP(launch_prefill_gemm_grouped(L->down_exps->data, L->down_exps->type, L->down_exps->expert_bytes, shd, hidden, L->down_exps->nb,
                                           (const uint8_t*)g.ap2.ptr, entries, G, plan, true, part, hidden, s, mt));
        MQ_HIP(launch_moe_combine(part, n, K, slots, hidden, wts, ids, E, sh.gate ? 1 : 0, L->sh_gate_inp_dev, x_dev, y_dev, s));
        return MQ_OK;
    }
    // the same launch quantizes x: extra workgroups next to the routing ones
    MQ_HIP(g.aq.reserve(aq_bytes(n, hidden / kQK)));
    MQ_HIP(g.ad.reserve(ad_count(n, hidden / kQK) * sizeof(float)));
    MQ_HIP(launch_route_and_group(logits_dev, E, n, K, L->route_mode, ids, wts, (uint32_t*)g.counters.ptr + 4095,
                                  r.group_expert, r.group_begin, r.n_groups, r.entry_token, r.entry_k,
                                  n > kDirectPairsMaxTokens, x_dev, hidden, hidden, (uint8_t*)g.aq.ptr, (float*)g.ad.ptr, s));
    // few tokens: nearly every (token, slot) pair has an expert of its own, so the pairs are the groups
    if (n <= kDirectPairsMaxTokens) r.direct_ids = ids;
    MQ_HIP(g.mid.reserve((size_t)n * slots * (size_t)inter * sizeof(float)));
    // the hidden rows leave gate/up in Q8_K, unless the token-major down launch quantizes what it reads itself
    const bool quantize_in_gateup = !token_major_down(L->down_exps, n, slots) && L->down_exps->type != kTypeQ80;
    if (int rc = run_moe_gateup(L->gate_exps, L->up_exps, sh, n, K, slots, L->silu_mode, r, (float*)g.mid.ptr, quantize_in_gateup, s))
        return rc;
    return run_moe_down(L->down_exps, sh, (const float*)g.mid.ptr, quantize_in_gateup, n, K, slots, r, ids, wts, L->sh_gate_inp_dev,
                        x_dev, y_dev, s);
}

// ---------------------------------------------------------------------------------- fused decoder layers
struct mq_decoder {
    DecoderLayerDev* dev_layers = nullptr;
    int n_layers = 0;
    int64_t max_tokens = 0, qkv_rows = 0;
    int hidden = 0, inter = 0, n_q = 0, n_experts = 0, top_k = 0, has_shared = 0, route_mode = 0;
    float eps = 0.0f;
    float* qkv = nullptr;
    float* o = nullptr;
    float* logits = nullptr;
    float* mid = nullptr;
    float* y = nullptr;
    uint32_t* sync = nullptr;
    int n_workgroups = 0;
    long long spin_ticks = 0;
};

namespace {

void decoder_release(mq_decoder* d) {
    for (void* q : {(void*)d->dev_layers, (void*)d->qkv, (void*)d->o, (void*)d->logits, (void*)d->mid, (void*)d->y, (void*)d->sync})
        if (q) (void)hipFree(q);
    delete d;
}

}  // namespace

int mq_decoder_create(const mq_decoder_layer_desc* layers, int n_layers, int64_t max_tokens, float eps, mq_decoder** out) {
    if (int rc = check_ready()) return rc;
    if (!out) return fail(MQ_ERR_INVALID, "mq_decoder_create: null output handle");
    *out = nullptr;
    if (!layers || n_layers <= 0) return fail(MQ_ERR_INVALID, "mq_decoder_create: no layers");
    if (max_tokens < 1 || max_tokens > 8) return fail(MQ_ERR_UNSUPPORTED, "mq_decoder_create: 1..8 tokens per step, asked for %lld", (long long)max_tokens);
    std::vector<DecoderLayerDev> host((size_t)n_layers);
    const mq_moe_layer_desc& m0 = layers[0].moe;
    if (int rc = check_weight(m0.gate_exps, "mq_decoder_create(gate_exps)")) return rc;
    if (int rc = check_weight(layers[0].wqkv, "mq_decoder_create(wqkv)")) return rc;
    if (int rc = check_weight(layers[0].wo, "mq_decoder_create(wo)")) return rc;
    const int64_t hidden = m0.gate_exps->cols, inter = m0.gate_exps->rows, E = m0.gate_exps->n_experts;
    const int64_t qkv_rows = layers[0].wqkv->rows, n_q = layers[0].wo->cols;
    const bool has_shared = m0.shared_gate != nullptr;
    if (E > kDecoderMaxExperts) return fail(MQ_ERR_UNSUPPORTED, "mq_decoder_create: at most %d experts", kDecoderMaxExperts);
    if (m0.top_k < 1 || m0.top_k > 8 || m0.top_k > E) return fail(MQ_ERR_INVALID, "mq_decoder_create: top_k %d", m0.top_k);
    if (m0.route_mode < 0 || m0.route_mode > 2) return fail(MQ_ERR_INVALID, "mq_decoder_create: bad route_mode");
    if (n_q > qkv_rows || (qkv_rows & 15) || (hidden & 15)) return fail(MQ_ERR_INVALID, "mq_decoder_create: n_q exceeds the qkv rows, or rows not a multiple of 16");
    for (int i = 0; i < n_layers; ++i) {
        const mq_decoder_layer_desc& L = layers[i];
        const mq_moe_layer_desc& m = L.moe;
        const mq_weight* all[8] = {L.wqkv, L.wo, m.gate_exps, m.up_exps, m.down_exps, m.shared_gate, m.shared_up, m.shared_down};
        for (int j = 0; j < 8; ++j) {
            if (j >= 5 && !has_shared) {
                if (all[j]) return fail(MQ_ERR_INVALID, "mq_decoder_create: layer %d has a shared expert, layer 0 has none", i);
                continue;
            }
            if (int rc = check_weight(all[j], "mq_decoder_create")) return rc;
            if (all[j]->type != kTypeQ4K) return fail(MQ_ERR_UNSUPPORTED, "mq_decoder_create: layer %d holds a non-Q4_K weight; run such layers node by node", i);
        }
        if (int rc = check_experts(m.gate_exps, m.up_exps, m.down_exps, m.top_k, "mq_decoder_create")) return rc;
        const bool same = L.wqkv->rows == qkv_rows && L.wqkv->cols == hidden && L.wqkv->n_experts == 1 && L.wo->rows == hidden &&
                          L.wo->cols == n_q && L.wo->n_experts == 1 && m.gate_exps->cols == hidden && m.gate_exps->rows == inter &&
                          m.gate_exps->n_experts == E && m.top_k == m0.top_k && m.route_mode == m0.route_mode && L.router_dev &&
                          (!has_shared || (m.shared_gate->rows == inter && m.shared_gate->cols == hidden && m.shared_up->rows == inter &&
                                           m.shared_up->cols == hidden && m.shared_down->rows == hidden && m.shared_down->cols == inter &&
                                           m.shared_gate->n_experts == 1 && m.shared_up->n_experts == 1 && m.shared_down->n_experts == 1));
        if (!same) return fail(MQ_ERR_INVALID, "mq_decoder_create: layer %d differs in shape from layer 0, or has no router", i);
        DecoderLayerDev& h = host[(size_t)i];
        h.wqkv = L.wqkv->data;
        h.wo = L.wo->data;
        h.qkv_rows = qkv_rows;
        h.attn_norm = L.attn_norm_dev;
        h.ffn_norm = L.ffn_norm_dev;
        h.router = L.router_dev;
        h.fixed_logits = L.fixed_logits_dev;
        h.gate_exps = m.gate_exps->data;
        h.up_exps = m.up_exps->data;
        h.down_exps = m.down_exps->data;
        h.gu_expert_bytes = m.gate_exps->expert_bytes;
        h.down_expert_bytes = m.down_exps->expert_bytes;
        if (m.up_exps->expert_bytes != m.gate_exps->expert_bytes) return fail(MQ_ERR_INVALID, "mq_decoder_create: gate/up expert strides differ");
        if (has_shared) {
            h.sh_gate = m.shared_gate->data;
            h.sh_up = m.shared_up->data;
            h.sh_down = m.shared_down->data;
            h.sh_gate_inp = m.sh_gate_inp_dev;
        }
    }
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    mq_decoder* d = new mq_decoder;
    d->n_layers = n_layers;
    d->max_tokens = max_tokens;
    d->qkv_rows = qkv_rows;
    d->hidden = (int)hidden, d->inter = (int)inter, d->n_q = (int)n_q, d->n_experts = (int)E, d->top_k = m0.top_k;
    d->has_shared = has_shared ? 1 : 0;
    d->route_mode = m0.route_mode;
    d->eps = eps;
    DecoderArgs probe;
    probe.n = (int)max_tokens, probe.hidden = d->hidden, probe.n_q = d->n_q;
    if (int rc = decoder_grid(decoder_layers_lds_bytes(probe), &d->n_workgroups, &d->spin_ticks)) {
        decoder_release(d);
        return rc;
    }
    const size_t slots = (size_t)d->top_k + (size_t)d->has_shared;
    const size_t sync_bytes = decoder_sync_bytes(d->n_workgroups);
    hipError_t e = hipMalloc(&d->dev_layers, host.size() * sizeof(DecoderLayerDev));
    if (e == hipSuccess) e = hipMemcpy(d->dev_layers, host.data(), host.size() * sizeof(DecoderLayerDev), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc(&d->qkv, (size_t)max_tokens * qkv_rows * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(&d->o, (size_t)max_tokens * hidden * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(&d->logits, (size_t)max_tokens * E * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(&d->mid, (size_t)max_tokens * slots * inter * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(&d->y, (size_t)max_tokens * hidden * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(&d->sync, sync_bytes);
    if (e == hipSuccess) e = hipMemset(d->sync, 0, sync_bytes);
    if (e != hipSuccess) {
        decoder_release(d);
        return fail(MQ_ERR_HIP, "mq_decoder_create: %s", hipGetErrorString(e));
    }
    *out = d;
    return MQ_OK;
}

int mq_decoder_step(mq_decoder* d, const float* x_dev, int64_t n, int silu_mode, float* out_dev, int32_t* ids_out_dev,
                    float* weights_out_dev, void* stream) {
    if (int rc = check_ready()) return rc;
    if (!d || !x_dev || !out_dev) return fail(MQ_ERR_INVALID, "mq_decoder_step: null argument");
    if (n < 1 || n > d->max_tokens) return fail(MQ_ERR_INVALID, "mq_decoder_step: %lld tokens, the handle holds 1..%lld", (long long)n, (long long)d->max_tokens);
    if (silu_mode < -1 || silu_mode > 2) return fail(MQ_ERR_INVALID, "mq_decoder_step: bad silu_mode");
    if ((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(out_dev)) & 3u) return fail(MQ_ERR_INVALID, "mq_decoder_step: unaligned pointer");
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    DecoderArgs a;
    a.layers = d->dev_layers;
    a.n_layers = d->n_layers;
    a.n = (int)n;
    a.hidden = d->hidden, a.inter = d->inter, a.n_q = d->n_q, a.n_experts = d->n_experts, a.top_k = d->top_k;
    a.has_shared = d->has_shared;
    // decode widths use the exact exponential, wider ones the polynomial (core/src/llm/moe/native.cpp:3614-3616)
    a.silu_mode = silu_mode >= 0 ? silu_mode : (n <= 4 ? MQ_SILU_EXACT : MQ_SILU_FAST);
    a.route_mode = d->route_mode;
    {
        // the expert gate/up launch of mq_moe_layer_q4k at this width: (token, slot) pairs up to eight tokens, expert
        // groups above, plus one pass of the shared expert; the kernel keeps that launch's summation order
        const int64_t pairs = n * (int64_t)d->top_k;
        const int64_t groups = (pairs < d->n_experts ? pairs : d->n_experts) + (d->has_shared ? (n + 7) / 8 : 0);
        a.gateup_order = n <= kDirectPairsMaxTokens ? moe_gateup_token_waves(d->hidden / kQK, d->inter, n, d->top_k + d->has_shared, kTypeQ4K)
                                                    : pick_waves(d->hidden / kQK, (int64_t)(d->inter / 16) * groups);
    }
    a.eps = d->eps;
    a.spin_ticks = d->spin_ticks;
    a.x_in = x_dev, a.out = out_dev;
    a.qkv = d->qkv, a.o = d->o, a.logits = d->logits, a.mid = d->mid, a.y = d->y;
    a.ids_out = ids_out_dev, a.wts_out = weights_out_dev;
    a.sync = d->sync;
    MQ_HIP(launch_decoder_layers(a, d->n_workgroups, (hipStream_t)stream));
    return MQ_OK;
}

int mq_debug_decoder_buffers(mq_decoder* d, float** qkv_dev, float** o_dev, float** logits_dev, float** hidden_dev, float** y_dev) {
    if (!d) return fail(MQ_ERR_INVALID, "mq_debug_decoder_buffers: null handle");
    if (qkv_dev) *qkv_dev = d->qkv;
    if (o_dev) *o_dev = d->o;
    if (logits_dev) *logits_dev = d->logits;
    if (hidden_dev) *hidden_dev = d->mid;
    if (y_dev) *y_dev = d->y;
    return MQ_OK;
}

int mq_debug_moe_hidden(float* hidden_out_dev, size_t count, void* stream) {
    if (int rc = check_ready()) return rc;
    if (!hidden_out_dev) return fail(MQ_ERR_INVALID, "mq_debug_moe_hidden: null output");
    Entry entry((hipStream_t)stream);
    if (entry.rc) return entry.rc;
    if (count * sizeof(float) > g.mid.cap) return fail(MQ_ERR_INVALID, "mq_debug_moe_hidden: the intermediate buffer holds %zu bytes", g.mid.cap);
    MQ_HIP(hipMemcpyAsync(hidden_out_dev, g.mid.ptr, count * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return MQ_OK;
}

int mq_decoder_status(mq_decoder* d) {
    if (int rc = check_ready()) return rc;
    if (!d) return fail(MQ_ERR_INVALID, "mq_decoder_status: null handle");
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    MQ_HIP(hipDeviceSynchronize());
    uint32_t flag = 0;
    MQ_HIP(hipMemcpy(&flag, d->sync + 128, sizeof flag, hipMemcpyDeviceToHost));
    if (flag == 0) return MQ_OK;
    // a barrier was abandoned: the outputs of that step are void; make the handle usable again
    MQ_HIP(hipMemset(d->sync, 0, decoder_sync_bytes(d->n_workgroups)));
    return fail(MQ_ERR_STATE, "mq_decoder_step: a device-wide barrier timed out (are all compute units free for this process?)");
}

int mq_decoder_set_patience(mq_decoder* d, int64_t microseconds) {
    if (int rc = check_ready()) return rc;
    if (!d || microseconds < 0) return fail(MQ_ERR_INVALID, "mq_decoder_set_patience: null handle or negative time");
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    int rate_khz = 0;
    if (hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, g.device) != hipSuccess || rate_khz <= 0) rate_khz = 100000;
    d->spin_ticks = (long long)rate_khz * microseconds / 1000;
    return MQ_OK;
}

void mq_decoder_free(mq_decoder* d) {
    if (!d) return;
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    (void)hipDeviceSynchronize();
    decoder_release(d);
}

// ---------------------------------------------------------------------------------- census
int mq_debug_set_dense_lds(int on) {
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    const int before = g_dense_lds;
    g_dense_lds = on & 1;
    g_gemm_pair = (on & 8) ? 0 : 1;
    g_moe_item_tiles = (on >> 8) & 0xf;      // bits 8..11: activation tiles per item of the expert-grouped GEMM (2, 4 or 8), 0 = by the rows per expert  // bit 3: gate and up as two GEMM launches and a SwiGLU pass instead of the pair form
    set_grouped_lds((on & 1) && !(on & 4));  // bit 2: only the expert-grouped launches go back to matmul_kernel
    g_skinny16 = (on & 0x1000) ? 0 : 1;      // bit 12: nine to 64 rows stay on the kernels with token tiles of eight (or the GEMM)
    g_dense_xf_rows = ((on >> 4) & 0xf) ? ((on >> 4) & 0xf) - 1 : kDenseXfRowsDefault;  // bits 4..7, experiments: widest product that quantizes its rows itself, plus one (0: the default)
    return before;
}

int mq_debug_set_skeleton(int on) {
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    const int before = g_skeleton;
    g_skeleton = on != 0;
    return before;
}

int mq_census_enable(int on) {
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    census.on = on != 0;
    return MQ_OK;
}
int mq_census_reset(void) {
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    if (census.used) (void)hipDeviceSynchronize();
    census.used = 0;
    return MQ_OK;
}
int mq_census_read(int kind, double* avg_us, double* min_us, double* max_us, int64_t* count) {
    if (int rc = check_ready()) return rc;
    if (kind < 0 || kind >= MQ_KIND_COUNT) return fail(MQ_ERR_INVALID, "mq_census_read: kind %d", kind);
    std::lock_guard<std::recursive_mutex> lock(g.mu);
    MQ_HIP(hipDeviceSynchronize());
    double sum = 0.0, lo = 1e30, hi = 0.0;
    int64_t n = 0;
    for (size_t i = 0; i < census.used; ++i) {
        if (census.pool[i].kind != kind) continue;
        float ms = 0.0f;
        MQ_HIP(hipEventElapsedTime(&ms, census.pool[i].start, census.pool[i].stop));
        const double us = (double)ms * 1000.0;
        sum += us;
        lo = us < lo ? us : lo;
        hi = us > hi ? us : hi;
        ++n;
    }
    if (avg_us) *avg_us = n ? sum / (double)n : 0.0;
    if (min_us) *min_us = n ? lo : 0.0;
    if (max_us) *max_us = hi;
    if (count) *count = n;
    return MQ_OK;
}

// ---------------------------------------------------------------------------------- memory helpers
int mq_device_malloc(void** ptr, size_t bytes) {
    if (int rc = check_ready()) return rc;
    if (!ptr) return fail(MQ_ERR_INVALID, "mq_device_malloc: null out pointer");
    MQ_HIP(hipMalloc(ptr, bytes ? bytes : 1));
    return MQ_OK;
}
int mq_device_free(void* ptr) {
    if (ptr) MQ_HIP(hipFree(ptr));
    return MQ_OK;
}
int mq_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes) {
    MQ_HIP(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
    return MQ_OK;
}
int mq_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes) {
    MQ_HIP(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
    return MQ_OK;
}
int mq_host_malloc(void** ptr, size_t bytes) {
    if (int rc = check_ready()) return rc;
    if (!ptr || bytes == 0) return fail(MQ_ERR_INVALID, "mq_host_malloc: null pointer or zero size");
    MQ_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return MQ_OK;
}
int mq_host_free(void* ptr) {
    if (ptr) MQ_HIP(hipHostFree(ptr));
    return MQ_OK;
}
int mq_memcpy_h2d_async(void* dst_dev, const void* src_pinned, size_t bytes, void* stream) {
    MQ_HIP(hipMemcpyAsync(dst_dev, src_pinned, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    return MQ_OK;
}
int mq_memcpy_d2h_async(void* dst_pinned, const void* src_dev, size_t bytes, void* stream) {
    MQ_HIP(hipMemcpyAsync(dst_pinned, src_dev, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    return MQ_OK;
}
int mq_stream_synchronize(void* stream) {
    MQ_HIP(hipStreamSynchronize((hipStream_t)stream));
    return MQ_OK;
}

}  // extern "C"
