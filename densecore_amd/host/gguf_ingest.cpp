// GGUF container reader for the Q4_K path (host C++, no HIP): see include/mi355_q4k_gguf.h.
#include "mi355_q4k_gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstring>
#include <initializer_list>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

thread_local std::string t_error;

int fail(const std::string& what) {
    t_error = what;
    return MQ_ERR_INVALID;
}

enum ValueType : uint32_t { U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 };

size_t scalar_size(uint32_t t) {
    switch (t) {
        case U8: case I8: case BOOL: return 1;
        case U16: case I16: return 2;
        case U32: case I32: case F32: return 4;
        case U64: case I64: case F64: return 8;
        default: return 0;
    }
}

// bytes per block and elements per block of the ggml types a Q4_K_M file contains
bool type_layout(int32_t t, size_t* block_bytes, int64_t* block_elems) {
    switch (t) {
        case 0: *block_bytes = 4, *block_elems = 1; return true;      // F32
        case 1: *block_bytes = 2, *block_elems = 1; return true;      // F16
        case 2: *block_bytes = 18, *block_elems = 32; return true;    // Q4_0
        case 8: *block_bytes = 34, *block_elems = 32; return true;    // Q8_0
        case 12: *block_bytes = 144, *block_elems = 256; return true; // Q4_K
        case 13: *block_bytes = 176, *block_elems = 256; return true; // Q5_K
        case 14: *block_bytes = 210, *block_elems = 256; return true; // Q6_K
        case 24: *block_bytes = 1, *block_elems = 1; return true;     // I8
        case 26: *block_bytes = 4, *block_elems = 1; return true;     // I32
        case 30: *block_bytes = 2, *block_elems = 1; return true;     // BF16
        default: return false;
    }
}

struct Cursor {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    template <typename T>
    T get() {
        T v{};
        if (!ok || (size_t)(end - p) < sizeof(T)) {
            ok = false;
            return v;
        }
        std::memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        return v;
    }
    std::string str() {
        const uint64_t n = get<uint64_t>();
        if (!ok || (uint64_t)(end - p) < n) {
            ok = false;
            return {};
        }
        std::string s(reinterpret_cast<const char*>(p), (size_t)n);
        p += n;
        return s;
    }
    void skip(uint64_t n) {
        if (!ok || (uint64_t)(end - p) < n) ok = false;
        else p += n;
    }
};

struct Meta {
    uint32_t type = 0;
    int64_t ival = 0;
    std::string sval;
};

}  // namespace

struct mq_gguf {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t size = 0;
    uint32_t version = 0;
    uint64_t alignment = 32;
    const uint8_t* data = nullptr;
    std::vector<std::string> names;
    std::vector<mq_gguf_tensor> tensors;
    std::unordered_map<std::string, int64_t> by_name;
    std::unordered_map<std::string, Meta> meta;
};

namespace {

bool skip_value(Cursor& c, uint32_t type, int depth = 0) {
    if (type == STRING) {
        c.str();
    } else if (type == ARRAY) {
        const uint32_t et = c.get<uint32_t>();
        const uint64_t n = c.get<uint64_t>();
        if (depth > 2) return false;
        if (et == STRING || et == ARRAY) {
            for (uint64_t i = 0; i < n && c.ok; ++i)
                if (!skip_value(c, et, depth + 1)) return false;
        } else {
            const size_t sz = scalar_size(et);
            if (!sz) return false;
            c.skip(n * sz);
        }
    } else {
        const size_t sz = scalar_size(type);
        if (!sz) return false;
        c.skip(sz);
    }
    return c.ok;
}

}  // namespace

extern "C" {

const char* mq_gguf_last_error(void) { return t_error.c_str(); }

int mq_gguf_open(const char* path, mq_gguf** out) {
    if (!path || !out) return fail("null argument");
    const int fd = ::open(path, O_RDONLY);
    if (fd < 0) return fail(std::string("cannot open ") + path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 24) {
        ::close(fd);
        return fail("file too short to be GGUF");
    }
    void* map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) {
        ::close(fd);
        return fail("mmap failed");
    }
    mq_gguf* g = new mq_gguf;
    g->fd = fd;
    g->map = static_cast<const uint8_t*>(map);
    g->size = (size_t)st.st_size;
    auto bail = [&](const std::string& why) {
        mq_gguf_close(g);
        return fail(why);
    };
    Cursor c{g->map, g->map + g->size};
    if (c.get<uint32_t>() != 0x46554747u) return bail("bad magic (not a GGUF file)");
    g->version = c.get<uint32_t>();
    if (g->version != 2 && g->version != 3) return bail("unsupported GGUF version " + std::to_string(g->version));
    const uint64_t n_tensors = c.get<uint64_t>();
    const uint64_t n_kv = c.get<uint64_t>();
    if (!c.ok || n_tensors > (1u << 24) || n_kv > (1u << 24)) return bail("implausible header counts");
    for (uint64_t i = 0; i < n_kv; ++i) {
        const std::string key = c.str();
        const uint32_t type = c.get<uint32_t>();
        if (!c.ok) return bail("truncated metadata");
        Meta m;
        m.type = type;
        switch (type) {
            case U8: m.ival = c.get<uint8_t>(); break;
            case I8: m.ival = c.get<int8_t>(); break;
            case U16: m.ival = c.get<uint16_t>(); break;
            case I16: m.ival = c.get<int16_t>(); break;
            case U32: m.ival = c.get<uint32_t>(); break;
            case I32: m.ival = c.get<int32_t>(); break;
            case BOOL: m.ival = c.get<uint8_t>() != 0; break;
            case U64: m.ival = (int64_t)c.get<uint64_t>(); break;
            case I64: m.ival = c.get<int64_t>(); break;
            case STRING: m.sval = c.str(); break;
            default:
                if (!skip_value(c, type)) return bail("unsupported metadata value for key " + key);
        }
        if (!c.ok) return bail("truncated metadata value for key " + key);
        g->meta.emplace(key, std::move(m));
    }
    auto al = g->meta.find("general.alignment");
    if (al != g->meta.end() && al->second.type == U32 && al->second.ival > 0) g->alignment = (uint64_t)al->second.ival;
    if (g->alignment & (g->alignment - 1)) return bail("general.alignment is not a power of two");
    g->names.reserve((size_t)n_tensors);
    g->tensors.resize((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; ++i) {
        g->names.push_back(c.str());
        mq_gguf_tensor& t = g->tensors[(size_t)i];
        t.n_dims = (int32_t)c.get<uint32_t>();
        if (!c.ok || t.n_dims < 1 || t.n_dims > 4) return bail("tensor with unsupported number of dimensions");
        for (int d = 0; d < 4; ++d) t.ne[d] = 1;
        for (int d = 0; d < t.n_dims; ++d) t.ne[d] = (int64_t)c.get<uint64_t>();
        t.ggml_type = (int32_t)c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        if (!c.ok) return bail("truncated tensor table");
        size_t bb = 0;
        int64_t be = 1;
        t.nbytes = 0;
        for (int d = 0; d < 4; ++d)
            if (t.ne[d] <= 0) return bail("tensor " + g->names.back() + ": dimension " + std::to_string(d) + " is not positive");
        if (type_layout(t.ggml_type, &bb, &be)) {
            if (t.ne[0] % be) return bail("tensor " + g->names.back() + ": row length is not a whole number of blocks");
            // the product of untrusted 64-bit fields: every step checked, so that a crafted table cannot wrap the size
            // to a small number and slip through the bounds test below
            uint64_t bytes = (uint64_t)(t.ne[0] / be);
            bool overflow = __builtin_mul_overflow(bytes, (uint64_t)bb, &bytes);
            for (int d = 1; d < 4; ++d) overflow = overflow || __builtin_mul_overflow(bytes, (uint64_t)t.ne[d], &bytes);
            if (overflow) return bail("tensor " + g->names.back() + ": size overflows 64 bits");
            t.nbytes = bytes;
        }
    }
    const uint64_t header = (uint64_t)(c.p - g->map);
    const uint64_t base = (header + g->alignment - 1) & ~(g->alignment - 1);
    if (base > g->size) return bail("data section starts past the end of the file");
    g->data = g->map + base;
    for (size_t i = 0; i < g->tensors.size(); ++i) {
        mq_gguf_tensor& t = g->tensors[i];
        t.name = g->names[i].c_str();
        if (t.offset % g->alignment) return bail("tensor " + g->names[i] + ": misaligned offset");
        // compare before adding: base + offset may wrap
        const uint64_t room = g->size - base;
        if (t.offset > room || t.nbytes > room - t.offset) return bail("tensor " + g->names[i] + ": data runs past the end of the file");
        t.data = g->data + t.offset;
        g->by_name.emplace(g->names[i], (int64_t)i);
    }
    *out = g;
    return MQ_OK;
}

int mq_gguf_close(mq_gguf* g) {
    if (!g) return MQ_OK;
    if (g->map) munmap(const_cast<uint8_t*>(g->map), g->size);
    if (g->fd >= 0) ::close(g->fd);
    delete g;
    return MQ_OK;
}

int64_t mq_gguf_tensor_count(const mq_gguf* g) { return g ? (int64_t)g->tensors.size() : 0; }

int mq_gguf_tensor_at(const mq_gguf* g, int64_t index, mq_gguf_tensor* out) {
    if (!g || !out || index < 0 || index >= (int64_t)g->tensors.size()) return fail("tensor index out of range");
    *out = g->tensors[(size_t)index];
    return MQ_OK;
}

int64_t mq_gguf_find_tensor(const mq_gguf* g, const char* name) {
    if (!g || !name) return -1;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? -1 : it->second;
}

int mq_gguf_get_int(const mq_gguf* g, const char* key, int64_t* out) {
    if (!g || !key || !out) return fail("null argument");
    auto it = g->meta.find(key);
    if (it == g->meta.end()) return fail(std::string("no metadata key ") + key);
    const uint32_t t = it->second.type;
    if (t == STRING || t == ARRAY || t == F32 || t == F64) return fail(std::string("metadata key ") + key + " is not an integer");
    *out = it->second.ival;
    return MQ_OK;
}

int mq_gguf_get_string(const mq_gguf* g, const char* key, const char** out, size_t* len) {
    if (!g || !key || !out) return fail("null argument");
    auto it = g->meta.find(key);
    if (it == g->meta.end() || it->second.type != STRING) return fail(std::string("no string metadata key ") + key);
    *out = it->second.sval.c_str();
    if (len) *len = it->second.sval.size();
    return MQ_OK;
}

namespace {
int load_kquant(const mq_gguf* g, const char* name, bool q4k_only, mq_weight** out) {
    if (!g || !name || !out) return fail("null argument");
    const int64_t idx = mq_gguf_find_tensor(g, name);
    if (idx < 0) return fail(std::string("no tensor ") + name);
    const mq_gguf_tensor& t = g->tensors[(size_t)idx];
    if (t.ggml_type != 12 && (q4k_only || (t.ggml_type != 13 && t.ggml_type != 14 && t.ggml_type != 8)))
        return fail(std::string("tensor ") + name + (q4k_only ? " is not GGML_TYPE_Q4_K" : " is not of type Q4_K, Q5_K, Q6_K or Q8_0"));
    if (t.n_dims > 3 || t.ne[3] != 1) return fail(std::string("tensor ") + name + " has more than three dimensions");
    if (t.ne[0] % 256) return fail(std::string("tensor ") + name + ": row length is not a multiple of 256");
    // bytes of 256 weights of a row: one K-quant super-block, or eight Q8_0 blocks
    const size_t row_bytes = (size_t)(t.ne[0] / 256) * (t.ggml_type == 12 ? 144 : t.ggml_type == 13 ? 176 : t.ggml_type == 14 ? 210 : 272);
    return mq_weight_upload_typed(t.ggml_type, t.data, t.ne[1], t.ne[0], t.ne[2], row_bytes, row_bytes * (size_t)t.ne[1], out);
}
}  // namespace

int mq_gguf_load_q4k(const mq_gguf* g, const char* name, mq_weight** out) { return load_kquant(g, name, true, out); }

int mq_gguf_load_weight(const mq_gguf* g, const char* name, mq_weight** out) { return load_kquant(g, name, false, out); }

namespace {

// The first of the reference's alternative names for a per-layer tensor that the file holds: "blk.<layer>.<suffix>"
// (get_layer_tensor_any, core/src/models/model_loader.cpp:3802-3811).
const mq_gguf_tensor* layer_tensor_any(const mq_gguf* g, int layer, std::initializer_list<const char*> suffixes) {
    for (const char* suffix : suffixes) {
        const std::string name = "blk." + std::to_string(layer) + "." + suffix;
        const int64_t idx = mq_gguf_find_tensor(g, name.c_str());
        if (idx >= 0) return &g->tensors[(size_t)idx];
    }
    return nullptr;
}

float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: normalise
            int e = -1;
            uint32_t m = man;
            do {
                ++e;
                m <<= 1;
            } while (!(m & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

// An F32 or F16 tensor of `count` elements as fp32 on the device.
int upload_f32(const mq_gguf_tensor* t, int64_t count, float** out_dev) {
    if (t->ggml_type != 0 && t->ggml_type != 1) return fail(std::string("tensor ") + t->name + " is neither F32 nor F16");
    if (t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3] != count) return fail(std::string("tensor ") + t->name + " has an unexpected shape");
    std::vector<float> host((size_t)count);
    if (t->ggml_type == 0) {
        std::memcpy(host.data(), t->data, (size_t)count * 4);
    } else {
        const uint16_t* h = static_cast<const uint16_t*>(t->data);
        for (int64_t i = 0; i < count; ++i) host[(size_t)i] = half_to_float(h[i]);
    }
    void* dev = nullptr;
    if (int rc = mq_device_malloc(&dev, (size_t)count * 4)) return rc;
    if (int rc = mq_memcpy_h2d(dev, host.data(), (size_t)count * 4)) {
        mq_device_free(dev);
        return rc;
    }
    *out_dev = static_cast<float*>(dev);
    return MQ_OK;
}

}  // namespace

int mq_gguf_free_moe_layer(mq_gguf_moe_layer* L) {
    if (!L) return MQ_OK;
    for (mq_weight*& w : L->owned) {
        if (w) mq_weight_free(w);
        w = nullptr;
    }
    if (L->router_dev) mq_device_free(L->router_dev);
    if (L->sh_gate_inp_dev) mq_device_free(L->sh_gate_inp_dev);
    *L = mq_gguf_moe_layer{};
    return MQ_OK;
}

int mq_gguf_load_moe_layer(const mq_gguf* g, int layer_index, mq_gguf_moe_layer* out) {
    if (!g || !out || layer_index < 0) return fail("null argument or negative layer");
    *out = mq_gguf_moe_layer{};
    // the stacked expert tensors (core/src/models/model_loader.cpp:231-235,4429-4440) ...
    const mq_gguf_tensor* ge = layer_tensor_any(g, layer_index, {"ffn_gate_exps.weight", "ffn_gate_exps", "experts.gate_proj.weight"});
    const mq_gguf_tensor* ue = layer_tensor_any(g, layer_index, {"ffn_up_exps.weight", "ffn_up_exps", "experts.up_proj.weight"});
    const mq_gguf_tensor* de = layer_tensor_any(g, layer_index, {"ffn_down_exps.weight", "ffn_down_exps", "experts.down_proj.weight"});
    if (!ge || !ue || !de) return fail("layer " + std::to_string(layer_index) + " holds no stacked ffn_{gate,up,down}_exps tensors");
    // ... the shared expert, the router and the shared expert's scalar gate (:3961-4001)
    const mq_gguf_tensor* sg = layer_tensor_any(g, layer_index, {"ffn_gate.weight", "ffn_gate_shexp.weight", "shared_expert.gate_proj.weight", "mlp.gate_proj.weight", "gate_proj.weight"});
    const mq_gguf_tensor* su = layer_tensor_any(g, layer_index, {"ffn_up.weight", "ffn_up_shexp.weight", "shared_expert.up_proj.weight", "mlp.up_proj.weight", "up_proj.weight"});
    const mq_gguf_tensor* sd = layer_tensor_any(g, layer_index, {"ffn_down.weight", "ffn_down_shexp.weight", "shared_expert.down_proj.weight", "mlp.down_proj.weight", "down_proj.weight"});
    const mq_gguf_tensor* sgi = layer_tensor_any(g, layer_index, {"ffn_gate_inp_shexp.weight", "shared_expert_gate.weight"});
    const mq_gguf_tensor* router = layer_tensor_any(g, layer_index, {"moe_gate.weight", "router.proj.weight", "mlp.gate.weight", "ffn_gate_inp.weight", "ffn_gate_inp"});
    // layout facts of the stacks (core/src/llm/moe/native.cpp:4546-4548,4589-4597): gate / up [n_embd, n_ff, n_expert],
    // down [n_ff, n_embd, n_expert]
    const int64_t hidden = ge->ne[0], inter = ge->ne[1], E = ge->ne[2];
    if (ue->ne[0] != hidden || ue->ne[1] != inter || ue->ne[2] != E || de->ne[0] != inter || de->ne[1] != hidden || de->ne[2] != E)
        return fail("layer " + std::to_string(layer_index) + ": the expert stacks do not fit each other");
    if ((sg || su || sd) && !(sg && su && sd)) return fail("layer " + std::to_string(layer_index) + ": an incomplete shared expert");
    if (sg && (sg->ne[0] != hidden || sg->ne[1] != inter || su->ne[0] != hidden || su->ne[1] != inter || sd->ne[0] != inter || sd->ne[1] != hidden))
        return fail("layer " + std::to_string(layer_index) + ": the shared expert does not have the routed experts' shape");
    int rc = load_kquant(g, ge->name, false, &out->owned[0]);
    if (rc == MQ_OK) rc = load_kquant(g, ue->name, false, &out->owned[1]);
    if (rc == MQ_OK) rc = load_kquant(g, de->name, false, &out->owned[2]);
    if (rc == MQ_OK && sg) rc = load_kquant(g, sg->name, false, &out->owned[3]);
    if (rc == MQ_OK && sg) rc = load_kquant(g, su->name, false, &out->owned[4]);
    if (rc == MQ_OK && sg) rc = load_kquant(g, sd->name, false, &out->owned[5]);
    if (rc == MQ_OK && router) {
        if (router->ne[0] != hidden || router->ne[1] != E) rc = fail(std::string("tensor ") + router->name + " is not [n_embd, n_expert]");
        else rc = upload_f32(router, hidden * E, &out->router_dev);
    }
    if (rc == MQ_OK && sgi) rc = upload_f32(sgi, hidden, &out->sh_gate_inp_dev);
    if (rc != MQ_OK) {
        mq_gguf_free_moe_layer(out);
        return rc;
    }
    out->desc.gate_exps = out->owned[0], out->desc.up_exps = out->owned[1], out->desc.down_exps = out->owned[2];
    out->desc.shared_gate = out->owned[3], out->desc.shared_up = out->owned[4], out->desc.shared_down = out->owned[5];
    out->desc.sh_gate_inp_dev = out->sh_gate_inp_dev;
    out->n_experts = E, out->hidden = hidden, out->inter = inter;
    // experts per token: "<architecture>.expert_used_count" (the key ggml model files carry)
    const char* arch = nullptr;
    size_t arch_len = 0;
    int64_t used = 0;
    if (mq_gguf_get_string(g, "general.architecture", &arch, &arch_len) == MQ_OK &&
        mq_gguf_get_int(g, (std::string(arch, arch_len) + ".expert_used_count").c_str(), &used) == MQ_OK && used > 0 && used <= 8)
        out->desc.top_k = (int)used;
    return MQ_OK;
}

}  // extern "C"
