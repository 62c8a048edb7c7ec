/*
 * mi355_q4k_gguf.h -- reads Q4_K tensors straight out of a .gguf file into mq_weight handles.
 *
 * DenseCore opens model files with ggml's gguf_init_from_file and walks the tensor table
 * (core/src/models/model_loader.cpp:2063-2125), then binds the stacked expert tensors
 * ffn_{gate,up,down}_exps [K, N, E] and the dense projections by name
 * (core/src/models/model_loader.cpp:4429-4434, core/src/llm/moe/native.cpp:4546-4548,4589-4597).
 * ggml itself is not part of this build, so the container is parsed here from its published
 * layout (GGUF v2/v3, little endian):
 *   u32 magic "GGUF", u32 version, u64 n_tensors, u64 n_kv,
 *   n_kv x { string key, u32 type, value }        string = u64 length + bytes; array = u32 type, u64 count, items
 *   n_tensors x { string name, u32 n_dims, u64 ne[n_dims], u32 ggml_type, u64 offset }
 *   padding to general.alignment (u32 key, default 32); tensor data at that base + offset.
 * Only what the hot path needs is exposed: the tensor table, the integer/string metadata a loader
 * looks up, and the upload of GGML_TYPE_Q4_K (12) tensors.  The file is memory-mapped read-only.
 */
#ifndef MI355_Q4K_GGUF_H
#define MI355_Q4K_GGUF_H

#include <stddef.h>
#include <stdint.h>

#include "mi355_q4k.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mq_gguf mq_gguf;

typedef struct {
    const char* name;   /* owned by the mq_gguf */
    int32_t ggml_type;  /* 0 = F32, 1 = F16, 12 = Q4_K, ... */
    int32_t n_dims;
    int64_t ne[4];      /* ne[0] innermost; unused dims are 1 */
    uint64_t offset;    /* from the start of the data section */
    uint64_t nbytes;    /* 0 when the type's block size is not known here */
    const void* data;   /* into the mapping */
} mq_gguf_tensor;

/* MQ_OK or MQ_ERR_INVALID (not a GGUF file, truncated, unsupported version); mq_gguf_last_error() explains. */
int mq_gguf_open(const char* path, mq_gguf** out);
const char* mq_gguf_last_error(void); /* of the calling thread */
int mq_gguf_close(mq_gguf* g);
int64_t mq_gguf_tensor_count(const mq_gguf* g);
int mq_gguf_tensor_at(const mq_gguf* g, int64_t index, mq_gguf_tensor* out);
/* index of the tensor called `name`, or -1 (gguf_find_tensor's contract) */
int64_t mq_gguf_find_tensor(const mq_gguf* g, const char* name);
/* Metadata: integer-valued keys of any integer/bool type, and strings.  Return MQ_ERR_INVALID when the key
 * is missing or of another kind. */
int mq_gguf_get_int(const mq_gguf* g, const char* key, int64_t* out);
int mq_gguf_get_string(const mq_gguf* g, const char* key, const char** out, size_t* len);
/* Uploads tensor `name` (GGML_TYPE_Q4_K; 2-D [K, N] -> one matrix of N rows, 3-D [K, N, E] -> an expert
 * stack) with mq_weight_upload.  mq_init must have been called. */
int mq_gguf_load_q4k(const mq_gguf* g, const char* name, mq_weight** out);
/* The same for a tensor of any type the product entry points multiply: GGML_TYPE_Q4_K, Q5_K or Q6_K, or a
 * dense (2-D) Q8_0 matrix (mq_weight_upload_typed).  A Q4_K_M file stores part of its down projections as Q5_K or
 * Q6_K. */
int mq_gguf_load_weight(const mq_gguf* g, const char* name, mq_weight** out);

/* One MoE layer of a model file bound to the descriptor mq_moe_layer_q4k takes: the stacked expert tensors
 * blk.<layer>.ffn_{gate,up,down}_exps [K, N, E] (any type the product entry points multiply), the shared expert
 * blk.<layer>.ffn_{gate,up,down}_shexp.weight when the layer has one, its scalar gate ffn_gate_inp_shexp.weight and the
 * router ffn_gate_inp.weight (F32 or F16, uploaded as fp32) -- each under the alternative names the reference's loader
 * tries, in its order (core/src/models/model_loader.cpp:231-235, 3961-4001, 4429-4440; stack layout
 * core/src/llm/moe/native.cpp:4546-4548,4589-4597).  desc.top_k comes from "<general.architecture>.expert_used_count"
 * when the file has it (else 0: the caller sets it); silu_mode and route_mode are left 0 for the caller.
 * Everything is owned by the struct until mq_gguf_free_moe_layer. */
typedef struct {
    mq_moe_layer_desc desc;
    mq_weight* owned[6];     /* gate_exps, up_exps, down_exps, shared gate / up / down (NULL without a shared expert) */
    float* router_dev;       /* fp32 [n_experts][hidden] on the device, or NULL when the file has no router tensor */
    float* sh_gate_inp_dev;  /* fp32 [hidden] or NULL */
    int64_t n_experts, hidden, inter;
} mq_gguf_moe_layer;
int mq_gguf_load_moe_layer(const mq_gguf* g, int layer_index, mq_gguf_moe_layer* out);
int mq_gguf_free_moe_layer(mq_gguf_moe_layer* layer);

#ifdef __cplusplus
}
#endif
#endif /* MI355_Q4K_GGUF_H */
