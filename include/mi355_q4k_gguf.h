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

#ifdef __cplusplus
}
#endif
#endif /* MI355_Q4K_GGUF_H */
