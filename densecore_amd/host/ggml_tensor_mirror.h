// Field-for-field mirror of the public `struct ggml_tensor` (ggml.h) for builds without a ggml
// header.  Only type, ne, nb, op_params, src, data and name are read by the adapters; the other
// members exist so that those sit at ggml's offsets.  A build inside DenseCore defines
// MQ_HAVE_GGML_H and includes the real header instead.
#pragma once
#ifdef MQ_HAVE_GGML_H
#include "ggml.h"
#else
#include <cstddef>
#include <cstdint>

extern "C" {
enum ggml_type : int { GGML_TYPE_F32 = 0, GGML_TYPE_F16 = 1, GGML_TYPE_Q8_0 = 8, GGML_TYPE_Q4_K = 12, GGML_TYPE_Q5_K = 13, GGML_TYPE_Q6_K = 14, GGML_TYPE_Q8_K = 15, GGML_TYPE_I32 = 26 };
#define GGML_MAX_DIMS 4
#define GGML_MAX_SRC 10
#define GGML_MAX_OP_PARAMS 64
#define GGML_MAX_NAME 64
struct ggml_backend_buffer;
struct ggml_tensor {
    enum ggml_type type;
    struct ggml_backend_buffer* buffer;
    int64_t ne[GGML_MAX_DIMS];  // elements per dimension, ne[0] innermost
    size_t nb[GGML_MAX_DIMS];   // strides in bytes
    int op;
    int32_t op_params[GGML_MAX_OP_PARAMS / sizeof(int32_t)];
    int32_t flags;
    struct ggml_tensor* src[GGML_MAX_SRC];
    struct ggml_tensor* view_src;
    size_t view_offs;
    void* data;
    char name[GGML_MAX_NAME];
    void* extra;
    char padding[8];
};
}
#endif
