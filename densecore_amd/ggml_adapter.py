"""ctypes view of the GGML_OP_CUSTOM adapters (libmi355q4k_ggml.so).

Builds `struct ggml_tensor` values over numpy buffers the way a ggml CPU graph would hold them
(host memory, ne[0] innermost, nb in bytes) and calls the adapters with the callback signature
`void fn(ggml_tensor* dst, int ith, int nth, void* userdata)`.  Used by the tests and as the
worked example of the binding a DenseCore maintainer adds (core/src/llm/matmul/graph_ops.cpp:212-227).
"""
import ctypes as C
import os

import numpy as np

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355q4k_ggml.so")

# every symbol include/mi355_q4k_ggml.h declares
CALLBACKS = [
    "mq_cb_gemv_custom", "mq_cb_gemv_batched_custom", "mq_cb_moe_gateup_swiglu", "mq_cb_moe_down_weighted_logits",
    "mq_cb_moe_fused_router", "mq_cb_moe_topk_weights_from_logits", "mq_cb_mul_mat_id",
]
CALLBACKS2 = ["mq_cb_silu_mul_fused", "mq_cb_apply_shared_scalar_gate"]   # ggml_custom2_op_t: (dst, a, b, ith, nth, userdata)
EXPORTS = CALLBACKS + CALLBACKS2 + [
    "mq_ggml_graph_begin", "mq_ggml_tensor_to_host", "mq_ggml_last_status", "mq_ggml_weight_cache_clear", "mq_ggml_weight_cache_size", "mq_ggml_weight_fingerprint",
    "mq_matmul_ggml_quantized_transb",
]

GGML_TYPE_F32, GGML_TYPE_Q4_K, GGML_TYPE_Q5_K, GGML_TYPE_Q6_K, GGML_TYPE_I32 = 0, 12, 13, 14, 26
GGML_TYPE_Q8_0 = 8
GGML_OP_CUSTOM_PLACEHOLDER = 0  # the adapters never read dst->op


class GgmlTensor(C.Structure):
    """Public layout of struct ggml_tensor (ggml.h)."""


GgmlTensor._fields_ = [
    ("type", C.c_int), ("buffer", C.c_void_p), ("ne", C.c_int64 * 4), ("nb", C.c_size_t * 4), ("op", C.c_int),
    ("op_params", C.c_int32 * 16), ("flags", C.c_int32), ("src", C.POINTER(GgmlTensor) * 10),
    ("view_src", C.POINTER(GgmlTensor)), ("view_offs", C.c_size_t), ("data", C.c_void_p), ("name", C.c_char * 64),
    ("extra", C.c_void_p), ("padding", C.c_char * 8),
]


class UserData(C.Structure):
    _fields_ = [("silu_mode", C.c_int), ("reserved", C.c_int), ("use_defaults", C.c_int), ("last_status", C.c_int),
                ("keep_hidden_on_device", C.c_int)]


class RouterState(C.Structure):
    """QwenNativeMoEFusedRouterState (core/src/llm/moe/native.cpp:602-608) as the fused router node's userdata."""
    _fields_ = [("n_experts", C.c_int64), ("n_tokens", C.c_int64), ("top_k", C.c_int64),
                ("normalized_weights", C.c_void_p), ("work_ctx", C.c_void_p)]


_handle = None


def lib():
    global _handle
    if _handle is None:
        try:
            _lib.lib()   # the C ABI library first, initialised on device 0: the adapter library links against it
        except _lib.MqError:
            _lib.load()  # no GPU: the host-only helpers (fingerprint, GGUF reader) still work, every node reports MQ_ERR_STATE
        if not os.path.exists(LIB_PATH):
            raise _lib.MqError(f"{LIB_PATH} is missing: run `make -C densecore_amd/host`")
        L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        cb = [C.POINTER(GgmlTensor), C.c_int, C.c_int, C.c_void_p]
        for name in CALLBACKS:
            getattr(L, name).argtypes = cb
            getattr(L, name).restype = None
        for name in CALLBACKS2:
            getattr(L, name).argtypes = [C.POINTER(GgmlTensor), C.POINTER(GgmlTensor), C.POINTER(GgmlTensor), C.c_int, C.c_int, C.c_void_p]
            getattr(L, name).restype = None
        L.mq_ggml_graph_begin.restype = None
        L.mq_ggml_tensor_to_host.argtypes = [C.POINTER(GgmlTensor)]
        L.mq_ggml_weight_cache_size.restype = C.c_int64
        L.mq_ggml_weight_fingerprint.argtypes = [C.c_void_p, C.c_size_t]
        L.mq_ggml_weight_fingerprint.restype = C.c_uint64
        L.mq_matmul_ggml_quantized_transb.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int32,
                                                      C.c_int64, C.c_int64, C.c_size_t, C.c_void_p, C.c_int64]
        _handle = L
    return _handle


def tensor(array: np.ndarray, ggml_type: int, ne, nb=None, name: bytes = b"") -> GgmlTensor:
    """A ggml_tensor over `array`'s memory (kept alive by the caller).  ne is ggml order (innermost first)."""
    t = GgmlTensor()
    t.type = ggml_type
    ne = list(ne) + [1] * (4 - len(ne))
    if nb is None:
        if ggml_type in (GGML_TYPE_Q4_K, GGML_TYPE_Q5_K, GGML_TYPE_Q6_K):
            bb = {GGML_TYPE_Q4_K: 144, GGML_TYPE_Q5_K: 176, GGML_TYPE_Q6_K: 210}[ggml_type]
            nb = [bb, bb * (ne[0] // 256)]
        elif ggml_type == GGML_TYPE_Q8_0:
            nb = [34, 34 * (ne[0] // 32)]
        else:
            nb = [4, 4 * ne[0]]
        while len(nb) < 4:
            nb.append(nb[-1] * ne[len(nb) - 1])
    nb = list(nb)
    while len(nb) < 4:
        nb.append(nb[-1] * ne[len(nb) - 1])
    for i in range(4):
        t.ne[i] = ne[i]
        t.nb[i] = nb[i]
    t.data = array.ctypes.data
    t.name = name
    t._keep = array
    return t


def set_src(dst: GgmlTensor, *srcs: GgmlTensor) -> None:
    for i, s in enumerate(srcs):
        dst.src[i] = C.pointer(s)
    dst._srcs = srcs
