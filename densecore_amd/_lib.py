"""ctypes loader for libmi355q4k.so (the C ABI declared in include/mi355_q4k.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355q4k.so")

# every symbol include/mi355_q4k.h declares
EXPORTS = [
    "mq_init", "mq_shutdown", "mq_last_error", "mq_device_info",
    "mq_weight_upload", "mq_weight_upload_typed", "mq_weight_synthetic", "mq_weight_synthetic_typed", "mq_weight_type", "mq_weight_download", "mq_weight_shape", "mq_weight_free",
    "mq_quantize_q8k", "mq_mul_mat_q4k", "mq_mul_mat_q4k_multi", "mq_mul_mat_q4k_noalloc", "mq_gemm_q4k", "mq_mul_mat_q4k_q8k", "mq_mul_mat_q4k_host", "mq_swiglu_mul_mat_q4k",
    "mq_ffn_swiglu_q4k", "mq_moe_gateup_swiglu_q4k", "mq_moe_down_weighted_q4k",
    "mq_moe_route_topk", "mq_moe_weights_from_logits", "mq_mul_mat_id_q4k", "mq_moe_layer_q4k",
    "mq_acts_create", "mq_acts_free", "mq_acts_quantize", "mq_mul_mat_q4k_acts", "mq_swiglu_mul_mat_q4k_acts",
    "mq_silu_mul_f32", "mq_scale_rows_sigmoid_f32", "mq_add_rmsnorm_f32", "mq_add_rmsnorm_q8k", "mq_router_logits_f32", "mq_add_rmsnorm_router_f32", "mq_rmsnorm_mul_mat_q4k",
    "mq_decoder_create", "mq_decoder_step", "mq_decoder_status", "mq_decoder_set_patience", "mq_decoder_free",
    "mq_device_malloc", "mq_device_free", "mq_memcpy_h2d", "mq_memcpy_d2h", "mq_host_malloc", "mq_host_free", "mq_memcpy_h2d_async", "mq_memcpy_d2h_async", "mq_stream_synchronize",
]
# every symbol include/mi355_q4k_debug.h declares (verification hooks and measurement instruments)
DEBUG_EXPORTS = [
    "mq_debug_block_sums", "mq_debug_moe_groups", "mq_debug_moe_hidden", "mq_debug_decoder_buffers",
    "mq_census_enable", "mq_census_reset", "mq_census_read", "mq_debug_set_dense_lds", "mq_debug_set_skeleton",
]


class MoELayerDesc(C.Structure):
    _fields_ = [
        ("gate_exps", C.c_void_p), ("up_exps", C.c_void_p), ("down_exps", C.c_void_p),
        ("shared_gate", C.c_void_p), ("shared_up", C.c_void_p), ("shared_down", C.c_void_p),
        ("sh_gate_inp_dev", C.c_void_p),
        ("top_k", C.c_int), ("silu_mode", C.c_int), ("route_mode", C.c_int),
    ]


class DecoderLayerDesc(C.Structure):
    _fields_ = [
        ("wqkv", C.c_void_p), ("wo", C.c_void_p), ("attn_norm_dev", C.c_void_p), ("ffn_norm_dev", C.c_void_p),
        ("router_dev", C.c_void_p), ("fixed_logits_dev", C.c_void_p), ("moe", MoELayerDesc),
    ]


class MqError(RuntimeError):
    pass


_lib = None
_inited = False


def load() -> C.CDLL:
    """Load the shared library (no GPU needed for this step)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MqError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                      "or `make -C densecore_amd/csrc`")
    L = C.CDLL(LIB_PATH)
    i64, vp, sz, ci = C.c_int64, C.c_void_p, C.c_size_t, C.c_int
    L.mq_last_error.restype = C.c_char_p
    L.mq_init.argtypes = [ci]
    L.mq_device_info.argtypes = [C.c_char_p, sz, C.POINTER(ci), C.POINTER(sz)]
    L.mq_weight_upload.argtypes = [vp, i64, i64, i64, sz, sz, C.POINTER(vp)]
    L.mq_weight_synthetic.argtypes = [C.c_uint64, i64, i64, i64, C.POINTER(vp)]
    L.mq_weight_upload_typed.argtypes = [C.c_int, vp, i64, i64, i64, sz, sz, C.POINTER(vp)]
    L.mq_weight_synthetic_typed.argtypes = [C.c_int, C.c_uint64, i64, i64, i64, C.POINTER(vp)]
    L.mq_weight_type.argtypes = [vp]
    L.mq_weight_download.argtypes = [vp, vp, sz, sz]
    L.mq_weight_shape.argtypes = [vp, C.POINTER(i64), C.POINTER(i64), C.POINTER(i64), C.POINTER(sz)]
    L.mq_weight_free.argtypes = [vp]
    L.mq_quantize_q8k.argtypes = [vp, i64, i64, i64, vp, vp]
    L.mq_mul_mat_q4k.argtypes = [vp, vp, i64, i64, vp, i64, vp]
    L.mq_mul_mat_q4k_multi.argtypes = [C.POINTER(vp), ci, vp, C.POINTER(vp), vp]
    L.mq_mul_mat_q4k_noalloc.argtypes = [vp, vp, i64, i64, vp, i64, vp]
    L.mq_gemm_q4k.argtypes = [vp, vp, i64, i64, vp, i64, vp]
    L.mq_mul_mat_q4k_q8k.argtypes = [vp, vp, i64, sz, vp, i64, vp]
    L.mq_mul_mat_q4k_host.argtypes = [vp, vp, i64, i64, vp, i64]
    L.mq_ffn_swiglu_q4k.argtypes = [vp, vp, vp, vp, i64, vp, ci, vp]
    L.mq_swiglu_mul_mat_q4k.argtypes = [vp, vp, vp, i64, i64, vp, i64, ci, vp]
    L.mq_moe_gateup_swiglu_q4k.argtypes = [vp, vp, vp, i64, vp, ci, ci, vp, vp]
    L.mq_moe_down_weighted_q4k.argtypes = [vp, vp, i64, vp, vp, ci, vp, vp]
    L.mq_moe_route_topk.argtypes = [vp, i64, i64, ci, ci, vp, vp, vp]
    L.mq_moe_weights_from_logits.argtypes = [vp, i64, i64, vp, ci, vp, vp]
    L.mq_mul_mat_id_q4k.argtypes = [vp, vp, i64, ci, vp, ci, vp, vp]
    L.mq_moe_layer_q4k.argtypes = [C.POINTER(MoELayerDesc), vp, vp, i64, vp, vp, vp, vp]
    L.mq_debug_block_sums.argtypes = [vp, vp, i64, i64, vp, vp, vp, i64, vp]
    L.mq_debug_moe_groups.argtypes = [vp, vp, i64, i64, ci, vp, vp, vp]
    L.mq_debug_moe_hidden.argtypes = [vp, sz, vp]
    L.mq_debug_decoder_buffers.argtypes = [vp] + [C.POINTER(vp)] * 5
    L.mq_silu_mul_f32.argtypes = [vp, vp, i64, i64, i64, i64, vp, i64, ci, vp]
    L.mq_scale_rows_sigmoid_f32.argtypes = [vp, i64, i64, i64, vp, i64, vp, i64, vp]
    L.mq_add_rmsnorm_f32.argtypes = [vp, vp, vp, i64, i64, C.c_float, vp, vp, vp]
    L.mq_add_rmsnorm_q8k.argtypes = [vp, vp, vp, i64, i64, C.c_float, vp, vp, vp, vp]
    L.mq_router_logits_f32.argtypes = [vp, i64, i64, vp, i64, i64, vp, vp]
    L.mq_rmsnorm_mul_mat_q4k.argtypes = [vp, vp, vp, vp, i64, C.c_float, vp, vp, i64, vp]
    L.mq_add_rmsnorm_router_f32.argtypes = [vp, vp, vp, i64, i64, C.c_float, vp, vp, vp, i64, vp, vp]
    L.mq_decoder_create.argtypes = [vp, ci, i64, C.c_float, C.POINTER(vp)]
    L.mq_decoder_step.argtypes = [vp, vp, i64, ci, vp, vp, vp, vp]
    L.mq_decoder_status.argtypes = [vp]
    L.mq_decoder_set_patience.argtypes = [vp, i64]
    L.mq_decoder_free.argtypes = [vp]
    L.mq_decoder_free.restype = None
    L.mq_acts_create.argtypes = [i64, i64, C.POINTER(vp)]
    L.mq_acts_free.argtypes = [vp]
    L.mq_acts_quantize.argtypes = [vp, vp, i64, i64, vp]
    L.mq_mul_mat_q4k_acts.argtypes = [vp, vp, vp, i64, vp]
    L.mq_swiglu_mul_mat_q4k_acts.argtypes = [vp, vp, vp, vp, i64, ci, vp]
    L.mq_census_enable.argtypes = [ci]
    L.mq_debug_set_skeleton.argtypes = [ci]
    L.mq_census_read.argtypes = [ci, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(i64)]
    L.mq_device_malloc.argtypes = [C.POINTER(vp), sz]
    L.mq_device_free.argtypes = [vp]
    L.mq_memcpy_h2d.argtypes = [vp, vp, sz]
    L.mq_memcpy_d2h.argtypes = [vp, vp, sz]
    L.mq_stream_synchronize.argtypes = [vp]
    for name in EXPORTS + DEBUG_EXPORTS:
        if name != "mq_last_error":
            getattr(L, name).restype = ci
    _lib = L
    return L


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise MqError(f"{what} failed (rc={rc}): {load().mq_last_error().decode()}")


def lib() -> C.CDLL:
    """Load and initialise on device 0; raises if there is no MI355X."""
    global _inited
    L = load()
    if not _inited:
        check(L.mq_init(0), "mq_init")
        _inited = True
    return L
