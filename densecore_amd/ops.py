"""Host-side operator surface over libmi355q4k.so, named after the DenseCore
functions each call stands in for.  Tensors are torch CUDA tensors (PyTorch is
used only to own device memory and the stream); all arithmetic happens in the
HIP library.  Every function raises if the library or the GPU is missing.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib
from .synth import BLOCK_BYTES, GGML_TYPE_Q4_K, GGML_TYPE_Q5_K, GGML_TYPE_Q6_K, GGML_TYPE_Q8_0, Q4K_BLOCK_BYTES, Q8K_BLOCK_BYTES, QK_K

SILU_EXACT, SILU_FAST, SILU_FAST_FMA = 0, 1, 2
ROUTE_FUSED, ROUTE_FLOOR, ROUTE_FLOOR_FINITE = 0, 1, 2


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: torch.Tensor) -> C.c_void_p:
    return C.c_void_p(t.data_ptr())


def _f32(x: torch.Tensor) -> torch.Tensor:
    if x.dtype != torch.float32 or not x.is_cuda:
        raise TypeError("expected a float32 CUDA tensor")
    return x.contiguous()


class Q4KWeight:
    """Device-resident Q4_K matrix or expert stack (GgmlQuantizedMatrixView's weight side,
    core/include/densecore/backend/cpu_backend.h:91-99)."""

    def __init__(self, handle: int, rows: int, cols: int, n_experts: int, ggml_type: int = GGML_TYPE_Q4_K):
        self._h = C.c_void_p(handle)
        self.rows, self.cols, self.n_experts, self.ggml_type = rows, cols, n_experts, ggml_type

    @property
    def block_bytes(self) -> int:
        return BLOCK_BYTES[self.ggml_type]

    @classmethod
    def from_ggml(cls, data: np.ndarray, cols: int, ggml_type: int = GGML_TYPE_Q4_K) -> "Q4KWeight":
        """data: uint8 [rows, row_bytes] or [n_experts, rows, row_bytes] in ggml block_q4_K (type 12),
        block_q5_K (type 13), block_q6_K (type 14) or -- dense matrices for mul_mat only -- Q8_0 (type 8) row layout."""
        a = np.ascontiguousarray(data, dtype=np.uint8)
        if a.ndim == 2:
            a = a[None]
        e, rows, row_bytes = a.shape
        h = C.c_void_p()
        _lib.check(_lib.lib().mq_weight_upload_typed(ggml_type, C.c_void_p(a.ctypes.data), rows, cols, e, row_bytes,
                                                     rows * row_bytes, C.byref(h)), "mq_weight_upload_typed")
        return cls(h.value, rows, cols, e, ggml_type)

    @classmethod
    def synthetic(cls, seed: int, rows: int, cols: int, n_experts: int = 1,
                  ggml_type: int = GGML_TYPE_Q4_K) -> "Q4KWeight":
        h = C.c_void_p()
        _lib.check(_lib.lib().mq_weight_synthetic_typed(ggml_type, C.c_uint64(seed & 0xFFFFFFFFFFFFFFFF), rows, cols,
                                                        n_experts, C.byref(h)), "mq_weight_synthetic_typed")
        return cls(h.value, rows, cols, n_experts, ggml_type)

    def to_ggml(self) -> np.ndarray:
        row_bytes = self.cols // QK_K * self.block_bytes
        out = np.zeros((self.n_experts, self.rows, row_bytes), np.uint8)
        _lib.check(_lib.lib().mq_weight_download(self._h, C.c_void_p(out.ctypes.data), row_bytes,
                                                 self.rows * row_bytes), "mq_weight_download")
        return out[0] if self.n_experts == 1 else out

    @property
    def ggml_bytes(self) -> int:
        return self.n_experts * self.rows * (self.cols // QK_K) * self.block_bytes

    def free(self) -> None:
        if self._h:
            _lib.lib().mq_weight_free(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def quantize_row_q8_k(x: torch.Tensor) -> torch.Tensor:
    """QuantizeRowQ8K_Hwy (core/include/densecore/simd/hwy_ops.h:255): fp32 [n, k] -> uint8 [n, k/256*292]."""
    x = _f32(x)
    if x.dim() == 1:
        x = x[None]
    n, k = x.shape
    if k % QK_K:
        raise ValueError("cols must be a multiple of 256")
    out = torch.empty((n, k // QK_K * Q8K_BLOCK_BYTES), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.lib().mq_quantize_q8k(_ptr(x), n, x.stride(0), k, _ptr(out), _stream()), "mq_quantize_q8k")
    return out


def mul_mat(w: Q4KWeight, x: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """ggml_mul_mat(Q4_K w, F32 x): y[m, r] = w[r] . q8k(x[m]).  cb_gemv_custom / cb_gemv_batched_custom
    (core/src/llm/matmul/gemv_exec.cpp:99, batched_exec.cpp:55) and MatMulGgmlQuantizedTransB."""
    x = _f32(x)
    if x.dim() == 1:
        x = x[None]
    n = x.shape[0]
    y = out if out is not None else torch.empty((n, w.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_mul_mat_q4k(w._h, _ptr(x), n, x.stride(0), _ptr(y), w.rows, _stream()), "mq_mul_mat_q4k")
    return y


def mul_mat_multi(ws, x: torch.Tensor, outs=None):
    """Several products of one activation row in one launch (mq_mul_mat_q4k_multi): the q, k and v projections of a
    layer as the graph emits them on one input (core/src/llm/graph/decoder.cpp:1092-1099).  Returns the list of y."""
    x = _f32(x).reshape(-1)
    ys = outs if outs is not None else [torch.empty((w.rows,), dtype=torch.float32, device=x.device) for w in ws]
    wl = (C.c_void_p * len(ws))(*[w._h for w in ws])
    yl = (C.c_void_p * len(ws))(*[y.data_ptr() for y in ys])
    _lib.check(_lib.lib().mq_mul_mat_q4k_multi(wl, len(ws), _ptr(x), yl, _stream()), "mq_mul_mat_q4k_multi")
    return ys


def gemm(w: Q4KWeight, x: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """The same product through the int8 matrix-core GEMM kernel at any n (RunQ4KRawBatchedDenseGemm,
    core/src/backend/cpu_backend_q4k_dense.cpp:57-101)."""
    x = _f32(x)
    n = x.shape[0]
    y = out if out is not None else torch.empty((n, w.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_gemm_q4k(w._h, _ptr(x), n, x.stride(0), _ptr(y), y.stride(0), _stream()), "mq_gemm_q4k")
    return y


class Q8KActs:
    """Device-resident Q8_K rows shared by several products (the reference's shared Q8 scratch,
    core/src/llm/matmul/gemv_exec.cpp:298-341)."""

    def __init__(self, max_rows: int, cols: int):
        h = C.c_void_p()
        _lib.check(_lib.lib().mq_acts_create(max_rows, cols, C.byref(h)), "mq_acts_create")
        self._h, self.max_rows, self.cols, self.n = h.value, max_rows, cols, 0

    def quantize(self, x: torch.Tensor) -> "Q8KActs":
        x = _f32(x)
        _lib.check(_lib.lib().mq_acts_quantize(self._h, _ptr(x), x.shape[0], x.stride(0), _stream()), "mq_acts_quantize")
        self.n = x.shape[0]
        return self

    def mul_mat(self, w: Q4KWeight, out: torch.Tensor = None) -> torch.Tensor:
        y = out if out is not None else torch.empty((self.n, w.rows), dtype=torch.float32, device="cuda")
        _lib.check(_lib.lib().mq_mul_mat_q4k_acts(w._h, self._h, _ptr(y), y.stride(0), _stream()), "mq_mul_mat_q4k_acts")
        return y

    def swiglu_mul_mat(self, gate: Q4KWeight, up: Q4KWeight, silu: int = 0, out: torch.Tensor = None) -> torch.Tensor:
        h = out if out is not None else torch.empty((self.n, gate.rows), dtype=torch.float32, device="cuda")
        _lib.check(_lib.lib().mq_swiglu_mul_mat_q4k_acts(gate._h, up._h, self._h, _ptr(h), h.stride(0), silu, _stream()),
                   "mq_swiglu_mul_mat_q4k_acts")
        return h

    def free(self) -> None:
        if self._h:
            _lib.lib().mq_acts_free(self._h)
            self._h = None


def mul_mat_q8k(w: Q4KWeight, q8: torch.Tensor) -> torch.Tensor:
    """RunMoEQ4KRawBatchedProjectionImpl (core/src/backend/cpu_backend_moe_raw_batched.inl:1352): Q8_K rows in."""
    n = q8.shape[0]
    y = torch.empty((n, w.rows), dtype=torch.float32, device=q8.device)
    _lib.check(_lib.lib().mq_mul_mat_q4k_q8k(w._h, _ptr(q8), n, q8.stride(0), _ptr(y), w.rows, _stream()),
               "mq_mul_mat_q4k_q8k")
    return y


def mul_mat_host(w: Q4KWeight, x: np.ndarray) -> np.ndarray:
    """What a GGML_OP_CUSTOM callback does when ith == 0: host buffers in, host buffers out."""
    x = np.ascontiguousarray(x, np.float32)
    if x.ndim == 1:
        x = x[None]
    y = np.zeros((x.shape[0], w.rows), np.float32)
    _lib.check(_lib.lib().mq_mul_mat_q4k_host(w._h, C.c_void_p(x.ctypes.data), x.shape[0], x.shape[1],
                                              C.c_void_p(y.ctypes.data), w.rows), "mq_mul_mat_q4k_host")
    return y


def debug_block_sums(w: Q4KWeight, x: torch.Tensor):
    """Production matmul with its per-super-block integer sums written out:
    (dot_scaled [rows, n, nb] int32, min_dot [rows, n, nb] int32, y [n, rows] fp32).  Q8_0 weights: dot_scaled is
    [rows, n, cols / 32], the integer sum of every 32-weight block, and min_dot stays zero."""
    x = _f32(x)
    n, nb = x.shape[0], w.cols // (32 if w.ggml_type == GGML_TYPE_Q8_0 else QK_K)
    ds = torch.zeros((w.rows, n, nb), dtype=torch.int32, device=x.device)
    md = torch.zeros_like(ds)
    y = torch.empty((n, w.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_debug_block_sums(w._h, _ptr(x), n, x.stride(0), _ptr(ds), _ptr(md), _ptr(y), w.rows,
                                              _stream()), "mq_debug_block_sums")
    return ds, md, y


def debug_moe_groups(n_experts: int, top_k: int, ids: torch.Tensor = None, logits: torch.Tensor = None) -> np.ndarray:
    """The expert-grouped work list the grouped kernels read, as int32 [entries, 3] = (expert, token, k) in list
    order (Qwen35BuildMoEAssignments, core/src/llm/moe/native.cpp:1664-1733).  ids int32 [n, top_k]: the grouping
    launch of the expert nodes; logits fp32 [n, n_experts]: the route-and-group launch of the MoE layer."""
    src = ids if ids is not None else logits
    n = src.shape[0]
    triples = torch.full((n * top_k, 3), -7, dtype=torch.int32, device=src.device)
    count = torch.zeros(1, dtype=torch.int32, device=src.device)
    _lib.check(_lib.lib().mq_debug_moe_groups(_ptr(_f32(logits)) if logits is not None else None,
                                              _ptr(ids.contiguous()) if ids is not None else None, n_experts, n, top_k,
                                              _ptr(triples), _ptr(count), _stream()), "mq_debug_moe_groups")
    return triples.cpu().numpy()[:int(count.item())]


def debug_moe_hidden(shape) -> torch.Tensor:
    """The fp32 intermediate of the last moe_layer / ffn_swiglu call (hidden rows [n, slots, inter] / [n, inter])."""
    out = torch.empty(shape, dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().mq_debug_moe_hidden(_ptr(out), out.numel(), _stream()), "mq_debug_moe_hidden")
    return out


def swiglu_mul_mat(gate: Q4KWeight, up: Q4KWeight, x: torch.Tensor, silu: int = SILU_EXACT) -> torch.Tensor:
    """FusedSwiGLUQ4KQ8KRows_Hwy (core/src/kernels/hwy/hwy_moe_quant.cc:359-380): silu(gate x) * (up x)."""
    x = _f32(x)
    n = x.shape[0]
    h = torch.empty((n, gate.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_swiglu_mul_mat_q4k(gate._h, up._h, _ptr(x), n, x.stride(0), _ptr(h), gate.rows, silu,
                                                _stream()), "mq_swiglu_mul_mat_q4k")
    return h


def ffn_swiglu(gate: Q4KWeight, up: Q4KWeight, down: Q4KWeight, x: torch.Tensor, silu: int = SILU_FAST_FMA):
    """down( silu(gate x) * (up x) ): the dense FFN block of core/src/llm/graph/decoder.cpp:2662-2730."""
    x = _f32(x)
    y = torch.empty((x.shape[0], down.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_ffn_swiglu_q4k(gate._h, up._h, down._h, _ptr(x), x.shape[0], _ptr(y), silu, _stream()),
               "mq_ffn_swiglu_q4k")
    return y


def moe_route_topk(logits: torch.Tensor, top_k: int, mode: int = ROUTE_FUSED):
    """ComputeQwenNativeMoEStableTopK (core/src/llm/moe/native.cpp:621): -> (ids int32 [n,k], weights f32 [n,k])."""
    logits = _f32(logits)
    n, e = logits.shape
    ids = torch.empty((n, top_k), dtype=torch.int32, device=logits.device)
    w = torch.empty((n, top_k), dtype=torch.float32, device=logits.device)
    _lib.check(_lib.lib().mq_moe_route_topk(_ptr(logits), e, n, top_k, mode, _ptr(ids), _ptr(w), _stream()),
               "mq_moe_route_topk")
    return ids, w


def moe_weights_from_logits(logits: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """Qwen35NativeMoEComputeTopKWeightsFromLogits (core/src/llm/moe/native.cpp:2305-2357): weights of given ids."""
    logits = _f32(logits)
    ids = ids.contiguous()
    n, e = logits.shape
    w = torch.empty(ids.shape, dtype=torch.float32, device=logits.device)
    _lib.check(_lib.lib().mq_moe_weights_from_logits(_ptr(logits), e, n, _ptr(ids), ids.shape[1], _ptr(w), _stream()),
               "mq_moe_weights_from_logits")
    return w


def mul_mat_id(w: Q4KWeight, x: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """ggml_mul_mat_id: x fp32 [n, cols] or [n, top_k, cols]; ids int32 [n, top_k] -> y [n, top_k, rows]."""
    x = _f32(x)
    ids = ids.contiguous()
    n, top_k = ids.shape
    slots = 1 if x.dim() == 2 else x.shape[1]
    y = torch.empty((n, top_k, w.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_mul_mat_id_q4k(w._h, _ptr(x), n, slots, _ptr(ids), top_k, _ptr(y), _stream()),
               "mq_mul_mat_id_q4k")
    return y


def moe_gateup_swiglu(gate_exps: Q4KWeight, up_exps: Q4KWeight, x: torch.Tensor, ids: torch.Tensor,
                      silu: int = SILU_EXACT) -> torch.Tensor:
    """cb_qwen35_native_moe_gateup_raw_qxk_swiglu (core/src/llm/moe/native.cpp:3929): -> hidden [n, top_k, inter]."""
    x = _f32(x)
    ids = ids.contiguous()
    n, top_k = ids.shape
    h = torch.empty((n, top_k, gate_exps.rows), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_moe_gateup_swiglu_q4k(gate_exps._h, up_exps._h, _ptr(x), n, _ptr(ids), top_k, silu,
                                                   _ptr(h), _stream()), "mq_moe_gateup_swiglu_q4k")
    return h


def moe_down_weighted(down_exps: Q4KWeight, hidden: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor):
    """cb_qwen35_native_moe_down_q5k_weighted_logits (core/src/llm/moe/native.cpp:3051): -> y [n, hidden]."""
    hidden = _f32(hidden)
    ids = ids.contiguous()
    weights = _f32(weights)
    n, top_k = ids.shape
    y = torch.empty((n, down_exps.rows), dtype=torch.float32, device=hidden.device)
    _lib.check(_lib.lib().mq_moe_down_weighted_q4k(down_exps._h, _ptr(hidden), n, _ptr(ids), _ptr(weights), top_k,
                                                   _ptr(y), _stream()), "mq_moe_down_weighted_q4k")
    return y


def moe_layer(gate_exps: Q4KWeight, up_exps: Q4KWeight, down_exps: Q4KWeight, x: torch.Tensor, logits: torch.Tensor,
              top_k: int, shared=None, silu: int = SILU_EXACT, route_mode: int = ROUTE_FUSED):
    """TryBuildQwen35NativeMoEGraph's four nodes plus the shared expert (core/src/llm/moe/native.cpp:4691).
    shared = (gate, up, down, gate_inp tensor or None).  Returns (y, ids, weights)."""
    x = _f32(x)
    logits = _f32(logits)
    n = x.shape[0]
    d = _lib.MoELayerDesc(gate_exps._h, up_exps._h, down_exps._h, None, None, None, None, top_k, silu, route_mode)
    keep = None
    if shared is not None:
        d.shared_gate, d.shared_up, d.shared_down = shared[0]._h, shared[1]._h, shared[2]._h
        if shared[3] is not None:
            keep = _f32(shared[3])
            d.sh_gate_inp_dev = keep.data_ptr()
    y = torch.empty((n, gate_exps.cols), dtype=torch.float32, device=x.device)
    ids = torch.empty((n, top_k), dtype=torch.int32, device=x.device)
    wts = torch.empty((n, top_k), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().mq_moe_layer_q4k(C.byref(d), _ptr(x), _ptr(logits), n, _ptr(y), _ptr(ids), _ptr(wts),
                                           _stream()), "mq_moe_layer_q4k")
    return y, ids, wts


KIND_DENSE, KIND_DENSE_SWIGLU, KIND_GROUPED, KIND_GROUPED_SWIGLU = 0, 1, 2, 3


def stream_synchronize() -> None:
    """Waits for the current stream and raises if a persistent launch on it gave up at a device-wide barrier."""
    _lib.check(_lib.lib().mq_stream_synchronize(_stream()), "mq_stream_synchronize")


def census_enable(on: bool) -> None:
    """Record a HIP event pair around every matmul-kernel launch (the GPU analogue of the reference's
    matmul dispatch census, core/src/llm/matmul/gemv_exec.cpp:203-276)."""
    _lib.check(_lib.lib().mq_census_enable(1 if on else 0), "mq_census_enable")


def census_reset() -> None:
    _lib.check(_lib.lib().mq_census_reset(), "mq_census_reset")


def census_read(kind: int) -> dict:
    avg, lo, hi, cnt = C.c_double(), C.c_double(), C.c_double(), C.c_int64()
    _lib.check(_lib.lib().mq_census_read(kind, C.byref(avg), C.byref(lo), C.byref(hi), C.byref(cnt)),
               "mq_census_read")
    return {"avg_us": avg.value, "min_us": lo.value, "max_us": hi.value, "count": cnt.value}
