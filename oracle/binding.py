"""ctypes binding to the C oracle (liboracle.so / liboracle_simd.so).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

ORDER_HWY, ORDER_AVX2, ORDER_SCALAR, ORDER_DOTPROD = 0, 1, 2, 3
ORDERS = {"hwy": 0, "avx2": 1, "scalar": 2, "dotprod": 3}
SILU_EXACT, SILU_FAST, SILU_FAST_FMA = 0, 1, 2

Q4K = 144
Q5K = 176
Q6K = 210
Q8K = 292


def build() -> None:
    subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)


def _load(name: str) -> C.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return C.CDLL(path)


_lib = None
_simd = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        L = _load("liboracle.so")
        L.orc_fp16_to_fp32.restype = C.c_float
        L.orc_fp16_to_fp32.argtypes = [C.c_uint16]
        L.orc_fp32_to_fp16.restype = C.c_uint16
        L.orc_fp32_to_fp16.argtypes = [C.c_float]
        L.orc_nearest_int.restype = C.c_int
        L.orc_nearest_int.argtypes = [C.c_float]
        L.orc_fast_exp.restype = C.c_float
        L.orc_fast_exp.argtypes = [C.c_float]
        L.orc_fast_exp_fma.restype = C.c_float
        L.orc_fast_exp_fma.argtypes = [C.c_float]
        L.orc_silu_mul.restype = C.c_float
        L.orc_silu_mul.argtypes = [C.c_float, C.c_float, C.c_int]
        L.orc_dot_q4k_q8k.restype = C.c_float
        L.orc_dot_q4k_q8k.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.orc_dot_dequant_f64.restype = C.c_double
        L.orc_dot_dequant_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.orc_dot_magnitude_f64.restype = C.c_double
        L.orc_dot_magnitude_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.orc_build_assignments.restype = C.c_int64
        L.orc_q5k_block_bytes.restype = C.c_size_t
        L.orc_q6k_block_bytes.restype = C.c_size_t
        L.orc_dot_dequant_q6k_f64.restype = C.c_double
        L.orc_dot_dequant_q6k_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.orc_dot_q5k_q8k.restype = C.c_float
        L.orc_dot_q5k_q8k.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.orc_dot_dequant_q5k_f64.restype = C.c_double
        L.orc_dot_dequant_q5k_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.orc_q80_block_bytes.restype = C.c_size_t
        L.orc_dot_typed_q8k.restype = C.c_float
        L.orc_dot_typed_q8k.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.orc_dot_dequant_q80_f64.restype = C.c_double
        L.orc_dot_dequant_q80_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        _lib = L
    return _lib


def host_has_vnni() -> bool:
    """AVX-512 VNNI with 256-bit vectors on this host (what liboracle_simd_vnni.so needs)."""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("flags"):
                flags = set(line.split(":", 1)[1].split())
                return {"avx512_vnni", "avx512vl", "avx512f", "avx512bw"} <= flags
    except OSError:
        pass
    return False


_simd_vnni = None


def simd(isa: str = "avx2") -> C.CDLL:
    """The threaded SIMD build: "avx2", "vnni" (AVX-512 VNNI; only load it where host_has_vnni()), or "best"."""
    global _simd, _simd_vnni
    if isa == "best":
        isa = "vnni" if host_has_vnni() else "avx2"
    if isa == "vnni":
        if _simd_vnni is None:
            _simd_vnni = _load("liboracle_simd_vnni.so")
        return _simd_vnni
    if _simd is None:
        _simd = _load("liboracle_simd.so")
    return _simd


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------- scalars
def fp16_to_fp32(h: int) -> float:
    return lib().orc_fp16_to_fp32(h)


def fp32_to_fp16(f: float) -> int:
    return lib().orc_fp32_to_fp16(f)


def nearest_int(v: float) -> int:
    return lib().orc_nearest_int(v)


def scales_kmask(packed12: np.ndarray):
    p = _c(packed12, np.uint8)
    s = np.zeros(8, np.uint8)
    m = np.zeros(8, np.uint8)
    lib().orc_q4k_scales_kmask(_p(p), _p(s), _p(m))
    return s, m


def scales_indexed(packed12: np.ndarray):
    p = _c(packed12, np.uint8)
    s = np.zeros(8, np.uint8)
    m = np.zeros(8, np.uint8)
    lib().orc_q4k_scales_indexed(_p(p), _p(s), _p(m))
    return s, m


# ---------------------------------------------------------------- quantizer
def quantize_rows_q8k(x: np.ndarray) -> np.ndarray:
    """fp32 [n, k] -> uint8 [n, k/256*292] (block_q8_K bytes)."""
    x = _c(x, np.float32)
    if x.ndim == 1:
        x = x[None, :]
    n, k = x.shape
    out = np.zeros((n, k // 256 * Q8K), np.uint8)
    rc = lib().orc_quantize_rows_q8k(_p(x), C.c_int64(n), C.c_int64(k), _p(out), C.c_int64(k))
    if rc:
        raise ValueError(f"orc_quantize_rows_q8k rc={rc}")
    return out


def split_q8k(q8: np.ndarray):
    """uint8 [n, nb*292] -> (d [n,nb] f32, qs [n,nb,256] i8, bsums [n,nb,16] i16)."""
    n = q8.shape[0]
    b = q8.reshape(n, -1, Q8K)
    d = b[:, :, 0:4].copy().view(np.float32).reshape(n, -1)
    qs = b[:, :, 4:260].copy().view(np.int8)
    bs = b[:, :, 260:292].copy().view(np.int16)
    return d, qs, bs


# ---------------------------------------------------------------- sums / dots
def matrix_block_sums(w: np.ndarray, cols: int, q8: np.ndarray):
    """w uint8 [rows, nb*144], q8 uint8 [n, nb*292] -> two int32 [rows, n, nb]."""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n, nb = w.shape[0], q8.shape[0], cols // 256
    ds = np.zeros((rows, n, nb), np.int32)
    md = np.zeros((rows, n, nb), np.int32)
    rc = lib().orc_matrix_block_sums(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                     C.c_int64(n), C.c_size_t(q8.shape[1]), _p(ds), _p(md))
    if rc:
        raise ValueError(f"orc_matrix_block_sums rc={rc}")
    return ds, md


def mul_mat_q4k_q8k(w: np.ndarray, cols: int, q8: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    """-> fp32 [n, rows]"""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n = w.shape[0], q8.shape[0]
    out = np.zeros((n, rows), np.float32)
    rc = lib().orc_mul_mat_q4k_q8k(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                   C.c_int64(n), C.c_size_t(q8.shape[1]), _p(out), C.c_int64(rows), C.c_int(order))
    if rc:
        raise ValueError(f"orc_mul_mat_q4k_q8k rc={rc}")
    return out


def mul_mat_q4k_f32(w: np.ndarray, cols: int, x: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    return mul_mat_q4k_q8k(w, cols, quantize_rows_q8k(x), order)


def dot_dequant_f64(w: np.ndarray, cols: int, q8: np.ndarray) -> np.ndarray:
    """double-precision dequantize-then-dot, [n, rows]."""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    L = lib()
    out = np.zeros((q8.shape[0], w.shape[0]), np.float64)
    for m in range(q8.shape[0]):
        for r in range(w.shape[0]):
            out[m, r] = L.orc_dot_dequant_f64(C.c_void_p(w[r].ctypes.data), C.c_void_p(q8[m].ctypes.data),
                                              C.c_int64(cols))
    return out


def dot_magnitude_f64(w: np.ndarray, cols: int, q8: np.ndarray) -> np.ndarray:
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    L = lib()
    out = np.zeros((q8.shape[0], w.shape[0]), np.float64)
    for m in range(q8.shape[0]):
        for r in range(w.shape[0]):
            out[m, r] = L.orc_dot_magnitude_f64(C.c_void_p(w[r].ctypes.data), C.c_void_p(q8[m].ctypes.data),
                                                C.c_int64(cols))
    return out


# ---------------------------------------------------------------- Q5_K weights
def q5k_matrix_block_sums(w: np.ndarray, cols: int, q8: np.ndarray):
    """w uint8 [rows, nb*176], q8 uint8 [n, nb*292] -> two int32 [rows, n, nb]."""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n, nb = w.shape[0], q8.shape[0], cols // 256
    ds = np.zeros((rows, n, nb), np.int32)
    md = np.zeros((rows, n, nb), np.int32)
    rc = lib().orc_q5k_matrix_block_sums(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                         C.c_int64(n), C.c_size_t(q8.shape[1]), _p(ds), _p(md))
    if rc:
        raise ValueError(f"orc_q5k_matrix_block_sums rc={rc}")
    return ds, md


def mul_mat_q5k_q8k(w: np.ndarray, cols: int, q8: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    """-> fp32 [n, rows]; order ORDER_HWY is the reference's own Q5_K kernel, anything else the per-block form."""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n = w.shape[0], q8.shape[0]
    out = np.zeros((n, rows), np.float32)
    rc = lib().orc_mul_mat_q5k_q8k(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                   C.c_int64(n), C.c_size_t(q8.shape[1]), _p(out), C.c_int64(rows), C.c_int(order))
    if rc:
        raise ValueError(f"orc_mul_mat_q5k_q8k rc={rc}")
    return out


def mul_mat_q5k_f32(w: np.ndarray, cols: int, x: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    return mul_mat_q5k_q8k(w, cols, quantize_rows_q8k(x), order)


def q5k_dot_dequant_f64(w: np.ndarray, cols: int, q8: np.ndarray, magnitude: bool = False) -> np.ndarray:
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    L = lib()
    out = np.zeros((q8.shape[0], w.shape[0]), np.float64)
    for m in range(q8.shape[0]):
        for r in range(w.shape[0]):
            out[m, r] = L.orc_dot_dequant_q5k_f64(C.c_void_p(w[r].ctypes.data), C.c_void_p(q8[m].ctypes.data),
                                                  C.c_int64(cols), C.c_int(int(magnitude)))
    return out


def q5k_from_q4k(w4: np.ndarray, qh: np.ndarray | None = None) -> np.ndarray:
    """[rows, nb*144] Q4_K rows -> [rows, nb*176] Q5_K rows with the same d, dmin, scales and nibbles and the
    given high-bit bytes ([rows, nb, 32], default zero)."""
    w4 = _c(w4, np.uint8)
    rows = w4.shape[0]
    b4 = w4.reshape(rows, -1, Q4K)
    nb = b4.shape[1]
    b5 = np.zeros((rows, nb, Q5K), np.uint8)
    b5[:, :, 0:16] = b4[:, :, 0:16]
    if qh is not None:
        b5[:, :, 16:48] = qh
    b5[:, :, 48:176] = b4[:, :, 16:144]
    return b5.reshape(rows, nb * Q5K)


# ---------------------------------------------------------------- Q6_K weights
def q6k_matrix_block_sums(w: np.ndarray, cols: int, q8: np.ndarray) -> np.ndarray:
    """w uint8 [rows, nb*210], q8 uint8 [n, nb*292] -> int32 [rows, n, nb]: sum_g scale_g * sum (q - 32) * y."""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n, nb = w.shape[0], q8.shape[0], cols // 256
    out = np.zeros((rows, n, nb), np.int32)
    rc = lib().orc_q6k_matrix_block_sums(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                         C.c_int64(n), C.c_size_t(q8.shape[1]), _p(out))
    if rc:
        raise ValueError(f"orc_q6k_matrix_block_sums rc={rc}")
    return out


def mul_mat_q6k_q8k(w: np.ndarray, cols: int, q8: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    """-> fp32 [n, rows]; ORDER_HWY is the reference's eight-lane kernel, anything else the per-block form."""
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n = w.shape[0], q8.shape[0]
    out = np.zeros((n, rows), np.float32)
    rc = lib().orc_mul_mat_q6k_q8k(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                   C.c_int64(n), C.c_size_t(q8.shape[1]), _p(out), C.c_int64(rows), C.c_int(order))
    if rc:
        raise ValueError(f"orc_mul_mat_q6k_q8k rc={rc}")
    return out


def mul_mat_q6k_f32(w: np.ndarray, cols: int, x: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    return mul_mat_q6k_q8k(w, cols, quantize_rows_q8k(x), order)


def q6k_dot_dequant_f64(w: np.ndarray, cols: int, q8: np.ndarray, magnitude: bool = False) -> np.ndarray:
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    L = lib()
    out = np.zeros((q8.shape[0], w.shape[0]), np.float64)
    for m in range(q8.shape[0]):
        for r in range(w.shape[0]):
            out[m, r] = L.orc_dot_dequant_q6k_f64(C.c_void_p(w[r].ctypes.data), C.c_void_p(q8[m].ctypes.data),
                                                  C.c_int64(cols), C.c_int(int(magnitude)))
    return out


# ---------------------------------------------------------------- FFN / router / MoE
# ---------------------------------------------------------------- Q8_0 weights (activations Q8_0 as well)
Q80 = 34
Q80_X86, Q80_SCALAR = 0, 1  # the two published forms of ggml's Q8_0 activation quantizer (parity unpinned)


def quantize_rows_q80(x: np.ndarray, variant: int = Q80_X86) -> np.ndarray:
    """fp32 [n, cols] -> uint8 [n, cols/32*34] Q8_0 rows."""
    x = _c(x, np.float32)
    n, cols = x.shape
    out = np.zeros((n, cols // 32 * Q80), np.uint8)
    rc = lib().orc_quantize_rows_q80(_p(x), C.c_int64(n), C.c_int64(cols), _p(out), C.c_int64(cols), C.c_int(variant))
    if rc:
        raise ValueError(f"orc_quantize_rows_q80 rc={rc}")
    return out


def q80_matrix_block_sums(w: np.ndarray, cols: int, q: np.ndarray) -> np.ndarray:
    """w uint8 [rows, cols/32*34], q uint8 [n, cols/32*34] -> int32 [rows, n, cols/32]."""
    w = _c(w, np.uint8)
    q = _c(q, np.uint8)
    rows, n = w.shape[0], q.shape[0]
    out = np.zeros((rows, n, cols // 32), np.int32)
    rc = lib().orc_q80_matrix_block_sums(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q),
                                         C.c_int64(n), C.c_size_t(q.shape[1]), _p(out))
    if rc:
        raise ValueError(f"orc_q80_matrix_block_sums rc={rc}")
    return out


def mul_mat_q80_q80(w: np.ndarray, cols: int, q: np.ndarray, order: int = ORDER_DOTPROD) -> np.ndarray:
    """-> fp32 [n, rows]; ORDER_HWY is the reference's eight-lane kernel, anything else the per-block form."""
    w = _c(w, np.uint8)
    q = _c(q, np.uint8)
    rows, n = w.shape[0], q.shape[0]
    out = np.zeros((n, rows), np.float32)
    rc = lib().orc_mul_mat_q80_q80(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q),
                                   C.c_int64(n), C.c_size_t(q.shape[1]), _p(out), C.c_int64(rows), C.c_int(order))
    if rc:
        raise ValueError(f"orc_mul_mat_q80_q80 rc={rc}")
    return out


def q80_dot_dequant_f64(w: np.ndarray, cols: int, q: np.ndarray, magnitude: bool = False) -> np.ndarray:
    w = _c(w, np.uint8)
    q = _c(q, np.uint8)
    L = lib()
    out = np.zeros((q.shape[0], w.shape[0]), np.float64)
    for m in range(q.shape[0]):
        for r in range(w.shape[0]):
            out[m, r] = L.orc_dot_dequant_q80_f64(C.c_void_p(w[r].ctypes.data), C.c_void_p(q[m].ctypes.data),
                                                  C.c_int64(cols), C.c_int(int(magnitude)))
    return out


def ffn_swiglu(gate, up, down, hidden: int, inter: int, x, order=ORDER_DOTPROD, silu=SILU_FAST_FMA,
               want_inter=False):
    gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
    x = _c(x, np.float32)
    n = x.shape[0]
    y = np.zeros((n, hidden), np.float32)
    mid = np.zeros((n, inter), np.float32)
    rc = lib().orc_ffn_swiglu_q4k(_p(gate), _p(up), _p(down), C.c_int64(hidden), C.c_int64(inter), _p(x),
                                  C.c_int64(n), _p(y), C.c_int(order), C.c_int(silu), _p(mid))
    if rc:
        raise ValueError(f"orc_ffn_swiglu_q4k rc={rc}")
    return (y, mid) if want_inter else y


def ffn_swiglu_typed(gu_type, down_type, gate, up, down, hidden: int, inter: int, x, order=ORDER_DOTPROD,
                     silu=SILU_FAST_FMA, want_inter=False):
    gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
    x = _c(x, np.float32)
    n = x.shape[0]
    y = np.zeros((n, hidden), np.float32)
    mid = np.zeros((n, inter), np.float32)
    rc = lib().orc_ffn_swiglu_typed(C.c_int(gu_type), C.c_int(down_type), _p(gate), _p(up), _p(down), C.c_int64(hidden),
                                    C.c_int64(inter), _p(x), C.c_int64(n), _p(y), C.c_int(order), C.c_int(silu), _p(mid))
    if rc:
        raise ValueError(f"orc_ffn_swiglu_typed rc={rc}")
    return (y, mid) if want_inter else y


def swiglu_mul_mat(gate, up, hidden: int, inter: int, x, order=ORDER_DOTPROD, silu=SILU_EXACT):
    gate, up = _c(gate, np.uint8), _c(up, np.uint8)
    x = _c(x, np.float32)
    out = np.zeros((x.shape[0], inter), np.float32)
    rc = lib().orc_swiglu_mul_mat_q4k_f32(_p(gate), _p(up), C.c_int64(inter), C.c_int64(hidden), _p(x),
                                          C.c_int64(x.shape[0]), _p(out), C.c_int(order), C.c_int(silu))
    if rc:
        raise ValueError(f"orc_swiglu_mul_mat_q4k_f32 rc={rc}")
    return out


def route_topk(logits, top_k: int, weights_mode: int = 0):
    logits = _c(logits, np.float32)
    n, e = logits.shape
    ids = np.zeros((n, top_k), np.int32)
    w = np.zeros((n, top_k), np.float32)
    rc = lib().orc_route_topk(_p(logits), C.c_int64(e), C.c_int64(n), C.c_int(top_k), C.c_int(weights_mode), _p(ids),
                              _p(w))
    if rc:
        raise ValueError(f"orc_route_topk rc={rc}")
    return ids, w


def route_weights_from_ids(logits, ids) -> np.ndarray:
    logits = _c(logits, np.float32)
    ids = _c(ids, np.int32)
    n, e = logits.shape
    w = np.zeros(ids.shape, np.float32)
    rc = lib().orc_route_weights_from_ids(_p(logits), C.c_int64(e), C.c_int64(n), _p(ids), C.c_int(ids.shape[1]), _p(w))
    if rc:
        raise ValueError(f"orc_route_weights_from_ids rc={rc}")
    return w


def build_assignments(ids, n_experts: int) -> np.ndarray:
    ids = _c(ids, np.int32)
    n, k = ids.shape
    out = np.zeros((n * k, 3), np.int32)
    cnt = lib().orc_build_assignments(_p(ids), C.c_int64(n), C.c_int(k), C.c_int64(n_experts), _p(out))
    return out[:cnt]


class _MoEWeights(C.Structure):
    _fields_ = [("hidden", C.c_int64), ("inter", C.c_int64), ("n_experts", C.c_int64), ("top_k", C.c_int),
                ("gate_exps", C.c_void_p), ("up_exps", C.c_void_p), ("down_exps", C.c_void_p),
                ("sh_gate", C.c_void_p), ("sh_up", C.c_void_p), ("sh_down", C.c_void_p),
                ("sh_gate_inp", C.c_void_p),
                ("gu_type", C.c_int), ("down_type", C.c_int), ("sh_gu_type", C.c_int), ("sh_down_type", C.c_int)]


def _moe_w(gate_exps, up_exps, down_exps, hidden, inter, top_k, keep, gu_type=12, down_type=12):
    n_exp = (gate_exps if gate_exps is not None else down_exps).shape[0]
    W = _MoEWeights(hidden, inter, n_exp, top_k, None, None, None, None, None, None, None, gu_type, down_type, 12, 12)
    for name, arr in (("gate_exps", gate_exps), ("up_exps", up_exps), ("down_exps", down_exps)):
        if arr is not None:
            a = _c(arr, np.uint8)
            keep.append(a)
            setattr(W, name, a.ctypes.data)
    return W


def moe_gateup_swiglu(gate_exps, up_exps, hidden, inter, x, ids, order=ORDER_DOTPROD, silu=SILU_EXACT, gu_type=12):
    """gu_type: ggml_type of both stacks (12 Q4_K, 13 Q5_K, 14 Q6_K); rows of the matching block size."""
    keep = []
    ids = _c(ids, np.int32)
    x = _c(x, np.float32)
    W = _moe_w(gate_exps, up_exps, None, hidden, inter, ids.shape[1], keep, gu_type=gu_type)
    out = np.zeros((x.shape[0], ids.shape[1], inter), np.float32)
    rc = lib().orc_moe_gateup_swiglu(C.byref(W), _p(x), _p(ids), C.c_int64(x.shape[0]), C.c_int(order), C.c_int(silu),
                                     _p(out))
    if rc:
        raise ValueError(f"orc_moe_gateup_swiglu rc={rc}")
    return out


def moe_down_weighted(down_exps, hidden, inter, hid, ids, weights, order=ORDER_DOTPROD, accumulate_mode=0, down_type=12):
    keep = []
    ids = _c(ids, np.int32)
    hid = _c(hid, np.float32)
    weights = _c(weights, np.float32)
    W = _moe_w(None, None, down_exps, hidden, inter, ids.shape[1], keep, down_type=down_type)
    y = np.zeros((ids.shape[0], hidden), np.float32)
    rc = lib().orc_moe_down_weighted(C.byref(W), _p(hid), _p(ids), _p(weights), C.c_int64(ids.shape[0]),
                                     C.c_int(order), C.c_int(accumulate_mode), _p(y))
    if rc:
        raise ValueError(f"orc_moe_down_weighted rc={rc}")
    return y


def moe_layer(gate_exps, up_exps, down_exps, hidden, inter, top_k, x, logits, shared=None, order=ORDER_DOTPROD,
              silu=SILU_EXACT, weights_mode=0, accumulate_mode=0, types=(12, 12, 12, 12)):
    """gate_exps/up_exps: uint8 [E, inter, hidden/256*144]; down_exps: uint8 [E, hidden, inter/256*144].
    shared: None or (gate, up, down, gate_inp[hidden] or None).
    types: ggml_type of (gate/up stacks, down stack, shared gate/up, shared down); rows of the matching block size.
    Returns dict(y, ids, weights, hidden)."""
    ge, ue, de = _c(gate_exps, np.uint8), _c(up_exps, np.uint8), _c(down_exps, np.uint8)
    x = _c(x, np.float32)
    logits = _c(logits, np.float32)
    n = x.shape[0]
    keep = [ge, ue, de, x, logits]
    W = _MoEWeights(hidden, inter, ge.shape[0], top_k, ge.ctypes.data, ue.ctypes.data, de.ctypes.data, None, None,
                    None, None, *types)
    if shared is not None:
        sg, su, sd = (_c(a, np.uint8) for a in shared[:3])
        keep += [sg, su, sd]
        W.sh_gate, W.sh_up, W.sh_down = sg.ctypes.data, su.ctypes.data, sd.ctypes.data
        if shared[3] is not None:
            gi = _c(shared[3], np.float32)
            keep.append(gi)
            W.sh_gate_inp = gi.ctypes.data
    y = np.zeros((n, hidden), np.float32)
    ids = np.zeros((n, top_k), np.int32)
    wts = np.zeros((n, top_k), np.float32)
    hid = np.zeros((n, top_k, inter), np.float32)
    rc = lib().orc_moe_layer(C.byref(W), _p(x), _p(logits), C.c_int64(n), _p(y), C.c_int(order), C.c_int(silu),
                             C.c_int(weights_mode), C.c_int(accumulate_mode), _p(ids), _p(wts), _p(hid))
    if rc:
        raise ValueError(f"orc_moe_layer rc={rc}")
    return {"y": y, "ids": ids, "weights": wts, "hidden": hid}


# ---------------------------------------------------------------- timed SIMD baseline
def simd_mul_mat_q4k_q8k(w, cols: int, q8, threads: int, isa: str = "avx2") -> np.ndarray:
    w = _c(w, np.uint8)
    q8 = _c(q8, np.uint8)
    rows, n = w.shape[0], q8.shape[0]
    out = np.zeros((n, rows), np.float32)
    rc = simd(isa).orc_simd_mul_mat_q4k_q8k(_p(w), C.c_int64(rows), C.c_int64(cols), C.c_size_t(w.shape[1]), _p(q8),
                                         C.c_int64(n), C.c_size_t(q8.shape[1]), _p(out), C.c_int64(rows),
                                         C.c_int(threads))
    if rc:
        raise ValueError(f"orc_simd_mul_mat_q4k_q8k rc={rc}")
    return out


def simd_ffn_swiglu(gate, up, down, hidden: int, inter: int, x, threads: int, silu=SILU_FAST_FMA, isa: str = "avx2") -> np.ndarray:
    gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
    x = _c(x, np.float32)
    y = np.zeros((x.shape[0], hidden), np.float32)
    rc = simd(isa).orc_simd_ffn_swiglu_q4k(_p(gate), _p(up), _p(down), C.c_int64(hidden), C.c_int64(inter), _p(x),
                                        C.c_int64(x.shape[0]), _p(y), C.c_int(threads), C.c_int(silu))
    if rc:
        raise ValueError(f"orc_simd_ffn_swiglu_q4k rc={rc}")
    return y
