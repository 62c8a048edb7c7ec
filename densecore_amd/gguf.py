"""ctypes view of the GGUF reader (include/mi355_q4k_gguf.h) and a minimal GGUF writer for tests and tools.

The reader is the C++ one in libmi355q4k_ggml.so; the writer below produces files in the same published
layout (GGUF v3, little endian) from numpy arrays and is only meant for fixtures and examples.
"""
import ctypes as C
import struct

import numpy as np

from . import _lib, ggml_adapter, ops

EXPORTS = [
    "mq_gguf_open", "mq_gguf_last_error", "mq_gguf_close", "mq_gguf_tensor_count", "mq_gguf_tensor_at",
    "mq_gguf_find_tensor", "mq_gguf_get_int", "mq_gguf_get_string", "mq_gguf_load_q4k", "mq_gguf_load_weight",
    "mq_gguf_load_moe_layer", "mq_gguf_free_moe_layer",
]

GGML_F32, GGML_F16, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_I32 = 0, 1, 12, 13, 14, 26
GGML_Q8_0 = 8


class TensorInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ggml_type", C.c_int32), ("n_dims", C.c_int32), ("ne", C.c_int64 * 4),
                ("offset", C.c_uint64), ("nbytes", C.c_uint64), ("data", C.c_void_p)]


class MoELayerStruct(C.Structure):
    """mq_gguf_moe_layer (include/mi355_q4k_gguf.h)."""
    _fields_ = [("desc", _lib.MoELayerDesc), ("owned", C.c_void_p * 6), ("router_dev", C.c_void_p), ("sh_gate_inp_dev", C.c_void_p),
                ("n_experts", C.c_int64), ("hidden", C.c_int64), ("inter", C.c_int64)]


class MoELayer:
    """A layer loaded by mq_gguf_load_moe_layer: .desc for mq_moe_layer_q4k, .weights as ops.Q4KWeight views (not owning)."""

    def __init__(self, raw: MoELayerStruct, types):
        self.raw = raw
        self.n_experts, self.hidden, self.inter = raw.n_experts, raw.hidden, raw.inter
        self.top_k = raw.desc.top_k
        shapes = [(self.inter, self.hidden, self.n_experts)] * 2 + [(self.hidden, self.inter, self.n_experts)] + \
                 [(self.inter, self.hidden, 1)] * 2 + [(self.hidden, self.inter, 1)]
        self.weights = [ops.Q4KWeight(raw.owned[i], r, c, e, types[i]) if raw.owned[i] else None
                        for i, (r, c, e) in enumerate(shapes)]
        self._freed = False

    def run(self, x, logits, silu: int = ops.SILU_EXACT, route_mode: int = ops.ROUTE_FUSED, top_k: int = 0):
        """mq_moe_layer_q4k on the loaded layer: returns (y, ids, weights)."""
        import torch
        self.raw.desc.top_k = top_k or self.top_k
        self.raw.desc.silu_mode, self.raw.desc.route_mode = silu, route_mode
        n, K = x.shape[0], self.raw.desc.top_k
        y = torch.empty((n, self.hidden), dtype=torch.float32, device="cuda")
        ids = torch.empty((n, K), dtype=torch.int32, device="cuda")
        wts = torch.empty((n, K), dtype=torch.float32, device="cuda")
        p = lambda t: C.c_void_p(t.data_ptr())
        _lib.check(_lib.lib().mq_moe_layer_q4k(C.byref(self.raw.desc), p(x), p(logits), n, p(y), p(ids), p(wts),
                                               C.c_void_p(torch.cuda.current_stream().cuda_stream)), "mq_moe_layer_q4k")
        return y, ids, wts

    def free(self):
        """Frees the layer's device memory; its weight views stop being usable."""
        if self._freed:
            return
        self._freed = True
        for w in self.weights:           # views: the layer owns the handles, a view must not free its own
            if w is not None:
                w._h = C.c_void_p()
        self.weights = []
        lib().mq_gguf_free_moe_layer(C.byref(self.raw))

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


_handle = None


def lib(need_gpu: bool = False):
    """The host library; the GPU library is only initialised when a tensor is to be uploaded."""
    global _handle
    if _handle is None:
        _lib.load()
        L = C.CDLL(ggml_adapter.LIB_PATH, mode=C.RTLD_GLOBAL)
        L.mq_gguf_open.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
        L.mq_gguf_last_error.restype = C.c_char_p
        L.mq_gguf_close.argtypes = [C.c_void_p]
        L.mq_gguf_tensor_count.argtypes = [C.c_void_p]
        L.mq_gguf_tensor_count.restype = C.c_int64
        L.mq_gguf_tensor_at.argtypes = [C.c_void_p, C.c_int64, C.POINTER(TensorInfo)]
        L.mq_gguf_find_tensor.argtypes = [C.c_void_p, C.c_char_p]
        L.mq_gguf_find_tensor.restype = C.c_int64
        L.mq_gguf_get_int.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64)]
        L.mq_gguf_get_string.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(C.c_size_t)]
        L.mq_gguf_load_q4k.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.mq_gguf_load_weight.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.mq_gguf_load_moe_layer.argtypes = [C.c_void_p, C.c_int, C.POINTER(MoELayerStruct)]
        L.mq_gguf_free_moe_layer.argtypes = [C.POINTER(MoELayerStruct)]
        _handle = L
    if need_gpu:
        _lib.lib()
    return _handle


class GgufFile:
    def __init__(self, path: str):
        h = C.c_void_p()
        if lib().mq_gguf_open(path.encode(), C.byref(h)) != 0:
            raise ValueError(f"{path}: {lib().mq_gguf_last_error().decode()}")
        self._h = h

    def close(self):
        if self._h:
            lib().mq_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def tensors(self):
        out = []
        for i in range(lib().mq_gguf_tensor_count(self._h)):
            t = TensorInfo()
            lib().mq_gguf_tensor_at(self._h, i, C.byref(t))
            out.append({"name": t.name.decode(), "type": t.ggml_type, "ne": list(t.ne)[:t.n_dims], "offset": t.offset,
                        "nbytes": t.nbytes, "data": t.data})
        return out

    def find(self, name: str) -> int:
        return lib().mq_gguf_find_tensor(self._h, name.encode())

    def get_int(self, key: str) -> int:
        v = C.c_int64()
        if lib().mq_gguf_get_int(self._h, key.encode(), C.byref(v)) != 0:
            raise KeyError(lib().mq_gguf_last_error().decode())
        return v.value

    def get_string(self, key: str) -> str:
        p, n = C.c_char_p(), C.c_size_t()
        if lib().mq_gguf_get_string(self._h, key.encode(), C.byref(p), C.byref(n)) != 0:
            raise KeyError(lib().mq_gguf_last_error().decode())
        return C.string_at(p, n.value).decode()

    def load_q4k(self, name: str) -> "ops.Q4KWeight":
        """Upload a GGML_TYPE_Q4_K tensor ([K, N] or [K, N, E]) to the GPU."""
        return self._load(name, "mq_gguf_load_q4k")

    def load_weight(self, name: str) -> "ops.Q4KWeight":
        """Upload a GGML_TYPE_Q4_K, Q5_K or Q6_K tensor ([K, N] or [K, N, E]) or a dense Q8_0 matrix to the GPU."""
        return self._load(name, "mq_gguf_load_weight")

    def load_moe_layer(self, layer: int) -> MoELayer:
        """Bind blk.<layer>'s expert stacks, shared expert, router and scalar gate to a MoE layer descriptor."""
        lib(need_gpu=True)
        raw = MoELayerStruct()
        rc = lib().mq_gguf_load_moe_layer(self._h, layer, C.byref(raw))
        if rc != 0:
            _lib.check(rc, f"mq_gguf_load_moe_layer({layer}): {lib().mq_gguf_last_error().decode()}")
        by_name = {t["name"]: t["type"] for t in self.tensors()}
        pick = lambda *sfx: next((by_name[f"blk.{layer}.{s}"] for s in sfx if f"blk.{layer}.{s}" in by_name), 12)
        types = [pick("ffn_gate_exps.weight", "ffn_gate_exps", "experts.gate_proj.weight"),
                 pick("ffn_up_exps.weight", "ffn_up_exps", "experts.up_proj.weight"),
                 pick("ffn_down_exps.weight", "ffn_down_exps", "experts.down_proj.weight"),
                 pick("ffn_gate.weight", "ffn_gate_shexp.weight", "shared_expert.gate_proj.weight", "mlp.gate_proj.weight", "gate_proj.weight"),
                 pick("ffn_up.weight", "ffn_up_shexp.weight", "shared_expert.up_proj.weight", "mlp.up_proj.weight", "up_proj.weight"),
                 pick("ffn_down.weight", "ffn_down_shexp.weight", "shared_expert.down_proj.weight", "mlp.down_proj.weight", "down_proj.weight")]
        return MoELayer(raw, types)

    def _load(self, name: str, entry: str) -> "ops.Q4KWeight":
        lib(need_gpu=True)
        idx = self.find(name)
        if idx < 0:
            raise KeyError(name)
        t = self.tensors()[idx]
        h = C.c_void_p()
        rc = getattr(lib(), entry)(self._h, name.encode(), C.byref(h))
        if rc != 0:
            _lib.check(rc, f"{entry}({name}): {lib().mq_gguf_last_error().decode()}")
        ne = t["ne"] + [1] * (3 - len(t["ne"]))
        return ops.Q4KWeight(h.value, ne[1], ne[0], ne[2], t["type"])


# ------------------------------------------------------------------------------------------ writer
_SCALAR = {"u8": (0, "<B"), "i8": (1, "<b"), "u16": (2, "<H"), "i16": (3, "<h"), "u32": (4, "<I"), "i32": (5, "<i"),
           "f32": (6, "<f"), "bool": (7, "<B"), "u64": (10, "<Q"), "i64": (11, "<q"), "f64": (12, "<d")}


def _s(b: bytes) -> bytes:
    return struct.pack("<Q", len(b)) + b


def write_gguf(path: str, metadata: dict, tensors: list, alignment: int = 32, version: int = 3) -> None:
    """metadata: key -> (kind, value) with kind in _SCALAR, "str", or ("arr", kind); tensors: list of
    (name, ggml_type, ne (innermost first), numpy array holding the raw bytes)."""
    out = bytearray()
    md = dict(metadata)
    if alignment != 32:
        md["general.alignment"] = ("u32", alignment)
    out += struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(md))
    for key, (kind, value) in md.items():
        out += _s(key.encode())
        if kind == "str":
            out += struct.pack("<I", 8) + _s(value.encode())
        elif isinstance(kind, tuple):
            ek = kind[1]
            out += struct.pack("<I", 9)
            if ek == "str":
                out += struct.pack("<IQ", 8, len(value)) + b"".join(_s(v.encode()) for v in value)
            else:
                out += struct.pack("<IQ", _SCALAR[ek][0], len(value)) + b"".join(struct.pack(_SCALAR[ek][1], v) for v in value)
        else:
            out += struct.pack("<I", _SCALAR[kind][0]) + struct.pack(_SCALAR[kind][1], value)
    offset, blobs = 0, []
    for name, ggml_type, ne, array in tensors:
        raw = np.ascontiguousarray(array).tobytes()
        out += _s(name.encode()) + struct.pack("<I", len(ne)) + b"".join(struct.pack("<Q", d) for d in ne)
        out += struct.pack("<IQ", ggml_type, offset)
        blobs.append(raw)
        offset += (len(raw) + alignment - 1) // alignment * alignment
    out += b"\0" * ((-len(out)) % alignment)
    for raw in blobs:
        out += raw + b"\0" * ((-len(raw)) % alignment)
    with open(path, "wb") as f:
        f.write(out)
