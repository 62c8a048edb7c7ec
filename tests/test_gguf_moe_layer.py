"""A MoE layer bound straight from a model file: mq_gguf_load_moe_layer resolves the reference's tensor names
(core/src/models/model_loader.cpp:231-235, 3961-4001, 4429-4440) and fills the descriptor mq_moe_layer_q4k takes.

The file comes from tests/golden/make_gguf_moe_layer.py, which states the container layout and the names without
anything of this repository and is pinned here by the SHA-256 of what it writes: Q4_K gate / up stacks [256, 256, 3],
a Q5_K down stack, a shared expert of the same types, its F32 scalar gate and an F16 router.  The CPU part checks the
table the reader makes of it; the GPU part runs the loaded layer against the CPU restatement on the file's own bytes."""
import ctypes as C
import hashlib
import importlib.util
import os

import numpy as np
import pytest

from densecore_amd import gguf

HERE = os.path.dirname(os.path.abspath(__file__))
SHA256 = "49e21c0fe5acdbb7bce9f3320175662d482e8d430465ce0007862380871cedcd"
H = I = 256
E, K = 3, 2


def maker():
    spec = importlib.util.spec_from_file_location("make_gguf_moe_layer", os.path.join(HERE, "golden", "make_gguf_moe_layer.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def layer_file(tmp_path_factory):
    blob = maker().moe_layer_file()
    assert hashlib.sha256(blob).hexdigest() == SHA256, "the fixture script no longer writes the pinned file"
    path = str(tmp_path_factory.mktemp("gguf") / "moe_layer.gguf")
    open(path, "wb").write(blob)
    return path


def test_the_reader_sees_the_layer(layer_file):
    mk = maker()
    with gguf.GgufFile(layer_file) as g:
        ts = {t["name"]: t for t in g.tensors()}
        assert g.get_string("general.architecture") == "qwen35moe" and g.get_int("qwen35moe.expert_used_count") == K
        want = {"blk.0.ffn_gate_exps.weight": (12, [H, I, E], mk._kquant_rows(11, I * E, 144)),
                "blk.0.ffn_up_exps.weight": (12, [H, I, E], mk._kquant_rows(12, I * E, 144)),
                "blk.0.ffn_down_exps.weight": (13, [I, H, E], mk._kquant_rows(13, H * E, 176)),
                "blk.0.ffn_gate_shexp.weight": (12, [H, I], mk._kquant_rows(14, I, 144)),
                "blk.0.ffn_up_shexp.weight": (12, [H, I], mk._kquant_rows(15, I, 144)),
                "blk.0.ffn_down_shexp.weight": (13, [I, H], mk._kquant_rows(16, H, 176))}
        for name, (ttype, ne, raw) in want.items():
            t = ts[name]
            assert (t["type"], t["ne"], t["nbytes"]) == (ttype, ne, len(raw)), name
            assert C.string_at(t["data"], len(raw)) == raw, name
        assert ts["blk.0.ffn_gate_inp.weight"]["type"] == 1 and ts["blk.0.ffn_gate_inp.weight"]["ne"] == [H, E]
        assert ts["blk.0.ffn_gate_inp_shexp.weight"]["ne"] == [H]


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 5, 20])
def test_loaded_layer_against_the_cpu_layer(layer_file, n):
    import torch
    from densecore_amd import _lib, synth
    from oracle import binding as orc
    mk = maker()
    rows = lambda seed, count, bb: np.frombuffer(mk._kquant_rows(seed, count, bb), np.uint8)
    ge, ue = rows(11, I * E, 144).reshape(E, I, 144), rows(12, I * E, 144).reshape(E, I, 144)
    de = rows(13, H * E, 176).reshape(E, H, 176)
    sg, su, sd = rows(14, I, 144).reshape(I, 144), rows(15, I, 144).reshape(I, 144), rows(16, H, 176).reshape(H, 176)
    gate_inp = np.array([((i * 37) % 64 - 32) / 512.0 for i in range(H)], np.float32)
    router = np.array([[(((e * H + i) * 29) % 256 - 128) / 256.0 for i in range(H)] for e in range(E)], np.float32)
    with gguf.GgufFile(layer_file) as g:
        layer = g.load_moe_layer(0)
        assert (layer.n_experts, layer.hidden, layer.inter, layer.top_k) == (E, H, I, K)
        assert [w.ggml_type for w in layer.weights] == [12, 12, 13, 12, 12, 13]
        # what went to the device is what the file holds: stacks bit for bit, router and scalar gate as fp32
        for w, raw in zip(layer.weights, (ge, ue, de, sg, su, sd)):
            assert np.array_equal(w.to_ggml(), raw)
        for ptr, want in ((layer.raw.router_dev, router), (layer.raw.sh_gate_inp_dev, gate_inp)):
            got = np.empty_like(want)
            _lib.check(_lib.lib().mq_memcpy_d2h(C.c_void_p(got.ctypes.data), C.c_void_p(ptr), got.nbytes), "mq_memcpy_d2h")
            assert np.array_equal(got, want)
        with pytest.raises(_lib.MqError):
            g.load_moe_layer(1)                       # the file has no blk.1
        x = synth.normal_f32(synth.tensor_seed("gguf-layer-x", n), (n, H))
        # the router projection through the library's own fp32 operator on the loaded router
        xd = torch.from_numpy(x).cuda()
        logits = torch.empty((n, E), device="cuda")
        p = lambda t: C.c_void_p(t.data_ptr())
        _lib.check(_lib.lib().mq_router_logits_f32(C.c_void_p(layer.raw.router_dev), E, H, p(xd), n, H, p(logits), None), "mq_router_logits_f32")
        lg = logits.cpu().numpy()
        assert np.allclose(lg, x.astype(np.float64) @ router.astype(np.float64).T, rtol=1e-5, atol=1e-5)
        y, ids, wts = layer.run(xd, logits, silu=0, route_mode=0)
        ref = orc.moe_layer(ge, ue, de, H, I, K, x, lg, shared=(sg, su, sd, gate_inp), silu=0, types=(12, 13, 12, 13))
        assert np.array_equal(ids.cpu().numpy(), ref["ids"])
        assert np.allclose(wts.cpu().numpy(), ref["weights"], rtol=3e-6)
        got = y.cpu().numpy()
        rel = np.max(np.abs(got - ref["y"]), axis=1) / np.max(np.abs(ref["y"]), axis=1)
        assert np.max(rel) <= 2e-3, np.max(rel)
        layer.free()
