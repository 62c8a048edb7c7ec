"""GGUF reader (include/mi355_q4k_gguf.h): files written by densecore_amd.gguf.write_gguf in the published
GGUF v3 layout are parsed by the C++ reader; metadata, tensor table, alignment and error paths on the
CPU, the upload of Q4_K tensors (2-D and stacked experts) on the GPU.

The reference reads these files through ggml's gguf_init_from_file (core/src/models/model_loader.cpp:2063),
which is not part of this build, and ships no .gguf fixture: agreement with ggml's own reader is not pinned
here beyond the published layout."""
import os
import struct

import numpy as np
import pytest

from densecore_amd import gguf, synth


def _write(tmp_path, alignment=32, version=3):
    rng = np.random.default_rng(1)
    f32 = rng.normal(size=(3, 8)).astype(np.float32)
    q2 = synth.q4k_matrix(11, 48, 512)                                   # [K=512, N=48]
    q3 = np.stack([synth.q4k_matrix(20 + e, 32, 256) for e in range(4)])   # [K=256, N=32, E=4]
    q5 = np.stack([synth.q5k_matrix(30 + e, 16, 512) for e in range(3)])   # [K=512, N=16, E=3], Q5_K
    q6 = synth.q6k_matrix(40, 32, 768)                                      # [K=768, N=32], Q6_K
    path = str(tmp_path / f"model_a{alignment}_v{version}.gguf")
    gguf.write_gguf(path, {
        "general.architecture": ("str", "qwen35moe"),
        "qwen35moe.block_count": ("u32", 40),
        "qwen35moe.expert_count": ("u32", 256),
        "qwen35moe.expert_used_count": ("i64", 8),
        "qwen35moe.rope.freq_base": ("f32", 1e6),
        "general.file_type": ("u16", 15),
        "flag": ("bool", 1),
        "tokenizer.ggml.tokens": (("arr", "str"), ["a", "bc", ""]),
        "tokenizer.ggml.scores": (("arr", "f32"), [0.5, -1.0, 2.0]),
    }, [
        ("token_embd.weight", gguf.GGML_F32, [8, 3], f32),
        ("blk.0.attn_q.weight", gguf.GGML_Q4_K, [512, 48], q2),
        ("blk.0.ffn_gate_exps.weight", gguf.GGML_Q4_K, [256, 32, 4], q3),
        ("blk.0.ffn_down_exps.weight", gguf.GGML_Q5_K, [512, 16, 3], q5),
        ("output.weight", gguf.GGML_Q6_K, [768, 32], q6),
    ], alignment=alignment, version=version)
    return path, f32, q2, q3, q5, q6


@pytest.mark.parametrize("alignment,version", [(32, 3), (64, 2), (4096, 3)])
def test_metadata_and_tensor_table(tmp_path, alignment, version):
    path, f32, q2, q3, q5, q6 = _write(tmp_path, alignment, version)
    with gguf.GgufFile(path) as g:
        assert g.get_string("general.architecture") == "qwen35moe"
        assert g.get_int("qwen35moe.block_count") == 40 and g.get_int("qwen35moe.expert_used_count") == 8
        assert g.get_int("general.file_type") == 15 and g.get_int("flag") == 1
        with pytest.raises(KeyError):
            g.get_int("qwen35moe.rope.freq_base")      # a float, not an integer
        with pytest.raises(KeyError):
            g.get_string("missing.key")
        ts = g.tensors()
        assert [t["name"] for t in ts] == ["token_embd.weight", "blk.0.attn_q.weight", "blk.0.ffn_gate_exps.weight",
                                           "blk.0.ffn_down_exps.weight", "output.weight"]
        assert [t["ne"] for t in ts] == [[8, 3], [512, 48], [256, 32, 4], [512, 16, 3], [768, 32]]
        assert [t["type"] for t in ts] == [0, 12, 12, 13, 14]
        assert [t["nbytes"] for t in ts] == [96, 48 * 2 * 144, 4 * 32 * 144, 3 * 16 * 2 * 176, 32 * 3 * 210]
        assert all(t["offset"] % alignment == 0 for t in ts)
        assert g.find("blk.0.attn_q.weight") == 1 and g.find("nope") == -1
        # the data pointers address the very bytes that were written
        import ctypes
        for t, ref in zip(ts, (f32, q2, q3, q5, q6)):
            assert ctypes.string_at(t["data"], t["nbytes"]) == ref.tobytes()


def test_rejects_what_is_not_gguf(tmp_path):
    path, *_ = _write(tmp_path)
    raw = open(path, "rb").read()
    cases = {
        "magic": b"GGML" + raw[4:],
        "version": raw[:4] + struct.pack("<I", 1) + raw[8:],
        "truncated_header": raw[:40],
        "truncated_data": raw[:-200],
    }
    for name, blob in cases.items():
        p = str(tmp_path / f"bad_{name}.gguf")
        open(p, "wb").write(blob)
        with pytest.raises(ValueError):
            gguf.GgufFile(p)
    with pytest.raises(ValueError):
        gguf.GgufFile(str(tmp_path / "does_not_exist.gguf"))


def test_library_exports_every_declared_symbol():
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(root, "include", "mi355_q4k_gguf.h")).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(mq_gguf_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(gguf.EXPORTS)
    L = gguf.lib()
    for name in declared:
        assert hasattr(L, name), name


@pytest.mark.gpu
def test_q4k_tensors_upload_and_multiply(tmp_path):
    import torch
    from densecore_amd import ops
    from oracle import binding as orc
    from tests._parity import assert_fp32_parity
    path, _, q2, q3, q5, q6 = _write(tmp_path)
    with gguf.GgufFile(path) as g:
        w2 = g.load_q4k("blk.0.attn_q.weight")
        w3 = g.load_weight("blk.0.ffn_gate_exps.weight")
        w5 = g.load_weight("blk.0.ffn_down_exps.weight")
        w6 = g.load_weight("output.weight")
        with pytest.raises(Exception):
            g.load_q4k("token_embd.weight")            # F32: not this path
        with pytest.raises(Exception):
            g.load_q4k("blk.0.ffn_down_exps.weight")   # Q5_K through the Q4_K-only entry
    assert (w5.rows, w5.cols, w5.n_experts, w5.ggml_type) == (16, 512, 3, 13) and np.array_equal(w5.to_ggml(), q5)
    xk = synth.normal_f32(6, (2, 3, 512))
    ids = np.array([[0, 1, 2], [2, 2, 0]], np.int32)
    yk = ops.mul_mat_id(w5, torch.from_numpy(xk).cuda(), torch.from_numpy(ids).cuda()).cpu().numpy()
    for t in range(2):
        for k in range(3):
            q8 = orc.quantize_rows_q8k(xk[t, k][None])
            assert_fp32_parity(yk[t, k][None], orc.mul_mat_q5k_q8k(q5[ids[t, k]], 512, q8),
                               orc.q5k_dot_dequant_f64(q5[ids[t, k]], 512, q8, magnitude=True))
    w5.free()
    assert (w6.rows, w6.cols, w6.ggml_type) == (32, 768, 14) and np.array_equal(w6.to_ggml(), q6)
    x6 = synth.normal_f32(7, (2, 768))
    q8 = orc.quantize_rows_q8k(x6)
    assert_fp32_parity(ops.mul_mat(w6, torch.from_numpy(x6).cuda()).cpu().numpy(), orc.mul_mat_q6k_q8k(q6, 768, q8),
                       orc.q6k_dot_dequant_f64(q6, 768, q8, magnitude=True))
    w6.free()
    assert (w2.rows, w2.cols, w2.n_experts) == (48, 512, 1) and (w3.rows, w3.cols, w3.n_experts) == (32, 256, 4)
    assert np.array_equal(w2.to_ggml(), q2) and np.array_equal(w3.to_ggml(), q3)
    x = synth.normal_f32(5, (3, 512))
    q8 = orc.quantize_rows_q8k(x)
    got = ops.mul_mat(w2, torch.from_numpy(x).cuda()).cpu().numpy()
    assert_fp32_parity(got, orc.mul_mat_q4k_q8k(q2, 512, q8, orc.ORDER_AVX2), orc.dot_magnitude_f64(q2, 512, q8))
    w2.free(), w3.free()


@pytest.mark.gpu
def test_q80_tensor_uploads_and_multiplies(tmp_path):
    """A dense Q8_0 matrix (e.g. the output head of a mixed-precision file) through the same loader."""
    import torch
    from densecore_amd import ops
    from oracle import binding as orc
    from tests._parity import assert_fp32_parity
    q80 = synth.q80_matrix(50, 24, 512)                                     # [K=512, N=24], Q8_0
    path = str(tmp_path / "q80.gguf")
    gguf.write_gguf(path, {"general.architecture": ("str", "qwen35moe")},
                    [("output.weight", gguf.GGML_Q8_0, [512, 24], q80)])
    with gguf.GgufFile(path) as g:
        assert g.tensors()[0]["type"] == 8 and g.tensors()[0]["nbytes"] == 24 * 16 * 34
        w = g.load_weight("output.weight")
        with pytest.raises(Exception):
            g.load_q4k("output.weight")
    assert (w.rows, w.cols, w.n_experts, w.ggml_type) == (24, 512, 1, 8) and np.array_equal(w.to_ggml(), q80)
    x = synth.normal_f32(51, (3, 512))
    q = orc.quantize_rows_q80(x)
    assert_fp32_parity(ops.mul_mat(w, torch.from_numpy(x).cuda()).cpu().numpy(), orc.mul_mat_q80_q80(q80, 512, q),
                       orc.q80_dot_dequant_f64(q80, 512, q, magnitude=True))
    w.free()
