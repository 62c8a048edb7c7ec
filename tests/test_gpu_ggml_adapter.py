"""The GGML_OP_CUSTOM adapters, driven as a ggml CPU graph would drive them (host tensors, strides,
ith/nth), checked against the oracle.  Mirrors the callback-level tests of the reference
(core/tests/... inference_test_hooks.inl:177-256: batched callback vs the reference dot <= 1e-4)."""
import ctypes as C

import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ga():
    from densecore_amd import ggml_adapter
    ggml_adapter.lib()
    yield ggml_adapter
    ggml_adapter.lib().mq_ggml_weight_cache_clear()


def _dense_ref(w, cols, x):
    return orc.mul_mat_q4k_q8k(w, cols, orc.quantize_rows_q8k(x), orc.ORDER_AVX2)


@pytest.mark.parametrize("m,pad", [(1, 0), (5, 0), (3, 64)])
def test_dense_node(ga, m, pad):
    rows, cols = 512, 1024
    w = synth.q4k_matrix(101, rows, cols)
    xbuf = np.zeros((m, cols + pad), np.float32)
    xbuf[:, :cols] = synth.normal_f32(102, (m, cols))
    ybuf = np.full((m, rows + pad), 7.0, np.float32)
    tw = ga.tensor(w, ga.GGML_TYPE_Q4_K, [cols, rows], name=b"blk.0.ffn_gate.weight")
    tx = ga.tensor(xbuf, ga.GGML_TYPE_F32, [cols, m], nb=[4, 4 * (cols + pad)])
    ty = ga.tensor(ybuf, ga.GGML_TYPE_F32, [rows, m], nb=[4, 4 * (rows + pad)])
    ga.set_src(ty, tx, tw)
    fn = ga.lib().mq_cb_gemv_custom if m == 1 else ga.lib().mq_cb_gemv_batched_custom
    fn(C.byref(ty), 1, 4, None)  # a worker other than 0 does nothing
    assert np.all(ybuf == 7.0)
    fn(C.byref(ty), 0, 4, None)
    assert ga.lib().mq_ggml_last_status() == 0
    x = np.ascontiguousarray(xbuf[:, :cols])
    ref = _dense_ref(w, cols, x)
    mag = orc.dot_magnitude_f64(w, cols, orc.quantize_rows_q8k(x))
    assert_fp32_parity(ybuf[:, :rows], ref, mag)
    assert np.all(ybuf[:, rows:] == 7.0)  # padding of a strided dst is not written
    before = ga.lib().mq_ggml_weight_cache_size()
    fn(C.byref(ty), 0, 4, None)  # second call reuses the uploaded weight
    assert ga.lib().mq_ggml_weight_cache_size() == before


def test_dense_node_rejects_mismatch(ga):
    rows, cols = 256, 512
    w = synth.q4k_matrix(111, rows, cols)
    x = synth.normal_f32(112, (1, cols))
    y = np.full((1, rows + 16), 3.0, np.float32)
    tw = ga.tensor(w, ga.GGML_TYPE_Q4_K, [cols, rows])
    tx = ga.tensor(x, ga.GGML_TYPE_F32, [cols, 1])
    ty = ga.tensor(y, ga.GGML_TYPE_F32, [rows + 16, 1])  # dst->ne[0] != weight->ne[1]
    ga.set_src(ty, tx, tw)
    ud = ga.UserData(0, 0, 1, 0)
    ga.lib().mq_cb_gemv_custom(C.byref(ty), 0, 1, C.byref(ud))
    assert ud.last_status != 0 and np.all(y == 3.0)
    tf = ga.tensor(np.zeros((rows, cols), np.float32), ga.GGML_TYPE_F32, [cols, rows])  # F32 weight: not this path
    ty2 = ga.tensor(np.full((1, rows), 3.0, np.float32), ga.GGML_TYPE_F32, [rows, 1])
    ga.set_src(ty2, tx, tf)
    ga.lib().mq_cb_gemv_custom(C.byref(ty2), 0, 1, C.byref(ud))
    assert ud.last_status != 0 and np.all(ty2._keep == 3.0)


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 6, 8, 9, 12, 16, 17, 33, 70, 200, 333])
def test_moe_nodes(ga, n):
    hidden, inter, n_exp, top_k = 512, 256, 8, 2
    gate = np.stack([synth.q4k_matrix(2010 + e, inter, hidden) for e in range(n_exp)])
    up = np.stack([synth.q4k_matrix(2020 + e, inter, hidden) for e in range(n_exp)])
    down = np.stack([synth.q4k_matrix(2030 + e, hidden, inter) for e in range(n_exp)])
    x = synth.normal_f32(204, (n, hidden))
    logits = synth.normal_f32(205, (n, n_exp))
    ids, _ = orc.route_topk(logits, top_k, 1)
    silu = orc.SILU_EXACT if n <= 4 else orc.SILU_FAST
    # gate/up node
    hid = np.zeros((n, top_k, inter), np.float32)
    tg = ga.tensor(gate, ga.GGML_TYPE_Q4_K, [hidden, inter, n_exp])
    tu = ga.tensor(up, ga.GGML_TYPE_Q4_K, [hidden, inter, n_exp])
    tx = ga.tensor(x, ga.GGML_TYPE_F32, [hidden, n])
    ts = ga.tensor(ids, ga.GGML_TYPE_I32, [top_k, n])
    th = ga.tensor(hid, ga.GGML_TYPE_F32, [inter, top_k, n])
    ga.set_src(th, tg, tu, tx, ts)
    ga.lib().mq_cb_moe_gateup_swiglu(C.byref(th), 0, 8, None)
    assert ga.lib().mq_ggml_last_status() == 0
    ref_hid = orc.moe_gateup_swiglu(gate, up, hidden, inter, x, ids, orc.ORDER_AVX2, silu)
    np.testing.assert_allclose(hid, ref_hid, rtol=2e-4, atol=2e-4 * np.abs(ref_hid).max())
    # down node, fed the oracle's hidden so that the stage is checked on identical inputs
    y = np.zeros((n, hidden), np.float32)
    td = ga.tensor(down, ga.GGML_TYPE_Q4_K, [inter, hidden, n_exp])
    th2 = ga.tensor(ref_hid, ga.GGML_TYPE_F32, [inter, top_k, n])
    tl = ga.tensor(logits, ga.GGML_TYPE_F32, [n_exp, n])
    ty = ga.tensor(y, ga.GGML_TYPE_F32, [hidden, n])
    ga.set_src(ty, td, th2, ts, tl)
    ga.lib().mq_cb_moe_down_weighted_logits(C.byref(ty), 0, 8, None)
    assert ga.lib().mq_ggml_last_status() == 0
    w_ref = orc.route_weights_from_ids(logits, ids)
    ref_y = orc.moe_down_weighted(down, hidden, inter, ref_hid, ids, w_ref, orc.ORDER_AVX2, 0)
    np.testing.assert_allclose(y, ref_y, rtol=2e-4, atol=2e-4 * np.abs(ref_y).max())


def test_moe_down_node_with_q5k_experts_and_q5k_dense_node(ga):
    """The down callback replaced is the reference's Q5_K one (cb_qwen35_native_moe_down_q5k_weighted_logits,
    core/src/llm/moe/native.cpp:3051): Q5_K expert stacks and Q5_K dense weights go through the same nodes."""
    n, hidden, inter, n_exp, top_k = 3, 512, 256, 6, 2
    down = np.stack([synth.q5k_matrix(2130 + e, hidden, inter) for e in range(n_exp)])
    hid = synth.normal_f32(2131, (n, top_k, inter))
    logits = synth.normal_f32(2132, (n, n_exp))
    ids, _ = orc.route_topk(logits, top_k, 1)
    y = np.zeros((n, hidden), np.float32)
    td = ga.tensor(down, ga.GGML_TYPE_Q5_K, [inter, hidden, n_exp])
    th = ga.tensor(hid, ga.GGML_TYPE_F32, [inter, top_k, n])
    ts = ga.tensor(ids, ga.GGML_TYPE_I32, [top_k, n])
    tl = ga.tensor(logits, ga.GGML_TYPE_F32, [n_exp, n])
    ty = ga.tensor(y, ga.GGML_TYPE_F32, [hidden, n])
    ga.set_src(ty, td, th, ts, tl)
    ga.lib().mq_cb_moe_down_weighted_logits(C.byref(ty), 0, 8, None)
    assert ga.lib().mq_ggml_last_status() == 0
    w_ref = orc.route_weights_from_ids(logits, ids)
    want = np.zeros((n, hidden))
    for t in range(n):
        for k in range(top_k):
            want[t] += np.float64(w_ref[t, k]) * orc.mul_mat_q5k_f32(down[ids[t, k]], inter, hid[t, k][None])[0]
    np.testing.assert_allclose(y, want, rtol=2e-4, atol=2e-4 * np.abs(want).max())
    # dense node
    rows, cols, m = 96, 768, 2
    w = synth.q5k_matrix(2140, rows, cols)
    x = synth.normal_f32(2141, (m, cols))
    out = np.zeros((m, rows), np.float32)
    tw = ga.tensor(w, ga.GGML_TYPE_Q5_K, [cols, rows])
    tx = ga.tensor(x, ga.GGML_TYPE_F32, [cols, m])
    to = ga.tensor(out, ga.GGML_TYPE_F32, [rows, m])
    ga.set_src(to, tx, tw)
    ga.lib().mq_cb_gemv_batched_custom(C.byref(to), 0, 1, None)
    assert ga.lib().mq_ggml_last_status() == 0
    q8 = orc.quantize_rows_q8k(x)
    assert_fp32_parity(out, orc.mul_mat_q5k_q8k(w, cols, q8), orc.q5k_dot_dequant_f64(w, cols, q8, magnitude=True))
    # library level
    c = np.zeros((m, rows), np.float32)
    assert ga.lib().mq_matmul_ggml_quantized_transb(x.ctypes.data, m, cols, cols, w.ctypes.data, ga.GGML_TYPE_Q5_K, rows,
                                                    cols, 176 * (cols // 256), c.ctypes.data, rows) == 1
    assert np.array_equal(c.view(np.uint32), out.view(np.uint32))


def test_dense_node_and_library_matmul_with_q6k_weights(ga):
    """Q6_K rows (210-byte blocks; the reference's kernel for the type is core/src/llm/matmul/q6_small_batch.h)."""
    rows, cols, m = 80, 1024, 3
    w = synth.q6k_matrix(2240, rows, cols)
    x = synth.normal_f32(2241, (m, cols))
    out = np.zeros((m, rows), np.float32)
    tw = ga.tensor(w, ga.GGML_TYPE_Q6_K, [cols, rows])
    tx = ga.tensor(x, ga.GGML_TYPE_F32, [cols, m])
    to = ga.tensor(out, ga.GGML_TYPE_F32, [rows, m])
    ga.set_src(to, tx, tw)
    ga.lib().mq_cb_gemv_batched_custom(C.byref(to), 0, 1, None)
    assert ga.lib().mq_ggml_last_status() == 0
    q8 = orc.quantize_rows_q8k(x)
    assert_fp32_parity(out, orc.mul_mat_q6k_q8k(w, cols, q8), orc.q6k_dot_dequant_f64(w, cols, q8, magnitude=True))
    c = np.zeros((m, rows), np.float32)
    assert ga.lib().mq_matmul_ggml_quantized_transb(x.ctypes.data, m, cols, cols, w.ctypes.data, ga.GGML_TYPE_Q6_K, rows,
                                                    cols, 210 * (cols // 256), c.ctypes.data, rows) == 1
    assert np.array_equal(c.view(np.uint32), out.view(np.uint32))


def test_dense_node_and_library_matmul_with_q80_weights(ga):
    """Q8_0 rows (34-byte blocks of 32; the reference's kernel for the type is core/src/llm/matmul/q8_small_batch.h);
    the activations are quantized to Q8_0 as the reference's vec_dot_type asks."""
    rows, cols, m = 80, 1024, 3
    w = synth.q80_matrix(2250, rows, cols)
    x = synth.normal_f32(2251, (m, cols))
    out = np.zeros((m, rows), np.float32)
    tw = ga.tensor(w, ga.GGML_TYPE_Q8_0, [cols, rows])
    tx = ga.tensor(x, ga.GGML_TYPE_F32, [cols, m])
    to = ga.tensor(out, ga.GGML_TYPE_F32, [rows, m])
    ga.set_src(to, tx, tw)
    ga.lib().mq_cb_gemv_batched_custom(C.byref(to), 0, 1, None)
    assert ga.lib().mq_ggml_last_status() == 0
    q = orc.quantize_rows_q80(x)
    assert_fp32_parity(out, orc.mul_mat_q80_q80(w, cols, q), orc.q80_dot_dequant_f64(w, cols, q, magnitude=True))
    c = np.zeros((m, rows), np.float32)
    assert ga.lib().mq_matmul_ggml_quantized_transb(x.ctypes.data, m, cols, cols, w.ctypes.data, ga.GGML_TYPE_Q8_0, rows,
                                                    cols, 34 * (cols // 32), c.ctypes.data, rows) == 1
    assert np.array_equal(c.view(np.uint32), out.view(np.uint32))


def test_library_level_matmul(ga):
    m, rows, cols = 7, 384, 768
    w = synth.q4k_matrix(301, rows, cols)
    a = synth.normal_f32(302, (m, cols))
    c = np.zeros((m, rows), np.float32)
    ok = ga.lib().mq_matmul_ggml_quantized_transb(a.ctypes.data, m, cols, cols, w.ctypes.data, ga.GGML_TYPE_Q4_K, rows,
                                                  cols, 144 * (cols // 256), c.ctypes.data, rows)
    assert ok == 1
    assert_fp32_parity(c, _dense_ref(w, cols, a), orc.dot_magnitude_f64(w, cols, orc.quantize_rows_q8k(a)))
    # a type other than Q4_K, Q5_K, Q6_K and Q8_0 is rejected like an unsupported ggml type
    assert ga.lib().mq_matmul_ggml_quantized_transb(a.ctypes.data, m, cols, cols, w.ctypes.data, 2, rows, cols,
                                                    144 * (cols // 256), c.ctypes.data, rows) == 0


@pytest.mark.parametrize("rows,cols", [(1000, 1024), (2048, 2048)])
def test_dense_node_at_every_width_equals_the_device_entry_point(ga, rows, cols):
    """The batched callback on host tensors with strided rows (NaN in the gaps of src, a sentinel in those of dst) at
    1..40 rows and three wider ones: the bits of mq_mul_mat_q4k on the same rows, nothing written outside them."""
    import torch
    from densecore_amd import ops
    w = synth.q4k_matrix(synth.tensor_seed("ga-w", rows, cols), rows, cols)
    W = ops.Q4KWeight.from_ggml(w, cols)
    tw = ga.tensor(w, ga.GGML_TYPE_Q4_K, [cols, rows], name=b"blk.1.attn_output.weight")
    xs = synth.normal_f32(synth.tensor_seed("ga-x", rows, cols), (130, cols))
    for m in list(range(1, 41)) + [49, 70, 130]:
        pad = 32 if m % 2 else 0
        xbuf = np.full((m, cols + pad), np.nan, np.float32)
        xbuf[:, :cols] = xs[:m]
        ybuf = np.full((m + 1, rows + pad), 7.0, np.float32)
        tx = ga.tensor(xbuf, ga.GGML_TYPE_F32, [cols, m], nb=[4, 4 * (cols + pad)])
        ty = ga.tensor(ybuf, ga.GGML_TYPE_F32, [rows, m], nb=[4, 4 * (rows + pad)])
        ga.set_src(ty, tx, tw)
        fn = ga.lib().mq_cb_gemv_custom if m == 1 else ga.lib().mq_cb_gemv_batched_custom
        fn(C.byref(ty), 0, 1, None)
        assert ga.lib().mq_ggml_last_status() == 0, f"m={m}"
        want = ops.mul_mat(W, torch.from_numpy(np.ascontiguousarray(xs[:m])).cuda()).cpu().numpy()
        assert np.array_equal(ybuf[:m, :rows].view(np.uint32), want.view(np.uint32)), f"m={m}"
        assert np.all(ybuf[:m, rows:] == 7.0) and np.all(ybuf[m] == 7.0), f"m={m}: written outside the rows"
    W.free()
