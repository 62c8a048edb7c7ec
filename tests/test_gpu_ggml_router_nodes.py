"""The remaining nodes of the native MoE graph as GGML_OP_CUSTOM adapters: the fused top-8 router
(cb_qwen_native_moe_fused_router, core/src/llm/moe/native.cpp:710-735), the weights-from-logits node
(cb_moe_topk_weights_from_logits, :800-868), a ggml_mul_mat_id node (core/src/llm/moe/native_gemma.cpp:1509-1559), the
down node with Q8_0 experts (:4611-4616, :3239-3245) and the opt-in hand-over of the hidden rows between the two
expert nodes on the device -- each over strided host tensors, against the oracle."""
import ctypes as C

import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ga():
    from densecore_amd import _lib, ggml_adapter
    _lib.lib()
    return ggml_adapter


@pytest.mark.parametrize("n,n_exp", [(1, 256), (5, 64), (1, 12)])
def test_fused_router_node(ga, n, n_exp):
    top_k = 8
    pad = 16 if n > 1 else 0  # logits rows with a longer stride
    buf = synth.normal_f32(5000 + n, (n, n_exp + pad))
    if n > 1:
        buf[1, 3] = buf[1, 7]            # a tie: the lower id goes first
        buf[2, 5] = np.inf               # a selected logit that is not finite: uniform weights
    logits = buf[:, :n_exp]
    sel = np.full((n, top_k), -7, np.int32)
    weights = np.full((n, top_k), -1.0, np.float32)
    state = ga.RouterState(n_exp, n, top_k, weights.ctypes.data, None)
    tl = ga.tensor(buf, ga.GGML_TYPE_F32, [n_exp, n], nb=[4, 4 * (n_exp + pad)])
    ts = ga.tensor(sel, ga.GGML_TYPE_I32, [top_k, n])
    ga.set_src(ts, tl)
    ga.lib().mq_cb_moe_fused_router(C.byref(ts), 0, 1, C.byref(state))
    assert ga.lib().mq_ggml_last_status() == 0
    ids_ref, w_ref = orc.route_topk(np.ascontiguousarray(logits), top_k, 0)
    assert np.array_equal(sel, ids_ref)
    np.testing.assert_allclose(weights, w_ref, rtol=3e-6, atol=1e-7)
    if n > 1:
        assert np.all(weights[2] == np.float32(1.0 / top_k))
    # ith > 0 does nothing; a state that does not match the tensors leaves the node alone
    sel[:] = -7
    ga.lib().mq_cb_moe_fused_router(C.byref(ts), 1, 2, C.byref(state))
    assert np.all(sel == -7)
    bad = ga.RouterState(n_exp + 1, n, top_k, weights.ctypes.data, None)
    ga.lib().mq_cb_moe_fused_router(C.byref(ts), 0, 1, C.byref(bad))
    assert np.all(sel == -7) and ga.lib().mq_ggml_last_status() != 0


@pytest.mark.parametrize("n", [1, 7])
def test_weights_from_logits_node(ga, n):
    n_exp, top_k = 40, 6
    logits = synth.normal_f32(5100 + n, (n, n_exp))
    ids, _ = orc.route_topk(logits, top_k, 1)
    ids = ids.copy()
    if n > 1:
        ids[1, 2] = -1          # an id outside the range weighs 0
        ids[2, 0] = n_exp + 3
        logits[3, ids[3, 1]] = -np.inf
    out = np.full((n, top_k, 1), 9.0, np.float32)  # ggml ne = [1, top_k, n_tokens]
    tl = ga.tensor(logits, ga.GGML_TYPE_F32, [n_exp, n])
    ts = ga.tensor(ids, ga.GGML_TYPE_I32, [top_k, n])
    to = ga.tensor(out, ga.GGML_TYPE_F32, [1, top_k, n])
    ga.set_src(to, tl, ts)
    ga.lib().mq_cb_moe_topk_weights_from_logits(C.byref(to), 0, 4, None)
    assert ga.lib().mq_ggml_last_status() == 0
    ref = orc.route_weights_from_ids(logits, ids)
    np.testing.assert_allclose(out[:, :, 0], ref, rtol=3e-6, atol=1e-7)
    if n > 1:
        assert out[1, 2, 0] == 0.0 and out[2, 0, 0] == 0.0


@pytest.mark.parametrize("wtype", ["q4k", "q5k"])
@pytest.mark.parametrize("n,x_slots", [(1, 1), (4, 1), (3, 2), (20, 2)])
def test_mul_mat_id_node(ga, n, x_slots, wtype):
    k_in, n_out, n_exp, top_k = 512, 96, 10, 2
    make, gtype, mul = ((synth.q4k_matrix, ga.GGML_TYPE_Q4_K, orc.mul_mat_q4k_f32) if wtype == "q4k" else
                        (synth.q5k_matrix, ga.GGML_TYPE_Q5_K, orc.mul_mat_q5k_f32))
    w = np.stack([make(5200 + e, n_out, k_in) for e in range(n_exp)])
    b = synth.normal_f32(5210 + n, (n, x_slots, k_in))
    logits = synth.normal_f32(5211 + n, (n, n_exp))
    ids, _ = orc.route_topk(logits, top_k, 1)
    ids = ids.copy()
    if n > 2:
        ids[2, 1] = -5  # comes back as a row of zeros
    out = np.full((n, top_k, n_out), 7.0, np.float32)
    tw = ga.tensor(w, gtype, [k_in, n_out, n_exp])
    tb = ga.tensor(b, ga.GGML_TYPE_F32, [k_in, x_slots, n])
    ts = ga.tensor(ids, ga.GGML_TYPE_I32, [top_k, n])
    to = ga.tensor(out, ga.GGML_TYPE_F32, [n_out, top_k, n])
    ga.set_src(to, tw, tb, ts)
    ga.lib().mq_cb_mul_mat_id(C.byref(to), 0, 4, None)
    assert ga.lib().mq_ggml_last_status() == 0
    for t in range(n):
        for k in range(top_k):
            if ids[t, k] < 0:
                assert np.all(out[t, k] == 0.0)
                continue
            row = b[t, k if x_slots > 1 else 0][None]
            ref = mul(w[ids[t, k]], k_in, row)[0]
            np.testing.assert_allclose(out[t, k], ref, rtol=2e-4, atol=2e-4 * np.abs(ref).max())
    # a b operand whose slot count is neither 1 nor n_used is refused and dst stays as it was
    bad = synth.normal_f32(1, (n, 3, k_in))
    tb2 = ga.tensor(bad, ga.GGML_TYPE_F32, [k_in, 3, n])
    out[:] = 7.0
    ga.set_src(to, tw, tb2, ts)
    ga.lib().mq_cb_mul_mat_id(C.byref(to), 0, 4, None)
    assert ga.lib().mq_ggml_last_status() != 0 and np.all(out == 7.0)


def _down_q80_reference(down, inter, hid, ids, w):
    """The down node on Q8_0 experts: every (token, k) hidden row is quantized to Q8_0 and multiplied by its expert
    (core/src/llm/moe/native.cpp:3239-3286), the results are summed in k order with the routing weights."""
    n, top_k = ids.shape
    y = np.zeros((n, down.shape[1]), np.float32)
    for t in range(n):
        for k in range(top_k):
            e = ids[t, k]
            if e < 0 or e >= down.shape[0] or w[t, k] == 0.0:
                continue
            q = orc.quantize_rows_q80(hid[t, k][None])
            y[t] += np.float32(w[t, k]) * orc.mul_mat_q80_q80(down[e], inter, q)[0].astype(np.float32)
    return y


@pytest.mark.parametrize("n", [1, 5, 20])
def test_down_node_with_q80_experts(ga, n):
    hidden, inter, n_exp, top_k = 384, 512, 6, 3
    down = np.stack([synth.q80_matrix(5300 + e, hidden, inter) for e in range(n_exp)])
    hid = synth.normal_f32(5310 + n, (n, top_k, inter))
    logits = synth.normal_f32(5311 + n, (n, n_exp))
    ids, _ = orc.route_topk(logits, top_k, 1)
    ids = ids.copy()
    if n > 2:
        ids[1, 1] = n_exp  # dropped pair
    y = np.zeros((n, hidden), np.float32)
    td = ga.tensor(down, ga.GGML_TYPE_Q8_0, [inter, hidden, n_exp])
    th = ga.tensor(hid, ga.GGML_TYPE_F32, [inter, top_k, n])
    ts = ga.tensor(ids, ga.GGML_TYPE_I32, [top_k, n])
    tl = ga.tensor(logits, ga.GGML_TYPE_F32, [n_exp, n])
    ty = ga.tensor(y, ga.GGML_TYPE_F32, [hidden, n])
    ga.set_src(ty, td, th, ts, tl)
    ga.lib().mq_cb_moe_down_weighted_logits(C.byref(ty), 0, 8, None)
    assert ga.lib().mq_ggml_last_status() == 0
    w_ref = orc.route_weights_from_ids(logits, ids)
    want = _down_q80_reference(down, inter, hid, ids, w_ref)
    np.testing.assert_allclose(y, want, rtol=2e-4, atol=2e-4 * np.abs(want).max())


@pytest.mark.parametrize("n", [1, 4, 12])
def test_hidden_rows_handed_over_on_the_device(ga, n):
    """keep_hidden_on_device: the gate/up node leaves dst untouched, the down node that follows finds the rows in HBM
    and returns the bits of the pair run with both host copies; a down node fed another tensor does not use them."""
    hidden, inter, n_exp, top_k = 512, 256, 8, 2
    gate = np.stack([synth.q4k_matrix(5410 + e, inter, hidden) for e in range(n_exp)])
    up = np.stack([synth.q4k_matrix(5420 + e, inter, hidden) for e in range(n_exp)])
    down = np.stack([synth.q4k_matrix(5430 + e, hidden, inter) for e in range(n_exp)])
    x = synth.normal_f32(5404 + n, (n, hidden))
    logits = synth.normal_f32(5405 + n, (n, n_exp))
    ids, _ = orc.route_topk(logits, top_k, 1)
    tg = ga.tensor(gate, ga.GGML_TYPE_Q4_K, [hidden, inter, n_exp])
    tu = ga.tensor(up, ga.GGML_TYPE_Q4_K, [hidden, inter, n_exp])
    td = ga.tensor(down, ga.GGML_TYPE_Q4_K, [inter, hidden, n_exp])
    tx = ga.tensor(x, ga.GGML_TYPE_F32, [hidden, n])
    ts = ga.tensor(ids, ga.GGML_TYPE_I32, [top_k, n])
    tl = ga.tensor(logits, ga.GGML_TYPE_F32, [n_exp, n])

    def run_pair(keep):
        hid = np.full((n, top_k, inter), 5.0, np.float32)
        y = np.zeros((n, hidden), np.float32)
        th = ga.tensor(hid, ga.GGML_TYPE_F32, [inter, top_k, n])
        ty = ga.tensor(y, ga.GGML_TYPE_F32, [hidden, n])
        ud = ga.UserData(0, 0, 1, 0, 1 if keep else 0)
        ga.set_src(th, tg, tu, tx, ts)
        ga.lib().mq_cb_moe_gateup_swiglu(C.byref(th), 0, 8, C.byref(ud))
        assert ud.last_status == 0
        ga.set_src(ty, td, th, ts, tl)
        ga.lib().mq_cb_moe_down_weighted_logits(C.byref(ty), 0, 8, C.byref(ud))
        assert ud.last_status == 0
        return hid, y

    hid_host, y_host = run_pair(False)
    hid_kept, y_kept = run_pair(True)
    assert np.all(hid_kept == 5.0), "with the hand-over the gate/up node must not write dst"
    assert not np.all(hid_host == 5.0)
    assert np.array_equal(y_host.view(np.uint32), y_kept.view(np.uint32))
    # the rows on the device belong to ONE following down node: another hidden tensor is uploaded as usual
    hid = np.full((n, top_k, inter), 5.0, np.float32)
    th = ga.tensor(hid, ga.GGML_TYPE_F32, [inter, top_k, n])
    ud = ga.UserData(0, 0, 1, 0, 1)
    ga.set_src(th, tg, tu, tx, ts)
    ga.lib().mq_cb_moe_gateup_swiglu(C.byref(th), 0, 8, C.byref(ud))
    other = hid_host.copy()
    y2 = np.zeros((n, hidden), np.float32)
    th2 = ga.tensor(other, ga.GGML_TYPE_F32, [inter, top_k, n])
    ty2 = ga.tensor(y2, ga.GGML_TYPE_F32, [hidden, n])
    ga.set_src(ty2, td, th2, ts, tl)
    ga.lib().mq_cb_moe_down_weighted_logits(C.byref(ty2), 0, 8, C.byref(ud))
    assert np.array_equal(y2.view(np.uint32), y_host.view(np.uint32))


def test_hand_over_followed_by_another_node(ga):
    """A gate/up node that handed its rows over returns while its uploads are still queued.  If the node after it is
    NOT its down node -- here a second gate/up node with other input, then a dense node -- that node first waits for
    the queued copies before it reuses the staging buffers: both results equal the runs without any hand-over."""
    hidden, inter, n_exp, top_k, n = 512, 256, 8, 2, 4
    gate = np.stack([synth.q4k_matrix(5610 + e, inter, hidden) for e in range(n_exp)])
    up = np.stack([synth.q4k_matrix(5620 + e, inter, hidden) for e in range(n_exp)])
    tg = ga.tensor(gate, ga.GGML_TYPE_Q4_K, [hidden, inter, n_exp])
    tu = ga.tensor(up, ga.GGML_TYPE_Q4_K, [hidden, inter, n_exp])
    xs = [synth.normal_f32(5630 + i, (n, hidden)) for i in range(2)]
    ids = [orc.route_topk(synth.normal_f32(5640 + i, (n, n_exp)), top_k, 1)[0] for i in range(2)]
    dense = synth.q4k_matrix(5650, 128, hidden)
    tw = ga.tensor(dense, ga.GGML_TYPE_Q4_K, [hidden, 128])

    def gateup(i, keep):
        hid = np.zeros((n, top_k, inter), np.float32)
        th = ga.tensor(hid, ga.GGML_TYPE_F32, [inter, top_k, n])
        tx = ga.tensor(xs[i], ga.GGML_TYPE_F32, [hidden, n])
        ts = ga.tensor(ids[i], ga.GGML_TYPE_I32, [top_k, n])
        ud = ga.UserData(0, 0, 1, 0, 1 if keep else 0)
        ga.set_src(th, tg, tu, tx, ts)
        ga.lib().mq_cb_moe_gateup_swiglu(C.byref(th), 0, 8, C.byref(ud))
        assert ud.last_status == 0
        return hid

    def dense_node(i):
        y = np.zeros((n, 128), np.float32)
        ty = ga.tensor(y, ga.GGML_TYPE_F32, [128, n])
        tx = ga.tensor(xs[i], ga.GGML_TYPE_F32, [hidden, n])
        ga.set_src(ty, tx, tw)
        ga.lib().mq_cb_gemv_batched_custom(C.byref(ty), 0, 1, None)
        assert ga.lib().mq_ggml_last_status() == 0
        return y

    want_hid, want_y = gateup(1, False), dense_node(0)
    for _ in range(3):
        gateup(0, True)                      # rows kept on the device, uploads still queued
        got_hid = gateup(1, False)           # another node reuses the same staging buffers
        assert np.array_equal(got_hid.view(np.uint32), want_hid.view(np.uint32))
        gateup(1, True)
        got_y = dense_node(0)
        assert np.array_equal(got_y.view(np.uint32), want_y.view(np.uint32))


def test_weight_cache_notices_new_contents_at_the_same_address(ga):
    """A model reloaded into the same buffer (same pointer, shape and strides, other bytes) must not be answered from
    the tiles of the old one: the cache key holds a fingerprint of the contents."""
    rows, cols, m = 64, 1024, 2
    buf = synth.q4k_matrix(5500, rows, cols).copy()
    x = synth.normal_f32(5501, (m, cols))

    def run():
        out = np.zeros((m, rows), np.float32)
        tw = ga.tensor(buf, ga.GGML_TYPE_Q4_K, [cols, rows])
        tx = ga.tensor(x, ga.GGML_TYPE_F32, [cols, m])
        to = ga.tensor(out, ga.GGML_TYPE_F32, [rows, m])
        ga.set_src(to, tx, tw)
        ga.lib().mq_cb_gemv_batched_custom(C.byref(to), 0, 1, None)
        assert ga.lib().mq_ggml_last_status() == 0
        return out

    first = run()
    size = ga.lib().mq_ggml_weight_cache_size()
    assert np.array_equal(run(), first) and ga.lib().mq_ggml_weight_cache_size() == size
    buf[:] = synth.q4k_matrix(5502, rows, cols)  # other weights, same address
    second = run()
    q8 = orc.quantize_rows_q8k(x)
    assert_fp32_parity(second, orc.mul_mat_q4k_q8k(buf, cols, q8), orc.dot_magnitude_f64(buf, cols, q8))
    assert not np.array_equal(first, second)
    assert ga.lib().mq_ggml_weight_cache_size() == size
