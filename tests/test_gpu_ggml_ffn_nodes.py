"""A dense FFN / shared expert as the reference's graph emits it -- three matmul nodes, the fused SiLU x mul node
(cb_silu_mul_fused, core/src/llm/graph/fused_ops.cpp:317-366), the scalar-gate node (cb_apply_shared_scalar_gate,
:437-475; graph at core/src/llm/graph/decoder.cpp:2426-2600) -- driven through the adapters with host tensors, once
with every node delivering to host memory and once with the intermediate tensors left on the device."""
import ctypes as C
import time

import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity
from tests.test_gpu_ffn_moe import assert_close_prod

pytestmark = pytest.mark.gpu

H, I = 2048, 512


@pytest.fixture(scope="module")
def ga():
    from densecore_amd import ggml_adapter
    ggml_adapter.lib()
    yield ggml_adapter
    ggml_adapter.lib().mq_ggml_weight_cache_clear()


@pytest.fixture(scope="module")
def weights():
    return tuple(synth.q4k_matrix(synth.tensor_seed("ffn-nodes", nm), r, c) for nm, r, c in (("g", I, H), ("u", I, H), ("d", H, I)))


def sigmoid(x):
    x = x.astype(np.float64)
    return np.where(x >= 0, 1 / (1 + np.exp(-x)), np.exp(x) / (1 + np.exp(x)))


class Chain:
    """The five nodes over fresh host buffers filled with a sentinel."""

    def __init__(self, ga, weights, x, logit, keep):
        g, u, d = weights
        n = x.shape[0]
        self.ga, self.n = ga, n
        self.bufs = {k: np.full(shape, 7.0, np.float32) for k, shape in
                     (("gate", (n, I)), ("up", (n, I)), ("h", (n, I)), ("y", (n, H)), ("out", (n, H)))}
        t = lambda a, ne: ga.tensor(a, ga.GGML_TYPE_F32, ne)
        self.tx, self.tl = t(x, [H, n]), t(logit, [1, n])
        self.tw = [ga.tensor(w, ga.GGML_TYPE_Q4_K, [c, r]) for w, r, c in ((g, I, H), (u, I, H), (d, H, I))]
        self.tg, self.tu, self.th = t(self.bufs["gate"], [I, n]), t(self.bufs["up"], [I, n]), t(self.bufs["h"], [I, n])
        self.ty, self.to = t(self.bufs["y"], [H, n]), t(self.bufs["out"], [H, n])
        ga.set_src(self.tg, self.tx, self.tw[0])
        ga.set_src(self.tu, self.tx, self.tw[1])
        ga.set_src(self.ty, self.th, self.tw[2])
        self.keep = ga.UserData(0, 0, 1, 0, 1) if keep else None
        self.dense = ga.lib().mq_cb_gemv_custom if n == 1 else ga.lib().mq_cb_gemv_batched_custom

    def run(self):
        L, ud = self.ga.lib(), (C.byref(self.keep) if self.keep else None)
        L.mq_ggml_graph_begin()
        self.dense(C.byref(self.tg), 0, 4, ud)
        self.dense(C.byref(self.tu), 0, 4, ud)
        L.mq_cb_silu_mul_fused(C.byref(self.th), C.byref(self.tg), C.byref(self.tu), 0, 4, ud)
        self.dense(C.byref(self.ty), 0, 4, ud)
        L.mq_cb_apply_shared_scalar_gate(C.byref(self.to), C.byref(self.ty), C.byref(self.tl), 0, 4, None)  # the host reads this one
        assert L.mq_ggml_last_status() == 0


@pytest.mark.parametrize("n", [1, 5, 20])
def test_shared_expert_through_nodes(ga, weights, n):
    g, u, d = weights
    x = synth.normal_f32(synth.tensor_seed("ffn-nodes-x", n), (n, H))
    logit = synth.normal_f32(synth.tensor_seed("ffn-nodes-l", n), (n, 1))
    host = Chain(ga, weights, x, logit, keep=False)
    host.run()
    # every stage against the CPU restatement, the GPU's own intermediate fed forward
    q8 = orc.quantize_rows_q8k(x)
    assert_fp32_parity(host.bufs["gate"], orc.mul_mat_q4k_q8k(g, H, q8), orc.dot_magnitude_f64(g, H, q8), "gate node")
    assert_fp32_parity(host.bufs["up"], orc.mul_mat_q4k_q8k(u, H, q8), orc.dot_magnitude_f64(u, H, q8), "up node")
    want_h = np.array([[orc.lib().orc_silu_mul(float(a), float(b), orc.SILU_FAST_FMA) for a, b in zip(ra, rb)]
                       for ra, rb in zip(host.bufs["gate"], host.bufs["up"])], np.float32)
    assert np.array_equal(host.bufs["h"].view(np.uint32), want_h.view(np.uint32)), "silu x mul node: the fused-multiply-add polynomial, bit for bit"
    hq = orc.quantize_rows_q8k(host.bufs["h"])
    assert_fp32_parity(host.bufs["y"], orc.mul_mat_q4k_q8k(d, I, hq), orc.dot_magnitude_f64(d, I, hq), "down node")
    gate = sigmoid(logit[:, 0])
    assert np.allclose(host.bufs["out"], host.bufs["y"].astype(np.float64) * gate[:, None], rtol=3e-7, atol=0)
    # end to end against the CPU FFN and gate
    ref = orc.ffn_swiglu(g, u, d, H, I, x, silu=orc.SILU_FAST_FMA).astype(np.float64) * gate[:, None]
    assert np.max(np.abs(host.bufs["out"] - ref)) <= 2e-3 * np.max(np.abs(ref))

    # the same graph with the four intermediate tensors left on the device: the same bits, and their host memory untouched
    dev = Chain(ga, weights, x, logit, keep=True)
    dev.run()
    assert np.array_equal(dev.bufs["out"].view(np.uint32), host.bufs["out"].view(np.uint32))
    for name in ("gate", "up", "h", "y"):
        assert np.all(dev.bufs[name] == 7.0), f"{name} was written although it stays on the device"
    # a consumer outside these nodes asks for a tensor: it arrives as the host-delivering run made it
    assert ga.lib().mq_ggml_tensor_to_host(C.byref(dev.th)) == 1
    assert np.array_equal(dev.bufs["h"].view(np.uint32), host.bufs["h"].view(np.uint32))
    assert ga.lib().mq_ggml_tensor_to_host(C.byref(dev.tx)) == 0      # never was on the device
    # a new graph compute forgets them: the down node then reads the host rows it is given
    ga.lib().mq_ggml_graph_begin()
    assert ga.lib().mq_ggml_tensor_to_host(C.byref(dev.tg)) == 0
    dev.bufs["h"][:] = 0.0
    dev.dense(C.byref(dev.ty), 0, 1, None)
    assert not dev.bufs["y"].any()


def test_silu_mul_node_strided_and_rejected(ga):
    n, cols, pad = 3, 768, 32
    a = np.zeros((n, cols + pad), np.float32)
    b = np.zeros((n, cols + pad), np.float32)
    a[:, :cols], b[:, :cols] = synth.normal_f32(1, (n, cols)) * 3, synth.normal_f32(2, (n, cols))
    out = np.full((n, cols + pad), 7.0, np.float32)
    ta, tb, to = (ga.tensor(v, ga.GGML_TYPE_F32, [cols, n], nb=[4, 4 * (cols + pad)]) for v in (a, b, out))
    ga.lib().mq_cb_silu_mul_fused(C.byref(to), C.byref(ta), C.byref(tb), 1, 2, None)     # not worker 0
    assert np.all(out == 7.0)
    ga.lib().mq_cb_silu_mul_fused(C.byref(to), C.byref(ta), C.byref(tb), 0, 2, None)
    assert ga.lib().mq_ggml_last_status() == 0
    # strided tensors: the reference's scalar branch with the exact exponential (fused_ops.cpp:364)
    want = np.array([[orc.lib().orc_silu_mul(float(p), float(q), orc.SILU_EXACT) for p, q in zip(ra, rb)]
                     for ra, rb in zip(a[:, :cols], b[:, :cols])], np.float32)
    assert_close_prod(out[:, :cols], want, "strided silu x mul")
    assert np.max(np.abs(out[:, :cols] - want)) <= 2e-6 * np.max(np.abs(want))
    assert np.all(out[:, cols:] == 7.0)
    # shapes that differ: dst untouched
    t_short = ga.tensor(np.zeros((n, cols - 256), np.float32), ga.GGML_TYPE_F32, [cols - 256, n])
    out[:] = 7.0
    ga.lib().mq_cb_silu_mul_fused(C.byref(to), C.byref(ta), C.byref(t_short), 0, 1, None)
    assert ga.lib().mq_ggml_last_status() != 0 and np.all(out == 7.0)


def test_scalar_gate_node_strided_logits(ga):
    n, hidden = 4, 512
    src = synth.normal_f32(3, (n, hidden))
    logits = np.zeros((n, 8), np.float32)                  # one logit per token, rows 32 bytes apart
    logits[:, 0] = np.array([-30.0, -0.5, 0.0, 12.0], np.float32)
    out = np.zeros((n, hidden), np.float32)
    ts, to = ga.tensor(src, ga.GGML_TYPE_F32, [hidden, n]), ga.tensor(out, ga.GGML_TYPE_F32, [hidden, n])
    tl = ga.tensor(logits, ga.GGML_TYPE_F32, [1, n], nb=[4, 32])
    ga.lib().mq_cb_apply_shared_scalar_gate(C.byref(to), C.byref(ts), C.byref(tl), 0, 1, None)
    assert ga.lib().mq_ggml_last_status() == 0
    want = src.astype(np.float64) * sigmoid(logits[:, 0])[:, None]
    assert np.allclose(out, want, rtol=3e-7, atol=1e-30)
    assert out[0].any()                                   # sigmoid(-30) is tiny, not zero: the two-sided form


def test_shared_expert_chain_time(ga, weights, capsys):
    """Not a pass/fail bound on speed: prints what the five nodes cost at one token with and without the hand-over."""
    x = synth.normal_f32(5, (1, H))
    logit = synth.normal_f32(6, (1, 1))
    out = {}
    for keep in (False, True):
        ch = Chain(ga, weights, x, logit, keep)
        for _ in range(20):
            ch.run()
        t = time.perf_counter()
        for _ in range(200):
            ch.run()
        out[keep] = (time.perf_counter() - t) / 200 * 1e6
    with capsys.disabled():
        print(f"\nshared expert through five nodes, one token: {out[False]:.1f} us per chain through host memory, "
              f"{out[True]:.1f} us with the intermediates left on the device")
    assert out[True] < out[False]
