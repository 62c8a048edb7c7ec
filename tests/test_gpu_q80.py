"""GPU parity: dense Q8_0 weights (34-byte blocks of 32 weights, weight = d * code) against Q8_0 activations.

The reference's own kernel for the type is Q8SmallBatchDot4 (core/src/llm/matmul/q8_small_batch.h:29-77).  The
integer sum of every 32-weight block must equal the oracle's bit for bit, given the same activation codes; fp32
within 1e-4 of both fp32 orders the oracle restates.  The activation quantizer is ggml's (a submodule the reference
tree does not carry): the GPU's codes and scales are compared with the oracle's restatement of ggml's published x86
form, whose parity with the reference build is unpinned.
"""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu

Q80 = synth.GGML_TYPE_Q8_0
ORDERS = {"eight-lane": orc.ORDER_HWY, "per-block": orc.ORDER_DOTPROD}


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("rows,cols", [(16, 256), (40, 1024), (1000, 2048), (7, 512)])
def test_q80_upload_download_round_trip_and_synthetic_fill(ops, rows, cols):
    raw = synth.q80_matrix(800 + rows, rows, cols)
    w = ops.Q4KWeight.from_ggml(raw, cols, Q80)
    assert w.ggml_type == Q80 and w.ggml_bytes == raw.size
    assert np.array_equal(w.to_ggml(), raw)
    w.free()
    seed = synth.tensor_seed("fill80", rows, cols)
    s = ops.Q4KWeight.synthetic(seed, rows, cols, 1, Q80)
    assert np.array_equal(s.to_ggml(), synth.q80_matrix(seed, rows, cols))
    s.free()


CASES = [(16, 256, 1), (40, 256, 3), (64, 1024, 1), (512, 2048, 4), (2048, 512, 8), (256, 4096, 16), (100, 768, 5),
         (48, 14336, 2), (4096, 4096, 1), (64, 1024, 17), (32, 512, 70)]


@pytest.mark.parametrize("rows,cols,n", CASES)
def test_q80_matmul_integer_sums_exact_and_fp32_within_tolerance(ops, rows, cols, n):
    w_np = synth.q80_matrix(synth.tensor_seed("mm80-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("mm80-x", rows, cols, n), (n, cols))
    w = ops.Q4KWeight.from_ggml(w_np, cols, Q80)
    sums, _, y_dbg = ops.debug_block_sums(w, cu(x))
    y = ops.mul_mat(w, cu(x)).cpu().numpy()
    assert np.array_equal(y.view(np.uint32), y_dbg.cpu().numpy().view(np.uint32))
    q = orc.quantize_rows_q80(x, orc.Q80_X86)
    assert np.array_equal(sums.cpu().numpy(), orc.q80_matrix_block_sums(w_np, cols, q))
    mag = orc.q80_dot_dequant_f64(w_np, cols, q, magnitude=True)
    for name, order in ORDERS.items():
        assert_fp32_parity(y, orc.mul_mat_q80_q80(w_np, cols, q, order), mag, f"q80 {name} {rows}x{cols} n={n}")
    assert_fp32_parity(y, orc.q80_dot_dequant_f64(w_np, cols, q), mag, "q80 vs double")
    w.free()


def test_q80_edge_inputs(ops):
    """Zero rows, a zero block inside a row, huge and tiny magnitudes, ties at .5 (round half to even)."""
    rows, cols = 32, 512
    w_np = synth.q80_matrix(81, rows, cols)
    x = synth.normal_f32(82, (6, cols))
    x[1] = 0.0
    x[2, 32:64] = 0.0
    x[3] *= np.float32(1000.0)
    x[4] *= np.float32(1e-30)
    x[5, :32] = np.arange(32, dtype=np.float32) + np.float32(0.5)   # amax 31.5: x * (127 / amax) lands near halves
    x[5, 31] = np.float32(127.0)                                      # amax 127: codes = rne(x) exactly, .5 ties
    w = ops.Q4KWeight.from_ggml(w_np, cols, Q80)
    sums, _, y = ops.debug_block_sums(w, cu(x))
    q = orc.quantize_rows_q80(x, orc.Q80_X86)
    assert np.array_equal(sums.cpu().numpy(), orc.q80_matrix_block_sums(w_np, cols, q))
    y = y.cpu().numpy()
    assert np.all(y[1] == 0.0)
    mag = orc.q80_dot_dequant_f64(w_np, cols, q, magnitude=True)
    assert_fp32_parity(y, orc.mul_mat_q80_q80(w_np, cols, q, orc.ORDER_DOTPROD), mag, "q80 edge")
    w.free()


def test_q80_is_refused_where_it_is_not_supported(ops):
    from densecore_amd import _lib
    w = ops.Q4KWeight.from_ggml(synth.q80_matrix(83, 256, 256), 256, Q80)
    x = cu(synth.normal_f32(84, (1, 256)))
    with pytest.raises(_lib.MqError):
        ops.swiglu_mul_mat(w, w, x, 0)
    # an expert stack uploads (the MoE down node takes Q8_0 experts, core/src/llm/moe/native.cpp:4611-4616) and comes
    # back bit for bit, but the K-quant expert products refuse it
    stack_np = synth.q80_matrix(85, 32, 256).reshape(2, 16, -1)
    stack = ops.Q4KWeight.from_ggml(stack_np, 256, Q80)
    assert stack.n_experts == 2 and np.array_equal(stack.to_ggml(), stack_np)
    ids = cu(np.zeros((1, 1), np.int32))
    with pytest.raises(_lib.MqError):
        ops.mul_mat_id(stack, x[:, None, :], ids)
    stack.free()
    w.free()


@pytest.mark.parametrize("n", [1, 3, 9, 24, 100, 300])
def test_moe_layer_with_q80_down_experts_and_shared_expert(ops, n):
    """Q4_K gate/up experts with Q8_0 down experts (an accepted pairing, core/src/llm/moe/native.cpp:4611-4616) through
    the whole MoE layer, shared expert included (up to eight tokens a workgroup column per pair, above that the pairs
    grouped by expert, eight rows to a pass; at 300 tokens gate and up run on the expert-grouped matrix-core GEMM and
    hand their fp32 rows to the same Q8_0 launches): the layer must equal its own gate/up node followed by the Q8_0 down
    arithmetic of the reference (hidden row -> Q8_0 -> dot -> += value * weight in k order, :3239-3286) and the
    sigmoid-gated shared expert."""
    import torch
    hidden, inter, E, K = 512, 256, 10, 4
    ge, ue = (np.stack([synth.q4k_matrix(synth.tensor_seed("q80moe", t, e), inter, hidden) for e in range(E)]) for t in "gu")
    de = np.stack([synth.q80_matrix(synth.tensor_seed("q80moe", "d", e), hidden, inter) for e in range(E)])
    sg, su = (synth.q4k_matrix(synth.tensor_seed("q80moe-sh", t), inter, hidden) for t in "gu")
    sd = synth.q80_matrix(synth.tensor_seed("q80moe-sh", "d"), hidden, inter)
    gate_inp = synth.normal_f32(8601, (hidden,)) * 0.05
    x = synth.normal_f32(8600 + n, (n, hidden))
    lg = synth.normal_f32(8700 + n, (n, E))
    GE, UE = ops.Q4KWeight.from_ggml(ge, hidden), ops.Q4KWeight.from_ggml(ue, hidden)
    DE = ops.Q4KWeight.from_ggml(de, inter, Q80)
    SG, SU = ops.Q4KWeight.from_ggml(sg, hidden), ops.Q4KWeight.from_ggml(su, hidden)
    SD = ops.Q4KWeight.from_ggml(sd, inter, Q80)
    xd, lgd = cu(x), cu(lg)
    y, ids, wts = ops.moe_layer(GE, UE, DE, xd, lgd, K, shared=(SG, SU, SD, cu(gate_inp)), silu=0)
    ids_ref, w_ref = orc.route_topk(lg, K, 0)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    # the layer's hidden rows, re-made by the gate/up node and the dense gate/up product on the same inputs
    hid = ops.moe_gateup_swiglu(GE, UE, xd, ids, 0).cpu().numpy()
    hid_sh = ops.swiglu_mul_mat(SG, SU, xd, 2).cpu().numpy()
    w = wts.cpu().numpy()
    want = np.zeros((n, hidden), np.float32)
    for t in range(n):
        for k in range(K):
            q = orc.quantize_rows_q80(hid[t, k][None])
            want[t] += np.float32(w[t, k]) * orc.mul_mat_q80_q80(de[ids_ref[t, k]], inter, q)[0].astype(np.float32)
        q = orc.quantize_rows_q80(hid_sh[t][None])
        gate = np.float32(1.0) / (np.float32(1.0) + np.exp(-np.float32(np.dot(gate_inp.astype(np.float64), x[t].astype(np.float64)))))
        want[t] += np.float32(gate) * orc.mul_mat_q80_q80(sd, inter, q)[0].astype(np.float32)
    got = y.cpu().numpy()
    assert np.max(np.abs(got - want)) <= 2e-4 * np.max(np.abs(want))
    for h in (GE, UE, DE, SG, SU, SD):
        h.free()
