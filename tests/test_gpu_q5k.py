"""GPU parity: Q5_K weights (block_q4_K plus one high bit per weight) through the same entry points.

The reference multiplies Q5_K tensors with the Q4_K kernel's arithmetic and 5-bit codes
(core/src/kernels/hwy/hwy_moe_quant.cc:145-258); Q4_K_M model files use the type for many down
projections. Integer per-super-block sums must equal the oracle's bit for bit; fp32 within 1e-4 of both
fp32 orders the reference has for the type.
"""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu

Q5 = synth.GGML_TYPE_Q5_K
Q5_ORDERS = {"hwy": orc.ORDER_HWY, "per-block": orc.ORDER_DOTPROD}


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def q5_mag(w, cols, x):
    return orc.q5k_dot_dequant_f64(w, cols, orc.quantize_rows_q8k(x), magnitude=True)


@pytest.mark.parametrize("rows,cols,experts", [(16, 256, 1), (40, 1024, 1), (1000, 2048, 1), (48, 512, 5)])
def test_q5k_upload_download_round_trip_and_synthetic_fill(ops, rows, cols, experts):
    raw = synth.q5k_matrix(500 + rows, rows * experts, cols).reshape(experts, rows, -1)
    w = ops.Q4KWeight.from_ggml(raw if experts > 1 else raw[0], cols, Q5)
    assert w.ggml_type == Q5 and w.ggml_bytes == raw.size
    assert np.array_equal(w.to_ggml(), raw if experts > 1 else raw[0])
    w.free()
    seed = synth.tensor_seed("fill5", rows, cols, experts)
    s = ops.Q4KWeight.synthetic(seed, rows, cols, experts, Q5)
    want = synth.q5k_matrix(seed, rows * experts, cols).reshape(experts, rows, -1)
    got = s.to_ggml()
    assert np.array_equal(got if experts > 1 else got[None], want)
    s.free()


CASES = [(16, 256, 1), (40, 256, 3), (64, 1024, 1), (512, 2048, 4), (2048, 512, 8), (256, 4096, 16), (100, 768, 5),
         (48, 14336, 2), (4096, 4096, 1), (64, 1024, 17), (64, 1024, 33), (32, 512, 70)]


@pytest.mark.parametrize("rows,cols,n", CASES)
def test_q5k_matmul_integer_sums_exact_and_fp32_within_tolerance(ops, rows, cols, n):
    import torch
    w_np = synth.q5k_matrix(synth.tensor_seed("mm5-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("mm5-x", rows, cols, n), (n, cols))
    w = ops.Q4KWeight.from_ggml(w_np, cols, Q5)
    ds, md, y_dbg = ops.debug_block_sums(w, cu(x))
    y = ops.mul_mat(w, cu(x))
    torch.cuda.synchronize()
    w.free()
    q8 = orc.quantize_rows_q8k(x)
    ods, omd = orc.q5k_matrix_block_sums(w_np, cols, q8)
    assert np.array_equal(ds.cpu().numpy(), ods), "dot_scaled differs"
    assert np.array_equal(md.cpu().numpy(), omd), "min_dot differs"
    y = y.cpu().numpy()
    if n < 48:
        assert np.array_equal(y_dbg.cpu().numpy().view(np.uint32), y.view(np.uint32)), "debug and production kernels disagree"
    else:  # from 48 rows the product runs on the matrix-core GEMM: the same integers, another summation order
        assert np.max(np.abs(y_dbg.cpu().numpy() - y)) <= 1e-5 * np.max(np.abs(y))
    mag = orc.q5k_dot_dequant_f64(w_np, cols, q8, magnitude=True)
    for name, order in Q5_ORDERS.items():
        assert_fp32_parity(y, orc.mul_mat_q5k_q8k(w_np, cols, q8, order), mag, f"order={name}")


def test_q5k_with_zero_high_bits_is_bitwise_the_q4k_result(ops):
    rows, cols, n = 272, 2048, 5
    w4 = synth.q4k_matrix(61, rows, cols)
    x = synth.normal_f32(62, (n, cols))
    W4 = ops.Q4KWeight.from_ggml(w4, cols)
    W5 = ops.Q4KWeight.from_ggml(orc.q5k_from_q4k(w4), cols, Q5)
    y4, y5 = ops.mul_mat(W4, cu(x)).cpu().numpy(), ops.mul_mat(W5, cu(x)).cpu().numpy()
    assert np.array_equal(y4.view(np.uint32), y5.view(np.uint32))
    W4.free()
    W5.free()


def test_q5k_extreme_blocks_do_not_overflow(ops):
    """All scales and mins 63, all codes 31, activations at +-full scale: the int32 bounds of the format."""
    rows, cols = 16, 512
    w_np = np.zeros((rows, cols // 256 * 176), np.uint8)
    blocks = w_np.reshape(rows, -1, 176)
    blocks[:, :, 0:2] = np.array([0.01], np.float16).view(np.uint8)
    blocks[:, :, 2:4] = np.array([0.01], np.float16).view(np.uint8)
    blocks[:, :, 4:] = 0xFF
    x = np.full((2, cols), 3.0, np.float32)
    x[1, 0::256] = -3.0
    w = ops.Q4KWeight.from_ggml(w_np, cols, Q5)
    ds, md, _ = ops.debug_block_sums(w, cu(x))
    ds, md = ds.cpu().numpy(), md.cpu().numpy()
    w.free()
    assert np.all(ds[:, 0, :] == -8 * 63 * 32 * 31 * 127)
    assert np.all(ds[:, 1, :] == 8 * 63 * 32 * 31 * 127 - 2 * 63 * 31 * 127)
    assert np.all(md[:, 0, :] == -16 * 16 * 127 * 63)


@pytest.mark.parametrize("n", [1, 4, 16])
def test_ffn_with_q5k_down_projection(ops, n):
    H, I = 1024, 1792
    g, u = (synth.q4k_matrix(synth.tensor_seed("ffn5", nm), I, H) for nm in ("g", "u"))
    d = synth.q5k_matrix(synth.tensor_seed("ffn5", "d"), H, I)
    x = synth.normal_f32(synth.tensor_seed("ffn5-x", n), (n, H))
    G, U, D = ops.Q4KWeight.from_ggml(g, H), ops.Q4KWeight.from_ggml(u, H), ops.Q4KWeight.from_ggml(d, I, Q5)
    h_gpu = ops.swiglu_mul_mat(G, U, cu(x), 2).cpu().numpy()
    y_gpu = ops.ffn_swiglu(G, U, D, cu(x), 2).cpu().numpy()
    assert np.array_equal(y_gpu.view(np.uint32), ops.mul_mat(D, cu(h_gpu)).cpu().numpy().view(np.uint32))
    mag = q5_mag(d, I, h_gpu)
    for name, order in Q5_ORDERS.items():
        assert_fp32_parity(y_gpu, orc.mul_mat_q5k_f32(d, I, h_gpu, order), mag, f"ffn-down order={name}")
    # end to end: the oracle's own intermediate through the oracle's Q5_K product
    h_ref = orc.swiglu_mul_mat(g, u, H, I, x, orc.ORDER_DOTPROD, 2)
    y_ref = orc.mul_mat_q5k_f32(d, I, h_ref)
    assert np.max(np.abs(y_gpu - y_ref)) <= 2e-3 * np.max(np.abs(y_ref))
    for w in (G, U, D):
        w.free()


def test_ffn_all_q5k(ops):
    H, I, n = 512, 768, 3
    g, u, d = (synth.q5k_matrix(synth.tensor_seed("ffn55", nm), r, c) for nm, r, c in
               (("g", I, H), ("u", I, H), ("d", H, I)))
    x = synth.normal_f32(7, (n, H))
    G, U, D = (ops.Q4KWeight.from_ggml(m, c, Q5) for m, c in ((g, H), (u, H), (d, I)))
    h_gpu = ops.swiglu_mul_mat(G, U, cu(x), 0).cpu().numpy()
    gq, uq = orc.mul_mat_q5k_f32(g, H, x), orc.mul_mat_q5k_f32(u, H, x)
    want = np.array([[orc.lib().orc_silu_mul(float(a), float(b), 0) for a, b in zip(gr, ur)] for gr, ur in zip(gq, uq)],
                    np.float32)
    floor = 1e-5 * np.sqrt(np.mean(want.astype(np.float64) ** 2, axis=-1, keepdims=True))
    assert np.all(np.abs(h_gpu - want) <= 2e-4 * np.abs(want) + floor)
    y = ops.ffn_swiglu(G, U, D, cu(x), 0).cpu().numpy()
    assert np.array_equal(y.view(np.uint32), ops.mul_mat(D, cu(h_gpu)).cpu().numpy().view(np.uint32))
    for w in (G, U, D):
        w.free()


@pytest.mark.parametrize("n", [1, 4, 16, 40, 300])
def test_moe_with_q5k_down_experts(ops, n):
    """Routed layer with Q4_K gate/up and Q5_K down experts plus a shared expert of the same types (300 tokens: a
    hundred rows per expert, every product on the expert-grouped matrix-core GEMM, the Q5_K ones with its third chain)."""
    E, H, I, K = 12, 1024, 512, 4
    ge = np.stack([synth.q4k_matrix(synth.tensor_seed("moe5-g", e), I, H) for e in range(E)])
    ue = np.stack([synth.q4k_matrix(synth.tensor_seed("moe5-u", e), I, H) for e in range(E)])
    de = np.stack([synth.q5k_matrix(synth.tensor_seed("moe5-d", e), H, I) for e in range(E)])
    sg, su = (synth.q4k_matrix(synth.tensor_seed("moe5-sh", nm), I, H) for nm in ("g", "u"))
    sd = synth.q5k_matrix(synth.tensor_seed("moe5-sh", "d"), H, I)
    gate_inp = synth.normal_f32(synth.tensor_seed("moe5-gi"), (H,)) * np.float32(0.02)
    x = synth.normal_f32(synth.tensor_seed("moe5-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("moe5-l", n), (n, E))
    GE, UE, DE = ops.Q4KWeight.from_ggml(ge, H), ops.Q4KWeight.from_ggml(ue, H), ops.Q4KWeight.from_ggml(de, I, Q5)
    SG, SU, SD = ops.Q4KWeight.from_ggml(sg, H), ops.Q4KWeight.from_ggml(su, H), ops.Q4KWeight.from_ggml(sd, I, Q5)

    ids_t, w_t = ops.moe_route_topk(cu(logits), K, 0)
    ids, wts = ids_t.cpu().numpy(), w_t.cpu().numpy()
    hid = ops.moe_gateup_swiglu(GE, UE, cu(x), ids_t, 0).cpu().numpy()
    # down per (token, slot) through mul_mat_id, against the oracle's Q5_K product on the same rows
    yk = ops.mul_mat_id(DE, cu(hid), ids_t).cpu().numpy()
    want = np.zeros((n, H), np.float64)
    mag = np.zeros((n, H), np.float64)
    for t in range(n):
        for k in range(K):
            q8 = orc.quantize_rows_q8k(hid[t, k][None])
            ref = orc.mul_mat_q5k_q8k(de[ids[t, k]], I, q8)
            m = orc.q5k_dot_dequant_f64(de[ids[t, k]], I, q8, magnitude=True)
            assert_fp32_parity(yk[t, k][None], ref, m, f"t{t}k{k}")
            want[t] += np.float64(wts[t, k]) * ref[0]
            mag[t] += abs(wts[t, k]) * m[0]
    y_routed = ops.moe_down_weighted(DE, cu(hid), ids_t, w_t).cpu().numpy()
    assert_fp32_parity(y_routed, want, mag, "weighted down")
    y_nosh, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=None, silu=0)
    assert np.array_equal(y_nosh.cpu().numpy().view(np.uint32), y_routed.view(np.uint32))
    y, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=(SG, SU, SD, cu(gate_inp)), silu=0)
    sh_gpu = ops.ffn_swiglu(SG, SU, SD, cu(x), 2).cpu().numpy()
    gate = 1.0 / (1.0 + np.exp(-(x.astype(np.float64) @ gate_inp.astype(np.float64))))
    full = y_routed.astype(np.float64) + sh_gpu.astype(np.float64) * gate[:, None]
    rel = np.max(np.abs(y.cpu().numpy() - full), axis=1) / np.max(np.abs(full), axis=1)
    assert np.max(rel) <= 2e-3 and np.median(rel) <= (2e-6 if n < 256 else 2e-5)   # wide: the shared expert's sums in another order
    for w in (GE, UE, DE, SG, SU, SD):
        w.free()


def test_q5k_rejections(ops):
    import torch
    from densecore_amd._lib import MqError
    w5 = ops.Q4KWeight.from_ggml(synth.q5k_matrix(1, 64, 512), 512, Q5)
    w4 = ops.Q4KWeight.from_ggml(synth.q4k_matrix(1, 64, 512), 512)
    x = torch.zeros((64, 512), device="cuda")
    with pytest.raises(MqError):
        ops.swiglu_mul_mat(w4, w5, x[:2], 0)                            # gate and up of different types
    with pytest.raises(MqError):
        ops.Q4KWeight.from_ggml(np.zeros((4, 144), np.uint8), 256, Q5)  # a Q5_K row needs 176 bytes
    with pytest.raises(MqError):
        ops.Q4KWeight.from_ggml(np.zeros((4, 84), np.uint8), 256, 10)   # Q2_K is not handled
    w4.free()
    w5.free()


# ----------------------------------------------------------------------------- matrix-core GEMM (prefill widths)
@pytest.mark.parametrize("rows,cols,n", [(96, 768, 64), (80, 4096, 50), (272, 2048, 130)])
def test_q5k_gemm_matches_oracle_and_decode_kernel(ops, rows, cols, n):
    """Prefill widths of Q5_K: the int8 matrix-core GEMM with a third MFMA chain for the fifth code bits (the second
    shape splits K into runs).  Against the oracle, against 16-row passes of the decode kernel, and through mq_mul_mat_q4k."""
    import torch
    w_np = synth.q5k_matrix(synth.tensor_seed("pf5-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("pf5-x", rows, cols, n), (n, cols))
    W = ops.Q4KWeight.from_ggml(w_np, cols, Q5)
    got = ops.gemm(W, cu(x))
    small = torch.cat([ops.mul_mat(W, cu(x[i:i + 16])) for i in range(0, n, 16)])
    # (up to 64 rows mq_mul_mat_q4k keeps the decode arithmetic, up to four tiles of sixteen where the shape has them)
    assert torch.equal(ops.mul_mat(W, cu(x)), got if n > 64 else small) or torch.equal(ops.mul_mat(W, cu(x)), got)
    assert (got - small).abs().max().item() <= 1e-5 * small.abs().max().item()
    q8 = orc.quantize_rows_q8k(x)
    mag = orc.q5k_dot_dequant_f64(w_np, cols, q8, magnitude=True)
    assert_fp32_parity(got.cpu().numpy(), orc.mul_mat_q5k_q8k(w_np, cols, q8, orc.ORDER_DOTPROD), mag, "Q5_K GEMM")
    W.free()


def test_q5k_gemm_integer_sums_are_exact(ops):
    """d = dmin = 1 and integer activations with a +-127 in every block: the output equals the oracle's integers."""
    rows, cols, n = 48, 768, 70
    nb = cols // 256
    w = synth.q5k_matrix(synth.tensor_seed("pf5-int", rows), rows, cols).reshape(rows, nb, 176).copy()
    w[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w[:, :, 2:4] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w = w.reshape(rows, nb * 176)
    rng = np.random.default_rng(11)
    x = rng.integers(-127, 128, size=(n, cols)).astype(np.float32)
    x.reshape(n, nb, 256)[:, :, 7] = rng.choice([-127.0, 127.0], size=(n, nb))
    q8 = orc.quantize_rows_q8k(x)
    d, _, _ = orc.split_q8k(q8)
    assert np.all(np.abs(d) == 1.0)
    ds, md = orc.q5k_matrix_block_sums(w, cols, q8)
    want = ((ds.astype(np.int64) - md.astype(np.int64)) * d.astype(np.int64)[None]).sum(axis=2).T
    assert np.abs(want).max() < 2 ** 24
    W = ops.Q4KWeight.from_ggml(w, cols, Q5)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    assert np.array_equal(got, want.astype(np.float32))
    W.free()


def test_q5k_gemm_extreme_blocks(ops):
    """All codes 31, scales and mins 63, activations at +-full scale: the largest bytes of all three operand sets."""
    rows, cols, n = 32, 512, 48
    w_np = np.zeros((rows, cols // 256 * 176), np.uint8)
    blocks = w_np.reshape(rows, -1, 176)
    blocks[:, :, 0:2] = np.array([0.01], np.float16).view(np.uint8)
    blocks[:, :, 2:4] = np.array([0.005], np.float16).view(np.uint8)
    blocks[:, :, 4:] = 0xFF
    x = np.ones((n, cols), np.float32)
    x[1::2] *= -1.0
    x[2, ::2] *= -1.0
    W = ops.Q4KWeight.from_ggml(w_np, cols, Q5)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    q8 = orc.quantize_rows_q8k(x)
    assert_fp32_parity(got, orc.mul_mat_q5k_q8k(w_np, cols, q8, orc.ORDER_DOTPROD),
                       orc.q5k_dot_dequant_f64(w_np, cols, q8, magnitude=True), "Q5_K extremes")
    W.free()
