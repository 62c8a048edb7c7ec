"""GPU parity: Q6_K weights (210-byte blocks, signed per-16 scales, weight = d * scale * (code - 32)) through the
same entry points.

The reference's own Q6_K x Q8_K kernel is ComputeQ6KQ8KM4Native (core/src/llm/matmul/q6_small_batch.h:36-92).
The per-super-block integer sum_g scale_g * sum (code - 32) * q8 must equal the oracle's bit for bit; fp32 within
1e-4 of both fp32 orders the oracle restates for the type.
"""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu

Q6 = synth.GGML_TYPE_Q6_K
Q6_ORDERS = {"eight-lane": orc.ORDER_HWY, "per-block": orc.ORDER_DOTPROD}


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("rows,cols,experts", [(16, 256, 1), (40, 1024, 1), (1000, 2048, 1), (48, 512, 5)])
def test_q6k_upload_download_round_trip_and_synthetic_fill(ops, rows, cols, experts):
    raw = synth.q6k_matrix(600 + rows, rows * experts, cols).reshape(experts, rows, -1)
    w = ops.Q4KWeight.from_ggml(raw if experts > 1 else raw[0], cols, Q6)
    assert w.ggml_type == Q6 and w.ggml_bytes == raw.size
    assert np.array_equal(w.to_ggml(), raw if experts > 1 else raw[0])
    w.free()
    seed = synth.tensor_seed("fill6", rows, cols, experts)
    s = ops.Q4KWeight.synthetic(seed, rows, cols, experts, Q6)
    want = synth.q6k_matrix(seed, rows * experts, cols).reshape(experts, rows, -1)
    got = s.to_ggml()
    assert np.array_equal(got if experts > 1 else got[None], want)
    s.free()


CASES = [(16, 256, 1), (40, 256, 3), (64, 1024, 1), (512, 2048, 4), (2048, 512, 8), (256, 4096, 16), (100, 768, 5),
         (48, 14336, 2), (4096, 4096, 1), (64, 1024, 17), (32, 512, 70)]


@pytest.mark.parametrize("rows,cols,n", CASES)
def test_q6k_matmul_integer_sums_exact_and_fp32_within_tolerance(ops, rows, cols, n):
    import torch
    w_np = synth.q6k_matrix(synth.tensor_seed("mm6-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("mm6-x", rows, cols, n), (n, cols))
    w = ops.Q4KWeight.from_ggml(w_np, cols, Q6)
    ds, md, y_dbg = ops.debug_block_sums(w, cu(x))
    y = ops.mul_mat(w, cu(x))
    torch.cuda.synchronize()
    w.free()
    q8 = orc.quantize_rows_q8k(x)
    assert np.array_equal(ds.cpu().numpy(), orc.q6k_matrix_block_sums(w_np, cols, q8)), "block sums differ"
    assert not md.cpu().numpy().any()
    y = y.cpu().numpy()
    if n < 48:
        assert np.array_equal(y_dbg.cpu().numpy().view(np.uint32), y.view(np.uint32)), "debug and production kernels disagree"
    else:  # from 48 rows the product runs on the matrix-core GEMM: the same integers, another summation order
        assert np.max(np.abs(y_dbg.cpu().numpy() - y)) <= 1e-5 * np.max(np.abs(y))
    mag = orc.q6k_dot_dequant_f64(w_np, cols, q8, magnitude=True)
    for name, order in Q6_ORDERS.items():
        assert_fp32_parity(y, orc.mul_mat_q6k_q8k(w_np, cols, q8, order), mag, f"order={name}")


def test_q6k_extreme_blocks_do_not_overflow(ops):
    """Scales -128, codes 0 (weight -32) and 63, activations at +-full scale: the int32 bounds of the format."""
    rows, cols = 16, 512
    w_np = np.zeros((rows, cols // 256 * 210), np.uint8)
    blocks = w_np.reshape(rows, -1, 210)
    blocks[:, :, 192:208] = np.int8(-128).view(np.uint8)
    blocks[:, :, 208:210] = np.array([0.01], np.float16).view(np.uint8)
    blocks[8:, :, 0:192] = 0xFF                  # rows 8..15: every code 63
    x = np.full((2, cols), 3.0, np.float32)      # every activation code -127
    x[1, 0::256] = -3.0                          # first element decides the sign: all other codes +127
    w = ops.Q4KWeight.from_ggml(w_np, cols, Q6)
    ds, _, _ = ops.debug_block_sums(w, cu(x))
    ds = ds.cpu().numpy()
    w.free()
    assert np.all(ds[:8, 0, :] == -128 * 256 * (-32) * (-127))
    assert np.all(ds[8:, 0, :] == -128 * 256 * 31 * (-127))
    assert np.all(ds[:8, 1, :] == -128 * (255 * (-32) * 127 + (-32) * (-127)))
    assert np.array_equal(ds, orc.q6k_matrix_block_sums(w_np, cols, orc.quantize_rows_q8k(x)))


@pytest.mark.parametrize("n", [1, 4, 16])
def test_ffn_with_q6k_down_projection(ops, n):
    H, I = 1024, 1792
    g, u = (synth.q4k_matrix(synth.tensor_seed("ffn6", nm), I, H) for nm in ("g", "u"))
    d = synth.q6k_matrix(synth.tensor_seed("ffn6", "d"), H, I)
    x = synth.normal_f32(synth.tensor_seed("ffn6-x", n), (n, H))
    G, U, D = ops.Q4KWeight.from_ggml(g, H), ops.Q4KWeight.from_ggml(u, H), ops.Q4KWeight.from_ggml(d, I, Q6)
    h_gpu = ops.swiglu_mul_mat(G, U, cu(x), 2).cpu().numpy()
    y_gpu = ops.ffn_swiglu(G, U, D, cu(x), 2).cpu().numpy()
    assert np.array_equal(y_gpu.view(np.uint32), ops.mul_mat(D, cu(h_gpu)).cpu().numpy().view(np.uint32))
    q8 = orc.quantize_rows_q8k(h_gpu)
    mag = orc.q6k_dot_dequant_f64(d, I, q8, magnitude=True)
    for name, order in Q6_ORDERS.items():
        assert_fp32_parity(y_gpu, orc.mul_mat_q6k_q8k(d, I, q8, order), mag, f"ffn-down order={name}")
    for w in (G, U, D):
        w.free()


def test_swiglu_with_q6k_gate_and_up(ops):
    H, I, n = 512, 768, 3
    g, u = (synth.q6k_matrix(synth.tensor_seed("gu6", nm), I, H) for nm in ("g", "u"))
    x = synth.normal_f32(8, (n, H))
    G, U = ops.Q4KWeight.from_ggml(g, H, Q6), ops.Q4KWeight.from_ggml(u, H, Q6)
    h_gpu = ops.swiglu_mul_mat(G, U, cu(x), 0).cpu().numpy()
    gq, uq = orc.mul_mat_q6k_f32(g, H, x), orc.mul_mat_q6k_f32(u, H, x)
    want = np.array([[orc.lib().orc_silu_mul(float(a), float(b), 0) for a, b in zip(gr, ur)] for gr, ur in zip(gq, uq)],
                    np.float32)
    floor = 1e-5 * np.sqrt(np.mean(want.astype(np.float64) ** 2, axis=-1, keepdims=True))
    assert np.all(np.abs(h_gpu - want) <= 2e-4 * np.abs(want) + floor)
    G.free()
    U.free()


@pytest.mark.parametrize("n", [1, 4, 40])
def test_moe_with_q6k_down_experts(ops, n):
    E, H, I, K = 12, 1024, 512, 4
    ge = np.stack([synth.q4k_matrix(synth.tensor_seed("moe6-g", e), I, H) for e in range(E)])
    ue = np.stack([synth.q4k_matrix(synth.tensor_seed("moe6-u", e), I, H) for e in range(E)])
    de = np.stack([synth.q6k_matrix(synth.tensor_seed("moe6-d", e), H, I) for e in range(E)])
    x = synth.normal_f32(synth.tensor_seed("moe6-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("moe6-l", n), (n, E))
    GE, UE, DE = ops.Q4KWeight.from_ggml(ge, H), ops.Q4KWeight.from_ggml(ue, H), ops.Q4KWeight.from_ggml(de, I, Q6)
    ids_t, w_t = ops.moe_route_topk(cu(logits), K, 0)
    ids, wts = ids_t.cpu().numpy(), w_t.cpu().numpy()
    hid = ops.moe_gateup_swiglu(GE, UE, cu(x), ids_t, 0).cpu().numpy()
    yk = ops.mul_mat_id(DE, cu(hid), ids_t).cpu().numpy()
    want = np.zeros((n, H), np.float64)
    mag = np.zeros((n, H), np.float64)
    for t in range(n):
        for k in range(K):
            q8 = orc.quantize_rows_q8k(hid[t, k][None])
            ref = orc.mul_mat_q6k_q8k(de[ids[t, k]], I, q8)
            m = orc.q6k_dot_dequant_f64(de[ids[t, k]], I, q8, magnitude=True)
            assert_fp32_parity(yk[t, k][None], ref, m, f"t{t}k{k}")
            want[t] += np.float64(wts[t, k]) * ref[0]
            mag[t] += abs(wts[t, k]) * m[0]
    y_routed = ops.moe_down_weighted(DE, cu(hid), ids_t, w_t).cpu().numpy()
    assert_fp32_parity(y_routed, want, mag, "weighted down")
    y_layer, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=None, silu=0)
    assert np.array_equal(y_layer.cpu().numpy().view(np.uint32), y_routed.view(np.uint32))
    for w in (GE, UE, DE):
        w.free()


def test_q6k_rejections(ops):
    import torch
    from densecore_amd._lib import MqError
    w6 = ops.Q4KWeight.from_ggml(synth.q6k_matrix(1, 64, 512), 512, Q6)
    w8 = ops.Q4KWeight.from_ggml(synth.q80_matrix(1, 64, 512), 512, synth.GGML_TYPE_Q8_0)
    x = torch.zeros((64, 512), device="cuda")
    with pytest.raises(MqError):
        ops.gemm(w8, x)                                                 # the matrix-core GEMM takes the three K-quant types only
    w8.free()
    with pytest.raises(MqError):
        ops.Q4KWeight.from_ggml(np.zeros((4, 176), np.uint8), 256, Q6)  # a Q6_K row needs 210 bytes
    w6.free()


# ----------------------------------------------------------------------------- matrix-core GEMM (prefill widths)
@pytest.mark.parametrize("rows,cols,n", [(96, 768, 64), (80, 4096, 50), (272, 2048, 130), (1000, 1024, 300)])
def test_q6k_gemm_matches_oracle_and_decode_kernel(ops, rows, cols, n):
    """48 rows and more of Q6_K: the int8 matrix-core GEMM with both factors of scale * (code - 32) cut in two digits
    (five MFMA chains; the second shape splits K into runs, the last has a ragged last row tile).  Against the oracle,
    against 16-row passes of the decode kernel, and through mq_mul_mat_q4k."""
    import torch
    w_np = synth.q6k_matrix(synth.tensor_seed("pf6-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("pf6-x", rows, cols, n), (n, cols))
    W = ops.Q4KWeight.from_ggml(w_np, cols, Q6)
    got = ops.gemm(W, cu(x))
    assert torch.equal(ops.mul_mat(W, cu(x)), got)
    small = torch.cat([ops.mul_mat(W, cu(x[i:i + 16])) for i in range(0, n, 16)])
    assert (got - small).abs().max().item() <= 1e-5 * small.abs().max().item()
    q8 = orc.quantize_rows_q8k(x)
    mag = orc.q6k_dot_dequant_f64(w_np, cols, q8, magnitude=True)
    assert_fp32_parity(got.cpu().numpy(), orc.mul_mat_q6k_q8k(w_np, cols, q8, orc.ORDER_DOTPROD), mag, "Q6_K GEMM")
    W.free()


def test_q6k_gemm_integer_sums_are_exact(ops):
    """d = 1 and integer activations with a +-127 in every block: the output equals the sum of the oracle's integers,
    so one wrong unit in any of the five chains, in any digit of any scale or code, changes it."""
    rows, cols, n = 48, 768, 70
    nb = cols // 256
    w = synth.q6k_matrix(synth.tensor_seed("pf6-int", rows), rows, cols).reshape(rows, nb, 210).copy()
    w[:, :, 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w[1::2, :, 208:210] = np.frombuffer(np.float16(-1.0).tobytes(), np.uint8)
    w = w.reshape(rows, nb * 210)
    rng = np.random.default_rng(12)
    x = rng.integers(-7, 8, size=(n, cols)).astype(np.float32)
    x.reshape(n, nb, 256)[:, :, 9] = rng.choice([-127.0, 127.0], size=(n, nb))
    q8 = orc.quantize_rows_q8k(x)
    d, _, _ = orc.split_q8k(q8)
    assert np.all(np.abs(d) == 1.0)
    isum = orc.q6k_matrix_block_sums(w, cols, q8).astype(np.int64)            # [rows, n, nb]
    sign = np.where(np.arange(rows) % 2 == 0, 1, -1)[:, None, None]
    want = (isum * sign * d.astype(np.int64)[None]).sum(axis=2).T
    assert np.abs(isum).sum(axis=2).max() < 2 ** 24
    W = ops.Q4KWeight.from_ggml(w, cols, Q6)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    assert np.array_equal(got, want.astype(np.float32))
    W.free()


@pytest.mark.parametrize("scale,code", [(-128, 0), (-128, 63), (127, 0), (127, 63), (-1, 31), (15, 40), (16, 24), (-16, 7)])
def test_q6k_gemm_extreme_blocks(ops, scale, code):
    """One scale and one code everywhere -- the corners of both digit pairs (scale + 128 = 0, 255, 143, 144, 112;
    code = 0, 63 and both sides of the digit boundaries) -- with activations at +-full scale."""
    rows, cols, n = 32, 512, 48
    w_np = np.zeros((rows, cols // 256 * 210), np.uint8)
    blocks = w_np.reshape(rows, -1, 210)
    blocks[:, :, 0:128] = (code & 15) | ((code & 15) << 4)
    top = code >> 4
    blocks[:, :, 128:192] = top | (top << 2) | (top << 4) | (top << 6)
    blocks[:, :, 192:208] = np.int8(scale).view(np.uint8)
    blocks[:, :, 208:210] = np.array([0.01], np.float16).view(np.uint8)
    x = np.ones((n, cols), np.float32)
    x[1::2] *= -1.0
    x[2, ::2] *= -1.0
    W = ops.Q4KWeight.from_ggml(w_np, cols, Q6)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    q8 = orc.quantize_rows_q8k(x)
    assert_fp32_parity(got, orc.mul_mat_q6k_q8k(w_np, cols, q8, orc.ORDER_DOTPROD),
                       orc.q6k_dot_dequant_f64(w_np, cols, q8, magnitude=True), "Q6_K extremes")
    W.free()
