"""Weights filled the way the reference's own micro-benchmark fills them (core/tests/benchmarks/q4_down_rowpair.cpp:38-58):
every byte of a block random, d and dmin SIGNED in [-1, 1] in steps of 1/1024 (zero included), rows padded to a longer
stride, Q8_K rows with arbitrary scales and codes down to -128 -- plus d / dmin drawn from all finite fp16 bit
patterns (subnormals, 65504, both zeros).  The benchmark configuration's d, dmin in +[0.001, 0.01] never reach
these cases.  Through the dense, the expert-grouped and the matrix-core kernels."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def reference_filler(seed, rows, cols, wide=False):
    """[rows, nb*144] Q4_K rows: random bytes, then d / dmin as the reference's filler draws them, or (wide) any
    finite fp16 bit pattern of magnitude up to 2048."""
    rng = np.random.default_rng(seed)
    nb = cols // 256
    w = rng.integers(0, 256, size=(rows, nb, 144), dtype=np.uint8)
    if wide:
        bits = rng.integers(0, 0x6800, size=(rows, nb, 2)).astype(np.uint16)      # 0 .. 2048, subnormals included
        bits |= (rng.integers(0, 2, size=(rows, nb, 2)).astype(np.uint16) << 15)  # either sign, -0 too
        w[:, :, 0:4] = bits.view(np.uint8).reshape(rows, nb, 4)
    else:
        dd = ((rng.integers(0, 2049, size=(rows, nb, 2)) - 1024) / 1024.0).astype(np.float16)
        w[:, :, 0:4] = dd.view(np.uint8).reshape(rows, nb, 4)
    return w.reshape(rows, nb * 144)


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("rows,cols,n", [(64, 512, 1), (96, 2048, 1), (2048, 2048, 3), (48, 14336, 1), (256, 4096, 8),
                                         (80, 2304, 16), (64, 1024, 64)])
def test_dense_and_gemm_with_signed_scales(ops, rows, cols, n, wide):
    w = reference_filler(rows * 31 + n, rows, cols, wide)
    x = synth.normal_f32(synth.tensor_seed("sg-x", rows, cols, n), (n, cols))
    W = ops.Q4KWeight.from_ggml(w, cols)
    q8 = orc.quantize_rows_q8k(x)
    ds, md, _ = ops.debug_block_sums(W, cu(x))
    ods, omd = orc.matrix_block_sums(w, cols, q8)
    assert np.array_equal(ds.cpu().numpy(), ods) and np.array_equal(md.cpu().numpy(), omd)
    mag = orc.dot_magnitude_f64(w, cols, q8)
    # scales spread over fourteen binades leave the four fp32 orders of the reference up to 2e-4 of the summed term
    # magnitudes apart from EACH OTHER (the scalar order rounds after every sub-block); there the outputs are held to
    # the value itself (the dequantized double-precision dot) and to the per-block order the kernels follow
    refs = {name: orc.mul_mat_q4k_q8k(w, cols, q8, order) for name, order in orc.ORDERS.items() if not wide or name == "dotprod"}
    refs["dequantized double"] = orc.dot_dequant_f64(w, cols, q8)
    for what, y in (("decode", ops.mul_mat(W, cu(x))), ("matrix-core", ops.gemm(W, cu(x)))):
        for name, ref in refs.items():
            assert_fp32_parity(y.cpu().numpy(), ref, mag, f"{what} order={name}")
    W.free()


@pytest.mark.parametrize("pad", [16, 64])
def test_padded_row_stride_and_foreign_q8k_rows(ops, pad):
    """Row starts `row_bytes` apart with padding after the blocks (q4_down_rowpair.cpp:59-63), and Q8_K rows that no
    quantizer wrote: any scale, codes over the whole int8 range."""
    rows, cols, n = 64, 768, 5
    nb = cols // 256
    w = reference_filler(pad, rows, cols)
    padded = np.full((rows, nb * 144 + pad), 0xA5, np.uint8)
    padded[:, :nb * 144] = w
    W = ops.Q4KWeight.from_ggml(padded, cols)
    assert np.array_equal(W.to_ggml(), w)
    rng = np.random.default_rng(pad)
    q8 = np.zeros((n, nb, 292), np.uint8)
    q8[:, :, 0:4] = ((rng.integers(0, 2049, size=(n, nb)) - 1024) / 1024.0).astype(np.float32).view(np.uint8).reshape(n, nb, 4)
    codes = rng.integers(-128, 128, size=(n, nb, 256)).astype(np.int8)
    q8[:, :, 4:260] = codes.view(np.uint8)
    q8[:, :, 260:292] = codes.reshape(n, nb, 16, 16).sum(axis=3).astype(np.int16).view(np.uint8).reshape(n, nb, 32)
    q8 = q8.reshape(n, nb * 292)
    y = ops.mul_mat_q8k(W, cu(q8)).cpu().numpy()
    mag = orc.dot_magnitude_f64(w, cols, q8)
    for name, order in orc.ORDERS.items():
        assert_fp32_parity(y, orc.mul_mat_q4k_q8k(w, cols, q8, order), mag, f"order={name}")
    W.free()


@pytest.mark.parametrize("n", [1, 6, 20])
def test_expert_nodes_with_signed_scales(ops, n):
    E, H, I, K = 10, 1024, 512, 4
    ge = np.stack([reference_filler(100 + e, I, H, e % 2 == 1) for e in range(E)])
    de = np.stack([reference_filler(200 + e, H, I, e % 2 == 0) for e in range(E)])
    GE, DE = ops.Q4KWeight.from_ggml(ge, H), ops.Q4KWeight.from_ggml(de, I)
    ids, wts = orc.route_topk(synth.normal_f32(synth.tensor_seed("sg-l", n), (n, E)), K, 0)
    x = synth.normal_f32(synth.tensor_seed("sg-xe", n), (n, H))
    y = ops.mul_mat_id(GE, cu(x), cu(ids)).cpu().numpy()
    for t in range(n):
        q8 = orc.quantize_rows_q8k(x[t:t + 1])
        for k in range(K):
            e = ids[t, k]
            assert_fp32_parity(y[t, k][None], orc.mul_mat_q4k_q8k(ge[e], H, q8), orc.dot_magnitude_f64(ge[e], H, q8), f"t{t} k{k}")
    hid = synth.normal_f32(synth.tensor_seed("sg-h", n), (n, K, I))
    yd = ops.moe_down_weighted(DE, cu(hid), cu(ids), cu(wts)).cpu().numpy()
    mag = np.zeros((n, H))
    for t in range(n):
        for k in range(K):
            mag[t] += abs(wts[t, k]) * orc.dot_magnitude_f64(de[ids[t, k]], I, orc.quantize_rows_q8k(hid[t, k][None]))[0]
    assert_fp32_parity(yd, orc.moe_down_weighted(de, H, I, hid, ids, wts, orc.ORDER_DOTPROD, 0), mag, "down node")
    GE.free(), DE.free()
