"""GPU parity: Q4_K x Q8_K matmul at decode widths, through the C ABI.

Integer per-super-block sums (dot_scaled, min_dot) must equal the oracle's bit for bit; fp32
outputs must sit within 1e-4 of every fp32 accumulation order the reference has.
"""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity, oracle_all_orders

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def _run(ops, w_np, cols, x):
    import torch
    w = ops.Q4KWeight.from_ggml(w_np, cols)
    ds, md, y = ops.debug_block_sums(w, torch.from_numpy(x).cuda())
    y2 = ops.mul_mat(w, torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    w.free()
    return ds.cpu().numpy(), md.cpu().numpy(), y.cpu().numpy(), y2.cpu().numpy()


CASES = [
    # rows, cols, n
    (16, 256, 1), (40, 256, 3), (64, 1024, 1), (512, 2048, 4), (2048, 512, 8), (256, 4096, 16),
    (100, 768, 5), (48, 14336, 2), (4096, 4096, 1),
    (64, 1024, 17), (64, 1024, 33), (32, 512, 64), (32, 512, 70),
]


@pytest.mark.parametrize("rows,cols,n", CASES)
def test_matmul_integer_sums_exact_and_fp32_within_tolerance(ops, rows, cols, n):
    w = synth.q4k_matrix(synth.tensor_seed("mm-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("mm-x", rows, cols, n), (n, cols))
    ds, md, y_dbg, y = _run(ops, w, cols, x)
    q8 = orc.quantize_rows_q8k(x)
    ods, omd = orc.matrix_block_sums(w, cols, q8)
    assert np.array_equal(ds, ods), "dot_scaled differs"
    assert np.array_equal(md, omd), "min_dot differs"
    if n < 48:
        assert np.array_equal(y_dbg.view(np.uint32), y.view(np.uint32)), "debug and production kernels disagree"
    else:   # from 48 rows up mq_mul_mat_q4k runs the matrix-core GEMM, whose fp32 update uses fused multiply-adds
        assert np.abs(y_dbg - y).max() <= 1e-5 * np.abs(y).max(), "decode and GEMM kernels disagree"
    mag = orc.dot_magnitude_f64(w, cols, q8)
    for name, ref in oracle_all_orders(w, cols, q8).items():
        assert_fp32_parity(y, ref, mag, f"order={name}")


@pytest.mark.parametrize("gtype", [synth.GGML_TYPE_Q4_K, synth.GGML_TYPE_Q5_K, synth.GGML_TYPE_Q6_K])
@pytest.mark.parametrize("rows,cols", [(17, 2304), (100, 5120), (1000, 14336), (4097, 4608), (48, 28672)])
def test_single_row_with_quantizer_inside_equals_the_two_launches(ops, rows, cols, gtype):
    """One activation row against long weight rows runs with the quantizer inside the decode kernel and without
    the lane's second activation row: the bits of quantize followed by the product from Q8_K rows, and the debug
    launch (the two-row arithmetic) too; ragged row counts take the several-row-tiles-per-workgroup path."""
    import torch
    make = {synth.GGML_TYPE_Q4_K: synth.q4k_matrix, synth.GGML_TYPE_Q5_K: synth.q5k_matrix, synth.GGML_TYPE_Q6_K: synth.q6k_matrix}[gtype]
    w_np = make(synth.tensor_seed("xq-w", rows, cols, gtype), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("xq-x", rows, cols), (1, cols))
    w = ops.Q4KWeight.from_ggml(w_np, cols, gtype)
    xd = torch.from_numpy(x).cuda()
    y = ops.mul_mat(w, xd).cpu().numpy()
    y_two = ops.mul_mat_q8k(w, ops.quantize_row_q8_k(xd)).cpu().numpy()
    _, _, y_dbg = ops.debug_block_sums(w, xd)
    assert np.array_equal(y.view(np.uint32), y_two.view(np.uint32))
    assert np.array_equal(y.view(np.uint32), y_dbg.cpu().numpy().view(np.uint32))
    w.free()


def test_matmul_zero_and_constant_activations(ops):
    rows, cols = 64, 1024
    w = synth.q4k_matrix(5, rows, cols)
    x = np.zeros((3, cols), np.float32)
    x[1] = 1.0
    x[2, :256] = -2.5
    ds, md, _, y = _run(ops, w, cols, x)
    q8 = orc.quantize_rows_q8k(x)
    ods, omd = orc.matrix_block_sums(w, cols, q8)
    assert np.array_equal(ds, ods) and np.array_equal(md, omd)
    assert not y[0].any()
    ref = orc.mul_mat_q4k_q8k(w, cols, q8, orc.ORDER_DOTPROD)
    assert_fp32_parity(y, ref, orc.dot_magnitude_f64(w, cols, q8) + 1e-30, "const")


def test_matmul_extreme_blocks_do_not_overflow(ops):
    """All scales/mins 63, all quants 15, activations at +-full scale: the int32 bounds of the format."""
    rows, cols = 16, 512
    w = np.zeros((rows, cols // 256 * 144), np.uint8)
    blocks = w.reshape(rows, -1, 144)
    blocks[:, :, 0:2] = np.array([0.01], np.float16).view(np.uint8)
    blocks[:, :, 2:4] = np.array([0.01], np.float16).view(np.uint8)
    blocks[:, :, 4:] = 0xFF
    x = np.full((2, cols), 3.0, np.float32)   # every code -127 (the extreme element maps to -127)
    x[1, 0::256] = -3.0                        # first element decides the sign: all other codes +127
    ds, md, _, y = _run(ops, w, cols, x)
    assert np.all(ds[:, 0, :] == -8 * 63 * 32 * 15 * 127)
    assert np.all(ds[:, 1, :] == 8 * 63 * 32 * 15 * 127 - 2 * 63 * 15 * 127)
    assert np.all(md[:, 0, :] == -16 * 16 * 127 * 63)
    q8 = orc.quantize_rows_q8k(x)
    ods, omd = orc.matrix_block_sums(w, cols, q8)
    assert np.array_equal(ds, ods) and np.array_equal(md, omd)


def test_matmul_with_external_q8k_rows_and_host_entry(ops):
    import torch
    rows, cols, n = 96, 2048, 6
    w_np = synth.q4k_matrix(9, rows, cols)
    x = synth.normal_f32(10, (n, cols))
    w = ops.Q4KWeight.from_ggml(w_np, cols)
    q8 = orc.quantize_rows_q8k(x)
    y_q8 = ops.mul_mat_q8k(w, torch.from_numpy(q8).cuda()).cpu().numpy()
    y_f32 = ops.mul_mat(w, torch.from_numpy(x).cuda()).cpu().numpy()
    y_host = ops.mul_mat_host(w, x)
    assert np.array_equal(y_q8.view(np.uint32), y_f32.view(np.uint32))
    assert np.array_equal(y_host.view(np.uint32), y_f32.view(np.uint32))
    w.free()


def test_matmul_rejects_bad_arguments(ops):
    import torch
    from densecore_amd._lib import MqError
    w = ops.Q4KWeight.from_ggml(synth.q4k_matrix(1, 16, 256), 256)
    with pytest.raises(MqError):
        ops.mul_mat(w, torch.zeros((1, 128), device="cuda"))            # fewer columns than the weight has
    with pytest.raises(MqError):
        ops.Q4KWeight.from_ggml(np.zeros((4, 100), np.uint8), 256)      # row shorter than one block
    with pytest.raises(MqError):
        ops.Q4KWeight.from_ggml(np.zeros((4, 144), np.uint8), 255)      # cols not a multiple of 256
    w.free()


def test_matmul_is_deterministic(ops):
    import torch
    rows, cols, n = 512, 4096, 4
    w = ops.Q4KWeight.synthetic(77, rows, cols)
    x = torch.from_numpy(synth.normal_f32(78, (n, cols))).cuda()
    a = ops.mul_mat(w, x).cpu().numpy()
    for _ in range(3):
        assert np.array_equal(ops.mul_mat(w, x).cpu().numpy().view(np.uint32), a.view(np.uint32))
    w.free()


def test_shared_activation_handle_matches_the_one_shot_entry_points():
    """mq_acts_*: quantize once, then mq_mul_mat_q4k_acts / mq_swiglu_mul_mat_q4k_acts must equal
    mq_mul_mat_q4k / mq_swiglu_mul_mat_q4k bit for bit (same kernels, same quantized rows)."""
    import torch
    from densecore_amd import ops
    rows, cols = 768, 1024
    g = ops.Q4KWeight.synthetic(501, rows, cols)
    u = ops.Q4KWeight.synthetic(502, rows, cols)
    acts = ops.Q8KActs(16, cols)
    for n in (16, 3):       # the second, smaller batch reuses the handle
        x = torch.from_numpy(synth.normal_f32(503 + n, (n, cols))).cuda()
        acts.quantize(x)
        assert torch.equal(acts.mul_mat(g), ops.mul_mat(g, x))
        assert torch.equal(acts.swiglu_mul_mat(g, u, 1), ops.swiglu_mul_mat(g, u, x, 1))
    with pytest.raises(Exception):
        acts.quantize(torch.zeros((17, cols), device="cuda"))
    acts.free(), g.free(), u.free()
