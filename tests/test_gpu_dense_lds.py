"""The dense kernel that stages the quantized activations in LDS (and quantizes up to four fp32 rows itself) against
the kernel that reads its operand from global memory at every stage: the same bits for every shape, row count and
weight type both take, incl. ragged row counts (a workgroup whose last row tiles do not exist), rows that fill the
160 KB of LDS, two token tiles, strided fp32 rows -- and, through the whole FFN, against the oracle."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    from densecore_amd import _lib, ops
    assert torch.cuda.is_available()
    yield torch, _lib, ops
    _lib.lib().mq_debug_set_dense_lds(1)


def both_ways(env, fn):
    torch, _lib, ops = env
    L = _lib.lib()
    L.mq_debug_set_dense_lds(0)
    want = fn().clone()
    L.mq_debug_set_dense_lds(1)
    got = fn().clone()
    torch.cuda.synchronize()
    return want.cpu().numpy(), got.cpu().numpy()


SHAPES = [(14336, 4096), (4096, 4096), (2048, 2048), (2560, 2048), (100, 512), (48, 8192), (64, 9216), (16, 256),
          (1000, 1024)]


@pytest.mark.parametrize("wtype", [12, 13, 14])
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_single_matrix_same_bits(env, rows, cols, wtype):
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("dl", wtype, rows, cols), rows, cols, ggml_type=wtype)
    for n in (1, 2, 3, 4, 5, 8, 9, 16):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("dl-x", rows, cols, n), (n, cols))).cuda()
        want, got = both_ways(env, lambda: ops.mul_mat(W, x))
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), f"n={n}"


@pytest.mark.parametrize("wtype", [12, 13, 14])
@pytest.mark.parametrize("rows,cols", [(14336, 4096), (512, 2048), (72, 1024), (304, 4096)])
@pytest.mark.parametrize("silu", [0, 1, 2])
def test_gate_up_same_bits(env, rows, cols, wtype, silu):
    torch, _lib, ops = env
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("dl-g", wtype, rows, cols), rows, cols, ggml_type=wtype)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("dl-u", wtype, rows, cols), rows, cols, ggml_type=wtype)
    for n in (1, 2, 4, 7, 8, 12, 16):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("dl-gx", rows, cols, n), (n, cols))).cuda()
        want, got = both_ways(env, lambda: ops.swiglu_mul_mat(G, U, x, silu))
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), f"n={n}"


def test_strided_rows(env):
    """fp32 rows with a stride longer than the row (the in-kernel quantizer reads them in place)."""
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(7, 640, 1024)
    for n in (2, 3, 4):
        buf = torch.from_numpy(synth.normal_f32(70 + n, (n, 1024 + 64))).cuda()
        x = buf[:, :1024]
        assert x.stride(0) == 1088

        def raw():  # ops.mul_mat would copy the rows together first
            y = torch.empty((n, W.rows), dtype=torch.float32, device="cuda")
            _lib.check(_lib.lib().mq_mul_mat_q4k(W._h, x.data_ptr(), n, x.stride(0), y.data_ptr(), W.rows, None), "mq_mul_mat_q4k")
            return y
        want, got = both_ways(env, raw)
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
        ref = ops.mul_mat(W, x.contiguous()).cpu().numpy()
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 8, 16])
def test_ffn_same_bits_and_oracle(env, n):
    """The whole FFN at the benchmark's shape: same bits both ways, and within the path's bound of the oracle."""
    torch, _lib, ops = env
    H, I = 4096, 14336
    g, u, d = (synth.q4k_matrix(synth.tensor_seed("dl-ffn", t), r, c) for t, r, c in (("g", I, H), ("u", I, H), ("d", H, I)))
    G, U, D = ops.Q4KWeight.from_ggml(g, H), ops.Q4KWeight.from_ggml(u, H), ops.Q4KWeight.from_ggml(d, I)
    x = synth.normal_f32(synth.tensor_seed("dl-ffn-x", n), (n, H))
    xd = torch.from_numpy(x).cuda()
    want, got = both_ways(env, lambda: ops.ffn_swiglu(G, U, D, xd, 2))
    assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    if n <= 2:  # the scalar oracle takes a few seconds per row at this size
        ref = orc.ffn_swiglu(g, u, d, H, I, x, orc.ORDER_DOTPROD, 2)
        assert np.max(np.abs(got - ref)) <= 2e-3 * np.max(np.abs(ref))
