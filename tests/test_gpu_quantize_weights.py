"""GPU parity: Q8_K quantizer bytes and the weight re-tiling, through the C ABI."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def _q8_gpu(ops, x):
    import torch
    return ops.quantize_row_q8_k(torch.from_numpy(x).cuda()).cpu().numpy()


@pytest.mark.parametrize("n,k", [(1, 256), (1, 4096), (3, 2048), (16, 4096), (5, 14336), (64, 512)])
def test_q8k_bytes_identical_to_oracle(ops, n, k):
    x = synth.normal_f32(100 + n * 7 + k, (n, k))
    assert np.array_equal(_q8_gpu(ops, x), orc.quantize_rows_q8k(x))


def test_q8k_edge_blocks(ops):
    x = synth.normal_f32(7, (6, 1024)) * np.float32(250.0)
    x[0, :256] = 0.0                       # all-zero block -> d = 0, codes 0, bsums 0
    x[1, 300], x[1, 400] = 9.0, -9.0       # equal magnitudes in different lanes: the first wins
    x[1, 256:512] = np.where(np.abs(x[1, 256:512]) > 9, 0, x[1, 256:512])
    x[2, 513], x[2, 512] = -4.0, 4.0       # equal magnitudes inside one lane's four values
    x[2, 512:768] = np.clip(x[2, 512:768], -4, 4)
    x[3] = np.float32(1e-30)               # tiny values: iscale overflows nothing, codes saturate to -127
    x[4, ::2] = 0.5                        # exact .5 ties after scaling
    x[4, 1::2] = -1.0
    x[5] = np.arange(1024, dtype=np.float32) - 511.5
    got, want = _q8_gpu(ops, x), orc.quantize_rows_q8k(x)
    assert np.array_equal(got, want)
    assert not got[0, :292].any()


def test_q8k_large_magnitudes_and_denormals(ops):
    x = synth.normal_f32(8, (4, 512))
    x[0] *= np.float32(1e30)
    x[1] *= np.float32(1e-38)              # denormal-range inputs
    x[2, 5] = np.float32(3.0e38)
    got, want = _q8_gpu(ops, x), orc.quantize_rows_q8k(x)
    assert np.array_equal(got, want)


def test_q8k_rejects_bad_arguments(ops):
    import ctypes as C

    import torch
    from densecore_amd import _lib
    with pytest.raises(ValueError):
        ops.quantize_row_q8_k(torch.zeros((1, 255), device="cuda"))
    L = _lib.lib()
    x = torch.zeros((2, 512), device="cuda")
    out = torch.zeros((2, 2 * 292), dtype=torch.uint8, device="cuda")
    bad = [
        (x.data_ptr(), 2, 512, 300, out.data_ptr()),      # k not a multiple of 256
        (x.data_ptr(), 2, 128, 256, out.data_ptr()),      # ldx < k
        (x.data_ptr() + 4, 1, 256, 256, out.data_ptr()),  # activations not 16-byte aligned
        (0, 1, 256, 256, out.data_ptr()),                 # null input
        (x.data_ptr(), 1, 256, 256, 0),                   # null output
    ]
    for xp, n, ldx, k, op in bad:
        assert L.mq_quantize_q8k(C.c_void_p(xp), n, ldx, k, C.c_void_p(op), None) == -1
        assert L.mq_last_error()


@pytest.mark.parametrize("rows,cols,experts", [(16, 256, 1), (40, 1024, 1), (4096, 4096, 1), (48, 512, 5)])
def test_weight_upload_download_round_trip(ops, rows, cols, experts):
    raw = synth.q4k_matrix(300 + rows, rows * experts, cols).reshape(experts, rows, -1)
    w = ops.Q4KWeight.from_ggml(raw if experts > 1 else raw[0], cols)
    back = w.to_ggml()
    assert np.array_equal(back, raw if experts > 1 else raw[0])
    w.free()


@pytest.mark.parametrize("rows,cols,experts", [(32, 512, 1), (20, 256, 3), (512, 2048, 4)])
def test_synthetic_fill_matches_numpy_recipe(ops, rows, cols, experts):
    seed = synth.tensor_seed("fill", rows, cols, experts)
    w = ops.Q4KWeight.synthetic(seed, rows, cols, experts)
    want = synth.q4k_matrix(seed, rows * experts, cols).reshape(experts, rows, -1)
    got = w.to_ggml()
    assert np.array_equal(got if experts > 1 else got[None], want)
    w.free()
