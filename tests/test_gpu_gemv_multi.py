"""GPU parity: several single-row products of one activation row in one launch (mq_mul_mat_q4k_multi), through the C ABI.

Every output must carry the bits of mq_mul_mat_q4k on its matrix alone (whose integer sums are checked against the
oracle in test_gpu_matmul.py) and sit within 1e-4 of every fp32 accumulation order the reference has.
"""
import ctypes as C

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


MAKE = {synth.GGML_TYPE_Q4_K: synth.q4k_matrix, synth.GGML_TYPE_Q5_K: synth.q5k_matrix, synth.GGML_TYPE_Q6_K: synth.q6k_matrix}

# (rows of each matrix), cols, types (None: all Q4_K)
CASES = [
    ((4096, 1024, 1024), 4096, None),            # q, k, v of a grouped-query layer: one launch
    ((512, 512), 2048, None),                    # gate and up of an expert-sized FFN
    ((40,), 256, None),                          # a single ragged matrix
    ((16, 100, 4096, 33, 48, 2048, 64, 17), 1024, None),   # the most the list takes, ragged row counts
    ((6144, 64), 4096, None),                    # different wave splits: a launch each
    ((256, 256, 256), 14336, None),              # rows too long for the single-row kernel: one by one
    ((512, 512, 512), 2048, (synth.GGML_TYPE_Q4_K, synth.GGML_TYPE_Q6_K, synth.GGML_TYPE_Q5_K)),  # other types go one by one
]


@pytest.mark.parametrize("rows_list,cols,types", CASES)
def test_multi_equals_one_call_per_matrix_and_the_oracle(ops, rows_list, cols, types):
    import torch
    types = types or (synth.GGML_TYPE_Q4_K,) * len(rows_list)
    w_np = [MAKE[t](synth.tensor_seed("multi-w", i, r, cols, t), r, cols) for i, (r, t) in enumerate(zip(rows_list, types))]
    ws = [ops.Q4KWeight.from_ggml(m, cols, t) for m, t in zip(w_np, types)]
    x = synth.normal_f32(synth.tensor_seed("multi-x", cols, len(rows_list)), (1, cols))
    xd = torch.from_numpy(x).cuda()
    ys = [y.cpu().numpy() for y in ops.mul_mat_multi(ws, xd)]
    singles = [ops.mul_mat(w, xd).cpu().numpy()[0] for w in ws]
    q8 = orc.quantize_rows_q8k(x)
    for i, (y, one) in enumerate(zip(ys, singles)):
        assert np.array_equal(y.view(np.uint32), one.view(np.uint32)), f"matrix {i}: bits differ from a launch of its own"
        if types[i] == synth.GGML_TYPE_Q4_K:
            mag = orc.dot_magnitude_f64(w_np[i], cols, q8)
            for name, ref in oracle_all_orders(w_np[i], cols, q8).items():
                assert_fp32_parity(y[None], ref, mag, f"matrix {i}, order={name}")
    for w in ws:
        w.free()


def test_multi_in_a_graph_replays_the_same_bits(ops):
    import torch
    cols = 2048
    ws = [ops.Q4KWeight.synthetic(synth.tensor_seed("multi-g", i), r, cols) for i, r in enumerate((2048, 512, 512))]
    xd = torch.from_numpy(synth.normal_f32(synth.tensor_seed("multi-gx"), (1, cols))).cuda()
    outs = [torch.zeros((w.rows,), dtype=torch.float32, device="cuda") for w in ws]
    eager = [y.clone() for y in ops.mul_mat_multi(ws, xd, outs)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        ops.mul_mat_multi(ws, xd, outs)
    for _ in range(3):
        for o in outs:
            o.fill_(7.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for o, e in zip(outs, eager):
            assert torch.equal(o, e)
    for w in ws:
        w.free()


def test_multi_rejects_bad_lists(ops):
    import torch
    from densecore_amd import _lib
    L = _lib.lib()
    a = ops.Q4KWeight.synthetic(1, 64, 1024)
    b = ops.Q4KWeight.synthetic(2, 64, 2048)
    e = ops.Q4KWeight.synthetic(3, 64, 1024, 4)
    x = torch.zeros((2048,), dtype=torch.float32, device="cuda")
    y = [torch.zeros((64,), dtype=torch.float32, device="cuda") for _ in range(9)]
    vp = C.c_void_p

    def call(ws, ys, count=None, xp=None):
        wl = (vp * max(len(ws), 1))(*[w._h if w is not None else None for w in ws])
        yl = (vp * max(len(ys), 1))(*[t.data_ptr() if t is not None else None for t in ys])
        return L.mq_mul_mat_q4k_multi(wl, len(ws) if count is None else count, vp(x.data_ptr()) if xp is None else xp, yl, None)

    assert call([], [], 0) == 0                      # an empty list is a no-op, as an empty product is
    assert call([a] * 9, y[:9]) != 0                 # more than eight
    assert call([a], y[:1], -1) != 0
    assert call([a, b], y[:2]) != 0                  # column counts differ
    assert call([a, e], y[:2]) != 0                  # an expert stack
    assert call([a, None], y[:2]) != 0
    assert call([a, a], [y[0], None]) != 0
    assert call([a], y[:1], xp=vp(0)) != 0
    assert b"mq_mul_mat_q4k_multi" in L.mq_last_error()
    assert call([a, a], y[:2]) == 0
    torch.cuda.synchronize()
    for w in (a, b, e):
        w.free()
