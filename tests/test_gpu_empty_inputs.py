"""Zero activation rows: every product entry point accepts them and does nothing (the reference's callbacks
return without touching dst when a tensor has no rows, core/src/llm/matmul/gemv_exec.cpp:102-143)."""
import numpy as np
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu


def test_zero_rows_through_every_entry_point():
    import torch
    from densecore_amd import ops
    H, I, E, K = 512, 256, 8, 2
    W = ops.Q4KWeight.from_ggml(synth.q4k_matrix(1, 64, H), H)
    G, U, D = (ops.Q4KWeight.synthetic(s, r, c) for s, r, c in ((2, I, H), (3, I, H), (4, H, I)))
    GE, UE, DE = (ops.Q4KWeight.synthetic(s, r, c, E) for s, r, c in ((5, I, H), (6, I, H), (7, H, I)))
    x = torch.zeros((0, H), device="cuda")
    assert ops.mul_mat(W, x).shape == (0, 64)
    assert ops.gemm(W, x).shape == (0, 64)
    assert ops.quantize_row_q8_k(x).shape[0] == 0
    assert ops.swiglu_mul_mat(G, U, x, 0).shape == (0, I)
    assert ops.ffn_swiglu(G, U, D, x, 2).shape == (0, H)
    ids = torch.zeros((0, K), dtype=torch.int32, device="cuda")
    logits = torch.zeros((0, E), device="cuda")
    i2, w2 = ops.moe_route_topk(logits, K, 0)
    assert i2.shape == (0, K) and w2.shape == (0, K)
    assert ops.mul_mat_id(GE, x, ids).shape == (0, K, I)
    assert ops.moe_gateup_swiglu(GE, UE, x, ids, 0).shape == (0, K, I)
    y, _, _ = ops.moe_layer(GE, UE, DE, x, logits, K, shared=None, silu=0)
    assert y.shape == (0, H)
    torch.cuda.synchronize()
    # and the library still works afterwards
    x1 = torch.from_numpy(synth.normal_f32(9, (1, H))).cuda()
    assert torch.isfinite(ops.mul_mat(W, x1)).all()
    for w in (W, G, U, D, GE, UE, DE):
        w.free()
