"""The routers inside the MoE launches -- in the token-major gate/up launch up to eight tokens, a token per
wavefront of the routing + grouping launch up to 64, a workgroup per token beyond: the ids and weights that
mq_moe_layer_q4k hands back against the oracle's stable top-k (core/src/llm/moe/native.cpp:610-676, :800-868) on rows
made to hit every branch of the one-pass selection: plain rows, a few candidates, ties at the top (lower id first),
ties that run across the cut, long runs of equal logits (more than 64 candidates: the round-by-round way), rows
of one value, NaN and infinities, and expert counts that leave lanes or whole groups of lanes without an expert."""
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


def rows_for(e, n, seed):
    logits = synth.normal_f32(seed, (n, e))
    kinds = ["plain", "top tie", "cut tie", "long run", "all equal", "nan", "inf", "descending"]
    for r in range(n):
        kind = kinds[(r + seed) % len(kinds)]
        row = logits[r]
        if kind == "top tie":
            row[[e - 1, 3, e // 2]] = row.max() + 1.0
        elif kind == "cut tie":          # ranks 6..13 share one value: the cut at eight goes through the run
            order = np.argsort(-row, kind="stable")
            row[order[6:14]] = row[order[6]]
        elif kind == "long run":         # min(e, 100) experts share the largest value: more candidates than lanes
            row[: min(e, 100)] = row.max() + 2.0
        elif kind == "all equal":
            row[:] = -0.25
        elif kind == "nan":
            row[::3] = np.nan
            row[1] = np.inf
        elif kind == "inf":
            row[:] = -np.inf
            row[e - 2] = 1.0
        elif kind == "descending":
            row[:] = -np.arange(e, dtype=np.float32)
    return logits


@pytest.mark.parametrize("e", [8, 40, 64, 100, 160, 256, 384, 512])
@pytest.mark.parametrize("n", [1, 3, 8, 16, 40, 64, 70])
def test_ids_and_weights_from_the_token_major_launch(ops, e, n):
    import torch
    hidden, inter, top_k = 256, 256, 8
    G = ops.Q4KWeight.synthetic(7001, inter, hidden, e)
    U = ops.Q4KWeight.synthetic(7002, inter, hidden, e)
    D = ops.Q4KWeight.synthetic(7003, hidden, inter, e)
    x = torch.from_numpy(synth.normal_f32(7004 + n, (n, hidden))).cuda()
    for seed in range(3):
        logits = rows_for(e, n, seed * 3 + e)
        for mode in (0, 1, 2):
            _, ids, w = ops.moe_layer(G, U, D, x, torch.from_numpy(logits).cuda(), top_k, route_mode=mode)
            oi, ow = orc.route_topk(logits, top_k, mode)
            assert np.array_equal(ids.cpu().numpy(), oi), f"ids: experts {e}, tokens {n}, seed {seed}, mode {mode}"
            assert np.allclose(w.cpu().numpy(), ow, rtol=3e-6, atol=1e-9, equal_nan=True), f"weights: mode {mode}"
