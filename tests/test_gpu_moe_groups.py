"""The expert-grouped work list ("gather tokens by expert") read back from the device and compared entry for entry
with the reference's sorted assignments (Qwen35BuildMoEAssignments, core/src/llm/moe/native.cpp:1664-1733, restated
as orc.build_assignments and pinned against `sorted` in tests/test_oracle_pins.py): (expert, token, k) ascending,
ids outside [0, n_experts) dropped, an expert named twice by one token kept twice in k order."""
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


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("n,e,k", [(1, 256, 8), (2, 256, 8), (4, 256, 8), (9, 256, 8), (16, 256, 8), (64, 256, 8),
                                   (257, 256, 8), (300, 64, 4), (7, 60, 4), (40, 12, 4), (3, 8, 8), (1100, 128, 8),
                                   (512, 256, 8), (1024, 256, 8), (2048, 256, 8), (4096, 256, 8), (4100, 64, 8),
                                   (3000, 512, 8)])
def test_group_lists_from_ids_equal_sorted_assignments(ops, n, e, k):
    """launch_build_groups: the grouping of mq_mul_mat_id_q4k and of the two expert nodes (token masks while they fit
    the LDS of a compute unit -- 4096 tokens at 256 experts --, the scan of earlier pairs beyond; ids in LDS up to 8192
    pairs, in global memory above)."""
    ids, _ = orc.route_topk(synth.normal_f32(synth.tensor_seed("grp", n, e, k), (n, e)), k, 0)
    got = ops.debug_moe_groups(e, k, ids=cu(ids))
    assert np.array_equal(got, orc.build_assignments(ids, e))
    assert len(got) == n * k


@pytest.mark.parametrize("n,e,k", [(5, 16, 4), (33, 256, 8), (70, 12, 6), (300, 40, 8), (1500, 256, 8)])
def test_group_lists_with_invalid_and_repeated_ids(ops, n, e, k):
    rng = np.random.default_rng(n * 1000 + e)
    ids = rng.integers(0, e, size=(n, k)).astype(np.int32)       # repeats inside a token are likely
    ids[0, 0] = -1
    ids[n - 1, k - 1] = e
    ids[n // 2, 1] = e + 1000
    ids[1, :] = 3                                                # one token names expert 3 k times
    ids[2, 0] = ids[2, k - 1] = 5
    got = ops.debug_moe_groups(e, k, ids=cu(ids))
    want = orc.build_assignments(ids, e)
    assert np.array_equal(got, want)
    assert len(got) == int(((ids >= 0) & (ids < e)).sum())


@pytest.mark.parametrize("n,e,k", [(1, 256, 8), (2, 256, 8), (3, 256, 8), (12, 256, 8), (16, 256, 8), (64, 256, 8),
                                   (200, 256, 8), (17, 60, 4), (31, 1000, 6), (512, 256, 8), (1024, 256, 8), (2048, 256, 8)])
def test_route_and_group_in_one_launch(ops, n, e, k):
    """launch_route_and_group: the first launch of mq_moe_layer_q4k above eight tokens (one workgroup up to two
    tokens, a last-arriver handshake above); ties in the logits keep the lower expert first."""
    logits = synth.normal_f32(synth.tensor_seed("grp-l", n, e, k), (n, e))
    if n > 2:
        logits[1, 3] = logits[1, e - 1] = logits[1].max() + 1.0
        logits[2, :] = 0.25
    ids, _ = orc.route_topk(logits, k, 0)
    got = ops.debug_moe_groups(e, k, logits=cu(logits))
    assert np.array_equal(got, orc.build_assignments(ids, e))
