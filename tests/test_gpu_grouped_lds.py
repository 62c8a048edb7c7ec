"""The expert-grouped kernel that gathers a group's activation rows into LDS once per eight wavefronts against the
expert-grouped form of the kernel that reads its operand from global memory at every stage: the same bits through
every entry point that groups by expert, at shapes with enough groups for one-wave workgroups -- groups of one row
and of more than eight rows (a second pass over the same weights), the shared expert's groups, ragged row counts (a
workgroup whose last wavefronts have no row tile, through mul_mat_id), ids outside the expert range, Q5_K / Q6_K down experts, the fused
Q8_K of the gate/up output -- and, through the whole layer, against the oracle (tests/test_gpu_moe_full_size.py runs
with the gathering kernel as well, it is the default)."""
import numpy as np
import pytest

from densecore_amd import synth

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
    L.mq_debug_set_dense_lds(5)  # expert-grouped launches on the kernel with the operand in global memory
    want = [t.clone() for t in fn()]
    L.mq_debug_set_dense_lds(1)
    got = [t.clone() for t in fn()]
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in want], [t.cpu().numpy() for t in got]


def same_bits(want, got, what):
    for i, (a, b) in enumerate(zip(want, got)):
        assert a.shape == b.shape
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"{what}: output {i} differs"


def route(torch, n, n_exp, top_k, seed, skew=0.0):
    """ids [n, top_k] int32: top-k of seeded logits; skew > 0 pulls the tokens towards the first experts (large groups)."""
    logits = synth.normal_f32(seed, (n, n_exp))
    logits = logits - skew * np.arange(n_exp, dtype=np.float32)[None, :]
    ids = np.argsort(-logits, axis=1, kind="stable")[:, :top_k].astype(np.int32)
    return torch.from_numpy(logits).cuda(), torch.from_numpy(np.ascontiguousarray(ids)).cuda()


# hidden, inter, experts, top_k, tokens, skew: every case has more than 1024 (row tile, group) pairs in both launches
CASES = [
    (2048, 512, 256, 8, 16, 0.0),    # the benchmark's MoE block: mostly one-row groups
    (2048, 512, 256, 8, 64, 0.0),
    (2048, 512, 256, 8, 40, 0.5),    # skewed routing: groups of more than eight rows, a second pass
    (512, 256, 64, 8, 24, 0.0),      # short rows: two super-blocks per row in gate/up, one in down
    (1024, 256, 128, 4, 33, 0.2),
]


@pytest.mark.parametrize("hidden,inter,n_exp,top_k,n,skew", CASES)
def test_gate_up_and_down_same_bits(env, hidden, inter, n_exp, top_k, n, skew):
    torch, _lib, ops = env
    seed = synth.tensor_seed("gl", hidden, inter, n_exp, n)
    G = ops.Q4KWeight.synthetic(seed + 1, inter, hidden, n_exp)
    U = ops.Q4KWeight.synthetic(seed + 2, inter, hidden, n_exp)
    x = torch.from_numpy(synth.normal_f32(seed + 3, (n, hidden))).cuda()
    logits, ids = route(torch, n, n_exp, top_k, seed + 4, skew)
    for silu in (0, 2):
        want, got = both_ways(env, lambda: [ops.moe_gateup_swiglu(G, U, x, ids, silu)])
        same_bits(want, got, f"gate/up silu={silu}")
    hid = torch.from_numpy(synth.normal_f32(seed + 5, (n, top_k, inter))).cuda()
    wts = ops.moe_weights_from_logits(logits, ids)
    if inter % 256 == 0:
        for wtype in (12, 13, 14):
            D = ops.Q4KWeight.synthetic(seed + 6 + wtype, hidden, inter, n_exp, ggml_type=wtype)
            want, got = both_ways(env, lambda: [ops.moe_down_weighted(D, hid, ids, wts)])
            same_bits(want, got, f"down type {wtype}")


@pytest.mark.parametrize("n", [16, 48])
def test_invalid_ids_same_bits(env, n):
    """ids outside [0, n_experts) are dropped by the grouping; both kernels leave the same rows untouched."""
    torch, _lib, ops = env
    hidden, inter, n_exp, top_k = 1024, 512, 160, 8
    G = ops.Q4KWeight.synthetic(9101, inter, hidden, n_exp)
    U = ops.Q4KWeight.synthetic(9102, inter, hidden, n_exp)
    x = torch.from_numpy(synth.normal_f32(9103 + n, (n, hidden))).cuda()
    _, ids = route(torch, n, n_exp, top_k, 9104 + n)
    ids = ids.clone()
    ids[1, 3] = -1
    ids[n - 1, 0] = n_exp + 7

    def run():
        h = ops.moe_gateup_swiglu(G, U, x, ids, 2)
        keep = torch.ones((n, top_k), dtype=torch.bool, device="cuda")
        keep[1, 3] = False
        keep[n - 1, 0] = False
        return [torch.where(keep[:, :, None], h, torch.zeros_like(h))]  # dropped rows are never written: mask them
    want, got = both_ways(env, run)
    same_bits(want, got, "gate/up with dropped ids")


@pytest.mark.parametrize("n", [12, 16, 32, 64, 100])
def test_layer_with_shared_expert_same_bits(env, n):
    """mq_moe_layer_q4k: router + grouping, gate/up with the fused Q8_K of its output, down, combine, shared expert."""
    torch, _lib, ops = env
    hidden, inter, n_exp, top_k = 2048, 512, 256, 8
    G = ops.Q4KWeight.synthetic(9201, inter, hidden, n_exp)
    U = ops.Q4KWeight.synthetic(9202, inter, hidden, n_exp)
    D = ops.Q4KWeight.synthetic(9203, hidden, inter, n_exp)
    sh = (ops.Q4KWeight.synthetic(9204, inter, hidden), ops.Q4KWeight.synthetic(9205, inter, hidden),
          ops.Q4KWeight.synthetic(9206, hidden, inter), None)
    x = torch.from_numpy(synth.normal_f32(9207 + n, (n, hidden))).cuda()
    logits = torch.from_numpy(synth.normal_f32(9208 + n, (n, n_exp))).cuda()
    want, got = both_ways(env, lambda: list(ops.moe_layer(G, U, D, x, logits, top_k, shared=sh, silu=1))[:1])
    same_bits(want, got, "layer")


@pytest.mark.parametrize("cols,rows,n_exp,top_k,n", [(2048, 512, 256, 8, 24),
                                                     (1024, 304, 64, 8, 24)])  # 19 row tiles: wavefronts without one
@pytest.mark.parametrize("x_slots_full", [False, True])
def test_mul_mat_id_same_bits(env, x_slots_full, cols, rows, n_exp, top_k, n):
    torch, _lib, ops = env
    for wtype in (12, 13, 14):
        W = ops.Q4KWeight.synthetic(9300 + wtype, rows, cols, n_exp, ggml_type=wtype)
        shape = (n, top_k, cols) if x_slots_full else (n, cols)
        x = torch.from_numpy(synth.normal_f32(9310 + wtype, shape)).cuda()
        _, ids = route(torch, n, n_exp, top_k, 9320 + wtype)
        want, got = both_ways(env, lambda: [ops.mul_mat_id(W, x, ids)])
        same_bits(want, got, f"mul_mat_id type {wtype}")
