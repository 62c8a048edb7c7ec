"""The MoE layer at every token count from 1 to 72 and at a few prefill widths: whatever launches the width selects
(token-major kernels with the router inside, expert-grouped decode kernels, the expert-grouped matrix-core GEMM), token
i's routing (ids and weights, exactly) and output row depend on token i alone.  The output to 1e-4 of the largest
entry: the widths differ in the order a row's super-blocks are summed in, and a last-bit difference in a hidden row can
move one of its Q8_K codes by one before the down product.  Few experts (groups of dozens of rows), an odd expert count, the cfg3
shape, sibling weight types in the down stack, with and without the shared expert."""
import numpy as np
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu

# (experts, hidden, inter, top_k, shared expert, gate/up type, down type)
CASES = [
    (5, 512, 256, 2, False, 12, 12),
    (60, 1024, 512, 4, True, 12, 12),
    (257, 2048, 512, 8, True, 12, 12),
    (33, 1024, 256, 8, True, 12, 14),
    (64, 1024, 512, 6, False, 13, 13),
    (16, 512, 512, 3, True, 12, 8),
]


@pytest.mark.parametrize("E,H,I,K,shared,gu_type,down_type", CASES)
def test_token_i_of_the_moe_layer_depends_on_token_i_alone(E, H, I, K, shared, gu_type, down_type):
    import torch
    from densecore_amd import ops
    tag = ("mw", E, H, I, K)
    ge = ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "g"), I, H, E, ggml_type=gu_type)
    ue = ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "u"), I, H, E, ggml_type=gu_type)
    de = ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "d"), H, I, E, ggml_type=down_type)
    sh = None
    if shared:
        sh = (ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "sg"), I, H, ggml_type=gu_type),
              ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "su"), I, H, ggml_type=gu_type),
              ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "sd"), H, I, ggml_type=down_type),
              torch.from_numpy(synth.normal_f32(synth.tensor_seed(*tag, "gi"), (H,)) * np.float32(0.02)).cuda())
    N = 620
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed(*tag, "x"), (N, H))).cuda()
    lg = torch.from_numpy(synth.normal_f32(synth.tensor_seed(*tag, "l"), (N, E))).cuda()
    run = lambda a, b: ops.moe_layer(ge, ue, de, x[a:b], lg[a:b], K, shared=sh, silu=ops.SILU_FAST)
    ones = [run(i, i + 1) for i in range(72)]
    y1, id1, w1 = (torch.cat([o[j] for o in ones], dim=0) for j in range(3))
    scale = y1.abs().max().item()
    for n in list(range(1, 73)):
        y, ids, wts = run(0, n)
        assert torch.equal(ids, id1[:n]) and torch.equal(wts, w1[:n]), f"routing n={n}"
        assert (y - y1[:n]).abs().max().item() <= 1e-4 * scale, f"n={n}"
    for n in (130, 200, 300, N):   # prefill widths, stage by stage against the same tokens taken 50 at a time
        cuts = [(a, min(a + 50, n)) for a in range(0, n, 50)]
        y, ids, wts = run(0, n)
        parts = [run(a, b) for a, b in cuts]
        yp, idp, wp = (torch.cat([p[j] for p in parts], dim=0) for j in range(3))
        assert torch.equal(ids, idp) and torch.equal(wts, wp), f"routing n={n}"
        h = ops.moe_gateup_swiglu(ge, ue, x[:n], ids, ops.SILU_FAST)
        hp = torch.cat([ops.moe_gateup_swiglu(ge, ue, x[a:b], ids[a:b], ops.SILU_FAST) for a, b in cuts], dim=0)
        assert (h - hp).abs().max().item() <= 2e-6 * hp.abs().max().item(), f"hidden rows n={n}"
        d = ops.moe_down_weighted(de, hp, ids, wts)
        dp = torch.cat([ops.moe_down_weighted(de, hp[a:b], ids[a:b], wts[a:b]) for a, b in cuts], dim=0)
        assert (d - dp).abs().max().item() <= 2e-6 * dp.abs().max().item(), f"down product of the same hidden rows n={n}"
        # the whole layer: a last-bit difference in a hidden row can move one of its codes (or a block's scale) in the
        # quantizer of the down product, in a few tokens
        err = (y - yp).abs().max(dim=1).values / yp.abs().max().item()
        assert err.max().item() <= 5e-4 and (err > 2e-5).sum().item() <= max(2, n // 50), f"n={n}"
    for w in (ge, ue, de) + (tuple(sh[:3]) if sh else ()):
        w.free()


@pytest.mark.parametrize("E,H,I,K,wtype", [(40, 1024, 512, 4, 12), (7, 512, 256, 3, 12), (40, 1024, 512, 4, 13), (24, 512, 512, 8, 14)])
def test_expert_nodes_with_given_ids_at_every_width(E, H, I, K, wtype):
    """mul_mat_id, the gate/up node and the down node with ids handed in -- some outside [0, E) (zero rows, skipped
    terms), some repeated within a token -- at 1..72 tokens and at prefill widths: (token, slot) rows depend on their
    own token alone (to rounding: the launches of different widths split a row's super-blocks over wavefronts
    differently)."""
    import torch
    from densecore_amd import ops
    tag = ("mwi", E, H, I, K, wtype)
    ge = ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "g"), I, H, E, ggml_type=wtype)
    ue = ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "u"), I, H, E, ggml_type=wtype)
    de = ops.Q4KWeight.synthetic(synth.tensor_seed(*tag, "d"), H, I, E, ggml_type=wtype)
    N = 520
    rng = np.random.default_rng(synth.tensor_seed(*tag, "ids") % (1 << 32))
    ids_h = rng.integers(0, E, size=(N, K)).astype(np.int32)
    ids_h[rng.random((N, K)) < 0.06] = -1
    ids_h[rng.random((N, K)) < 0.03] = E + 3
    ids_h[5, :] = ids_h[5, 0]           # one expert in every slot of a token
    ids_h[9, :] = -1                    # a token with no valid slot
    ids = torch.from_numpy(ids_h).cuda()
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed(*tag, "x"), (N, H))).cuda()
    hid = torch.from_numpy(synth.normal_f32(synth.tensor_seed(*tag, "h"), (N, K, I))).cuda()
    wts = torch.from_numpy(np.abs(synth.normal_f32(synth.tensor_seed(*tag, "w"), (N, K)))).cuda()
    fns = {
        "mul_mat_id": lambda a, b: ops.mul_mat_id(ge, x[a:b], ids[a:b]),
        "mul_mat_id per slot": lambda a, b: ops.mul_mat_id(de, hid[a:b], ids[a:b]),
        "gate/up node": lambda a, b: ops.moe_gateup_swiglu(ge, ue, x[a:b], ids[a:b], ops.SILU_FAST),
        "down node": lambda a, b: ops.moe_down_weighted(de, hid[a:b], ids[a:b], wts[a:b]),
    }
    invalid = torch.from_numpy((ids_h < 0) | (ids_h >= E)).cuda()
    for name, fn in fns.items():
        one = torch.cat([fn(i, i + 1) for i in range(72)], dim=0)
        if one.dim() == 3:
            assert (one[invalid[:72]] == 0).all(), f"{name}: rows of invalid ids are zero"
        scale = one.abs().max().item()
        for n in range(1, 73):
            y = fn(0, n)
            assert (y - one[:n]).abs().max().item() <= 2e-6 * scale, f"{name} n={n}"
            if y.dim() == 3:
                assert (y[invalid[:n]] == 0).all(), f"{name} n={n}: rows of invalid ids are zero"
        for n in (200, 333, N):
            whole = fn(0, n)
            parts = torch.cat([fn(a, min(a + 40, n)) for a in range(0, n, 40)], dim=0)
            assert (whole - parts).abs().max().item() <= 2e-6 * parts.abs().max().item(), f"{name} n={n}"
            if whole.dim() == 3:
                assert (whole[invalid[:n]] == 0).all(), f"{name} n={n}: rows of invalid ids are zero"
    ge.free(), ue.free(), de.free()
