"""The MoE block at the benchmark's shape (hidden 2048, 256 experts + 1 shared, intermediate 512, top-8) at the
token-major widths, two to eight tokens, where the launches change shape with the token count: gate/up with a
workgroup per (token, slot, row tile) or, when a row takes one wavefront, per (token, row tile) with a wavefront per
slot and x quantized once per workgroup; down with one, two or four row tiles of a token per workgroup and the
hidden rows quantized once per workgroup.

Hidden rows and output against the CPU restatement (fp32 tolerance of tests/test_gpu_ffn_moe.py), ids exact; and the
down launch of n tokens bit-equal to n single-token launches (one row tile per workgroup, every wavefront quantizing
for itself): the same terms in the same order, for Q4_K / Q5_K / Q6_K experts, with ids out of range and zero
weights among them."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests.test_gpu_ffn_moe import END_TO_END_REL, assert_close_prod

pytestmark = pytest.mark.gpu

E, H, I, K = 256, 2048, 512, 8


@pytest.fixture(scope="module")
def layer():
    import torch
    from densecore_amd import ops
    assert torch.cuda.is_available()
    dev = [ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", nm), r, c, E) for nm, r, c in
           (("g", I, H), ("u", I, H), ("d", H, I))]
    sh = [ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3-sh", nm), r, c) for nm, r, c in
          (("g", I, H), ("u", I, H), ("d", H, I))]
    host = [w.to_ggml() for w in dev]
    sh_host = [w.to_ggml() for w in sh]
    gate_inp = synth.normal_f32(synth.tensor_seed("cfg3-gi"), (H,)) * np.float32(0.02)
    yield ops, dev, sh, host, sh_host, gate_inp
    for w in dev + sh:
        w.free()


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("n,silu", [(2, 0), (3, 1), (4, 0), (5, 2), (6, 0), (7, 1), (8, 0)])
def test_layer_against_the_cpu_layer(layer, n, silu):
    ops, (GE, UE, DE), (SG, SU, SD), (ge, ue, de), (sg, su, sd), gate_inp = layer
    x = synth.normal_f32(synth.tensor_seed("tm-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("tm-l", n), (n, E))
    y, ids, wts = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=(SG, SU, SD, cu(gate_inp)), silu=silu)
    oi, ow = orc.route_topk(logits, K, 0)
    assert np.array_equal(ids.cpu().numpy(), oi)
    assert np.allclose(wts.cpu().numpy(), ow, rtol=3e-6)
    hid = ops.debug_moe_hidden((n, K + 1, I)).cpu().numpy()
    assert_close_prod(hid[:, :K], orc.moe_gateup_swiglu(ge, ue, H, I, x, oi, orc.ORDER_DOTPROD, silu), "gate/up")
    assert_close_prod(hid[:, K], orc.swiglu_mul_mat(sg, su, H, I, x, orc.ORDER_DOTPROD, 2), "shared gate/up")
    ref = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=(sg, su, sd, gate_inp), silu=silu)
    y = y.cpu().numpy()
    rel = np.max(np.abs(y - ref["y"]), axis=1) / np.max(np.abs(ref["y"]), axis=1)
    assert np.max(rel) <= END_TO_END_REL and np.median(rel) <= 2e-5, (np.max(rel), np.median(rel))


@pytest.mark.parametrize("wtype", [12, 13, 14])
@pytest.mark.parametrize("n", [3, 4, 5, 8])
def test_down_of_n_tokens_is_n_single_token_launches(layer, n, wtype):
    import torch
    ops = layer[0]
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("tm-d", wtype), H, I, 32, ggml_type=wtype)
    hid = torch.from_numpy(synth.normal_f32(synth.tensor_seed("tm-h", n, wtype), (n, K, I))).cuda()
    logits = synth.normal_f32(synth.tensor_seed("tm-dl", n), (n, 32))
    ids_np, w_np = orc.route_topk(logits, K, 0)
    ids_np, w_np = ids_np.copy(), w_np.copy()
    ids_np[0, 2] = -1          # dropped: below the range
    ids_np[n - 1, 7] = 32 + 5  # dropped: above it
    w_np[1, 0] = 0.0           # skipped: zero weight
    ids, wts = torch.from_numpy(ids_np).cuda(), torch.from_numpy(w_np).cuda()
    together = ops.moe_down_weighted(D, hid, ids, wts).cpu().numpy()
    for t in range(n):
        alone = ops.moe_down_weighted(D, hid[t:t + 1].contiguous(), ids[t:t + 1].contiguous(), wts[t:t + 1].contiguous()).cpu().numpy()
        assert np.array_equal(together[t].view(np.uint32), alone[0].view(np.uint32)), f"token {t}"
    D.free()
