"""The MoE block at the benchmark's own shape -- hidden 2048, 256 experts + 1 shared, expert intermediate 512,
top-8 -- above eight tokens, where the expert-grouped gate/up launch lets a one-wavefront workgroup take two or
four row tiles and counts 16 / 2 or 16 / 4 arrivals per 256-row block for the fused Q8_K of its output
(widths 12..64 take two row tiles, 72 -- and 64 with the shared expert's groups added -- four).

Stage by stage against the CPU restatement with the GPU's own intermediate fed forward (a Q8_K re-quantization sits
between the stages; see tests/test_gpu_ffn_moe.py), the one-call layer bit-equal to its stages, and end to end."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity
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


@pytest.mark.parametrize("n,silu", [(12, 1), (16, 1), (32, 1), (64, 1), (72, 2), (9, 0)])
def test_cfg3_layer_stagewise(layer, n, silu):
    ops, (GE, UE, DE), (SG, SU, SD), (ge, ue, de), (sg, su, sd), gate_inp = layer
    x = synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E))
    ids_t, w_t = ops.moe_route_topk(cu(logits), K, 0)
    ids, wts = ids_t.cpu().numpy(), w_t.cpu().numpy()
    oi, ow = orc.route_topk(logits, K, 0)
    assert np.array_equal(ids, oi) and np.allclose(wts, ow, rtol=3e-6)

    # stage 1: expert-grouped gate/up + SwiGLU (several row tiles per workgroup at these widths)
    hid = ops.moe_gateup_swiglu(GE, UE, cu(x), ids_t, silu).cpu().numpy()
    assert_close_prod(hid, orc.moe_gateup_swiglu(ge, ue, H, I, x, ids, orc.ORDER_DOTPROD, silu), "gate/up")

    # stage 2: expert-grouped down + combine on the GPU's own hidden rows and weights
    y_routed = ops.moe_down_weighted(DE, cu(hid), ids_t, w_t).cpu().numpy()
    mag = np.zeros((n, H))
    hq = orc.quantize_rows_q8k(hid.reshape(n * K, I)).reshape(n, K, -1)
    for t in range(n):
        for k in range(K):
            mag[t] += abs(wts[t, k]) * orc.dot_magnitude_f64(de[ids[t, k]], I, hq[t, k][None])[0]
    assert_fp32_parity(y_routed, orc.moe_down_weighted(de, H, I, hid, ids, wts, orc.ORDER_DOTPROD, 0), mag, "down")

    # the one-call layer without the shared expert: the same bits as its stages (its gate/up leaves the hidden rows
    # in Q8_K through the arrival counters, its hidden rows are the stage's)
    y_nosh, ids2, w2 = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=None, silu=silu)
    assert np.array_equal(ids2.cpu().numpy(), ids) and np.array_equal(w2.cpu().numpy().view(np.uint32), wts.view(np.uint32))
    assert np.array_equal(ops.debug_moe_hidden((n, K, I)).cpu().numpy().view(np.uint32), hid.view(np.uint32))
    assert np.array_equal(y_nosh.cpu().numpy().view(np.uint32), y_routed.view(np.uint32))

    # with the shared expert (more groups in both launches): hidden rows of the routed slots unchanged, the shared
    # slot against the dense SwiGLU of the same matrices, the output end to end against the CPU layer
    y, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=(SG, SU, SD, cu(gate_inp)), silu=silu)
    hid_sh = ops.debug_moe_hidden((n, K + 1, I)).cpu().numpy()
    assert np.array_equal(hid_sh[:, :K].view(np.uint32), hid.view(np.uint32))
    assert_close_prod(hid_sh[:, K], orc.swiglu_mul_mat(sg, su, H, I, x, orc.ORDER_DOTPROD, 2), "shared gate/up")
    ref = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=(sg, su, sd, gate_inp), silu=silu)
    y = y.cpu().numpy()
    rel = np.max(np.abs(y - ref["y"]), axis=1) / np.max(np.abs(ref["y"]), axis=1)
    assert np.max(rel) <= END_TO_END_REL and np.median(rel) <= 2e-5, (np.max(rel), np.median(rel))


@pytest.mark.parametrize("n", [400, 1024])
def test_cfg3_layer_at_prefill_widths_on_the_grouped_gemm(layer, n):
    """The full-size block (256 + 1 experts, 2048 x 512, top-8) at widths where the expert products run on the
    matrix-core GEMM in its expert-grouped form: routing bit for bit; the routed part against the decode kernels' own
    stages on the same ids (other summation order, see below); a sample of tokens end to end against
    the CPU layer, which depends on those tokens' own rows only."""
    import torch
    ops, (GE, UE, DE), (SG, SU, SD), (ge, ue, de), (sg, su, sd), gate_inp = layer
    x = synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E))
    oi, ow = orc.route_topk(logits, K, 0)
    y_nosh, ids, w = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=None, silu=1)
    assert np.array_equal(ids.cpu().numpy(), oi) and np.allclose(w.cpu().numpy(), ow, rtol=3e-6)
    # the decode kernels' stages on the same ids, in chunks of 128 tokens (below the width where the nodes switch to
    # the GEMM themselves).  The hidden rows are re-quantized to Q8_K for the down product: a last-bit difference
    # between the two paths' SwiGLU rows can move a code by one step, so single tokens differ at the end-to-end
    # tolerance, most by far less
    xs, parts = cu(x), []
    for i in range(0, n, 128):
        hid = ops.moe_gateup_swiglu(GE, UE, xs[i:i + 128], ids[i:i + 128], 1)
        parts.append(ops.moe_down_weighted(DE, hid, ids[i:i + 128], w[i:i + 128]))
    y_stage = torch.cat(parts)
    rel = ((y_nosh - y_stage).abs() / y_stage.abs().max(dim=1, keepdim=True).values).max(dim=1).values
    assert rel.max().item() <= END_TO_END_REL and rel.median().item() <= 2e-5, (rel.max().item(), rel.median().item())
    # and the nodes at the full width (the GEMM): bit for bit the layer
    hid = ops.moe_gateup_swiglu(GE, UE, xs, ids, 1)
    assert torch.equal(ops.moe_down_weighted(DE, hid, ids, w), y_nosh)
    y, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=(SG, SU, SD, cu(gate_inp)), silu=1)
    pick = np.unique(np.concatenate([np.arange(0, n, max(1, n // 6)), [n - 1]]))
    ref = orc.moe_layer(ge, ue, de, H, I, K, x[pick], logits[pick], shared=(sg, su, sd, gate_inp), silu=1)
    got = y.cpu().numpy()[pick]
    rel = np.max(np.abs(got - ref["y"]), axis=1) / np.max(np.abs(ref["y"]), axis=1)
    assert np.max(rel) <= END_TO_END_REL, np.max(rel)


def test_prefill_width_paths_replay_from_a_graph(layer):
    """The MoE block on the expert-grouped GEMM and the wide dense FFN, captured once and replayed several times with
    eager work of the same entries in between: every replay returns the eager bits."""
    import torch
    ops, (GE, UE, DE), (SG, SU, SD), _, _, gate_inp = layer
    n = 512
    x = cu(synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H)))
    logits = cu(synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E)))
    sh = (SG, SU, SD, cu(gate_inp))
    y_eager, ids_eager, _ = ops.moe_layer(GE, UE, DE, x, logits, K, shared=sh, silu=1)
    f_eager = ops.ffn_swiglu(SG, SU, SD, x, 2)
    y_eager, f_eager, ids_eager = y_eager.clone(), f_eager.clone(), ids_eager.clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        y_g, ids_g, _ = ops.moe_layer(GE, UE, DE, x, logits, K, shared=sh, silu=1)
        f_g = ops.ffn_swiglu(SG, SU, SD, x, 2)
    for rep in range(4):
        y_g.zero_(), f_g.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_eager) and torch.equal(f_g, f_eager) and torch.equal(ids_g, ids_eager), f"replay {rep}"
        # eager work of other widths through the same workspaces between the replays
        ops.moe_layer(GE, UE, DE, x[:64], logits[:64], K, shared=sh, silu=1)
        ops.ffn_swiglu(SG, SU, SD, x[:100], 2)
        torch.cuda.synchronize()
