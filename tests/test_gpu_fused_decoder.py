"""mq_decoder_step (a run of decoder layers as one persistent launch) against the node-by-node entry points.

The fused kernel keeps the arithmetic and the summation orders of the kernels it replaces and always splits a
row's super-blocks over eight wavefronts.  Where the node-by-node kernels split the same way (one token at the
full-size shape, every width at the small shapes) its outputs equal those of DecodeStep -- which
tests/test_gpu_decode_step.py checks against the CPU restatement -- bit for bit: residual stream, routed experts,
routing weights of every layer.  Where they split K over fewer wavefronts (wider steps at the full-size shape)
only the fp32 summation order differs: same experts, outputs within the end-to-end bound of a MoE layer, and
a direct comparison with the CPU restatement.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ds():
    import torch
    from densecore_amd import decode_step
    assert torch.cuda.is_available()
    return decode_step


def _pair(ds, cfg, n, seed, fixed=False):
    import torch
    cfg.synthetic_logits = fixed
    step = ds.DecodeStep(cfg, n)
    fused = ds.FusedDecodeStep(cfg, n, step.layers, step.fixed_logits)
    x = torch.randn((n, cfg.hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(seed))
    return step, fused, x


END_TO_END_REL = 2e-3   # a 1-ulp difference before a re-quantization can flip a Q8_K code


def _assert_same(step, fused, x, exact=True):
    import torch
    want = step.run(x).clone()
    got = fused.run(x).clone()
    fused.status()
    assert torch.equal(fused.ids, step.ids), "routed experts differ"
    assert torch.isfinite(got).all()
    if exact:
        assert torch.equal(fused.wts, step.wts), "routing weights differ"
        assert torch.equal(got, want), f"max |diff| {(got - want).abs().max().item():.3e}"
    else:
        assert torch.allclose(fused.wts, step.wts, rtol=1e-4, atol=1e-7), "routing weights differ"
        rel = ((got - want).abs().amax(dim=1) / want.abs().amax(dim=1)).max().item()
        assert rel <= END_TO_END_REL, f"relative difference {rel:.3e}"


@pytest.mark.parametrize("n", [1, 3, 4, 8])
@pytest.mark.parametrize("n_layers", [1, 4])
def test_small_layers_bitwise_equal_to_node_by_node(ds, n, n_layers):
    cfg = ds.StepConfig(n_layers=n_layers, hidden=512, n_experts=16, inter=256, top_k=4, n_q=512, n_kv=128, seed=7)
    step, fused, x = _pair(ds, cfg, n, 100 + n)
    _assert_same(step, fused, x)
    fused.free()
    step.free()


def test_no_shared_expert_and_wide_inter(ds):
    cfg = ds.StepConfig(n_layers=2, hidden=1024, n_experts=24, inter=768, top_k=8, n_q=768, n_kv=256,
                        shared_expert=False, seed=8)
    step, fused, x = _pair(ds, cfg, 2, 21)
    _assert_same(step, fused, x)
    fused.free()
    step.free()


@pytest.mark.parametrize("n,fixed", [(1, False), (1, True), (4, False), (8, True)])
def test_full_size_layers_bitwise_equal(ds, n, fixed):
    """hidden 2048, 256 experts + shared, inter 512, top-8, 16 query / 2 KV heads of 128: three layers."""
    cfg = ds.StepConfig(n_layers=3, seed=11)
    step, fused, x = _pair(ds, cfg, n, 5 + n, fixed)
    # the fused kernel adds a row tile's super-blocks in the order of the node-by-node gate/up launch of this width
    _assert_same(step, fused, x)
    fused.free()
    step.free()


@pytest.mark.parametrize("n", [1, 4])
def test_full_size_layer_against_cpu_restatement(ds, n):
    import torch
    from oracle import decode_step as ref_step
    from tests.test_gpu_decode_step import close, host_weights
    cfg = ds.StepConfig(n_layers=1, seed=12)
    step, fused, x = _pair(ds, cfg, n, 40 + n)
    out = fused.run(x).cpu().numpy()
    fused.status()
    r = ref_step.layer_forward(host_weights(step.layers[0]), x.cpu().numpy(), None, cfg, step.silu_mode())
    assert np.array_equal(fused.ids[0].cpu().numpy(), r["ids"])
    close(fused.wts[0].cpu().numpy(), r["weights"], 1e-5, "routing weights")
    close(out, r["x"] + r["y"], END_TO_END_REL, "layer output")
    fused.free()
    step.free()


def test_graph_replays_and_repeated_steps(ds):
    import torch
    cfg = ds.StepConfig(n_layers=4, hidden=512, n_experts=16, inter=256, top_k=4, n_q=512, n_kv=128, seed=9)
    step, fused, x = _pair(ds, cfg, 4, 77)
    want = step.run(x).clone()
    fused.x.copy_(x)
    fused.capture()
    for rep in range(3):
        fused.x.copy_(x)
        got = fused.replay().clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {rep}"
        assert torch.equal(fused.run(x), want)   # eager launches between the replays
        torch.cuda.synchronize()
    x2 = x * 0.5 + 1.0
    assert torch.equal(fused.run(x2), step.run(x2))
    fused.status()
    fused.free()
    step.free()


def test_abandoned_barrier_is_reported_and_the_handle_recovers(ds):
    """With no patience every workgroup that has to wait gives up at its first barrier: the launch drains by
    itself, the status call reports it, and the next step is right again."""
    import torch
    from densecore_amd import _lib
    cfg = ds.StepConfig(n_layers=2, hidden=512, n_experts=16, inter=256, top_k=4, n_q=512, n_kv=128, seed=13)
    step, fused, x = _pair(ds, cfg, 2, 55)
    want = step.run(x).clone()
    assert torch.equal(fused.run(x), want)
    fused.status()
    _lib.check(_lib.lib().mq_decoder_set_patience(fused._h, 0), "mq_decoder_set_patience")
    fused.run(x)
    with pytest.raises(_lib.MqError):
        fused.status()
    _lib.check(_lib.lib().mq_decoder_set_patience(fused._h, 200000), "mq_decoder_set_patience")
    assert torch.equal(fused.run(x), want)
    fused.status()
    fused.free()
    step.free()


def test_rejections(ds):
    import torch
    from densecore_amd import _lib, ops, synth
    cfg = ds.StepConfig(n_layers=1, hidden=512, n_experts=16, inter=256, top_k=4, n_q=512, n_kv=128, seed=3)
    step = ds.DecodeStep(cfg, 2)
    with pytest.raises(_lib.MqError):
        ds.FusedDecodeStep(cfg, 9, step.layers)                      # more than 8 tokens per step
    fused = ds.FusedDecodeStep(cfg, 2, step.layers)
    x = torch.zeros((4, cfg.hidden), device="cuda")
    with pytest.raises(_lib.MqError):
        _lib.check(_lib.lib().mq_decoder_step(fused._h, C.c_void_p(x.data_ptr()), 4, -1, C.c_void_p(x.data_ptr()), None,
                                              None, None), "mq_decoder_step")   # more tokens than the handle holds
    fused.free()
    # a Q5_K projection keeps the layer on the node-by-node path
    ly = step.layers[0]
    keep = ly.wo
    ly.wo = ops.Q4KWeight.synthetic(5, cfg.hidden, cfg.n_q, 1, synth.GGML_TYPE_Q5_K)
    with pytest.raises(_lib.MqError):
        ds.FusedDecodeStep(cfg, 2, step.layers)
    ly.wo.free()
    ly.wo = keep
    step.free()
