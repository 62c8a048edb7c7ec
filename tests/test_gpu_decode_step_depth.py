"""The 40-layer, 256-expert decoder step at its full size (18.5 GB of Q4_K weights) against the CPU restatement at
depth: layers 0, 19 and 39, teacher-forced on the GPU's own residual stream.

The residual stream that enters layer L is read off a run of the first L layers (same weights, same launches: its
final residual add forms exactly the sum layer L's first launch would form).  Layer L alone on that input must route
exactly as layer L did inside the full step -- which ties the single-layer run to the 40-layer one -- and its stages
are compared with oracle/decode_step.py on the same input: ids exactly, products within the tolerances of
tests/test_gpu_decode_step.py.  The last layer's output is the full step's output, bit for bit."""
import dataclasses

import numpy as np
import pytest

from oracle import decode_step as ref_step
from tests.test_gpu_decode_step import STAGE_REL, close, host_weights

pytestmark = pytest.mark.gpu

DEPTHS = (0, 19, 39)


@pytest.fixture(scope="module")
def model():
    import torch
    from densecore_amd import decode_step as ds
    assert torch.cuda.is_available()
    cfg = ds.StepConfig(synthetic_logits=True)       # router logits N(0,1): the configuration the benchmark times
    assert cfg.n_layers == 40 and cfg.n_experts == 256
    base = ds.DecodeStep(cfg, 1)
    host = {L: host_weights(base.layers[L]) for L in DEPTHS}
    yield ds, cfg, base, host
    base.free()


@pytest.mark.parametrize("n", [1, 4, 8])
def test_full_depth_step_teacher_forced(model, n):
    import torch
    ds, cfg, base, host = model
    full = base if n == 1 else ds.DecodeStep(cfg, n, layers=base.layers)
    x = torch.randn((n, cfg.hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(40 + n))
    out_full = full.run(x).clone()
    ids_full = full.ids.cpu().numpy()
    assert torch.isfinite(out_full).all()
    for L in DEPTHS:
        if L == 0:
            x_in = x
        else:
            head = ds.DecodeStep(dataclasses.replace(cfg, n_layers=L), n, layers=base.layers[:L])
            head.fixed_logits = full.fixed_logits[:L]
            x_in = head.run(x).clone()
            assert np.array_equal(head.ids.cpu().numpy(), ids_full[:L]), f"first {L} layers route differently alone"
            head.free()
        one = ds.DecodeStep(dataclasses.replace(cfg, n_layers=1), n, layers=[base.layers[L]])
        one.fixed_logits = full.fixed_logits[L:L + 1]
        out_one = one.run(x_in).clone()
        assert np.array_equal(one.ids[0].cpu().numpy(), ids_full[L]), f"layer {L} routes differently alone"
        if L == cfg.n_layers - 1:
            assert torch.equal(out_one, out_full), "the last layer on the step's own residual stream is the step's output"
        r = ref_step.layer_forward(host[L], x_in.cpu().numpy(), None, cfg, full.silu_mode(),
                                   fixed_logits=full.fixed_logits[L].cpu().numpy())
        assert np.array_equal(ids_full[L], r["ids"]), f"layer {L}: ids differ from the CPU restatement"
        close(full.wts[L].cpu().numpy(), r["weights"], 1e-5, f"layer {L} routing weights")
        close(one.qkv.cpu().numpy(), r["qkv"], STAGE_REL, f"layer {L} qkv")
        close(one.o.cpu().numpy(), r["o"], STAGE_REL, f"layer {L} wo")
        close(one.logits.cpu().numpy(), r["logits"], 1e-5, f"layer {L} router projection")
        close(one.y.cpu().numpy(), r["y"], 2e-3, f"layer {L} moe block")
        close(out_one.cpu().numpy(), r["x"] + r["y"], 2e-3, f"layer {L} output")
        one.free()
    if full is not base:
        full.free()
