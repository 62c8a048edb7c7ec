"""The operators either side of the projections at every width: residual add + RMSNorm fused with a projection
(mq_rmsnorm_mul_mat_q4k) and with the router (mq_add_rmsnorm_router_f32) must return, bit for bit, what their unfused
sequences return -- mq_add_rmsnorm_f32 followed by mq_mul_mat_q4k / mq_router_logits_f32 -- at 1..72 rows and two
prefill widths, with and without the residual delta, the norm weight and the sum output, on ragged row counts and the
three K-quant types; and the norm itself against numpy in double precision."""
import ctypes as C

import numpy as np
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu
EPS = 1e-6


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


@pytest.mark.parametrize("rows,cols,wtype", [(2560, 2048, 12), (1000, 1024, 12), (72, 4096, 12), (520, 2048, 13), (1000, 1024, 14),
                                             (14336 + 8, 4096, 12)])
def test_norm_fused_projection_equals_norm_then_projection(rows, cols, wtype):
    import torch
    from densecore_amd import _lib, ops
    L = _lib.lib()
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("nw", rows, cols, wtype), rows, cols, ggml_type=wtype)
    xs = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nw-x", rows, cols), (300, cols))).cuda()
    ds = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nw-d", rows, cols), (300, cols)) * np.float32(0.3)).cuda()
    wn = torch.from_numpy(1.0 + 0.1 * synth.normal_f32(synth.tensor_seed("nw-w", cols), (cols,))).cuda()
    for n in list(range(1, 73)) + [130, 300]:
        variant = n % 4   # 0: delta + weight + sum, 1: no delta, 2: no weight, 3: no sum output
        x, d = xs[:n].contiguous(), (ds[:n].contiguous() if variant != 1 else None)
        w = wn if variant != 2 else None
        s_ref = torch.empty_like(x)
        h_ref = torch.empty_like(x)
        _lib.check(L.mq_add_rmsnorm_f32(_p(x), _p(d), _p(w), n, cols, C.c_float(EPS), _p(s_ref), _p(h_ref), None), "mq_add_rmsnorm_f32")
        want = ops.mul_mat(W, h_ref)
        s_got = torch.full_like(x, 7.0) if variant != 3 else None
        ldy = rows + 8
        y = torch.full((n + 1, ldy), 7.0, dtype=torch.float32, device="cuda")
        _lib.check(L.mq_rmsnorm_mul_mat_q4k(W._h, _p(x), _p(d), _p(w), n, C.c_float(EPS), _p(s_got), _p(y), ldy, None), "mq_rmsnorm_mul_mat_q4k")
        assert torch.equal(y[:n, :rows], want), f"n={n} variant {variant}"
        assert (y[:n, rows:] == 7.0).all() and (y[n] == 7.0).all(), f"n={n}: written outside the rows"
        if s_got is not None:
            assert torch.equal(s_got, s_ref), f"n={n}: sum"
        # the norm against numpy in double precision
        if n in (1, 7, 40):
            sd = x.double().cpu().numpy() + (d.double().cpu().numpy() if d is not None else 0.0)
            hd = sd / np.sqrt((sd * sd).mean(axis=1, keepdims=True) + EPS) * (w.double().cpu().numpy() if w is not None else 1.0)
            assert np.abs(h_ref.cpu().numpy() - hd).max() <= 2e-6 * np.abs(hd).max(), f"n={n}: norm"
    W.free()


@pytest.mark.parametrize("cols,n_experts", [(2048, 256), (1024, 60), (4096, 7), (256, 300), (512, 1)])
def test_norm_fused_router_equals_norm_then_router(cols, n_experts):
    import torch
    from densecore_amd import _lib
    L = _lib.lib()
    xs = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nr-x", cols), (300, cols))).cuda()
    ds = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nr-d", cols), (300, cols)) * np.float32(0.3)).cuda()
    wn = torch.from_numpy(1.0 + 0.1 * synth.normal_f32(synth.tensor_seed("nr-w", cols), (cols,))).cuda()
    router = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nr-r", cols, n_experts), (n_experts, cols)) * np.float32(0.05)).cuda()
    for n in list(range(1, 73)) + [130, 300]:
        variant = n % 3   # 0: delta + weight, 1: no delta, 2: no weight
        x, d = xs[:n].contiguous(), (ds[:n].contiguous() if variant != 1 else None)
        w = wn if variant != 2 else None
        s_ref, h_ref = torch.empty_like(x), torch.empty_like(x)
        _lib.check(L.mq_add_rmsnorm_f32(_p(x), _p(d), _p(w), n, cols, C.c_float(EPS), _p(s_ref), _p(h_ref), None), "mq_add_rmsnorm_f32")
        lg_ref = torch.empty((n, n_experts), dtype=torch.float32, device="cuda")
        _lib.check(L.mq_router_logits_f32(_p(router), n_experts, cols, _p(h_ref), n, cols, _p(lg_ref), None), "mq_router_logits_f32")
        s_got, h_got = torch.full_like(x, 7.0), torch.full_like(x, 7.0)
        lg = torch.full((n + 1, n_experts), 7.0, dtype=torch.float32, device="cuda")
        _lib.check(L.mq_add_rmsnorm_router_f32(_p(x), _p(d), _p(w), n, cols, C.c_float(EPS), _p(s_got), _p(h_got), _p(router), n_experts,
                                               _p(lg), None), "mq_add_rmsnorm_router_f32")
        assert torch.equal(s_got, s_ref) and torch.equal(h_got, h_ref), f"n={n}: sum / normalised rows"
        assert torch.equal(lg[:n], lg_ref), f"n={n}: logits"
        assert (lg[n] == 7.0).all(), f"n={n}: written past the last row"
        if n in (1, 9, 72):
            want = h_ref.double().cpu().numpy() @ router.double().cpu().numpy().T
            assert np.abs(lg_ref.cpu().numpy() - want).max() <= 2e-6 * max(np.abs(want).max(), 1e-30), f"n={n}: router"


@pytest.mark.parametrize("n", [3, 12, 24, 50, 100])
def test_norm_fused_projection_replayed_from_a_graph(n):
    """Every width's launch sequence (norm inside the GEMV, norm + Q8_K + decode kernel, norm + quantizer + tiles of
    sixteen, norm + GEMM) captured into a HIP graph: three replays with eager work in between equal the eager result."""
    import torch
    from densecore_amd import _lib, ops
    L = _lib.lib()
    rows, cols = 2560, 2048
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("nwg", rows, cols), rows, cols)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nwg-x", n), (n, cols))).cuda()
    d = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nwg-d", n), (n, cols))).cuda()
    s_out, y = torch.empty_like(x), torch.empty((n, rows), dtype=torch.float32, device="cuda")
    def run():
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        _lib.check(L.mq_rmsnorm_mul_mat_q4k(W._h, _p(x), _p(d), None, n, C.c_float(EPS), _p(s_out), _p(y), rows, st), "mq_rmsnorm_mul_mat_q4k")
    run()
    torch.cuda.synchronize()
    eager = y.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run()
    for rep in range(3):
        y.fill_(0.0)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {rep}"
        other = torch.from_numpy(synth.normal_f32(synth.tensor_seed("nwg-o", rep), (7 + rep, cols))).cuda()
        ops.mul_mat(W, other)          # eager work on the same workspaces between the replays
        torch.cuda.synchronize()
    W.free()
