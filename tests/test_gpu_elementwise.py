"""add + RMSNorm and the fp32 router projection against plain numpy (float64 accumulation)."""
import ctypes as C

import numpy as np
import pytest

from oracle import decode_step as ref_step

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,cols", [(1, 2048), (5, 512), (3, 768)])
@pytest.mark.parametrize("with_delta", [False, True])
def test_add_rmsnorm(n, cols, with_delta):
    import torch
    from densecore_amd import _lib
    rng = np.random.default_rng(n * cols)
    x = rng.normal(size=(n, cols)).astype(np.float32) * 3
    d = rng.normal(size=(n, cols)).astype(np.float32) if with_delta else None
    xs, hs = ref_step.add_rmsnorm(x, d, 1e-6)
    xt = torch.from_numpy(x).cuda()
    dt = torch.from_numpy(d).cuda() if with_delta else None
    h = torch.empty_like(xt)
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    # the sum is written in place over x, as the decoder step does
    _lib.check(_lib.lib().mq_add_rmsnorm_f32(p(xt), p(dt), None, n, cols, C.c_float(1e-6), p(xt), p(h), None), "rms")
    torch.cuda.synchronize()
    assert np.array_equal(xt.cpu().numpy(), xs)
    np.testing.assert_allclose(h.cpu().numpy(), hs, rtol=2e-6, atol=1e-7)
    # with a weight vector
    w = rng.normal(size=cols).astype(np.float32)
    xt2 = torch.from_numpy(x).cuda()
    _lib.check(_lib.lib().mq_add_rmsnorm_f32(p(xt2), p(dt), p(torch.from_numpy(w).cuda()), n, cols, C.c_float(1e-6),
                                             None, p(h), None), "rms")
    np.testing.assert_allclose(h.cpu().numpy(), hs * w, rtol=3e-6, atol=1e-7)


@pytest.mark.parametrize("n", [1, 9])
def test_router_logits(n):
    import torch
    from densecore_amd import _lib
    rng = np.random.default_rng(n)
    w = rng.normal(size=(256, 2048)).astype(np.float32)
    x = rng.normal(size=(n, 2048)).astype(np.float32)
    out = torch.empty((n, 256), device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    wt, xt = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
    _lib.check(_lib.lib().mq_router_logits_f32(p(wt), 256, 2048, p(xt), n, 2048, p(out), None), "router")
    ref = ref_step.router_logits(w, x)
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=0, atol=2e-5 * np.abs(ref).max())


@pytest.mark.parametrize("n,cols", [(1, 2048), (6, 512)])
def test_add_rmsnorm_q8k_equals_norm_then_quantize(n, cols):
    """mq_add_rmsnorm_q8k: same fp32 rows as mq_add_rmsnorm_f32, and products from its Q8_K handle equal the
    products from quantizing those fp32 rows separately, bit for bit."""
    import torch
    from densecore_amd import _lib, ops
    rng = np.random.default_rng(n + cols)
    x = torch.from_numpy(rng.normal(size=(n, cols)).astype(np.float32) * 2).cuda()
    d = torch.from_numpy(rng.normal(size=(n, cols)).astype(np.float32)).cuda()
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    ref_sum, ref_h = torch.empty_like(x), torch.empty_like(x)
    _lib.check(_lib.lib().mq_add_rmsnorm_f32(p(x), p(d), None, n, cols, C.c_float(1e-6), p(ref_sum), p(ref_h), None), "f32")
    acts = ops.Q8KActs(n, cols)
    got_sum, got_h = torch.empty_like(x), torch.empty_like(x)
    _lib.check(_lib.lib().mq_add_rmsnorm_q8k(p(x), p(d), None, n, cols, C.c_float(1e-6), p(got_sum), p(got_h),
                                             C.c_void_p(acts._h), None), "q8k")
    acts.n = n
    assert torch.equal(got_sum, ref_sum) and torch.equal(got_h, ref_h)
    w = ops.Q4KWeight.synthetic(9, 128, cols)
    assert torch.equal(acts.mul_mat(w), ops.mul_mat(w, ref_h))
    # without the fp32 copy and with the sum written in place
    x2 = x.clone()
    _lib.check(_lib.lib().mq_add_rmsnorm_q8k(p(x2), p(d), None, n, cols, C.c_float(1e-6), p(x2), None,
                                             C.c_void_p(acts._h), None), "q8k in place")
    assert torch.equal(x2, ref_sum) and torch.equal(acts.mul_mat(w), ops.mul_mat(w, ref_h))
    acts.free(), w.free()


@pytest.mark.parametrize("n,cols,n_experts,with_delta,with_weight", [(1, 2048, 256, True, False), (4, 2048, 256, True, True),
                                                                      (3, 512, 10, False, True), (8, 4096, 64, True, False)])
def test_add_rmsnorm_router_equals_the_two_launches(n, cols, n_experts, with_delta, with_weight):
    """mq_add_rmsnorm_router_f32: the bits of mq_add_rmsnorm_f32 followed by mq_router_logits_f32."""
    import torch
    from densecore_amd import _lib
    g = torch.Generator(device="cuda").manual_seed(n * 1000 + cols)
    x = torch.randn((n, cols), device="cuda", generator=g)
    d = torch.randn((n, cols), device="cuda", generator=g) if with_delta else None
    w = (torch.rand((cols,), device="cuda", generator=g) + 0.5) if with_weight else None
    router = torch.randn((n_experts, cols), device="cuda", generator=g) * 0.05
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    L = _lib.lib()
    ref_sum, ref_h = torch.empty_like(x), torch.empty_like(x)
    ref_lg = torch.empty((n, n_experts), device="cuda")
    _lib.check(L.mq_add_rmsnorm_f32(p(x), p(d), p(w), n, cols, C.c_float(1e-6), p(ref_sum), p(ref_h), None), "norm")
    _lib.check(L.mq_router_logits_f32(p(router), n_experts, cols, p(ref_h), n, cols, p(ref_lg), None), "router")
    got_sum, got_h = torch.empty_like(x), torch.empty_like(x)
    got_lg = torch.empty((n, n_experts), device="cuda")
    _lib.check(L.mq_add_rmsnorm_router_f32(p(x), p(d), p(w), n, cols, C.c_float(1e-6), p(got_sum), p(got_h), p(router),
                                           n_experts, p(got_lg), None), "fused")
    torch.cuda.synchronize()
    assert torch.equal(got_sum, ref_sum) and torch.equal(got_h, ref_h)
    assert torch.equal(got_lg, ref_lg), f"max |diff| {(got_lg - ref_lg).abs().max().item():.3e}"
    # the sum may not overwrite an input: every workgroup of a row reads x and delta
    with pytest.raises(_lib.MqError):
        _lib.check(L.mq_add_rmsnorm_router_f32(p(x), p(d), p(w), n, cols, C.c_float(1e-6), p(x), p(got_h), p(router),
                                               n_experts, p(got_lg), None), "fused in place")


@pytest.mark.parametrize("n,rows,cols,with_delta,with_weight", [(1, 2560, 2048, True, False), (1, 512, 4096, False, True),
                                                                 (1, 64, 512, True, True), (3, 2560, 2048, True, False)])
def test_rmsnorm_mul_mat_equals_norm_then_product(n, rows, cols, with_delta, with_weight):
    """mq_rmsnorm_mul_mat_q4k: the bits of mq_add_rmsnorm_q8k followed by mq_mul_mat_q4k_acts (one launch at one row)."""
    import torch
    from densecore_amd import _lib, ops
    g = torch.Generator(device="cuda").manual_seed(rows + cols + n)
    x = torch.randn((n, cols), device="cuda", generator=g)
    d = torch.randn((n, cols), device="cuda", generator=g) if with_delta else None
    w = (torch.rand((cols,), device="cuda", generator=g) + 0.5) if with_weight else None
    W = ops.Q4KWeight.synthetic(rows * 7 + cols, rows, cols)
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    L = _lib.lib()
    acts = ops.Q8KActs(n, cols)
    ref_sum = torch.empty_like(x)
    _lib.check(L.mq_add_rmsnorm_q8k(p(x), p(d), p(w), n, cols, C.c_float(1e-6), p(ref_sum), None, C.c_void_p(acts._h), None), "norm")
    ref_y = acts.mul_mat(W, out=torch.empty((n, rows), device="cuda"))
    got_sum = torch.empty_like(x)
    got_y = torch.empty((n, rows), device="cuda")
    _lib.check(L.mq_rmsnorm_mul_mat_q4k(W._h, p(x), p(d), p(w), n, C.c_float(1e-6), p(got_sum), p(got_y), rows, None), "fused")
    torch.cuda.synchronize()
    assert torch.equal(got_sum, ref_sum)
    assert torch.equal(got_y, ref_y), f"max |diff| {(got_y - ref_y).abs().max().item():.3e}"
    with pytest.raises(_lib.MqError):
        _lib.check(L.mq_rmsnorm_mul_mat_q4k(W._h, p(x), p(d), p(w), n, C.c_float(1e-6), p(x), p(got_y), rows, None), "in place")
    acts.free()
    W.free()


@pytest.mark.parametrize("n,rows,cols", [(70, 2560, 2048), (40, 4096, 14336)])
def test_rmsnorm_mul_mat_at_prefill_widths_is_norm_then_gemm(n, rows, cols):
    """Where mq_mul_mat_q4k takes the matrix-core GEMM (65 rows; 33 where the rows do not pass through LDS as tiles of
    sixteen) the fused entry does too: the bits of mq_add_rmsnorm_f32 followed by mq_gemm_q4k on the normalised rows."""
    import torch
    from densecore_amd import _lib, ops
    g = torch.Generator(device="cuda").manual_seed(rows + cols + n)
    x = torch.randn((n, cols), device="cuda", generator=g)
    d = torch.randn((n, cols), device="cuda", generator=g)
    w = torch.rand((cols,), device="cuda", generator=g) + 0.5
    W = ops.Q4KWeight.synthetic(rows * 3 + cols, rows, cols)
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    L = _lib.lib()
    ref_sum, ref_h = torch.empty_like(x), torch.empty_like(x)
    _lib.check(L.mq_add_rmsnorm_f32(p(x), p(d), p(w), n, cols, C.c_float(1e-6), p(ref_sum), p(ref_h), None), "norm")
    ref_y = ops.gemm(W, ref_h)
    got_sum = torch.empty_like(x)
    got_y = torch.empty((n, rows), device="cuda")
    _lib.check(L.mq_rmsnorm_mul_mat_q4k(W._h, p(x), p(d), p(w), n, C.c_float(1e-6), p(got_sum), p(got_y), rows, None), "fused")
    torch.cuda.synchronize()
    assert torch.equal(got_sum, ref_sum) and torch.equal(got_y, ref_y)
    W.free()
