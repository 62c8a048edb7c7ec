"""Strided operands at every width: activation rows ldx floats apart with NaN in the gaps, results written ldy floats
apart into a buffer pre-filled with a sentinel, two spare rows after the last one.  Every entry point that takes
strides must produce the bits of the contiguous call and leave the gaps, the padding columns and the spare rows alone
(a NaN read from a gap, or a store past a row's end, shows at once).  Rows 1..72 and two prefill widths, ragged row
counts, the four weight types."""
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu

SENTINEL = 12345.678


def _strided_x(torch, x, pad):
    n, cols = x.shape
    buf = torch.full((n, cols + pad), float("nan"), dtype=torch.float32, device="cuda")
    buf[:, :cols] = x
    return buf


def _check(torch, ybuf, n, rows, want, what, exact=True):
    if exact:
        assert torch.equal(ybuf[:n, :rows], want), what + ": result"
    else:   # the handle's products stay on the decode kernels where the plain entry point moves to the GEMM: to rounding
        assert (ybuf[:n, :rows] - want).abs().max().item() <= 1e-5 * want.abs().max().item(), what + ": result"
    assert (ybuf[:n, rows:] == SENTINEL).all(), what + ": padding columns written"
    assert (ybuf[n:] == SENTINEL).all(), what + ": rows past the last one written"


@pytest.mark.parametrize("rows,cols,wtype", [(1000, 1024, 12), (4096, 4096, 12), (520, 2048, 13), (1000, 1024, 14), (1000, 1024, 8),
                                             (14336 + 24, 4096, 12)])
def test_products_with_strided_rows(rows, cols, wtype):
    import torch
    from densecore_amd import _lib, ops
    L = _lib.lib()
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("sb", rows, cols, wtype), rows, cols, ggml_type=wtype)
    xs = torch.from_numpy(synth.normal_f32(synth.tensor_seed("sb-x", rows, cols), (300, cols))).cuda()
    acts = ops.Q8KActs(64, cols) if wtype != 8 else None
    for n in list(range(1, 73)) + [130, 300]:
        x = xs[:n].contiguous()
        xb = _strided_x(torch, x, 64)
        ldy = rows + 40
        want = ops.mul_mat(W, x)
        yb = torch.full((n + 2, ldy), SENTINEL, dtype=torch.float32, device="cuda")
        _lib.check(L.mq_mul_mat_q4k(W._h, xb.data_ptr(), n, xb.stride(0), yb.data_ptr(), ldy, None), "mq_mul_mat_q4k")
        _check(torch, yb, n, rows, want, f"mq_mul_mat_q4k n={n}")
        if wtype != 8:
            want = ops.gemm(W, x)
            yb.fill_(SENTINEL)
            _lib.check(L.mq_gemm_q4k(W._h, xb.data_ptr(), n, xb.stride(0), yb.data_ptr(), ldy, None), "mq_gemm_q4k")
            _check(torch, yb, n, rows, want, f"mq_gemm_q4k n={n}")
        if acts is not None and n <= 64:
            yb.fill_(SENTINEL)
            _lib.check(L.mq_acts_quantize(acts._h, xb.data_ptr(), n, xb.stride(0), None), "mq_acts_quantize")
            _lib.check(L.mq_mul_mat_q4k_acts(W._h, acts._h, yb.data_ptr(), ldy, None), "mq_mul_mat_q4k_acts")
            _check(torch, yb, n, rows, ops.mul_mat(W, x), f"mq_mul_mat_q4k_acts n={n}", exact=n <= 16)
    if acts is not None:
        acts.free()
    W.free()


@pytest.mark.parametrize("rows,cols,wtype", [(1000, 1024, 12), (3000, 2048, 12), (14336, 4096, 12), (520, 1024, 13), (776, 1024, 14)])
def test_gate_up_with_strided_rows(rows, cols, wtype):
    import torch
    from densecore_amd import _lib, ops
    L = _lib.lib()
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("sb-g", rows, cols, wtype), rows, cols, ggml_type=wtype)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("sb-u", rows, cols, wtype), rows, cols, ggml_type=wtype)
    xs = torch.from_numpy(synth.normal_f32(synth.tensor_seed("sb-gx", rows, cols), (300, cols))).cuda()
    acts = ops.Q8KActs(64, cols)
    for n in list(range(1, 73)) + [130, 300]:
        x = xs[:n].contiguous()
        xb = _strided_x(torch, x, 64)
        ldh = rows + 24        # (rows of 16-byte alignment: the wide form's contract)
        want = ops.swiglu_mul_mat(G, U, x, 2)
        hb = torch.full((n + 2, ldh), SENTINEL, dtype=torch.float32, device="cuda")
        _lib.check(L.mq_swiglu_mul_mat_q4k(G._h, U._h, xb.data_ptr(), n, xb.stride(0), hb.data_ptr(), ldh, 2, None), "mq_swiglu_mul_mat_q4k")
        _check(torch, hb, n, rows, want, f"mq_swiglu_mul_mat_q4k n={n}")
        if n <= 64:
            hb.fill_(SENTINEL)
            _lib.check(L.mq_acts_quantize(acts._h, xb.data_ptr(), n, xb.stride(0), None), "mq_acts_quantize")
            _lib.check(L.mq_swiglu_mul_mat_q4k_acts(G._h, U._h, acts._h, hb.data_ptr(), ldh, 2, None), "mq_swiglu_mul_mat_q4k_acts")
            _check(torch, hb, n, rows, want, f"mq_swiglu_mul_mat_q4k_acts n={n}", exact=n <= 16)
    acts.free(), G.free(), U.free()
