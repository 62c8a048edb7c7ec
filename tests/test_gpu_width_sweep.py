"""Every row count from 1 to 72 through `mq_mul_mat_q4k` on a handful of shapes and the three weight types: whatever
kernel the width selects (single-row GEMV with the quantizer inside, the fused few-row GEMV, the LDS-staged and the
global-operand decode kernels, one to four activation tiles of sixteen, 16-row passes, the matrix-core GEMM), row i of
the result depends on row i of x alone.  The decode kernels share one arithmetic, so up to the width where the GEMM
takes over row i equals the one-row product of x[i] bit for bit; the GEMM sums a row's super-blocks in another order and
agrees to rounding (1e-5 of the largest entry).  Shapes with ragged row counts, one and several stages per wavefront,
and a matrix large enough for the GEMM's lower threshold."""
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu

# (rows, cols, weight type, first width of the matrix-core GEMM)
CASES = [
    (4096, 4096, 12, 65), (2048, 2048, 12, 65), (1000, 1024, 12, 65), (72, 2048, 12, 65), (3000, 6144, 12, 33),
    (14336, 4096, 12, 65), (4096, 14336, 12, 33),
    (4096, 4096, 13, 48), (1000, 1024, 13, 48), (14336, 4096, 13, 17),
    (4096, 4096, 14, 48), (1000, 1024, 14, 48), (4096, 14336, 14, 17),
]


@pytest.mark.parametrize("rows,cols,wtype,gemm_from", CASES)
def test_row_i_of_the_result_depends_on_row_i_alone_at_every_width(rows, cols, wtype, gemm_from):
    import torch
    from densecore_amd import ops
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("ws", rows, cols, wtype), rows, cols, ggml_type=wtype)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("ws-x", rows, cols), (72, cols))).cuda()
    single = torch.cat([ops.mul_mat(W, x[i:i + 1]) for i in range(72)], dim=0)
    scale = single.abs().max().item()
    for n in range(1, 73):
        y = ops.mul_mat(W, x[:n])
        if n < gemm_from:
            assert torch.equal(y, single[:n]), f"n={n}: rows {(y != single[:n]).any(dim=1).nonzero().flatten().tolist()[:8]}"
        else:
            assert (y - single[:n]).abs().max().item() <= 1e-5 * scale, f"n={n}"
    W.free()


def _rows_alone(fn, x, n_max, exact_to):
    import torch
    single = torch.cat([fn(x[i:i + 1]) for i in range(n_max)], dim=0)
    scale = single.abs().max().item()
    for n in range(1, n_max + 1):
        y = fn(x[:n])
        if n <= exact_to:
            assert torch.equal(y, single[:n]), f"n={n}"
        elif not torch.equal(y, single[:n]):    # a width of the matrix-core GEMM: to rounding
            assert (y - single[:n]).abs().max().item() <= 2e-5 * scale, f"n={n}"


@pytest.mark.parametrize("rows,cols", [(14336, 4096), (1024, 4096), (2048, 2048), (3000, 2048)])
@pytest.mark.parametrize("silu", [0, 2])
def test_gate_up_rows_alone_at_every_width(rows, cols, silu):
    import torch
    from densecore_amd import ops
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("ws-g", rows, cols), rows, cols)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("ws-u", rows, cols), rows, cols)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("ws-gx", rows, cols), (72, cols))).cuda()
    _rows_alone(lambda t: ops.swiglu_mul_mat(G, U, t, silu), x, 72, 16)
    G.free(), U.free()


@pytest.mark.parametrize("hidden,inter", [(4096, 14336), (2048, 512), (1024, 3072)])
def test_ffn_rows_alone_at_every_width(hidden, inter):
    import torch
    from densecore_amd import ops
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("ws-fg", hidden, inter), inter, hidden)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("ws-fu", hidden, inter), inter, hidden)
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("ws-fd", hidden, inter), hidden, inter)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("ws-fx", hidden, inter), (72, hidden))).cuda()
    _rows_alone(lambda t: ops.ffn_swiglu(G, U, D, t, ops.SILU_FAST_FMA), x, 72, 16)
    G.free(), U.free(), D.free()


@pytest.mark.parametrize("rows,cols", [(3000, 2048), (1000, 1024), (72, 2048), (14336 + 8, 1024)])
def test_wide_gate_up_and_product_on_row_counts_that_are_no_multiple_of_a_super_block(rows, cols):
    """Prefill widths on matrices whose row count is no multiple of 256 (nor of the 64 and 128 rows of a GEMM workgroup):
    the SwiGLU rows are formed by the pair launch, or from two planes where K is split into runs -- every column of
    every row against the same rows taken sixteen at a time."""
    import torch
    from densecore_amd import ops
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("wr-g", rows, cols), rows, cols)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("wr-u", rows, cols), rows, cols)
    for n in (49, 100, 300, 601):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("wr-x", rows, cols, n), (n, cols))).cuda()
        for fn in (lambda t: ops.swiglu_mul_mat(G, U, t, 0), lambda t: ops.swiglu_mul_mat(G, U, t, 2), lambda t: ops.mul_mat(G, t)):
            whole = fn(x)
            split = torch.cat([fn(x[i:i + 16]) for i in range(0, n, 16)], dim=0)
            assert (whole - split).abs().max().item() <= 2e-5 * split.abs().max().item(), f"n={n}"
    G.free(), U.free()


@pytest.mark.parametrize("hidden,inter,gu_type,down_type", [(1024, 3072, 12, 13), (1024, 3072, 12, 14), (2048, 512, 13, 13),
                                                           (2048, 512, 14, 14), (4096, 14336, 12, 14)])
def test_ffn_with_sibling_types_equals_its_two_nodes_at_every_width(hidden, inter, gu_type, down_type):
    """mq_ffn_swiglu_q4k against the gate/up entry point followed by the down product, as a graph that keeps the three
    nodes apart would run them: bit for bit up to sixteen rows (every kernel there shares one arithmetic and the
    quantizers one block routine); beyond, the fused entry point may take other launches (the matrix-core GEMM, the
    SwiGLU product formed in its quantizer), whose last-bit differences in a hidden row can move a code of the down
    product's quantizer in a few rows."""
    import torch
    from densecore_amd import ops
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("fs-g", hidden, inter, gu_type), inter, hidden, ggml_type=gu_type)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("fs-u", hidden, inter, gu_type), inter, hidden, ggml_type=gu_type)
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("fs-d", hidden, inter, down_type), hidden, inter, ggml_type=down_type)
    xs = torch.from_numpy(synth.normal_f32(synth.tensor_seed("fs-x", hidden, inter), (300, hidden))).cuda()
    for n in list(range(1, 73)) + [130, 300]:
        x = xs[:n]
        y = ops.ffn_swiglu(G, U, D, x, ops.SILU_FAST_FMA)
        want = ops.mul_mat(D, ops.swiglu_mul_mat(G, U, x, ops.SILU_FAST_FMA))
        if n <= 16:
            assert torch.equal(y, want), f"n={n}"
        else:
            err = (y - want).abs().max(dim=1).values / want.abs().max().item()
            assert err.max().item() <= 5e-4 and (err > 2e-5).sum().item() <= max(2, n // 40), f"n={n}: {err.max().item()}"
    G.free(), U.free(), D.free()
