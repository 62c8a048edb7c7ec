"""Dense Q4_K (and Q5_K, Q6_K) products of nine to sixteen rows as ONE activation tile of sixteen (skinny16_kernel) against the kernels
that take the same rows as two token tiles of eight: the same bits for every wave split the kernel has (one, two, four
and eight wavefronts per row tile), ragged row counts, strided rows, the fused gate/up form and the whole FFN -- and
within 1e-4 of every fp32 accumulation order the reference has."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity, oracle_all_orders

pytestmark = pytest.mark.gpu

TWO_TILES_OF_EIGHT = 1 | 0x1000   # mq_debug_set_dense_lds: LDS-staged kernels on, the sixteen-row tile off


@pytest.fixture(scope="module")
def env():
    import torch
    from densecore_amd import _lib, ops
    assert torch.cuda.is_available()
    yield torch, _lib, ops
    _lib.lib().mq_debug_set_dense_lds(1)


def three_ways(env, fn):
    """global-operand kernel, LDS-staged kernel with two token tiles, the sixteen-row tile"""
    torch, _lib, ops = env
    L = _lib.lib()
    out = []
    for mode in (0, TWO_TILES_OF_EIGHT, 1):
        L.mq_debug_set_dense_lds(mode)
        out.append(fn().clone())
    torch.cuda.synchronize()
    L.mq_debug_set_dense_lds(1)
    return [o.cpu().numpy() for o in out]


# rows, cols: wavefronts per row tile 2 (896 row tiles), 8, 8 with a ragged last tile, 4, 1, 2 with workgroups past the end,
# 8 with all of LDS in use; then odd stage counts: one stage per wavefront (2048 x 2048, 1000 x 1024), seven with the
# activation tiles read from global memory (the FFN's down projection: 56 super-blocks do not fit LDS), an even count
# from global memory, and a wave split the kernel does not have (six: falls back to two token tiles)
SHAPES = [(14336, 4096), (4096, 4096), (1000, 4096), (6144, 4096), (20480, 1024), (14000, 2048), (2048, 8192),
          (2048, 2048), (1000, 1024), (4096, 14336), (512, 16384), (2560, 3072)]


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_single_matrix_same_bits(env, rows, cols):
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s16", rows, cols), rows, cols)
    for n in (9, 11, 16):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16-x", rows, cols, n), (n, cols))).cuda()
        a, b, c = three_ways(env, lambda: ops.mul_mat(W, x))
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32)), f"n={n}: against the global-operand kernel"
        assert np.array_equal(b.view(np.uint32), c.view(np.uint32)), f"n={n}: against two token tiles in LDS"
    W.free()


@pytest.mark.parametrize("rows,cols", [(14336, 4096), (1024, 4096), (3000, 2048)])
@pytest.mark.parametrize("silu", [0, 1, 2])
def test_gate_up_same_bits(env, rows, cols, silu):
    torch, _lib, ops = env
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-g", rows, cols), rows, cols)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-u", rows, cols), rows, cols)
    for n in (9, 13, 16):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16-gx", rows, cols, n), (n, cols))).cuda()
        a, b, c = three_ways(env, lambda: ops.swiglu_mul_mat(G, U, x, silu))
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32)), f"n={n}"
        assert np.array_equal(b.view(np.uint32), c.view(np.uint32)), f"n={n}"
    G.free(), U.free()


def test_strided_rows_and_strided_output(env):
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(11, 1024, 4096)
    n = 14
    buf = torch.from_numpy(synth.normal_f32(1100 + n, (n, 4096 + 64))).cuda()
    x = buf[:, :4096]

    def raw():
        y = torch.full((n, W.rows + 32), 7.0, dtype=torch.float32, device="cuda")
        _lib.check(_lib.lib().mq_mul_mat_q4k(W._h, x.data_ptr(), n, x.stride(0), y.data_ptr(), y.stride(0), None), "mq_mul_mat_q4k")
        return y
    a, b, c = three_ways(env, raw)
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))
    assert np.all(c[:, W.rows:] == 7.0)
    ref = ops.mul_mat(W, x.contiguous()).cpu().numpy()
    assert np.array_equal(ref.view(np.uint32), c[:, :W.rows].view(np.uint32))
    W.free()


@pytest.mark.parametrize("hidden,inter", [(4096, 14336), (4096, 4096)])
def test_ffn_same_bits_and_graph_replay(env, hidden, inter):
    """gate/up on the sixteen-row tile with its rows in LDS; down on it as well, its rows in LDS (inter 4096) or read
    from global memory a stage ahead (inter 14336)."""
    torch, _lib, ops = env
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-fg", inter), inter, hidden)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-fu", inter), inter, hidden)
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-fd", inter), hidden, inter)
    for n in (10, 16):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16-fx", n), (n, hidden))).cuda()
        a, b, c = three_ways(env, lambda: ops.ffn_swiglu(G, U, D, x, ops.SILU_FAST))
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32)), f"n={n}"
        assert np.array_equal(b.view(np.uint32), c.view(np.uint32)), f"n={n}"
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16-fx", 16), (16, hidden))).cuda()
    eager = ops.ffn_swiglu(G, U, D, x, ops.SILU_FAST).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    out = {}
    with torch.cuda.graph(g, stream=side):
        out["y"] = ops.ffn_swiglu(G, U, D, x, ops.SILU_FAST)
    for _ in range(3):
        out["y"].fill_(3.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out["y"], eager)
    G.free(), U.free(), D.free()


def test_against_the_oracle(env):
    torch, _lib, ops = env
    rows, cols, n = 272, 4096, 13   # 17 row tiles, eight wavefronts per row tile
    w_np = synth.q4k_matrix(synth.tensor_seed("s16-ow"), rows, cols)
    W = ops.Q4KWeight.from_ggml(w_np, cols, synth.GGML_TYPE_Q4_K)
    x = synth.normal_f32(synth.tensor_seed("s16-ox"), (n, cols))
    y = ops.mul_mat(W, torch.from_numpy(x).cuda()).cpu().numpy()
    q8 = orc.quantize_rows_q8k(x)
    mag = orc.dot_magnitude_f64(w_np, cols, q8)
    for name, ref in oracle_all_orders(w_np, cols, q8).items():
        assert_fp32_parity(y, ref, mag, f"order={name}")
    W.free()


def test_shared_activation_handle_keeps_its_tile_of_sixteen_current(env):
    """A handle of more than eight rows carries the rows' tile of sixteen beside the A-major rows: mq_acts_quantize
    writes both, mq_add_rmsnorm_q8k only the A-major ones -- a product from the handle must then not read the stale
    tile.  Both ways the product equals the one-shot entry point on the same fp32 rows."""
    import ctypes as C
    torch, _lib, ops = env
    L = _lib.lib()
    rows, cols, n = 4096, 4096, 12
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-hw"), rows, cols)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s16-hu"), rows, cols)
    x1 = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16-h1"), (n, cols))).cuda()
    x2 = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16-h2"), (n, cols))).cuda()
    acts = ops.Q8KActs(16, cols)
    acts.quantize(x1)
    assert torch.equal(acts.mul_mat(W), ops.mul_mat(W, x1))
    assert torch.equal(acts.swiglu_mul_mat(W, U, 2), ops.swiglu_mul_mat(W, U, x1, 2))
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    normed = torch.empty_like(x2)
    _lib.check(L.mq_add_rmsnorm_q8k(p(x2), None, None, n, cols, C.c_float(1e-6), None, p(normed), C.c_void_p(acts._h), None), "norm")
    acts.n = n
    assert torch.equal(acts.mul_mat(W), ops.mul_mat(W, normed))
    acts.quantize(x2[:9])
    assert torch.equal(acts.mul_mat(W), ops.mul_mat(W, x2[:9]))
    acts.free(), W.free(), U.free()


# ---- seventeen to thirty-two rows: two tiles of sixteen per weight tile ----------------------------------------------

SMALL = [(4096, 4096), (2048, 2048), (1000, 4096), (6144, 4096), (20480, 1024), (2048, 8192), (512, 16384), (2560, 3072)]


@pytest.mark.parametrize("rows,cols", SMALL)
def test_two_tiles_single_matrix_same_bits_as_the_sixteen_row_passes(env, rows, cols):
    """Matrices below the GEMM's size threshold: the other decode kernel runs 17 to 32 rows as passes of sixteen in one
    launch (switch 0), the LDS-staged ones do not take them (switch 0x1001 ends on the same kernel)."""
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s32", rows, cols), rows, cols)
    for n in (17, 25, 32):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s32-x", rows, cols, n), (n, cols))).cuda()
        a, b, c = three_ways(env, lambda: ops.mul_mat(W, x))
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32)), f"n={n}"
        assert np.array_equal(b.view(np.uint32), c.view(np.uint32)), f"n={n}"
    W.free()


@pytest.mark.parametrize("rows,cols", [(1024, 4096), (3000, 2048), (512, 1024)])
@pytest.mark.parametrize("silu", [0, 2])
def test_two_tiles_gate_up_same_bits(env, rows, cols, silu):
    torch, _lib, ops = env
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s32-g", rows, cols), rows, cols)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s32-u", rows, cols), rows, cols)
    for n in (18, 32):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s32-gx", rows, cols, n), (n, cols))).cuda()
        a, b, c = three_ways(env, lambda: ops.swiglu_mul_mat(G, U, x, silu))
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32)), f"n={n}"
    G.free(), U.free()


@pytest.mark.parametrize("n", [17, 23, 32])
def test_two_tiles_on_ffn_sized_matrices_equal_the_rows_taken_sixteen_at_a_time(env, n):
    """Matrices of 24 MB and more used to go to the matrix-core GEMM from 17 rows (another fp32 update, other bits); up to
    32 rows they now stay on the decode arithmetic.  Every row's result is independent of the rows beside it, so the
    product and the whole FFN must equal the same rows handed over sixteen at a time, bit for bit -- and the oracle."""
    torch, _lib, ops = env
    hidden, inter = 4096, 14336
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s32-fg"), inter, hidden)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s32-fu"), inter, hidden)
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("s32-fd"), hidden, inter)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s32-fx", n), (n, hidden))).cuda()
    h = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s32-fh", n), (n, inter))).cuda()
    parts = lambda fn, t: torch.cat([fn(t[:16]), fn(t[16:])], dim=0)
    for name, fn, t in (("gate", lambda t: ops.mul_mat(G, t), x), ("down (rows read from global memory)", lambda t: ops.mul_mat(D, t), h),
                        ("gate/up", lambda t: ops.swiglu_mul_mat(G, U, t, 1), x), ("ffn", lambda t: ops.ffn_swiglu(G, U, D, t, ops.SILU_FAST), x)):
        whole, split = fn(t), parts(fn, t)
        assert torch.equal(whole, split), name
    # the oracle on sampled rows of the down projection (K = 14336: 56 super-blocks, seven per wavefront)
    w_np = synth.q4k_matrix(synth.tensor_seed("s32-ow"), 64, inter)
    W = ops.Q4KWeight.from_ggml(w_np, inter, synth.GGML_TYPE_Q4_K)
    hx = h.cpu().numpy()
    y = ops.mul_mat(W, h).cpu().numpy()
    q8 = orc.quantize_rows_q8k(hx)
    mag = orc.dot_magnitude_f64(w_np, inter, q8)
    for name, ref in oracle_all_orders(w_np, inter, q8).items():
        assert_fp32_parity(y, ref, mag, f"order={name}")
    for w in (G, U, D, W):
        w.free()


# ---- 33 to 64 rows: three and four tiles of sixteen, the activation tiles passing through LDS in runs of super-blocks ----

def _sixteen_at_a_time(fn, t):
    import torch
    return torch.cat([fn(t[i:i + 16]) for i in range(0, t.shape[0], 16)], dim=0)


# wavefronts per row tile 2 (two runs of super-blocks), 4 (two runs), 1 (not taken: 16-row passes or the GEMM), 4 (one run), 8 (two runs of one stage
# each), a single stage per wavefront whose tiles fit LDS in one run (twice), and three stages per wavefront whose tiles
# do not (falls back to the 16-row passes or the GEMM)
WIDE = [(14336, 4096), (6144, 4096), (20480, 1024), (8192, 2048), (4096, 4096), (2048, 2048), (2560, 2048), (2048, 6144)]


@pytest.mark.parametrize("rows,cols", WIDE)
def test_three_and_four_tiles_equal_the_rows_taken_sixteen_at_a_time(env, rows, cols):
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s64", rows, cols), rows, cols)
    takes = (rows, cols) not in ((2048, 6144), (20480, 1024))   # (... and more than 1,024 row tiles: the GEMM from 33 rows)
    for n in (33, 40, 48, 64):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s64-x", rows, cols, n), (n, cols))).cuda()
        whole, split = ops.mul_mat(W, x), _sixteen_at_a_time(lambda t: ops.mul_mat(W, t), x)
        if takes or n < 48:     # (the fallback below 48 rows is the 16-row passes: the same bits; from 48 the GEMM: to rounding)
            assert torch.equal(whole, split), f"n={n}"
        else:
            assert (whole - split).abs().max().item() <= 1e-5 * split.abs().max().item(), f"n={n}"
    W.free()


@pytest.mark.parametrize("wtype", [12, 13, 14])
@pytest.mark.parametrize("rows,cols", [(14336, 4096), (8192, 2048), (2048, 2048), (4096, 4096), (6144, 4096)])
@pytest.mark.parametrize("n", [40, 64])
def test_three_and_four_tiles_gate_up(env, rows, cols, n, wtype):
    torch, _lib, ops = env
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-g", rows, cols, wtype), rows, cols, ggml_type=wtype)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-u", rows, cols, wtype), rows, cols, ggml_type=wtype)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s64-gx", rows, cols, n), (n, cols))).cuda()
    # not built (the GEMM, to rounding): four tiles of a pair with eight wavefronts per row tile (2048 and 4096 rows here);
    # in runs of an odd number of stages (4096 x 4096: runs of one) the Q6_K forms and the Q5_K pair of four tiles
    gemm = (rows in (2048, 4096) and n == 64) or ((rows, cols) == (4096, 4096) and wtype == 14)
    for silu in (0, 1):
        fn = lambda t: ops.swiglu_mul_mat(G, U, t, silu)
        whole, split = fn(x), _sixteen_at_a_time(fn, x)
        if gemm:
            assert (whole - split).abs().max().item() <= 1e-5 * split.abs().max().item(), f"silu={silu}"
        else:
            assert torch.equal(whole, split), f"silu={silu}"
    G.free(), U.free()


@pytest.mark.parametrize("n", [40, 64])
def test_ffn_at_33_to_64_rows_and_graph_replay(env, n):
    """gate/up on three or four tiles of sixteen; the down projection's rows (56 super-blocks, seven per wavefront) do not
    pass through LDS in runs, so it goes to the matrix-core GEMM on the SwiGLU rows: equal to rounding."""
    torch, _lib, ops = env
    hidden, inter = 4096, 14336
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-fg"), inter, hidden)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-fu"), inter, hidden)
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-fd"), hidden, inter)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s64-fx", n), (n, hidden))).cuda()
    fn = lambda t: ops.ffn_swiglu(G, U, D, t, ops.SILU_FAST)
    whole, split = fn(x).clone(), _sixteen_at_a_time(fn, x)
    assert (whole - split).abs().max().item() <= 1e-5 * split.abs().max().item()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    out = {}
    with torch.cuda.graph(g, stream=side):
        out["y"] = fn(x)
    for _ in range(3):
        out["y"].fill_(3.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out["y"], whole)
    G.free(), U.free(), D.free()


def test_three_tiles_against_the_oracle(env):
    torch, _lib, ops = env
    rows, cols, n = 17000, 1024, 45   # 1063 row tiles: one wavefront per row tile, four stages each
    w_np = synth.q4k_matrix(synth.tensor_seed("s64-ow"), rows, cols)
    W = ops.Q4KWeight.from_ggml(w_np, cols, synth.GGML_TYPE_Q4_K)
    x = synth.normal_f32(synth.tensor_seed("s64-ox"), (n, cols))
    y = ops.mul_mat(W, torch.from_numpy(x).cuda()).cpu().numpy()
    pick = np.r_[0:64, 8000:8064, rows - 40:rows]
    q8 = orc.quantize_rows_q8k(x)
    w_pick = np.ascontiguousarray(w_np.reshape(rows, -1)[pick])
    mag = orc.dot_magnitude_f64(w_pick, cols, q8)
    for name, ref in oracle_all_orders(w_pick, cols, q8).items():
        assert_fp32_parity(y[:, pick], ref, mag, f"order={name}")
    W.free()


def test_shared_activation_handle_up_to_64_rows(env):
    torch, _lib, ops = env
    rows, cols = 6144, 4096
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-hw"), rows, cols)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s64-hu"), rows, cols)
    acts = ops.Q8KActs(64, cols)
    for n in (64, 20, 40, 5):      # every later batch reuses the handle
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s64-hx", n), (n, cols))).cuda()
        acts.quantize(x)
        assert torch.equal(acts.mul_mat(W), ops.mul_mat(W, x)), f"n={n}"
        assert torch.equal(acts.swiglu_mul_mat(W, U, 1), ops.swiglu_mul_mat(W, U, x, 1)), f"n={n}"
    acts.free(), W.free(), U.free()


# ---- Q5_K and Q6_K: one and two tiles of sixteen (Q5_K: a third MFMA chain for the fifth code bits; Q6_K: sixteen
# K = 32 MFMAs, one per 16-weight scale group, as the passes of eight multiply it) ----

@pytest.mark.parametrize("wtype", [13, 14])
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_sibling_types_single_matrix_same_bits_as_the_passes_of_eight(env, rows, cols, wtype):
    torch, _lib, ops = env
    L = _lib.lib()
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s16q5", rows, cols, wtype), rows, cols, ggml_type=wtype)
    for n in (9, 13, 16, 17, 25, 32):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16q5-x", rows, cols, n), (n, cols))).cuda()
        got = ops.mul_mat(W, x)
        L.mq_debug_set_dense_lds(TWO_TILES_OF_EIGHT)
        want = torch.cat([ops.mul_mat(W, x[i:i + 8]) for i in range(0, n, 8)], dim=0)
        L.mq_debug_set_dense_lds(1)
        assert torch.equal(got, want), f"n={n}"
    W.free()


@pytest.mark.parametrize("wtype", [13, 14])
@pytest.mark.parametrize("rows,cols", WIDE)
def test_sibling_types_three_and_four_tiles_equal_the_rows_taken_sixteen_at_a_time(env, rows, cols, wtype):
    """Q5_K single matrices wherever Q4_K ones take three and four tiles, Q6_K ones except in runs of an odd number of
    stages (4096 x 4096: runs of one); otherwise the 16-row passes (the same bits) or, from 48 rows, the GEMM."""
    torch, _lib, ops = env
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("s64", rows, cols, wtype), rows, cols, ggml_type=wtype)
    for n in (33, 40, 48, 64):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s64-x", rows, cols, n), (n, cols))).cuda()
        whole, split = ops.mul_mat(W, x), _sixteen_at_a_time(lambda t: ops.mul_mat(W, t), x)
        if not torch.equal(whole, split):
            assert torch.equal(whole, ops.gemm(W, x)), f"n={n}: neither the tiles of sixteen nor the GEMM"
            assert (whole - split).abs().max().item() <= 1e-5 * split.abs().max().item(), f"n={n}"
    # the shapes that must take the tiles (not the one with a wavefront per row tile, nor the one whose tiles do not fit LDS)
    if (rows, cols) not in ((2048, 6144), (20480, 1024)) and (wtype == 13 or (rows, cols) != (4096, 4096)):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s64-x", rows, cols, 64), (64, cols))).cuda()
        assert torch.equal(ops.mul_mat(W, x), _sixteen_at_a_time(lambda t: ops.mul_mat(W, t), x))
    W.free()


@pytest.mark.parametrize("wtype", [13, 14])
@pytest.mark.parametrize("rows,cols", [(14336, 4096), (1024, 4096), (3000, 2048), (512, 8192)])
@pytest.mark.parametrize("silu", [0, 2])
def test_sibling_types_gate_up_same_bits(env, rows, cols, silu, wtype):
    torch, _lib, ops = env
    L = _lib.lib()
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("s16q5-g", rows, cols, wtype), rows, cols, ggml_type=wtype)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("s16q5-u", rows, cols, wtype), rows, cols, ggml_type=wtype)
    for n in (9, 16, 17, 32):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("s16q5-gx", rows, cols, n), (n, cols))).cuda()
        got = ops.swiglu_mul_mat(G, U, x, silu)
        L.mq_debug_set_dense_lds(TWO_TILES_OF_EIGHT)
        want = torch.cat([ops.swiglu_mul_mat(G, U, x[i:i + 8], silu) for i in range(0, n, 8)], dim=0)
        L.mq_debug_set_dense_lds(1)
        # (8192 columns: the two tiles of a Q5_K / Q6_K pair do not fit LDS in one run -- 16-row passes, the same bits)
        assert torch.equal(got, want), f"n={n}"
    G.free(), U.free()


@pytest.mark.parametrize("wtype", [13, 14])
def test_sibling_types_against_the_oracle(env, wtype):
    torch, _lib, ops = env
    rows, cols = 1000, 2048
    make, mul, mag_of = ((synth.q5k_matrix, orc.mul_mat_q5k_q8k, orc.q5k_dot_dequant_f64) if wtype == 13 else
                         (synth.q6k_matrix, orc.mul_mat_q6k_q8k, orc.q6k_dot_dequant_f64))
    w = make(synth.tensor_seed("s16q5-o", wtype), rows, cols)
    W = ops.Q4KWeight.from_ggml(w, cols, ggml_type=wtype)
    for n in (12, 29):
        x = synth.normal_f32(synth.tensor_seed("s16q5-ox", n), (n, cols))
        q8 = orc.quantize_rows_q8k(x)
        got = ops.mul_mat(W, torch.from_numpy(x).cuda()).cpu().numpy()
        mag = mag_of(w, cols, q8, magnitude=True)
        for order in orc.ORDERS.values():
            assert_fp32_parity(got, mul(w, cols, q8, order), mag, f"n={n} order {order}")
    W.free()


@pytest.mark.parametrize("wtype", [12, 14])
def test_output_projection_sized_matrix(env, wtype):
    """128,256 x 4,096 (a vocabulary's output projection, Q6_K in a Q4_K_M file): more than 1,024 row tiles, a wavefront
    per row tile.  Nine to 32 rows are one and two tiles of sixteen -- the bits of the passes of eight --, from 33 the GEMM."""
    torch, _lib, ops = env
    L = _lib.lib()
    rows, cols = 128256, 4096
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("lmhead", wtype), rows, cols, ggml_type=wtype)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("lmhead-x"), (40, cols))).cuda()
    for n in (12, 16, 27):
        got = ops.mul_mat(W, x[:n])
        L.mq_debug_set_dense_lds(TWO_TILES_OF_EIGHT)
        want = torch.cat([ops.mul_mat(W, x[i:min(i + 8, n)]) for i in range(0, n, 8)], dim=0)
        L.mq_debug_set_dense_lds(1)
        assert torch.equal(got, want), f"n={n}"
    assert torch.equal(ops.mul_mat(W, x), ops.gemm(W, x))
    W.free()
