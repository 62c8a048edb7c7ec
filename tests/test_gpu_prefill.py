"""The matrix-core prefill GEMM (mq_gemm_q4k) against the oracle and against the decode kernel.

Reference counterpart: RunQ4KRawBatchedDenseGemm behind MatMulGgmlQuantizedTransB
(core/src/backend/cpu_backend_q4k_dense.cpp:57-101); its own test compares with the dequantized
double-precision dot at 1e-4 (core/tests/test_moe_ops.cpp:170-201,428-430), as assert_fp32_parity does."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("n", [1, 5, 16, 17, 130, 200])
@pytest.mark.parametrize("rows,cols", [(48, 256), (272, 1024), (40, 512)])
def test_gemm_matches_oracle(ops, n, rows, cols):
    w = synth.q4k_matrix(synth.tensor_seed("pf-w", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("pf-x", n, cols), (n, cols))
    W = ops.Q4KWeight.from_ggml(w, cols)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    q8 = orc.quantize_rows_q8k(x)
    mag = orc.dot_magnitude_f64(w, cols, q8)
    for name, order in orc.ORDERS.items():
        assert_fp32_parity(got, orc.mul_mat_q4k_q8k(w, cols, q8, order), mag, f"order={name}")
    assert_fp32_parity(got, orc.dot_dequant_f64(w, cols, q8), mag, "dequantized double")
    W.free()


def test_gemm_extreme_codes_do_not_overflow_the_byte_digits(ops):
    """All nibbles 15, scales and mins 63, activations +-max: the largest (s1*q4) and (s0*q4) bytes
    (105), the largest sub-block code sums (+-4064 -> digits h = +-32, l = 0..127) and the largest
    int32 sums of a super-block."""
    rows, cols, n = 32, 512, 40
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(0.005).tobytes(), np.uint8)
    blk[4:16] = 0xFF
    blk[16:] = 0xFF
    w = np.tile(blk, (rows, cols // 256))
    x = np.ones((n, cols), np.float32)
    x[1::2] *= -1.0            # every code -127 / +127
    x[2, ::2] *= -1.0          # alternating signs: sub-block sums of 0
    x[3, :300] = 0.0
    W = ops.Q4KWeight.from_ggml(w, cols)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    q8 = orc.quantize_rows_q8k(x)
    ref = orc.mul_mat_q4k_q8k(w, cols, q8, orc.ORDER_SCALAR)
    assert_fp32_parity(got, ref, orc.dot_magnitude_f64(w, cols, q8), "extremes")
    W.free()


@pytest.mark.parametrize("n", [3, 64, 150])
def test_gemm_integer_sums_are_exact(ops, n):
    """With d = dmin = 1 and integer activations whose largest magnitude per block is 127, the Q8_K codes
    are the activations themselves (scale +-1) and every fp32 operation of the kernel is exact, so the
    output must EQUAL sum_b yd_b * (dot_scaled_b - min_dot_b) built from the oracle's integers: a single
    wrong unit in either integer sum of any super-block shows up."""
    rows, cols = 80, 768
    nb = cols // 256
    w = synth.q4k_matrix(synth.tensor_seed("pf-int", rows), rows, cols).reshape(rows, nb, 144).copy()
    w[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w[:, :, 2:4] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w = w.reshape(rows, nb * 144)
    rng = np.random.default_rng(n)
    x = rng.integers(-127, 128, size=(n, cols)).astype(np.float32)
    x.reshape(n, nb, 256)[:, :, 7] = rng.choice([-127.0, 127.0], size=(n, nb))
    q8 = orc.quantize_rows_q8k(x)
    d, qs, _ = orc.split_q8k(q8)
    assert np.all(np.abs(d) == 1.0) and np.array_equal(qs.reshape(n, cols) * d.repeat(256, axis=1), x)
    ds, md = orc.matrix_block_sums(w, cols, q8)            # [rows, n, nb]
    want = ((ds.astype(np.int64) - md.astype(np.int64)) * d.astype(np.int64)[None]).sum(axis=2).T
    assert np.abs(want).max() < 2 ** 24
    W = ops.Q4KWeight.from_ggml(w, cols)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, want.astype(np.float32))
    W.free()


def test_gemm_agrees_with_decode_kernel_and_dispatch(ops):
    import torch
    rows, cols, n = 512, 2048, 96
    W = ops.Q4KWeight.synthetic(77, rows, cols)
    x = cu(synth.normal_f32(78, (n, cols)))
    big = ops.gemm(W, x)
    assert torch.equal(ops.mul_mat(W, x), big)          # n >= 48 is routed to the GEMM kernel
    small = torch.cat([ops.mul_mat(W, x[i:i + 16]) for i in range(0, n, 16)])
    scale = small.abs().max().item()
    assert (big - small).abs().max().item() <= 1e-5 * scale   # same integers, fp32 rounding only
    # strided input rows and a padded output are honoured
    xp = torch.zeros((n, cols + 256), device="cuda")
    xp[:, :cols] = x
    assert torch.equal(ops.gemm(W, xp[:, :cols]), big)
    W.free()


@pytest.mark.parametrize("rows,cols,n", [(64, 4096, 50), (48, 14336, 130), (272, 2048, 33), (4096, 14336, 48)])
def test_gemm_with_k_in_runs_matches_oracle_and_decode_kernel(ops, rows, cols, n):
    """Few weight rows and a long K: the launch splits K into runs of super-blocks whose sums are added in order by
    a second launch (64 x 4096: four runs; 48 x 14336: fourteen; 272 x 2048: two; 4096 x 14336 at 48 rows: eight).
    Against the oracle on a sample of weight rows, and against the decode kernel on all of them."""
    import torch
    w = synth.q4k_matrix(synth.tensor_seed("pf-split", rows, cols), rows, cols)
    x = synth.normal_f32(synth.tensor_seed("pf-split-x", n, cols), (n, cols))
    W = ops.Q4KWeight.from_ggml(w, cols)
    got = ops.gemm(W, cu(x))
    small = torch.cat([ops.mul_mat(W, cu(x[i:i + 16])) for i in range(0, n, 16)])
    scale = small.abs().max().item()
    assert (got - small).abs().max().item() <= 1e-5 * scale
    pick = np.unique(np.concatenate([np.arange(0, rows, max(1, rows // 40)), [rows - 1]]))
    q8 = orc.quantize_rows_q8k(x)
    ref = orc.mul_mat_q4k_q8k(w[pick], cols, q8, orc.ORDER_SCALAR)
    assert_fp32_parity(got.cpu().numpy()[:, pick], ref, orc.dot_magnitude_f64(w[pick], cols, q8), "K in runs")
    # a padded output keeps its padding
    yp = torch.full((n, rows + 8), 7.0, device="cuda")
    ops.gemm(W, cu(x), out=yp[:, :rows])
    assert torch.equal(yp[:, :rows], got) and bool((yp[:, rows:] == 7.0).all())
    W.free()


def test_gemm_integer_sums_are_exact_with_k_in_runs(ops):
    """The exactness construction of test_gemm_integer_sums_are_exact on a shape whose K is split (32 rows x 4096
    columns: four runs of four super-blocks): every partial sum is an integer below 2^24, so the planes add exactly."""
    rows, cols, n = 32, 4096, 20
    nb = cols // 256
    w = synth.q4k_matrix(synth.tensor_seed("pf-int-split", rows), rows, cols).reshape(rows, nb, 144).copy()
    w[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w[:, :, 2:4] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w[:, :, 4:16] &= 0x1F   # scales and mins below 32: the sixteen super-block sums stay below 2^24 in all
    w = w.reshape(rows, nb * 144)
    rng = np.random.default_rng(5)
    x = rng.integers(-127, 128, size=(n, cols)).astype(np.float32)
    x.reshape(n, nb, 256)[:, :, 7] = rng.choice([-127.0, 127.0], size=(n, nb))
    q8 = orc.quantize_rows_q8k(x)
    d, qs, _ = orc.split_q8k(q8)
    assert np.all(np.abs(d) == 1.0)
    ds, md = orc.matrix_block_sums(w, cols, q8)
    want = ((ds.astype(np.int64) - md.astype(np.int64)) * d.astype(np.int64)[None]).sum(axis=2).T
    assert np.abs(want).max() < 2 ** 24
    W = ops.Q4KWeight.from_ggml(w, cols)
    got = ops.gemm(W, cu(x)).cpu().numpy()
    assert np.array_equal(got, want.astype(np.float32))
    W.free()


def test_large_matrices_take_the_gemm_beyond_the_widths_of_the_decode_kernels(ops):
    """24 MB of weights and more: Q4_K rows up to 64 stay on the decode arithmetic (up to four tiles of sixteen per weight
    tile: a row's result is the one it has when the rows are handed over sixteen at a time, bit for bit); from 65 rows
    mul_mat hands them to the matrix-core GEMM (matrices whose rows do not pass through LDS that way from 33; Q5_K
    and Q6_K matrices as Q4_K ones, Q6_K not in runs of an odd number of stages)."""
    import torch
    W = ops.Q4KWeight.synthetic(4, 14336, 4096)
    x = torch.randn((70, 4096), device="cuda", generator=torch.Generator(device="cuda").manual_seed(20))
    pieces = lambda t: torch.cat([ops.mul_mat(W, t[i:i + 16]) for i in range(0, t.shape[0], 16)])
    assert torch.equal(ops.mul_mat(W, x[:20]), pieces(x[:20]))
    assert torch.equal(ops.mul_mat(W, x[:40]), pieces(x[:40]))
    big = ops.gemm(W, x)
    assert torch.equal(ops.mul_mat(W, x), big)
    small = pieces(x)
    assert (big - small).abs().max().item() <= 1e-5 * small.abs().max().item()
    W.free()
    W = ops.Q4KWeight.synthetic(7, 4096, 14336)   # 56 super-blocks, seven per wavefront: two tiles read from global memory, then the GEMM
    x = torch.randn((40, 14336), device="cuda", generator=torch.Generator(device="cuda").manual_seed(23))
    assert torch.equal(ops.mul_mat(W, x[:30]), torch.cat([ops.mul_mat(W, x[:16]), ops.mul_mat(W, x[16:30])]))
    assert torch.equal(ops.mul_mat(W, x), ops.gemm(W, x))
    W.free()
    # the other types: Q5_K like Q4_K (up to four tiles of sixteen, then the GEMM); Q6_K likewise except where the tiles would
    # pass through LDS in runs of an odd number of stages (4096 x 4096: runs of one): two tiles, then 16-row passes up to 47 rows
    x = torch.randn((70, 4096), device="cuda", generator=torch.Generator(device="cuda").manual_seed(22))
    pieces = lambda t: torch.cat([ops.mul_mat(W, t[i:i + 16]) for i in range(0, t.shape[0], 16)])
    for rows in (4096, 14336):
        W = ops.Q4KWeight.synthetic(6, rows, 4096, ggml_type=synth.GGML_TYPE_Q5_K)
        assert torch.equal(ops.mul_mat(W, x[:20]), pieces(x[:20]))
        assert torch.equal(ops.mul_mat(W, x[:48]), pieces(x[:48]))
        assert torch.equal(ops.mul_mat(W, x), ops.gemm(W, x))
        assert torch.equal(ops.mul_mat(W, x[:16]), torch.cat([ops.mul_mat(W, x[:8]), ops.mul_mat(W, x[8:16])]))
        W.free()
    W = ops.Q4KWeight.synthetic(6, 4096, 4096, ggml_type=synth.GGML_TYPE_Q6_K)
    assert torch.equal(ops.mul_mat(W, x[:40]), pieces(x[:40]))
    assert torch.equal(ops.mul_mat(W, x[:48]), ops.gemm(W, x[:48]))
    W.free()
    W = ops.Q4KWeight.synthetic(8, 14336, 4096, ggml_type=synth.GGML_TYPE_Q6_K)   # (runs of four stages: up to four tiles)
    assert torch.equal(ops.mul_mat(W, x[:33]), pieces(x[:33]))
    assert torch.equal(ops.mul_mat(W, x[:64]), pieces(x[:64]))
    assert torch.equal(ops.mul_mat(W, x), ops.gemm(W, x))
    assert torch.equal(ops.mul_mat(W, x[:16]), torch.cat([ops.mul_mat(W, x[:8]), ops.mul_mat(W, x[8:16])]))
    W.free()
    W = ops.Q4KWeight.synthetic(5, 4096, 4096)
    x = torch.randn((20, 4096), device="cuda", generator=torch.Generator(device="cuda").manual_seed(21))
    assert torch.equal(ops.mul_mat(W, x), torch.cat([ops.mul_mat(W, x[:16]), ops.mul_mat(W, x[16:])]))
    W.free()


@pytest.mark.parametrize("m", [512, 2048])
def test_gemm_full_size_rows_against_decode_kernel(ops, m):
    """W 4096 -> 14336 at M = 512 / 2048: every 37th activation row is recomputed by the decode kernel,
    whose integer sums are pinned bit-exactly elsewhere; plus linearity in the activations' sign."""
    import torch
    rows, cols = 14336, 4096
    W = ops.Q4KWeight.synthetic(4, rows, cols)
    g = torch.Generator(device="cuda").manual_seed(m)
    x = torch.randn((m, cols), device="cuda", generator=g)
    y = ops.gemm(W, x)
    pick = torch.arange(0, m, 37, device="cuda")
    ref = torch.cat([ops.mul_mat(W, x[pick[i:i + 16]]) for i in range(0, len(pick), 16)])
    scale = ref.abs().max().item()
    assert (y[pick] - ref).abs().max().item() <= 1e-5 * scale
    # Q8_K quantization is odd (codes and scale flip sign together), so the product is too, exactly
    assert torch.equal(ops.gemm(W, -x), -y)
    W.free()


@pytest.mark.parametrize("m", [512, 2048])
def test_gemm_full_size_sampled_rows_against_the_oracle(ops, m):
    """W 4096 -> 14336 at M = 512 / 2048 against the CPU restatement itself: every 61st activation row (and the last)
    over all 14336 outputs, the AVX2-order build for speed plus the Highway order on two of them."""
    import torch
    rows, cols = 14336, 4096
    W = ops.Q4KWeight.synthetic(4, rows, cols)
    w = W.to_ggml()
    x = synth.normal_f32(synth.tensor_seed("pf-full", m), (m, cols))
    y = ops.gemm(W, cu(x)).cpu().numpy()
    pick = sorted(set(range(0, m, 61)) | {m - 1})
    q8 = orc.quantize_rows_q8k(x[pick])
    ref = orc.simd_mul_mat_q4k_q8k(w, cols, q8, 8)
    mag = np.stack([orc.dot_magnitude_f64(w, cols, q8[i:i + 1])[0] for i in range(len(pick))])
    assert_fp32_parity(y[pick], ref, mag, "sampled rows (AVX2 order)")
    assert_fp32_parity(y[pick[:2]], orc.mul_mat_q4k_q8k(w, cols, q8[:2], orc.ORDER_HWY), mag[:2], "Highway order")
    W.free()


@pytest.mark.parametrize("n,E,K", [(400, 16, 4), (300, 10, 8), (1030, 24, 3)])
def test_rows_quantized_once_and_copied_to_their_groups_give_the_bits_of_rows_quantized_per_slot(ops, n, E, K):
    """mul_mat_id at a width that takes the expert-grouped GEMM.  With one activation row per token the row is
    quantized once and its codes are copied to every group it is routed to; with the same rows replicated per slot by
    the caller every (token, slot) row is quantized by itself.  Same quantizer, same codes: the outputs must agree bit
    for bit (ragged token counts, a last tile of padding rows, ids outside the expert range)."""
    import torch
    rows, cols = 64, 1024
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("once-w", n, E), rows, cols, E)
    x = synth.normal_f32(synth.tensor_seed("once-x", n, cols), (n, cols))
    rng = np.random.default_rng(synth.tensor_seed("once-ids", n, E, K) & 0xffffffff)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(n)]).astype(np.int32)
    ids[3, 0] = -1
    ids[n - 1, K - 1] = E + 5
    xd, idd = cu(x), cu(ids)
    once = ops.mul_mat_id(W, xd, idd).cpu().numpy()
    per_slot = ops.mul_mat_id(W, xd[:, None, :].expand(n, K, cols).contiguous(), idd).cpu().numpy()
    assert np.array_equal(once.view(np.uint32), per_slot.view(np.uint32))
    assert not np.any(once[3, 0]) and not np.any(once[n - 1, K - 1])
    # and against the oracle on a sample of pairs
    w_np = W.to_ggml()
    q8 = orc.quantize_rows_q8k(x)
    for t, k in ((0, 0), (7, K - 1), (n - 2, 1), (n // 2, 0)):
        e = int(ids[t, k])
        ref = orc.mul_mat_q4k_q8k(w_np[e], cols, q8[t:t + 1], orc.ORDERS["avx2"])
        mag = orc.dot_magnitude_f64(w_np[e], cols, q8[t:t + 1])
        assert_fp32_parity(once[t, k][None], ref, mag, f"pair ({t}, {k})")
    W.free()


def _with_pair(on):
    from densecore_amd import _lib
    _lib.lib().mq_debug_set_dense_lds(1 if on else 9)  # bit 3: gate and up as two GEMM launches and a SwiGLU pass


@pytest.mark.parametrize("n", [48, 130, 512, 1000])
@pytest.mark.parametrize("silu", [0, 1, 2])
def test_pair_gemm_of_gate_and_up_gives_the_bits_of_two_launches_and_a_swiglu_pass(ops, n, silu):
    """Dense FFN and SwiGLU product at prefill widths: one GEMM launch whose epilogue stores silu(gate) * up against the
    two launches + SwiGLU pass it replaces (the same accumulators, the same SiLU function on the same values)."""
    import torch
    hidden, inter = 1024, 2560
    G = ops.Q4KWeight.synthetic(synth.tensor_seed("pair-g"), inter, hidden)
    U = ops.Q4KWeight.synthetic(synth.tensor_seed("pair-u"), inter, hidden)
    D = ops.Q4KWeight.synthetic(synth.tensor_seed("pair-d"), hidden, inter)
    x = cu(synth.normal_f32(synth.tensor_seed("pair-x", n), (n, hidden)))
    try:
        _with_pair(True)
        h1 = ops.swiglu_mul_mat(G, U, x, silu).cpu().numpy()
        y1 = ops.ffn_swiglu(G, U, D, x, silu).cpu().numpy()
        _with_pair(False)
        h0 = ops.swiglu_mul_mat(G, U, x, silu).cpu().numpy()
        y0 = ops.ffn_swiglu(G, U, D, x, silu).cpu().numpy()
    finally:
        _with_pair(True)
    assert np.array_equal(h1.view(np.uint32), h0.view(np.uint32))
    assert np.array_equal(y1.view(np.uint32), y0.view(np.uint32))
    for w in (G, U, D):
        w.free()


@pytest.mark.parametrize("n,down_type", [(300, synth.GGML_TYPE_Q4_K), (520, synth.GGML_TYPE_Q6_K), (300, synth.GGML_TYPE_Q8_0)])
def test_pair_gemm_in_the_moe_block_gives_the_bits_of_two_launches(ops, n, down_type):
    """The expert-grouped form, in the MoE layer (rows in the plan's order for a GEMM down product, scattered to their
    (token, slot) places for a down stack with a kernel of its own) and in the gate/up entry point, shared expert included."""
    import torch
    E, H, I, K = 12, 1024, 512, 4
    ge = ops.Q4KWeight.synthetic(synth.tensor_seed("pairm-g"), I, H, E)
    ue = ops.Q4KWeight.synthetic(synth.tensor_seed("pairm-u"), I, H, E)
    de = ops.Q4KWeight.synthetic(synth.tensor_seed("pairm-d", down_type), H, I, E, down_type)
    sh = (ops.Q4KWeight.synthetic(synth.tensor_seed("pairm-sg"), I, H), ops.Q4KWeight.synthetic(synth.tensor_seed("pairm-su"), I, H),
          ops.Q4KWeight.synthetic(synth.tensor_seed("pairm-sd", down_type), H, I, 1, down_type),
          cu(synth.normal_f32(synth.tensor_seed("pairm-gi"), (H,)) * np.float32(0.02)))
    x = cu(synth.normal_f32(synth.tensor_seed("pairm-x", n), (n, H)))
    lg = cu(synth.normal_f32(synth.tensor_seed("pairm-l", n), (n, E)))
    out = {}
    try:
        for on in (True, False):
            _with_pair(on)
            y, ids, wts = ops.moe_layer(ge, ue, de, x, lg, K, shared=sh, silu=ops.SILU_FAST)
            h = ops.moe_gateup_swiglu(ge, ue, x, ids, ops.SILU_FAST)
            out[on] = (y.cpu().numpy(), h.cpu().numpy(), ids.cpu().numpy())
    finally:
        _with_pair(True)
    assert np.array_equal(out[True][2], out[False][2])
    assert np.array_equal(out[True][1].view(np.uint32), out[False][1].view(np.uint32))
    assert np.array_equal(out[True][0].view(np.uint32), out[False][0].view(np.uint32))
    for w in (ge, ue, de) + sh[:3]:
        w.free()


@pytest.mark.parametrize("n,E,K,down_type", [(300, 12, 4, synth.GGML_TYPE_Q4_K), (700, 64, 8, synth.GGML_TYPE_Q6_K), (260, 20, 2, synth.GGML_TYPE_Q5_K)])
def test_items_of_two_four_and_eight_tiles_give_the_same_bits(ops, n, E, K, down_type):
    """The expert-grouped GEMM cuts an expert's rows into items of two, four or eight 16-row tiles (chosen by the rows per
    expert); an output's accumulator walks K the same way in both, so the MoE block must not change by a bit -- gate/up
    in the pair form and as single products, down of every type, experts with more rows than an item."""
    from densecore_amd import _lib
    E_, H, I = E, 1024, 512
    ge = ops.Q4KWeight.synthetic(synth.tensor_seed("mt-g", E), I, H, E_)
    ue = ops.Q4KWeight.synthetic(synth.tensor_seed("mt-u", E), I, H, E_)
    de = ops.Q4KWeight.synthetic(synth.tensor_seed("mt-d", E, down_type), H, I, E_, down_type)
    x = cu(synth.normal_f32(synth.tensor_seed("mt-x", n), (n, H)))
    lg = cu(synth.normal_f32(synth.tensor_seed("mt-l", n, E), (n, E_)))
    out = {}
    try:
        for mode in (1 | (2 << 8), 1 | (4 << 8), 1 | (8 << 8), 9 | (2 << 8), 9 | (4 << 8), 1):
            _lib.lib().mq_debug_set_dense_lds(mode)
            y, ids, wts = ops.moe_layer(ge, ue, de, x, lg, K, silu=ops.SILU_FAST)
            yk = ops.mul_mat_id(ge, x, ids)
            out[mode] = (y.cpu().numpy(), yk.cpu().numpy())
    finally:
        _lib.lib().mq_debug_set_dense_lds(1)
    ref = out[1 | (8 << 8)]
    for mode, got in out.items():
        assert np.array_equal(got[0].view(np.uint32), ref[0].view(np.uint32)), f"layer, mode {mode}"
        assert np.array_equal(got[1].view(np.uint32), ref[1].view(np.uint32)), f"mul_mat_id, mode {mode}"
    for w in (ge, ue, de):
        w.free()
