"""Integer sums of EVERY decode kernel pinned through the public entry points by an exactness construction.

Weights get d = +-2^a and dmin = +-2^b (any sign, fp16 subnormals included) and the activations are small integers
whose largest magnitude in every super-block is exactly 127.  Then the Q8_K codes are the activations themselves
with a block scale of +-1, and every fp32 operation of the kernels -- d * yd, the products with the two integer sums,
their difference, the accumulation over the super-blocks, the reduction across wavefronts, routing weights that are
powers of two -- is exact whatever its order.  The output must therefore EQUAL
    sum_b yd_b * (d * dot_scaled_b - dmin * min_dot_b)
built from the CPU restatement's integers (orc.matrix_block_sums, itself pinned by an int64 brute force in
tests/test_oracle_pins.py): one wrong unit in either integer sum of any super-block of any row changes the result.
The polynomial SiLU flavours are plain fp32 arithmetic in a fixed order, so after an exact gate and up product the
SwiGLU output is compared bit for bit as well.

Kernels reached: the expert-grouped matmul_kernel (mq_mul_mat_id_q4k, the gate/up node, the down node above eight
tokens), moe_gateup_token_kernel and moe_down_token_kernel (mq_moe_layer_q4k / the down node up to eight tokens),
gemv1_fused / gemvn_fused and their norm forms (short rows, 1..4 tokens), the XQ and J = 1 forms of the dense kernel
(one token, long rows), the two-token-tile form (9..16 tokens), and the persistent decoder-layer kernel phase by phase.
"""
import ctypes as C

import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc

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


def f16_bytes(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def exact_matrix(seed, rows, cols, d=1.0, dmin=1.0, alternate_signs=False):
    """Seeded Q4_K rows with every block's d, dmin set to the given powers of two (row-alternating signs on request)."""
    nb = cols // 256
    w = synth.q4k_matrix(seed, rows, cols).reshape(rows, nb, 144).copy()
    w[:, :, 0:2] = f16_bytes(d)
    w[:, :, 2:4] = f16_bytes(dmin)
    if alternate_signs:
        w[1::2, :, 0:2] = f16_bytes(-d)
        w[::3, :, 2:4] = f16_bytes(-dmin)
    return w.reshape(rows, nb * 144)


def exact_acts(seed, shape, small=15):
    """Integers in [-small, small] with one +-127 per super-block (position varies), as fp32."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-small, small + 1, size=shape).astype(np.float32)
    blocks = x.reshape(-1, 256)
    pos = rng.integers(0, 256, size=blocks.shape[0])
    blocks[np.arange(blocks.shape[0]), pos] = rng.choice([-127.0, 127.0], size=blocks.shape[0])
    return x


def expected(w, cols, x):
    """sum_b yd_b (d ds_b - dmin md_b) in float64 from the oracle's integers -> [n, rows]; asserts the construction."""
    rows, nb, n = w.shape[0], cols // 256, x.shape[0]
    q8 = orc.quantize_rows_q8k(x)
    yd, qs, _ = orc.split_q8k(q8)
    assert np.all(np.abs(yd) == 1.0) and np.array_equal(qs.reshape(n, cols) * yd.repeat(256, axis=1), x)
    ds, md = orc.matrix_block_sums(w, cols, q8)                      # [rows, n, nb]
    blk = w.reshape(rows, nb, 144)
    d = blk[:, :, 0:2].copy().view(np.float16).astype(np.float64).reshape(rows, 1, nb)
    dm = blk[:, :, 2:4].copy().view(np.float16).astype(np.float64).reshape(rows, 1, nb)
    terms = (d * ds - dm * md) * yd.astype(np.float64)[None]
    want = terms.sum(axis=2).T
    # exactness of every partial sum: all terms are multiples of one power of two and stay below 2^24 of them
    unit = min(v for v in (np.abs(d[d != 0]).min(initial=np.inf), np.abs(dm[dm != 0]).min(initial=np.inf)))
    assert np.abs(terms).sum(axis=2).max() / unit < 2 ** 24
    return want


def assert_equal_exact(got, want, what):
    got = np.asarray(got)
    assert got.dtype == np.float32
    assert np.array_equal(got.astype(np.float64), want), f"{what}: {np.abs(got - want).max()} off"


# d and dmin stay within a few powers of two of each other (d * dot_scaled - dmin * min_dot must fit 24 bits);
# signs alternate over the rows, 2^-17 and 2^-24 are fp16 subnormals, 1024 a large half
SCALES = [(1.0, 1.0, False), (2.0 ** -17, 2.0 ** -15, True), (1024.0, 512.0, True), (2.0 ** -24, 2.0 ** -23, True)]


@pytest.mark.parametrize("d,dmin,alt", SCALES)
@pytest.mark.parametrize("rows,cols,n", [(2048, 2048, 1), (2048, 2048, 2), (2048, 2048, 3), (2048, 2048, 4),
                                         (272, 1024, 4), (64, 14336, 1), (1000, 4608, 1), (512, 2048, 8),
                                         (256, 4096, 16), (96, 768, 11)])
def test_dense_product_is_exact(ops, rows, cols, n, d, dmin, alt):
    """gemv1_fused (n = 1) and gemvn_fused (2..4) on short rows, the quantizer-inside form of the dense kernel on
    long rows, the plain and the two-token-tile forms."""
    w = exact_matrix(synth.tensor_seed("ex-w", rows, cols), rows, cols, d, dmin, alt)
    x = exact_acts(rows + n, (n, cols))
    W = ops.Q4KWeight.from_ggml(w, cols)
    assert_equal_exact(ops.mul_mat(W, cu(x)).cpu().numpy(), expected(w, cols, x), "mul_mat")
    W.free()


@pytest.mark.parametrize("n", [1, 2, 4, 8])
def test_norm_inside_the_product_is_exact(ops, n):
    """mq_rmsnorm_mul_mat_q4k (gemv1_norm_fused, gemvn_fused with the norm, norm + product launches at 8 rows): rows
    of +-1 have mean square 1, so with eps = 0 the normalised row is +-weight: integers again."""
    import torch
    from densecore_amd import _lib
    rows, cols = 2560, 2048
    w = exact_matrix(synth.tensor_seed("ex-norm"), rows, cols, 2.0 ** -3, 2.0 ** -1, True)
    rng = np.random.default_rng(n)
    x = rng.choice([-1.0, 1.0], size=(n, cols)).astype(np.float32)
    delta = np.zeros((n, cols), np.float32)
    flip = rng.random((n, cols)) < 0.25
    delta[flip] = -2.0 * x[flip]                                     # x + delta is +-1 as well
    weight = exact_acts(77, (1, cols))[0]
    W = ops.Q4KWeight.from_ggml(w, cols)
    xd, dd, wd = cu(x), cu(delta), cu(weight)
    s_out = torch.empty((n, cols), device="cuda")
    y = torch.empty((n, rows), device="cuda")
    _lib.check(_lib.lib().mq_rmsnorm_mul_mat_q4k(W._h, C.c_void_p(xd.data_ptr()), C.c_void_p(dd.data_ptr()), C.c_void_p(wd.data_ptr()),
                                                 n, C.c_float(0.0), C.c_void_p(s_out.data_ptr()), C.c_void_p(y.data_ptr()), rows,
                                                 C.c_void_p(torch.cuda.current_stream().cuda_stream)), "mq_rmsnorm_mul_mat_q4k")
    assert np.array_equal(s_out.cpu().numpy(), x + delta)
    assert_equal_exact(y.cpu().numpy(), expected(w, cols, (x + delta) * weight[None]), "norm + product")
    W.free()


def make_exact_experts(tag, E, rows, cols, d, dmin):
    return np.stack([exact_matrix(synth.tensor_seed(tag, e), rows, cols, d, dmin, True) for e in range(E)])


@pytest.mark.parametrize("n", [1, 4, 16, 40])
def test_mul_mat_id_is_exact(ops, n):
    """The expert-grouped kernel (groups of one row and of several, one wavefront per row tile and more)."""
    E, H, I, K = 12, 2048, 512, 4
    ge = make_exact_experts("ex-id-g", E, I, H, 1.0, 2.0 ** -2)
    de = make_exact_experts("ex-id-d", E, H, I, 2.0 ** -16, 2.0 ** -16)
    GE, DE = ops.Q4KWeight.from_ggml(ge, H), ops.Q4KWeight.from_ggml(de, I)
    ids, _ = orc.route_topk(synth.normal_f32(synth.tensor_seed("ex-id-l", n), (n, E)), K, 0)
    x = exact_acts(n, (n, H))
    xk = exact_acts(100 + n, (n, K, I))
    y = ops.mul_mat_id(GE, cu(x), cu(ids)).cpu().numpy()
    yk = ops.mul_mat_id(DE, cu(xk), cu(ids)).cpu().numpy()
    for t in range(n):
        for k in range(K):
            assert_equal_exact(y[t, k][None], expected(ge[ids[t, k]], H, x[t:t + 1]), f"gate t{t} k{k}")
            assert_equal_exact(yk[t, k][None], expected(de[ids[t, k]], I, xk[t, k][None]), f"down t{t} k{k}")
    GE.free(), DE.free()


@pytest.mark.parametrize("n", [1, 3, 8, 16, 33])
def test_down_node_with_power_of_two_weights_is_exact(ops, n):
    """moe_down_token_kernel up to eight tokens (hidden rows quantized inside), the expert-grouped launch and the
    combine above; routing weights 2^-k, one of them zero (skipped), so the k-ordered sum is exact too."""
    E, H, I, K = 16, 1024, 512, 8
    de = make_exact_experts("ex-dn", E, H, I, 2.0 ** -4, 2.0 ** -4)
    DE = ops.Q4KWeight.from_ggml(de, I)
    ids, _ = orc.route_topk(synth.normal_f32(synth.tensor_seed("ex-dn-l", n), (n, E)), K, 0)
    hid = exact_acts(n, (n, K, I))
    wts = np.tile(np.array([1.0, 0.5, 0.25, 0.5, 1.0, 0.0, 0.25, 0.125], np.float32), (n, 1))
    y = ops.moe_down_weighted(DE, cu(hid), cu(ids), cu(wts)).cpu().numpy()
    want, total = np.zeros((n, H)), np.zeros((n, H))
    for t in range(n):
        for k in range(K):
            part = expected(de[ids[t, k]], I, hid[t, k][None])[0]
            want[t] += float(wts[t, k]) * part
            total[t] += float(wts[t, k]) * np.abs(part)
    assert total.max() / (2.0 ** -4 * 0.125) < 2 ** 24       # every partial sum of the k-ordered combine is exact
    assert_equal_exact(y, want, "down node")
    DE.free()


@pytest.mark.parametrize("silu", [1, 2])
@pytest.mark.parametrize("n", [1, 2, 4, 8, 16])
def test_gateup_swiglu_bits_after_exact_products(ops, n, silu):
    """mq_swiglu_mul_mat_q4k (dense), the gate/up node (expert-grouped) and mq_moe_layer_q4k's hidden rows
    (moe_gateup_token_kernel up to eight tokens): gate and up products exact, then the polynomial SiLU in fp32 -- the
    output bit for bit.  d = 2^-17 keeps the gate in the range where the sigmoid is neither 0 nor 1."""
    E, H, I, K = 16, 2048, 512, 8
    ge = make_exact_experts("ex-gu-g", E, I, H, 2.0 ** -17, 2.0 ** -17)
    ue = make_exact_experts("ex-gu-u", E, I, H, 2.0 ** -15, 2.0 ** -16)
    de = make_exact_experts("ex-gu-d", E, H, I, 1.0, 1.0)
    GE, UE, DE = (ops.Q4KWeight.from_ggml(a, c) for a, c in ((ge, H), (ue, H), (de, I)))
    x = exact_acts(n + 7, (n, H))
    logits = synth.normal_f32(synth.tensor_seed("ex-gu-l", n), (n, E))
    ids, _ = orc.route_topk(logits, K, 0)

    def want_rows(g, u, xs):
        a, b = expected(g, H, xs).astype(np.float32), expected(u, H, xs).astype(np.float32)
        L = orc.lib()
        return np.array([[L.orc_silu_mul(float(p), float(q), silu) for p, q in zip(ra, rb)] for ra, rb in zip(a, b)], np.float32)

    want = np.stack([np.stack([want_rows(ge[ids[t, k]], ue[ids[t, k]], x[t:t + 1])[0] for k in range(K)]) for t in range(n)])
    node = ops.moe_gateup_swiglu(GE, UE, cu(x), cu(ids), silu).cpu().numpy()
    assert np.array_equal(node.view(np.uint32), want.view(np.uint32)), "gate/up node"
    _, ids2, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, silu=silu)
    assert np.array_equal(ids2.cpu().numpy(), ids)
    layer_hidden = ops.debug_moe_hidden((n, K, I)).cpu().numpy()
    assert np.array_equal(layer_hidden.view(np.uint32), want.view(np.uint32)), "layer hidden rows"
    G0, U0 = ops.Q4KWeight.from_ggml(ge[0], H), ops.Q4KWeight.from_ggml(ue[0], H)
    dense = ops.swiglu_mul_mat(G0, U0, cu(x), silu).cpu().numpy()
    assert np.array_equal(dense.view(np.uint32), want_rows(ge[0], ue[0], x).view(np.uint32)), "dense swiglu"
    for w in (GE, UE, DE, G0, U0):
        w.free()


def selection_matrix(rows, cols, pick, d=1.0):
    """Q4_K rows with a single weight of d (scale 1, nibble 1) at column pick[r] and zeros elsewhere (mins 0)."""
    nb = cols // 256
    w = np.zeros((rows, nb, 144), np.uint8)
    w[:, :, 0:2] = f16_bytes(d)
    for r in range(rows):
        b, e = divmod(int(pick[r]), 256)
        g, i = divmod(e, 32)                       # sub-block, element
        sc = w[r, b, 4:16]
        if g < 4:
            sc[g] = 1
        else:
            sc[g + 4] = 1                          # low four bits of the scale of sub-blocks 4..7
        w[r, b, 16 + 32 * (g // 2) + i] = 1 << (4 * (g % 2))
    return w.reshape(rows, nb * 144)


@pytest.mark.parametrize("n", [1, 4, 8])
def test_persistent_decoder_layer_phase_by_phase(ops, n):
    """decoder_layers_kernel, one layer, every product phase read from the handle's exchange buffers.

    x = +-1 and eps = 0 make rmsnorm(x) * attn_norm integer (qkv exact).  wqkv's first n_q rows select single
    activations, so the q part of qkv is small integers again and wo's product is exact.  wo . q is made to vanish
    in a second handle (wo = 0), which leaves x + o = +-1 for the FFN norm: the expert gate and up products are exact
    and the hidden rows are compared bit for bit (polynomial SiLU).  The down phase then sees hidden rows that are
    not integers; it is compared bit for bit with the down node (pinned above) on the kernel's own hidden rows, ids
    and weights."""
    import torch
    from densecore_amd import _lib
    hidden, inter, E, K, n_q, n_kv = 512, 256, 16, 4, 512, 128
    L = _lib.lib()
    rng = np.random.default_rng(40 + n)
    x = rng.choice([-1.0, 1.0], size=(n, hidden)).astype(np.float32)
    attn_norm, ffn_norm = exact_acts(41, (1, hidden))[0], exact_acts(42, (1, hidden))[0]
    pick = rng.permutation(hidden)[:n_q] if n_q <= hidden else rng.integers(0, hidden, n_q)
    for b in range(n_q // 256):                    # every super-block of q must hold one +-127 for its Q8_K scale to be 1
        pick[b * 256] = int(np.argmax(np.abs(attn_norm) == 127.0))
    wqkv = np.concatenate([selection_matrix(n_q, hidden, pick), exact_matrix(43, 2 * n_kv, hidden, 2.0 ** -2, 2.0 ** -3, True)])
    wo = exact_matrix(44, hidden, n_q, 2.0 ** -5, 2.0 ** -4, True)
    ge = make_exact_experts("ex-dec-g", E, inter, hidden, 2.0 ** -16, 2.0 ** -17)
    ue = make_exact_experts("ex-dec-u", E, inter, hidden, 2.0 ** -14, 2.0 ** -15)
    de = make_exact_experts("ex-dec-d", E, hidden, inter, 2.0 ** -6, 2.0 ** -7)
    router = synth.normal_f32(45, (E, hidden)) * np.float32(0.05)
    dev = {k: ops.Q4KWeight.from_ggml(v, c) for k, (v, c) in dict(wqkv=(wqkv, hidden), wo=(wo, n_q), wo0=(np.zeros_like(wo), n_q),
                                                                 ge=(ge, hidden), ue=(ue, hidden), de=(de, inter)).items()}
    an, fn, rt, xd = cu(attn_norm), cu(ffn_norm), cu(router), cu(x)

    def run(wo_key):
        table = (_lib.DecoderLayerDesc * 1)()
        table[0].wqkv, table[0].wo = dev["wqkv"]._h, dev[wo_key]._h
        table[0].attn_norm_dev, table[0].ffn_norm_dev, table[0].router_dev = an.data_ptr(), fn.data_ptr(), rt.data_ptr()
        table[0].moe = _lib.MoELayerDesc(dev["ge"]._h, dev["ue"]._h, dev["de"]._h, None, None, None, None, K, 1, ops.ROUTE_FLOOR)
        h = C.c_void_p()
        _lib.check(L.mq_decoder_create(table, 1, n, C.c_float(0.0), C.byref(h)), "mq_decoder_create")
        out = torch.empty((n, hidden), device="cuda")
        ids = torch.empty((1, n, K), dtype=torch.int32, device="cuda")
        wts = torch.empty((1, n, K), device="cuda")
        p = lambda t: C.c_void_p(t.data_ptr())
        _lib.check(L.mq_decoder_step(h, p(xd), n, 1, p(out), p(ids), p(wts), None), "mq_decoder_step")
        _lib.check(L.mq_decoder_status(h), "mq_decoder_status")
        ptrs = [C.c_void_p() for _ in range(5)]
        _lib.check(L.mq_debug_decoder_buffers(h, *[C.byref(q) for q in ptrs]), "mq_debug_decoder_buffers")
        shapes = [(n, n_q + 2 * n_kv), (n, hidden), (n, E), (n, K, inter), (n, hidden)]
        bufs = []
        for q, shp in zip(ptrs, shapes):
            host = np.empty(shp, np.float32)
            _lib.check(L.mq_memcpy_d2h(C.c_void_p(host.ctypes.data), q, host.nbytes), "mq_memcpy_d2h")
            bufs.append(host)
        L.mq_decoder_free(h)
        return bufs, out.cpu().numpy(), ids.cpu().numpy()[0], wts[0]

    h1 = x * attn_norm[None]
    # handle A: qkv and wo phases
    (qkv, o, _, _, _), _, _, _ = run("wo")
    assert_equal_exact(qkv, expected(wqkv, hidden, h1), "qkv phase")
    assert np.array_equal(qkv[:, :n_q], h1[:, pick])
    assert_equal_exact(o, expected(wo, n_q, qkv[:, :n_q]), "wo phase")
    # handle B: wo = 0, the MoE phases
    (_, o0, logits, hid, y), out, ids, wts_t = run("wo0")
    assert not o0.any()
    h2 = x * ffn_norm[None]
    assert np.allclose(logits, h2 @ router.T, rtol=1e-5, atol=1e-4)
    oi, _ = orc.route_topk(logits, K, 1)
    assert np.array_equal(ids, oi)
    Lo = orc.lib()
    for t in range(n):
        for k in range(K):
            e = ids[t, k]
            a = expected(ge[e], hidden, h2[t:t + 1]).astype(np.float32)[0]
            b = expected(ue[e], hidden, h2[t:t + 1]).astype(np.float32)[0]
            want = np.array([Lo.orc_silu_mul(float(p), float(q), 1) for p, q in zip(a, b)], np.float32)
            assert np.array_equal(hid[t, k].view(np.uint32), want.view(np.uint32)), f"hidden rows t{t} k{k}"
    y_node = ops.moe_down_weighted(dev["de"], cu(hid), cu(ids), wts_t).cpu().numpy()
    assert np.array_equal(y.view(np.uint32), y_node.view(np.uint32)), "down phase vs the down node"
    assert np.array_equal(out, x + y)
    for w in dev.values():
        w.free()
