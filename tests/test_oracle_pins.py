"""Pins the CPU oracle against what fixes each function independently of it.

The reference holds no stored vectors for this path (its kernel tests are
differential and execute ggml, which is absent), so each oracle function is
pinned by a library routine, an invariant of the format, a closed form or a
brute-force evaluation written separately here in numpy.
"""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc


# ----------------------------------------------------------------- helpers
def np_unpack_q4k(w):
    """Independent decode of block_q4_K rows -> (d, dmin, scales[8], mins[8], q[256]).

    Written from the published format: 12 packed bytes hold eight 6-bit scales
    and eight 6-bit mins; each 32-byte chunk of qs holds sub-block 2c in the low
    nibbles and 2c+1 in the high nibbles.
    """
    b = w.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64)[:, 0]
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float64)[:, 0]
    p = b[:, 4:16].astype(np.int64)
    sc = np.zeros((b.shape[0], 8), np.int64)
    mn = np.zeros((b.shape[0], 8), np.int64)
    for j in range(8):
        if j < 4:
            sc[:, j] = p[:, j] & 63
            mn[:, j] = p[:, j + 4] & 63
        else:
            sc[:, j] = (p[:, j + 4] & 0xF) | ((p[:, j - 4] >> 6) << 4)
            mn[:, j] = (p[:, j + 4] >> 4) | ((p[:, j] >> 6) << 4)
    qs = b[:, 16:144].reshape(-1, 4, 32).astype(np.int64)
    q = np.stack([qs & 0xF, qs >> 4], axis=2).reshape(-1, 256)  # [blk, chunk, lo/hi, 32]
    return d, dmin, sc, mn, q


def brute_block_sums(w, q8):
    d, dmin, sc, mn, q = np_unpack_q4k(w)
    yd, yq, ybs = orc.split_q8k(q8)
    rows = w.shape[0]
    nb = w.shape[1] // 144
    q = q.reshape(rows, nb, 8, 32)
    sc = sc.reshape(rows, nb, 8)
    mn = mn.reshape(rows, nb, 8)
    yq = yq.astype(np.int64).reshape(q8.shape[0], nb, 8, 32)
    sub = np.einsum("rbgi,mbgi->rmbg", q, yq)
    ds = np.einsum("rmbg,rbg->rmb", sub, sc)
    gsum = yq.sum(axis=3)  # recomputed from qs, independent of bsums
    md = np.einsum("mbg,rbg->rmb", gsum, mn)
    return ds, md


# ----------------------------------------------------------------- fp16
def test_fp16_to_fp32_exhaustive_against_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([np.float32(orc.fp16_to_fp32(int(h))).view(np.uint32) for h in allh], dtype=np.uint32)
    nan = np.isnan(allh.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float32)))


def test_fp32_to_fp16_against_numpy():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, 6.1035e-5],
                 np.float32),
        np.arange(2048, dtype=np.uint16).view(np.float16).astype(np.float32),  # every subnormal/small half
    ])
    # exact ties between adjacent halves
    h = np.arange(1, 30000, 7, dtype=np.uint16)
    ties = (h.view(np.float16).astype(np.float64) + (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2
    vals = np.concatenate([vals, ties.astype(np.float32)])
    want = vals.astype(np.float16).view(np.uint16)
    got = np.array([orc.fp32_to_fp16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ----------------------------------------------------------------- nearest int
def test_nearest_int_is_round_half_even():
    grid = np.concatenate([
        np.arange(-130.0, 130.0, 0.25, dtype=np.float32),  # includes every +-x.5 tie
        np.random.default_rng(2).uniform(-4e6, 4e6, 5000).astype(np.float32),
        np.nextafter(np.arange(-128, 128, dtype=np.float32) + np.float32(0.5), np.float32(1e9)),
        np.nextafter(np.arange(-128, 128, dtype=np.float32) + np.float32(0.5), np.float32(-1e9)),
    ])
    want = np.rint(grid.astype(np.float64)).astype(np.int64)
    got = np.array([orc.nearest_int(float(v)) for v in grid], dtype=np.int64)
    assert np.array_equal(got, want)


# ----------------------------------------------------------------- Q8_K quantizer
def test_q8k_invariants_on_normal_input():
    x = synth.normal_f32(11, (8, 2048))
    q8 = orc.quantize_rows_q8k(x)
    d, qs, bs = orc.split_q8k(q8)
    assert qs.min() >= -127 and qs.max() <= 127
    assert np.array_equal(bs.astype(np.int64), qs.astype(np.int64).reshape(8, 8, 16, 16).sum(-1))
    xb = x.reshape(8, 8, 256)
    amax_idx = np.abs(xb).argmax(-1)  # numpy argmax returns the first maximum
    picked = np.take_along_axis(qs, amax_idx[..., None], -1)[..., 0]
    assert np.all(picked == -127)  # iscale = -127/max maps the extreme element to exactly -127
    # d = 1/iscale = max/-127 up to two roundings; reconstruction within half a step
    recon = d[..., None].astype(np.float64) * qs
    assert np.all(np.abs(recon - xb) <= np.abs(d[..., None]) * 0.5000001 + 1e-12)
    # sign of d is minus the sign of the extreme element
    mx = np.take_along_axis(xb, amax_idx[..., None], -1)[..., 0]
    assert np.all(np.sign(d) == -np.sign(mx))


def test_q8k_zero_block_and_sign_symmetry_and_tie_break():
    x = synth.normal_f32(12, (1, 512))
    x[0, :256] = 0.0
    q8 = orc.quantize_rows_q8k(x)
    assert not q8[0, :292].any()  # all-zero block: d = 0, qs = 0, bsums = 0
    # quant(-x): same codes, d negated
    qn = orc.quantize_rows_q8k(-x)
    d0, q0, b0 = orc.split_q8k(q8)
    d1, q1, b1 = orc.split_q8k(qn)
    assert np.array_equal(q0, q1) and np.array_equal(b0, b1) and np.array_equal(d0, -d1)
    # first of two equal magnitudes decides the sign
    y = np.zeros((2, 256), np.float32)
    y[0, 10], y[0, 200] = 3.0, -3.0
    y[1, 10], y[1, 200] = -3.0, 3.0
    d, qs, _ = orc.split_q8k(orc.quantize_rows_q8k(y))
    assert qs[0, 0, 10] == -127 and qs[0, 0, 200] == 127 and d[0, 0] < 0
    assert qs[1, 0, 10] == -127 and qs[1, 0, 200] == 127 and d[1, 0] > 0


def test_q8k_matches_numpy_restatement():
    """Same recipe in numpy float32 (division, multiply and rint are IEEE on both sides)."""
    x = synth.normal_f32(13, (4, 1024)) * np.float32(3.7)
    xb = x.reshape(-1, 256)
    idx = np.abs(xb).argmax(-1)
    mx = xb[np.arange(xb.shape[0]), idx]
    iscale = (np.float32(-127.0) / mx).astype(np.float32)
    q = np.minimum(127, np.rint((iscale[:, None] * xb).astype(np.float32))).astype(np.int8)
    d = (np.float32(1.0) / iscale).astype(np.float32)
    gd, gq, gb = orc.split_q8k(orc.quantize_rows_q8k(x))
    assert np.array_equal(gq.reshape(-1, 256), q)
    assert np.array_equal(gd.reshape(-1), d)
    assert np.array_equal(gb.reshape(-1, 16), q.astype(np.int32).reshape(-1, 16, 16).sum(-1))


def test_q8k_rejects_bad_shapes():
    with pytest.raises(ValueError):
        orc.quantize_rows_q8k(np.zeros((1, 255), np.float32))


# ----------------------------------------------------------------- scales
def test_scale_unpack_two_formulas_agree_and_one_hot_fields():
    rng = np.random.default_rng(3)
    for _ in range(2000):
        p = rng.integers(0, 256, 12, dtype=np.uint8)
        s0, m0 = orc.scales_kmask(p)
        s1, m1 = orc.scales_indexed(p)
        assert np.array_equal(s0, s1) and np.array_equal(m0, m1)
        assert s0.max() < 64 and m0.max() < 64
    # every one of the 96 input bits lands in exactly one output bit, and all 96 are distinct
    seen = set()
    for bit in range(96):
        p = np.zeros(12, np.uint8)
        p[bit // 8] = 1 << (bit % 8)
        s, m = orc.scales_kmask(p)
        out = np.concatenate([s, m]).astype(np.int64)
        nz = np.nonzero(out)[0]
        assert len(nz) == 1 and bin(int(out[nz[0]])).count("1") == 1
        seen.add((int(nz[0]), int(out[nz[0]])))
    assert len(seen) == 96
    # spot values from the format: byte j<4 low 6 bits = scale j; byte j+4 low 6 bits = min j
    p = np.zeros(12, np.uint8)
    p[2], p[6] = 45, 33
    s, m = orc.scales_kmask(p)
    assert s[2] == 45 and m[2] == 33
    p = np.zeros(12, np.uint8)
    p[9] = 0xA7          # low nibble -> scale 5 low bits, high nibble -> min 5 low bits
    p[1] = 0b11 << 6     # top bits of byte 1 -> scale 5 high bits
    p[5] = 0b10 << 6     # top bits of byte 5 -> min 5 high bits
    s, m = orc.scales_kmask(p)
    assert s[5] == (0x7 | (3 << 4)) and m[5] == (0xA | (2 << 4))


# ----------------------------------------------------------------- integer sums
def test_block_sums_against_brute_force():
    w = synth.q4k_matrix(21, 24, 1024)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(22, (5, 1024)))
    ds, md = orc.matrix_block_sums(w, 1024, q8)
    bds, bmd = brute_block_sums(w, q8)
    assert np.array_equal(ds, bds) and np.array_equal(md, bmd)


def test_block_sums_closed_form_extremes():
    blk = np.zeros((1, 144), np.uint8)
    blk[0, 4:16] = 0xFF   # every scale and min = 63
    blk[0, 16:] = 0xFF    # every quant = 15
    q8 = np.zeros((1, 292), np.uint8)
    q8[0, 4:260] = np.int8(127).view(np.uint8)
    q8[0, 260:292] = np.full(16, 16 * 127, np.int16).view(np.uint8)
    ds, md = orc.matrix_block_sums(blk, 256, q8)
    assert ds[0, 0, 0] == 8 * 63 * 32 * 15 * 127
    assert md[0, 0, 0] == 16 * (16 * 127) * 63
    q8[0, 4:260] = np.int8(-127).view(np.uint8)
    ds, _ = orc.matrix_block_sums(blk, 256, q8)
    assert ds[0, 0, 0] == -8 * 63 * 32 * 15 * 127


def test_block_sums_single_element_placement():
    """One non-zero weight nibble and one non-zero activation: only the matching element contributes,
    and it is scaled by that sub-block's scale (catches nibble-order and scale-index slips)."""
    rng = np.random.default_rng(4)
    for _ in range(300):
        e = int(rng.integers(0, 256))
        blk = np.zeros((1, 144), np.uint8)
        packed = rng.integers(0, 256, 12, dtype=np.uint8)
        blk[0, 4:16] = packed
        chunk, within = e // 64, e % 64
        byte = 16 + 32 * chunk + (within % 32)
        blk[0, byte] = 9 if within < 32 else 9 << 4
        q8 = np.zeros((1, 292), np.uint8)
        for probe in (e, (e + 32) % 256):
            q8[:] = 0
            q8[0, 4 + probe] = np.int8(-5).view(np.uint8)
            ds, _ = orc.matrix_block_sums(blk, 256, q8)
            sc, _ = orc.scales_indexed(packed)
            assert ds[0, 0, 0] == (int(sc[e // 32]) * 9 * -5 if probe == e else 0)


# ----------------------------------------------------------------- fp32 dots
@pytest.mark.parametrize("cols", [256, 2048, 4096])
def test_all_fp32_orders_close_to_double_dequant(cols):
    w = synth.q4k_matrix(31 + cols, 48, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(32 + cols, (3, cols)))
    ref = orc.dot_dequant_f64(w, cols, q8)
    mag = orc.dot_magnitude_f64(w, cols, q8)
    for name, order in orc.ORDERS.items():
        got = orc.mul_mat_q4k_q8k(w, cols, q8, order).astype(np.float64)
        assert np.max(np.abs(got - ref) / mag) < 2e-6, name  # a few fp32 ulps of the summed magnitudes
        ok = np.abs(ref) > 1e-3 * mag                         # well-conditioned outputs
        assert np.max(np.abs(got - ref)[ok] / np.abs(ref)[ok]) < 1e-4, name


def test_double_dequant_matches_numpy_dequant():
    cols = 1024
    w = synth.q4k_matrix(41, 16, cols)
    x = synth.normal_f32(42, (2, cols))
    q8 = orc.quantize_rows_q8k(x)
    d, dmin, sc, mn, q = np_unpack_q4k(w)
    wq = (d[:, None, None] * sc[:, :, None] * q.reshape(-1, 8, 32) - dmin[:, None, None] * mn[:, :, None])
    wq = wq.reshape(16, cols)
    yd, yq, _ = orc.split_q8k(q8)
    act = (yd[..., None].astype(np.float64) * yq).reshape(2, cols)
    want = act @ wq.T
    got = orc.dot_dequant_f64(w, cols, q8)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    # and the quantized product approximates the unquantized one (sanity of the whole chain)
    dense = x.astype(np.float64) @ wq.T
    assert np.max(np.abs(dense - want)) / np.max(np.abs(dense)) < 0.02


def test_simd_baseline_is_bitwise_the_avx2_order():
    cols = 2048
    w = synth.q4k_matrix(51, 96, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(52, (19, cols)))  # 19 rows: one full tile of 16 plus a ragged one
    ref = orc.mul_mat_q4k_q8k(w, cols, q8, orc.ORDER_AVX2)
    for threads in (1, 3, 8):
        got = orc.simd_mul_mat_q4k_q8k(w, cols, q8, threads)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.skipif(not orc.host_has_vnni(), reason="this host has no AVX-512 VNNI")
def test_vnni_build_of_the_baseline_is_bitwise_the_avx2_build():
    """The reference's VNNI kernel (cpu_backend_moe_raw_batched.inl:562-616) keeps the AVX2 kernel's eight lanes: the
    two builds of the baseline must agree bit for bit, for a product and for the whole FFN."""
    assert orc.simd("vnni").orc_simd_isa() == 2 and orc.simd("avx2").orc_simd_isa() == 1
    cols, rows = 2048, 96
    w = synth.q4k_matrix(271, rows, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(272, (5, cols)))
    a = orc.simd_mul_mat_q4k_q8k(w, cols, q8, 3, isa="avx2")
    b = orc.simd_mul_mat_q4k_q8k(w, cols, q8, 3, isa="vnni")
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(a.view(np.uint32), orc.mul_mat_q4k_q8k(w, cols, q8, orc.ORDER_AVX2).view(np.uint32))
    H, I = 512, 768
    g, u, d = synth.q4k_matrix(273, I, H), synth.q4k_matrix(274, I, H), synth.q4k_matrix(275, H, I)
    x = synth.normal_f32(276, (3, H))
    assert np.array_equal(orc.simd_ffn_swiglu(g, u, d, H, I, x, 2, isa="vnni").view(np.uint32),
                          orc.simd_ffn_swiglu(g, u, d, H, I, x, 2, isa="avx2").view(np.uint32))


def test_simd_ffn_baseline_matches_scalar_oracle():
    H, I, n = 512, 768, 3
    g, u, d = synth.q4k_matrix(55, I, H), synth.q4k_matrix(56, I, H), synth.q4k_matrix(57, H, I)
    x = synth.normal_f32(58, (n, H))
    want = orc.ffn_swiglu(g, u, d, H, I, x, orc.ORDER_AVX2, orc.SILU_FAST_FMA)
    got = orc.simd_ffn_swiglu(g, u, d, H, I, x, threads=4)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ----------------------------------------------------------------- activation
def test_fast_exp_known_answers_from_the_references_literals():
    """The cubic's three coefficients and log2(e) as the reference spells them
    (core/src/backend/cpu_backend_internal.h:103 kLog2E, :108 the three coefficients;
    core/src/kernels/hwy/hwy_fastexp.h:31-33 c0, c1, c2): the restatement must return, bit for bit, what those
    literals give when every step is rounded to fp32 in the written order -- a wrong digit in any of them shows."""
    f32 = np.float32
    log2e, c0, c1, c2 = f32(1.4426950408889634), f32(0.6960656421638072), f32(0.224494337302845), f32(0.07944023841053369)
    xs = np.concatenate([np.linspace(-60, 60, 2401), [0.0, -0.0, 1e-8, 49.999, 50.0, 50.001, -50.001]]).astype(f32)
    xc = np.clip(xs, f32(-50), f32(50))
    y = xc * log2e
    fl = np.floor(y)
    f = y - fl
    two_i = ((fl.astype(np.int32) + 127) << 23).view(f32)
    plain = two_i * (f32(1) + f * (c0 + f * (c1 + f * c2)))                      # unfused Horner, fp32 at every step
    got = np.array([orc.lib().orc_fast_exp(float(v)) for v in xs], f32)
    assert np.array_equal(got.view(np.uint32), plain.view(np.uint32))
    # the fused form: each multiply-add rounded once (a double holds the exact product and, here, the exact sum)
    fma = lambda a, b, c: (a.astype(np.float64) * b.astype(np.float64) + np.float64(c)).astype(f32)
    p = fma(f, np.full_like(f, c2), c1)
    p = fma(f, p, c0)
    p = fma(f, p, f32(1))
    got = np.array([orc.lib().orc_fast_exp_fma(float(v)) for v in xs], f32)
    assert np.array_equal(got.view(np.uint32), (two_i * p).view(np.uint32))
    # closed form: at f = 1/2 the cubic is 1 + c0/2 + c1/4 + c2/8, a 2e-4-accurate sqrt(2)
    half = orc.lib().orc_fast_exp(float(f32(0.5) / log2e))
    assert abs(half - (1 + 0.6960656421638072 / 2 + 0.224494337302845 / 4 + 0.07944023841053369 / 8)) < 2e-6
    assert abs(half - 2 ** 0.5) < 3e-4


def test_fast_exp_error_class_and_silu_flavours():
    xs = np.linspace(-20, 20, 4001, dtype=np.float32)
    fe = np.array([orc.lib().orc_fast_exp(float(v)) for v in xs])
    ff = np.array([orc.lib().orc_fast_exp_fma(float(v)) for v in xs])
    ex = np.exp(xs.astype(np.float64))
    assert np.max(np.abs(fe - ex) / ex) < 2e-3 and np.max(np.abs(fe - ex) / ex) > 1e-5  # a cubic, not libm
    assert np.max(np.abs(ff - fe) / ex) < 1e-6                                          # fused vs unfused: ulps
    # exact at integer powers of two of e**x where f == 0:  x = i*ln2 gives p(0) = 1
    assert orc.lib().orc_fast_exp(0.0) == 1.0
    for g, u in [(0.5, 2.0), (-3.0, 1.5), (7.0, -0.25)]:
        want = g / (1 + np.exp(-g)) * u
        assert abs(orc.lib().orc_silu_mul(g, u, orc.SILU_EXACT) - want) < 1e-6 * abs(want)
        assert abs(orc.lib().orc_silu_mul(g, u, orc.SILU_FAST) - want) < 3e-3 * abs(want)
        assert abs(orc.lib().orc_silu_mul(g, u, orc.SILU_FAST_FMA) - want) < 3e-3 * abs(want)


# ----------------------------------------------------------------- router
def np_route(logits, k):
    n, e = logits.shape
    ids = np.zeros((n, k), np.int32)
    for t in range(n):
        row = logits[t]
        key = sorted(range(e), key=lambda i: (np.isnan(row[i]), -row[i] if not np.isnan(row[i]) else 0.0, i))
        ids[t] = key[:k]
    return ids


def test_router_topk_matches_sort_and_softmax():
    logits = synth.normal_f32(61, (16, 256))
    logits[3, 40] = logits[3, 7] = logits[3].max() + 1.0      # tie at the top: lower id first
    logits[5, 100] = np.nan                                    # NaN sorts last
    logits[6, :] = 0.25                                        # all equal: ids 0..7
    ids, w = orc.route_topk(logits, 8, 0)
    assert np.array_equal(ids, np_route(logits, 8))
    assert list(ids[3, :2]) == [7, 40] and list(ids[6]) == list(range(8)) and 100 not in ids[5]
    sel = np.take_along_axis(logits.astype(np.float64), ids.astype(np.int64), 1)
    sm = np.exp(sel - sel.max(1, keepdims=True))
    sm /= sm.sum(1, keepdims=True)
    assert np.allclose(w, sm, rtol=2e-6, atol=1e-8)
    # restricted softmax equals full softmax renormalised over the selected set
    full = np.exp(logits[0].astype(np.float64) - logits[0].max())
    full /= full.sum()
    assert np.allclose(w[0], full[ids[0]] / full[ids[0]].sum(), rtol=2e-6)
    for mode in (1, 2):
        _, wm = orc.route_topk(logits, 8, mode)
        assert np.allclose(wm, sm, rtol=2e-6, atol=1e-8)


def test_router_degenerate_rows():
    logits = np.full((2, 16), -np.inf, np.float32)
    logits[1, :] = np.inf
    ids, w = orc.route_topk(logits, 8, 0)
    assert np.allclose(w, 1.0 / 8)                       # uniform fallback
    assert np.array_equal(ids[0], np.arange(8))


def test_assignments_sorted_by_expert_token_k():
    ids, _ = orc.route_topk(synth.normal_f32(62, (13, 32)), 4, 0)
    got = orc.build_assignments(ids, 32)
    want = sorted((int(ids[t, k]), t, k) for t in range(13) for k in range(4))
    assert [tuple(r) for r in got.tolist()] == want
    ids[2, 1] = -1
    ids[4, 0] = 99
    assert len(orc.build_assignments(ids, 32)) == 13 * 4 - 2


# ----------------------------------------------------------------- composition
def np_dequant(w, cols):
    d, dmin, sc, mn, q = np_unpack_q4k(w)
    return (d[:, None, None] * sc[:, :, None] * q.reshape(-1, 8, 32) - dmin[:, None, None] * mn[:, :, None]).reshape(
        w.shape[0], cols)


def np_q8_dequant(x):
    d, q, _ = orc.split_q8k(orc.quantize_rows_q8k(x))
    return (d[..., None].astype(np.float64) * q).reshape(x.shape[0], -1)


def test_tiny_moe_layer_against_double_brute_force():
    H, I, E, K, n = 256, 256, 4, 2, 3
    ge = np.stack([synth.q4k_matrix(synth.tensor_seed("g", e), I, H) for e in range(E)])
    ue = np.stack([synth.q4k_matrix(synth.tensor_seed("u", e), I, H) for e in range(E)])
    de = np.stack([synth.q4k_matrix(synth.tensor_seed("d", e), H, I) for e in range(E)])
    sh = (synth.q4k_matrix(71, I, H), synth.q4k_matrix(72, I, H), synth.q4k_matrix(73, H, I),
          synth.normal_f32(74, (H,)) * np.float32(0.05))
    x = synth.normal_f32(75, (n, H))
    logits = synth.normal_f32(76, (n, E))
    for acc_mode in (0, 1):
        r = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=sh, silu=orc.SILU_EXACT, accumulate_mode=acc_mode)
        ids, wts = orc.route_topk(logits, K, 0)
        assert np.array_equal(r["ids"], ids)
        xq = np_q8_dequant(x)
        y = np.zeros((n, H))
        for t in range(n):
            for k in range(K):
                e = ids[t, k]
                g = np_dequant(ge[e], H) @ xq[t]
                u = np_dequant(ue[e], H) @ xq[t]
                h = g / (1 + np.exp(-g)) * u
                assert np.allclose(r["hidden"][t, k], h, rtol=2e-4, atol=1e-5 * np.abs(h).max())
                hq = np_q8_dequant(r["hidden"][t, k][None, :])[0]
                y[t] += wts[t, k] * (np_dequant(de[e], I) @ hq)
        # shared expert (fast-exp SiLU is ~1e-3 off exact, so compare with matching tolerance)
        g = xq @ np_dequant(sh[0], H).T
        u = xq @ np_dequant(sh[1], H).T
        hs = g / (1 + np.exp(-g)) * u
        ysh = np_q8_dequant(hs.astype(np.float32)) @ np_dequant(sh[2], I).T
        gate = 1 / (1 + np.exp(-(x.astype(np.float64) @ sh[3].astype(np.float64))))
        y_full = y + ysh * gate[:, None]
        scale = np.abs(y_full).max()
        assert np.max(np.abs(r["y"] - y_full)) < 5e-3 * scale
        # routed part alone, tight
        r2 = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=None, silu=orc.SILU_EXACT, accumulate_mode=acc_mode)
        assert np.max(np.abs(r2["y"] - y)) < 1e-5 * np.abs(y).max()


def test_ffn_against_double_brute_force():
    H, I, n = 512, 768, 2
    g, u, d = synth.q4k_matrix(81, I, H), synth.q4k_matrix(82, I, H), synth.q4k_matrix(83, H, I)
    x = synth.normal_f32(84, (n, H))
    y, mid = orc.ffn_swiglu(g, u, d, H, I, x, silu=orc.SILU_EXACT, want_inter=True)
    xq = np_q8_dequant(x)
    gg, uu = xq @ np_dequant(g, H).T, xq @ np_dequant(u, H).T
    h = gg / (1 + np.exp(-gg)) * uu
    assert np.allclose(mid, h, rtol=2e-4, atol=1e-5 * np.abs(h).max())
    want = np_q8_dequant(mid) @ np_dequant(d, I).T
    assert np.max(np.abs(y - want)) < 1e-5 * np.abs(want).max()


def test_weights_from_ids_agree_with_router_and_double_softmax():
    """orc_route_weights_from_ids: on the router's own selection it must reproduce the router's FLOOR-mode
    weights bit for bit (two restatements of one formula in the reference, native.cpp:822-866 vs :2305-2357,
    on finite logits) and equal a double-precision softmax restricted to the selected set; invalid ids weigh 0."""
    rng = np.random.default_rng(77)
    logits = rng.normal(size=(33, 64)).astype(np.float32)
    ids, w_router = orc.route_topk(logits, 8, 1)
    w = orc.route_weights_from_ids(logits, ids)
    assert np.array_equal(w, w_router)
    sel = np.take_along_axis(logits.astype(np.float64), ids.astype(np.int64), axis=1)
    ref = np.exp(sel - sel.max(axis=1, keepdims=True))
    ref /= ref.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(w, ref, rtol=2e-6)
    bad = ids.copy()
    bad[:, 3] = -1
    bad[:, 5] = 64
    wb = orc.route_weights_from_ids(logits, bad)
    assert np.all(wb[:, 3] == 0) and np.all(wb[:, 5] == 0)
    np.testing.assert_allclose(wb.sum(axis=1), 1.0, rtol=1e-6)
    # arbitrary (unsorted) ids: any permutation of the selection gives the permuted weights up to summation order
    perm = rng.permutation(8)
    np.testing.assert_allclose(orc.route_weights_from_ids(logits, ids[:, perm]), w[:, perm], rtol=1e-6)


# ----------------------------------------------------------------- Q5_K weights
def np_unpack_q5k(w):
    """Independent decode of block_q5_K rows, from the published format: the Q4_K fields with 32 qh bytes
    between the packed scales and the nibbles; bit s of qh[l] is worth 16 in element l of sub-block s."""
    b = w.reshape(-1, 176)
    as_q4 = np.concatenate([b[:, 0:16], b[:, 48:176]], axis=1)
    d, dmin, sc, mn, q = np_unpack_q4k(as_q4)
    qh = b[:, 16:48].astype(np.int64)                                        # [blk, l]
    hi = (qh[:, None, :] >> np.arange(8)[None, :, None]) & 1                 # [blk, s, l]
    return d, dmin, sc, mn, q + 16 * hi.reshape(-1, 256)


def test_q5k_layout_and_zero_high_bits_reduce_to_q4k():
    assert orc.lib().orc_q5k_block_bytes() == 176
    cols = 1024
    w4 = synth.q4k_matrix(301, 12, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(302, (3, cols)))
    w5 = orc.q5k_from_q4k(w4)
    ds4, md4 = orc.matrix_block_sums(w4, cols, q8)
    ds5, md5 = orc.q5k_matrix_block_sums(w5, cols, q8)
    assert np.array_equal(ds4, ds5) and np.array_equal(md4, md5)
    for order in (orc.ORDER_HWY, orc.ORDER_DOTPROD):
        assert np.array_equal(orc.mul_mat_q4k_q8k(w4, cols, q8, order), orc.mul_mat_q5k_q8k(w5, cols, q8, order))


def test_q5k_all_high_bits_closed_form_and_single_bit_placement():
    """Every qh bit set adds 16 * scale_s * (sum of sub-block s of the activations), which the Q8_K block
    carries as bsums; one set bit adds 16 * scale_s * y[32 s + l] and nothing else."""
    cols = 512
    w4 = synth.q4k_matrix(311, 6, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(312, (2, cols)))
    ds4, md4 = orc.matrix_block_sums(w4, cols, q8)
    full = orc.q5k_from_q4k(w4, np.full((6, 2, 32), 0xFF, np.uint8))
    ds5, md5 = orc.q5k_matrix_block_sums(full, cols, q8)
    _, _, sc, _, _ = np_unpack_q4k(w4)
    _, yq, ybs = orc.split_q8k(q8)
    sub = ybs.astype(np.int64).reshape(2, 2, 8, 2).sum(axis=3)               # [m, b, s]
    extra = 16 * np.einsum("rbs,mbs->rmb", sc.reshape(6, 2, 8), sub)
    assert np.array_equal(ds5, ds4 + extra) and np.array_equal(md5, md4)
    rng = np.random.default_rng(5)
    for _ in range(200):
        r, b, s, l = (int(rng.integers(0, n)) for n in (6, 2, 8, 32))
        qh = np.zeros((6, 2, 32), np.uint8)
        qh[r, b, l] = 1 << s
        ds1, _ = orc.q5k_matrix_block_sums(orc.q5k_from_q4k(w4, qh), cols, q8)
        want = ds4.copy()
        want[r, :, b] += 16 * sc.reshape(6, 2, 8)[r, b, s] * yq.reshape(2, 2, 256)[:, b, 32 * s + l].astype(np.int64)
        assert np.array_equal(ds1, want)


def test_q5k_sums_brute_force_and_fp32_against_double():
    cols = 2048
    w = synth.q5k_matrix(321, 20, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(322, (3, cols)))
    d, dmin, sc, mn, q = np_unpack_q5k(w)
    assert q.min() == 0 and q.max() == 31
    nb = cols // 256
    _, yq, _ = orc.split_q8k(q8)
    yq = yq.astype(np.int64).reshape(3, nb, 8, 32)
    sub = np.einsum("rbgi,mbgi->rmbg", q.reshape(20, nb, 8, 32), yq)
    bds = np.einsum("rmbg,rbg->rmb", sub, sc.reshape(20, nb, 8))
    bmd = np.einsum("mbg,rbg->rmb", yq.sum(axis=3), mn.reshape(20, nb, 8))
    ds, md = orc.q5k_matrix_block_sums(w, cols, q8)
    assert np.array_equal(ds, bds) and np.array_equal(md, bmd)
    # dequantize in numpy, dot in double
    wq = d[:, None, None] * sc[:, :, None] * q.reshape(-1, 8, 32) - dmin[:, None, None] * mn[:, :, None]
    yd, yq8, _ = orc.split_q8k(q8)
    act = (yd[..., None].astype(np.float64) * yq8).reshape(3, cols)
    want = act @ wq.reshape(20, cols).T
    ref = orc.q5k_dot_dequant_f64(w, cols, q8)
    assert np.allclose(ref, want, rtol=1e-12, atol=1e-12)
    mag = orc.q5k_dot_dequant_f64(w, cols, q8, magnitude=True)
    for order in (orc.ORDER_HWY, orc.ORDER_DOTPROD):
        got = orc.mul_mat_q5k_q8k(w, cols, q8, order).astype(np.float64)
        assert np.max(np.abs(got - ref) / mag) < 2e-6
        ok = np.abs(ref) > 1e-3 * mag
        assert np.max(np.abs(got - ref)[ok] / np.abs(ref)[ok]) < 1e-4


# ----------------------------------------------------------------- Q6_K weights
def np_unpack_q6k(w):
    """Independent decode of block_q6_K rows -> (d, scales[16], q[256] unsigned codes), from the published format."""
    b = w.reshape(-1, 210)
    ql = b[:, 0:128].astype(np.int64).reshape(-1, 2, 2, 32)      # [blk, j, half of the 64 bytes, l]
    qh = b[:, 128:192].astype(np.int64).reshape(-1, 2, 32)       # [blk, j, l]
    sc = b[:, 192:208].copy().view(np.int8).astype(np.int64)
    d = b[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]
    q = np.zeros((b.shape[0], 2, 4, 32), np.int64)               # [blk, j, z, l]
    for z in range(4):
        nib = ql[:, :, z & 1, :] & 15 if z < 2 else ql[:, :, z & 1, :] >> 4
        q[:, :, z, :] = nib | (((qh >> (2 * z)) & 3) << 4)
    return d, sc, q.reshape(-1, 256)


def test_q6k_layout_sums_brute_force_and_closed_forms():
    assert orc.lib().orc_q6k_block_bytes() == 210
    cols = 1024
    w = synth.q6k_matrix(401, 10, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(402, (3, cols)))
    d, sc, q = np_unpack_q6k(w)
    assert q.min() == 0 and q.max() == 63 and sc.min() < -100 and sc.max() > 100
    nb = cols // 256
    _, yq, ybs = orc.split_q8k(q8)
    yq = yq.astype(np.int64).reshape(3, nb, 16, 16)
    sub = np.einsum("rbgi,mbgi->rmbg", (q - 32).reshape(10, nb, 16, 16), yq)
    want = np.einsum("rmbg,rbg->rmb", sub, sc.reshape(10, nb, 16))
    assert np.array_equal(orc.q6k_matrix_block_sums(w, cols, q8), want)
    # every code 32 -> weights are all zero; every code 0 -> -32 * sum_g scale_g * bsums_g
    blocks = w.reshape(10, nb, 210).copy()
    blocks[:, :, 0:128] = 0
    blocks[:, :, 128:192] = 0xAA          # each two-bit field = 2 -> code 32
    assert not orc.q6k_matrix_block_sums(blocks.reshape(10, -1), cols, q8).any()
    blocks[:, :, 128:192] = 0
    got = orc.q6k_matrix_block_sums(blocks.reshape(10, -1), cols, q8)
    closed = -32 * np.einsum("rbg,mbg->rmb", sc.reshape(10, nb, 16), ybs.astype(np.int64).reshape(3, nb, 16))
    assert np.array_equal(got, closed)


def test_q6k_single_element_placement():
    rng = np.random.default_rng(6)
    for _ in range(300):
        e = int(rng.integers(0, 256))
        blk = np.zeros((1, 210), np.uint8)
        blk[0, 128:192] = 0xAA                               # every code 32: contributes nothing
        scales = rng.integers(-128, 128, 16).astype(np.int8)
        blk[0, 192:208] = scales.view(np.uint8)
        code = int(rng.integers(0, 64))
        j, z, l = e // 128, (e // 32) % 4, e % 32
        byte = 64 * j + 32 * (z & 1) + l
        blk[0, byte] = (code & 15) if z < 2 else (code & 15) << 4
        hb = 128 + 32 * j + l
        blk[0, hb] = (int(blk[0, hb]) & (0xFF ^ (3 << (2 * z)))) | ((code >> 4) << (2 * z))
        # the nibble that shares the byte belongs to element e +- 64 and must read as code 32 there: its top bits stay 2
        q8 = np.zeros((1, 292), np.uint8)
        for probe in (e, (e + 64) % 256, (e + 32) % 256):
            q8[:] = 0
            q8[0, 4 + probe] = np.int8(-7).view(np.uint8)
            got = orc.q6k_matrix_block_sums(blk, 256, q8)[0, 0, 0]
            if probe == e:
                assert got == int(scales[e // 16]) * (code - 32) * -7
            elif probe == (e + 64) % 256 and (e // 128) == (probe // 128):
                # same ql byte, other nibble: zero nibble with top bits 2 -> code 32 -> nothing
                assert got == 0
            else:
                assert got == 0


@pytest.mark.parametrize("cols", [256, 2048])
def test_q6k_fp32_orders_against_double(cols):
    w = synth.q6k_matrix(411 + cols, 24, cols)
    q8 = orc.quantize_rows_q8k(synth.normal_f32(412 + cols, (3, cols)))
    d, sc, q = np_unpack_q6k(w)
    wq = (d[:, None] * np.repeat(sc, 16, axis=1) * (q - 32)).reshape(24, cols)
    yd, yq8, _ = orc.split_q8k(q8)
    act = (yd[..., None].astype(np.float64) * yq8).reshape(3, cols)
    want = act @ wq.T
    ref = orc.q6k_dot_dequant_f64(w, cols, q8)
    assert np.allclose(ref, want, rtol=1e-12, atol=1e-12)
    mag = orc.q6k_dot_dequant_f64(w, cols, q8, magnitude=True)
    for order in (orc.ORDER_HWY, orc.ORDER_DOTPROD):
        got = orc.mul_mat_q6k_q8k(w, cols, q8, order).astype(np.float64)
        assert np.max(np.abs(got - ref) / mag) < 2e-6
        ok = np.abs(ref) > 1e-3 * mag
        assert np.max(np.abs(got - ref)[ok] / np.abs(ref)[ok]) < 1e-4


# ----------------------------------------------------------------- expert stacks of the sibling types
def np_dequant_typed(w, cols, t):
    """Independent numpy dequantization of Q4_K / Q5_K / Q6_K rows in double."""
    if t == 14:
        d, sc, q = np_unpack_q6k(w)
        return (d[:, None, None] * sc.reshape(-1, 16)[:, :, None] * (q - 32).reshape(-1, 16, 16)).reshape(w.shape[0], cols)
    d, dmin, sc, mn, q = np_unpack_q5k(w) if t == 13 else np_unpack_q4k(w)
    return (d[:, None, None] * sc[:, :, None] * q.reshape(-1, 8, 32) - dmin[:, None, None] * mn[:, :, None]).reshape(
        w.shape[0], cols)


@pytest.mark.parametrize("types", [(13, 13, 13, 13), (13, 14, 12, 14), (12, 14, 13, 12), (14, 12, 12, 12)])
def test_tiny_moe_layer_with_typed_stacks_against_double_brute_force(types):
    """The MoE layer with gate/up, down and shared-expert stacks of Q5_K / Q6_K (what the loader admits,
    core/src/llm/moe/native.cpp:4611-4620): every stage against numpy's own decode of the blocks in double."""
    H, I, E, K, n = 256, 512, 5, 3, 4
    gen = {12: synth.q4k_matrix, 13: synth.q5k_matrix, 14: synth.q6k_matrix}
    gu, dn, sgu, sdn = types
    ge = np.stack([gen[gu](synth.tensor_seed("tg", e), I, H) for e in range(E)])
    ue = np.stack([gen[gu](synth.tensor_seed("tu", e), I, H) for e in range(E)])
    de = np.stack([gen[dn](synth.tensor_seed("td", e), H, I) for e in range(E)])
    sh = (gen[sgu](171, I, H), gen[sgu](172, I, H), gen[sdn](173, H, I), synth.normal_f32(174, (H,)) * np.float32(0.05))
    x = synth.normal_f32(175, (n, H))
    logits = synth.normal_f32(176, (n, E))
    r = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=sh, silu=orc.SILU_EXACT, types=types)
    ids, wts = orc.route_topk(logits, K, 0)
    assert np.array_equal(r["ids"], ids)
    hid = orc.moe_gateup_swiglu(ge, ue, H, I, x, ids, silu=orc.SILU_EXACT, gu_type=gu)
    assert np.array_equal(hid.view(np.uint32), r["hidden"].view(np.uint32))
    xq = np_q8_dequant(x)
    y = np.zeros((n, H))
    for t in range(n):
        for k in range(K):
            e = ids[t, k]
            g = np_dequant_typed(ge[e], H, gu) @ xq[t]
            u = np_dequant_typed(ue[e], H, gu) @ xq[t]
            h = g / (1 + np.exp(-g)) * u
            assert np.allclose(hid[t, k], h, rtol=2e-4, atol=1e-5 * np.abs(h).max())
            hq = np_q8_dequant(hid[t, k][None, :])[0]
            y[t] += wts[t, k] * (np_dequant_typed(de[e], I, dn) @ hq)
    routed = orc.moe_down_weighted(de, H, I, hid, ids, wts, down_type=dn)
    assert np.max(np.abs(routed - y)) < 1e-5 * np.abs(y).max()
    r2 = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=None, silu=orc.SILU_EXACT, types=types)
    assert np.array_equal(r2["y"].view(np.uint32), routed.view(np.uint32))
    # shared expert: the typed dense FFN against the same decode
    ysh, mid = orc.ffn_swiglu_typed(sgu, sdn, sh[0], sh[1], sh[2], H, I, x, silu=orc.SILU_EXACT, want_inter=True)
    g = xq @ np_dequant_typed(sh[0], H, sgu).T
    u = xq @ np_dequant_typed(sh[1], H, sgu).T
    hs = g / (1 + np.exp(-g)) * u
    assert np.allclose(mid, hs, rtol=2e-4, atol=1e-5 * np.abs(hs).max())
    want_sh = np_q8_dequant(mid) @ np_dequant_typed(sh[2], I, sdn).T
    assert np.max(np.abs(ysh - want_sh)) < 1e-5 * np.abs(want_sh).max()
    # the layer's own shared expert uses the fast-exp SiLU (~1e-3 off the exact one): looser end to end
    gate = 1 / (1 + np.exp(-(x.astype(np.float64) @ sh[3].astype(np.float64))))
    y_full = y + (np_q8_dequant(hs.astype(np.float32)) @ np_dequant_typed(sh[2], I, sdn).T) * gate[:, None]
    assert np.max(np.abs(r["y"] - y_full)) < 5e-3 * np.abs(y_full).max()


def test_typed_layer_with_q4k_types_is_bitwise_the_q4k_layer():
    """Stacks declared Q4_K go through the typed row product and the typed shared-expert FFN: the same bits as the
    plain Q4_K functions they stand beside."""
    H, I, E, K, n = 256, 256, 4, 2, 3
    ge, ue, de = (np.stack([synth.q4k_matrix(synth.tensor_seed(nm, e), r, c) for e in range(E)])
                  for nm, r, c in (("g", I, H), ("u", I, H), ("d", H, I)))
    sh = (synth.q4k_matrix(71, I, H), synth.q4k_matrix(72, I, H), synth.q4k_matrix(73, H, I), None)
    x = synth.normal_f32(75, (n, H))
    logits = synth.normal_f32(76, (n, E))
    want = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=sh, silu=orc.SILU_FAST)["y"]
    routed = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=None, silu=orc.SILU_FAST)["y"]
    shy = orc.ffn_swiglu(sh[0], sh[1], sh[2], H, I, x, silu=orc.SILU_FAST_FMA)
    assert np.array_equal((routed + shy).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(orc.ffn_swiglu_typed(12, 12, sh[0], sh[1], sh[2], H, I, x).view(np.uint32), shy.view(np.uint32))


# ---------------------------------------------------------------- Q8_0 x Q8_0 (core/src/llm/matmul/q8_small_batch.h)
def np_unpack_q80(rows_u8: np.ndarray):
    """-> (d float64 [rows, blocks], codes int64 [rows, blocks, 32]) by an independent numpy decode."""
    b = rows_u8.reshape(rows_u8.shape[0], -1, 34)
    d = np.ascontiguousarray(b[:, :, 0:2]).view(np.float16)[..., 0].astype(np.float64)
    return d, np.ascontiguousarray(b[:, :, 2:]).view(np.int8).astype(np.int64)


def test_q80_layout_sums_brute_force_and_closed_forms():
    assert orc.lib().orc_q80_block_bytes() == 34                      # q8_small_batch.h:13-14
    cols = 1024
    w = synth.q80_matrix(801, 10, cols)
    q = orc.quantize_rows_q80(synth.normal_f32(802, (3, cols)))
    _, wq = np_unpack_q80(w)
    _, yq = np_unpack_q80(q)
    assert wq.min() == -127 and wq.max() == 127
    assert np.array_equal(orc.q80_matrix_block_sums(w, cols, q), np.einsum("rbi,mbi->rmb", wq, yq))
    # all codes one -> the block sum is the sum of the activation codes; a single non-zero pair -> its product
    ones = w.reshape(10, -1, 34).copy()
    ones[:, :, 2:] = 1
    assert np.array_equal(orc.q80_matrix_block_sums(ones.reshape(10, -1), cols, q),
                          np.broadcast_to(yq.sum(-1)[None], (10, 3, cols // 32)))
    rng = np.random.default_rng(8)
    for _ in range(100):
        e, a, b = int(rng.integers(0, 256)), int(rng.integers(-127, 128)), int(rng.integers(-127, 128))
        wr, qr = np.zeros((1, 8 * 34), np.uint8), np.zeros((1, 8 * 34), np.uint8)
        wr[0, (e // 32) * 34 + 2 + e % 32] = np.int8(a).view(np.uint8)
        qr[0, (e // 32) * 34 + 2 + e % 32] = np.int8(b).view(np.uint8)
        got = orc.q80_matrix_block_sums(wr, 256, qr)[0, 0]
        assert got[e // 32] == a * b and got.sum() == a * b


@pytest.mark.parametrize("cols", [256, 2048])
def test_q80_fp32_orders_against_double(cols):
    w = synth.q80_matrix(811 + cols, 24, cols)
    q = orc.quantize_rows_q80(synth.normal_f32(812 + cols, (3, cols)))
    wd, wq = np_unpack_q80(w)
    yd, yq = np_unpack_q80(q)
    want = (yd[..., None] * yq).reshape(3, cols) @ (wd[..., None] * wq).reshape(24, cols).T
    ref = orc.q80_dot_dequant_f64(w, cols, q)
    assert np.allclose(ref, want, rtol=1e-12, atol=1e-12)
    mag = orc.q80_dot_dequant_f64(w, cols, q, magnitude=True)
    for order in (orc.ORDER_HWY, orc.ORDER_DOTPROD):
        got = orc.mul_mat_q80_q80(w, cols, q, order).astype(np.float64)
        assert np.max(np.abs(got - ref) / mag) < 2e-6
        ok = np.abs(ref) > 1e-3 * mag
        assert np.max(np.abs(got[ok] - ref[ok]) / np.abs(ref[ok])) < 1e-4


@pytest.mark.parametrize("variant", [orc.Q80_X86, orc.Q80_SCALAR])
def test_q80_activation_quantizer_invariants(variant):
    """ggml's Q8_0 quantizer is third-party code the reference tree does not carry (parity unpinned): what is
    checked is what either published form must satisfy."""
    x = synth.normal_f32(821, (5, 512))
    x[1] = 0.0
    x[2, 64:96] = 0.0
    x[3] *= np.float32(300.0)
    q = orc.quantize_rows_q80(x, variant)
    d, codes = np_unpack_q80(q)
    xb = x.reshape(5, 16, 32).astype(np.float64)
    amax = np.abs(xb).max(-1)
    assert np.abs(codes).max() <= 127
    assert not q[1].any() and not codes[2, 2].any() and d[2, 2] == 0.0
    live = amax > 0
    first = np.abs(xb).argmax(-1)
    extreme = np.take_along_axis(codes, first[..., None], -1)[..., 0]
    assert np.all(np.abs(extreme[live]) == 127)                          # the extreme element maps to +-127
    assert np.all(np.sign(extreme[live]) == np.sign(np.take_along_axis(xb, first[..., None], -1)[..., 0][live]))
    d32 = (amax / 127.0).astype(np.float32)
    assert np.array_equal(d.astype(np.float16), d32.astype(np.float16))  # stored scale = fp16(amax / 127)
    # reconstruction with the unrounded scale within half a step (plus fp32 rounding of the product)
    assert np.all(np.abs(codes * d32[..., None].astype(np.float64) - xb) <= 0.5 * d32[..., None] * (1 + 1e-5))
    qn = orc.quantize_rows_q80(-x, variant)                                 # sign symmetry
    dn, cn = np_unpack_q80(qn)
    assert np.array_equal(cn, -codes) and np.array_equal(dn, d)


def test_q80_quantizer_variants_differ_only_at_ties():
    x = synth.normal_f32(831, (4, 1024))
    a = np_unpack_q80(orc.quantize_rows_q80(x, orc.Q80_X86))[1]
    b = np_unpack_q80(orc.quantize_rows_q80(x, orc.Q80_SCALAR))[1]
    assert np.abs(a - b).max() <= 1 and np.mean(a != b) < 1e-3
