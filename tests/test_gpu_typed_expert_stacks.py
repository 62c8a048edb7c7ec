"""Expert stacks of the sibling types through every MoE kernel family, at the benchmark's own block shape.

The loader admits Q4_K and Q5_K gate/up stacks and Q4_K / Q5_K / Q6_K / Q8_0 down stacks
(core/src/llm/moe/native.cpp:4611-4620); a Q4_K_M file usually carries Q5_K or Q6_K down experts.  Here gate/up are
Q5_K (their own kernel instantiations: the fifth code bit in the decode tile, a third MFMA chain in the GEMM) and the
down stack Q5_K or Q6_K, at hidden 2048, 256 experts + 1 shared, intermediate 512, top-8:

  n = 1, 4, 8   token-major launches (moe_gateup_token / _slots, moe_down_token / _rows)
  n = 16, 64    expert-grouped launches (grouped_lds_kernel<2>, grouped matmul_kernel, combine)
  n = 400       the expert-grouped matrix-core GEMM for every stack it takes

stage by stage against the CPU restatement with the GPU's own intermediate fed forward, the one-call layer against its
stages, and end to end.  The integer sums of the Q5_K gate/up kernels are pinned by the exactness construction of
tests/test_gpu_integer_exactness.py through the gate/up node and mq_mul_mat_id_q4k at decode and prefill widths."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity
from tests.test_gpu_ffn_moe import END_TO_END_REL, assert_close_prod

pytestmark = pytest.mark.gpu

E, H, I, K = 256, 2048, 512, 8
Q4, Q5, Q6 = 12, 13, 14
MAG = {Q4: lambda w, c, q: orc.dot_magnitude_f64(w, c, q),
       Q5: lambda w, c, q: orc.q5k_dot_dequant_f64(w, c, q, magnitude=True),
       Q6: lambda w, c, q: orc.q6k_dot_dequant_f64(w, c, q, magnitude=True)}


def cu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module", params=[(Q5, Q5), (Q5, Q6), (Q4, Q6)], ids=["q5k-gateup-q5k-down", "q5k-gateup-q6k-down", "q4k-gateup-q6k-down"])
def layer(request):
    import torch
    from densecore_amd import ops
    assert torch.cuda.is_available()
    gu, dn = request.param
    types = (gu, gu, dn)
    dev = [ops.Q4KWeight.synthetic(synth.tensor_seed("typed", nm, t), r, c, E, t) for (nm, r, c), t in
           zip((("g", I, H), ("u", I, H), ("d", H, I)), types)]
    sh = [ops.Q4KWeight.synthetic(synth.tensor_seed("typed-sh", nm, t), r, c, 1, t) for (nm, r, c), t in
          zip((("g", I, H), ("u", I, H), ("d", H, I)), types)]
    host = [w.to_ggml() for w in dev]
    sh_host = [w.to_ggml() for w in sh]
    gate_inp = synth.normal_f32(synth.tensor_seed("typed-gi"), (H,)) * np.float32(0.02)
    yield ops, gu, dn, dev, sh, host, sh_host, gate_inp
    for w in dev + sh:
        w.free()


def down_reference(de, dn, hid, ids, wts):
    """(reference, magnitude) of the weighted down product on the given hidden rows."""
    n = hid.shape[0]
    ref = orc.moe_down_weighted(de, H, I, hid, ids, wts, orc.ORDER_DOTPROD, 0, down_type=dn)
    hq = orc.quantize_rows_q8k(hid.reshape(n * K, I)).reshape(n, K, -1)
    mag = np.zeros((n, H))
    for t in range(n):
        for k in range(K):
            mag[t] += abs(wts[t, k]) * MAG[dn](de[ids[t, k]], I, hq[t, k][None])[0]
    return ref, mag


@pytest.mark.parametrize("n,silu", [(1, 0), (4, 0), (8, 1), (16, 1), (64, 1)])
def test_typed_stacks_stagewise_and_end_to_end(layer, n, silu):
    ops, gu, dn, (GE, UE, DE), (SG, SU, SD), (ge, ue, de), (sg, su, sd), gate_inp = layer
    x = synth.normal_f32(synth.tensor_seed("typed-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("typed-l", n), (n, E))
    ids_t, w_t = ops.moe_route_topk(cu(logits), K, 0)
    ids, wts = ids_t.cpu().numpy(), w_t.cpu().numpy()
    oi, ow = orc.route_topk(logits, K, 0)
    assert np.array_equal(ids, oi) and np.allclose(wts, ow, rtol=3e-6)

    # stage 1: the gate/up node (expert-grouped launches at every width)
    hid = ops.moe_gateup_swiglu(GE, UE, cu(x), ids_t, silu).cpu().numpy()
    assert_close_prod(hid, orc.moe_gateup_swiglu(ge, ue, H, I, x, ids, orc.ORDER_DOTPROD, silu, gu_type=gu), "gate/up node")
    # stage 2: the down node on the GPU's own hidden rows
    y_routed = ops.moe_down_weighted(DE, cu(hid), ids_t, w_t).cpu().numpy()
    ref, mag = down_reference(de, dn, hid, ids, wts)
    assert_fp32_parity(y_routed, ref, mag, "down node")

    # the one-call layer (token-major launches up to eight tokens, expert-grouped above): its hidden rows against the
    # CPU restatement as well, its output against the down reference on ITS hidden rows
    y_nosh, ids2, w2 = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=None, silu=silu)
    assert np.array_equal(ids2.cpu().numpy(), ids) and np.allclose(w2.cpu().numpy(), wts, rtol=1e-6)
    hid_l = ops.debug_moe_hidden((n, K, I)).cpu().numpy()
    assert_close_prod(hid_l, orc.moe_gateup_swiglu(ge, ue, H, I, x, ids, orc.ORDER_DOTPROD, silu, gu_type=gu), "layer hidden rows")
    ref_l, mag_l = down_reference(de, dn, hid_l, ids, w2.cpu().numpy())
    assert_fp32_parity(y_nosh.cpu().numpy(), ref_l, mag_l, "layer output on its own hidden rows")

    # with the shared expert, end to end against the CPU layer of the same types
    y, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=(SG, SU, SD, cu(gate_inp)), silu=silu)
    hid_sh = ops.debug_moe_hidden((n, K + 1, I)).cpu().numpy()
    sh_ref = orc.ffn_swiglu_typed(gu, dn, sg, su, sd, H, I, x, silu=2, want_inter=True)[1]
    assert_close_prod(hid_sh[:, K], sh_ref, "shared gate/up")
    full = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=(sg, su, sd, gate_inp), silu=silu, types=(gu, dn, gu, dn))
    y = y.cpu().numpy()
    rel = np.max(np.abs(y - full["y"]), axis=1) / np.max(np.abs(full["y"]), axis=1)
    assert np.max(rel) <= END_TO_END_REL and np.median(rel) <= 2e-5, (np.max(rel), np.median(rel))


def test_typed_stacks_at_a_prefill_width(layer):
    """400 tokens: a dozen routed rows per expert, the width from which the expert products leave the decode kernels
    for the matrix-core GEMM (every stack of a type it takes).  Routing bit for bit; the gate/up node, mq_mul_mat_id_q4k
    over the gate stack and the down node against the CPU restatement on a sample of tokens; the layer end to end."""
    import torch
    ops, gu, dn, (GE, UE, DE), (SG, SU, SD), (ge, ue, de), (sg, su, sd), gate_inp = layer
    n, silu = 400, 1
    x = synth.normal_f32(synth.tensor_seed("typed-x", n), (n, H))
    logits = synth.normal_f32(synth.tensor_seed("typed-l", n), (n, E))
    oi, ow = orc.route_topk(logits, K, 0)
    y_nosh, ids_t, w_t = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=None, silu=silu)
    assert np.array_equal(ids_t.cpu().numpy(), oi) and np.allclose(w_t.cpu().numpy(), ow, rtol=3e-6)
    pick = np.unique(np.concatenate([np.arange(0, n, 57), [n - 1]]))

    hid = ops.moe_gateup_swiglu(GE, UE, cu(x), ids_t, silu)
    hid_np = hid.cpu().numpy()
    assert_close_prod(hid_np[pick], orc.moe_gateup_swiglu(ge, ue, H, I, x[pick], oi[pick], orc.ORDER_DOTPROD, silu, gu_type=gu),
                      "gate/up node")
    # the gate stack alone through mul_mat_id
    gk = ops.mul_mat_id(GE, cu(x), ids_t).cpu().numpy()
    q8 = orc.quantize_rows_q8k(x[pick])
    for i, t in enumerate(pick[:3]):
        for k in range(K):
            w = ge[oi[t, k]]
            refk = np.array([[orc.lib().orc_dot_typed_q8k(gu, w[r].ctypes.data, q8[i].ctypes.data, H, orc.ORDER_DOTPROD) for r in range(0, I, 7)]])
            assert_fp32_parity(gk[t, k][None, 0:I:7], refk, MAG[gu](w[0:I:7], H, q8[i][None]), f"mul_mat_id t{t} k{k}")
    y_node = ops.moe_down_weighted(DE, hid, ids_t, w_t)
    ref, mag = down_reference(de, dn, hid_np[pick], oi[pick], w_t.cpu().numpy()[pick])
    assert_fp32_parity(y_node.cpu().numpy()[pick], ref, mag, "down node")
    # the layer without the shared expert is its two nodes
    rel = ((y_nosh - y_node).abs() / y_node.abs().max(dim=1, keepdim=True).values).max(dim=1).values
    assert rel.max().item() <= END_TO_END_REL and rel.median().item() <= 2e-5, (rel.max().item(), rel.median().item())
    y, _, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), K, shared=(SG, SU, SD, cu(gate_inp)), silu=silu)
    full = orc.moe_layer(ge, ue, de, H, I, K, x[pick], logits[pick], shared=(sg, su, sd, gate_inp), silu=silu, types=(gu, dn, gu, dn))
    got = y.cpu().numpy()[pick]
    rel = np.max(np.abs(got - full["y"]), axis=1) / np.max(np.abs(full["y"]), axis=1)
    assert np.max(rel) <= END_TO_END_REL, np.max(rel)


# ------------------------------------------------------------------------------------------- exactness construction
def f16_bytes(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def exact_q5k_experts(tag, n_exp, rows, cols, d, dmin):
    """Seeded Q5_K stacks with every block's d / dmin a power of two, signs alternating over the rows."""
    nb = cols // 256
    out = []
    for e in range(n_exp):
        w = synth.q5k_matrix(synth.tensor_seed(tag, e), rows, cols).reshape(rows, nb, 176).copy()
        w[:, :, 0:2] = f16_bytes(d)
        w[:, :, 2:4] = f16_bytes(dmin)
        w[1::2, :, 0:2] = f16_bytes(-d)
        w[::3, :, 2:4] = f16_bytes(-dmin)
        out.append(w.reshape(rows, nb * 176))
    return np.stack(out)


def exact_acts(seed, shape, small=7):
    rng = np.random.default_rng(seed)
    x = rng.integers(-small, small + 1, size=shape).astype(np.float32)
    blocks = x.reshape(-1, 256)
    pos = rng.integers(0, 256, size=blocks.shape[0])
    blocks[np.arange(blocks.shape[0]), pos] = rng.choice([-127.0, 127.0], size=blocks.shape[0])
    return x


def expected_q5k(w, cols, x):
    """sum_b yd_b (d ds_b - dmin md_b) in float64 from the CPU restatement's Q5_K integers -> [n, rows]."""
    rows, nb, n = w.shape[0], cols // 256, x.shape[0]
    q8 = orc.quantize_rows_q8k(x)
    yd, qs, _ = orc.split_q8k(q8)
    assert np.all(np.abs(yd) == 1.0) and np.array_equal(qs.reshape(n, cols) * yd.repeat(256, axis=1), x)
    ds, md = orc.q5k_matrix_block_sums(w, cols, q8)
    blk = w.reshape(rows, nb, 176)
    d = blk[:, :, 0:2].copy().view(np.float16).astype(np.float64).reshape(rows, 1, nb)
    dm = blk[:, :, 2:4].copy().view(np.float16).astype(np.float64).reshape(rows, 1, nb)
    terms = (d * ds - dm * md) * yd.astype(np.float64)[None]
    unit = min(np.abs(d).min(), np.abs(dm).min())
    assert np.abs(terms).sum(axis=2).max() / unit < 2 ** 24      # every partial sum exact whatever the order
    return terms.sum(axis=2).T


@pytest.mark.parametrize("n", [1, 3, 8, 16, 40, 384])
def test_q5k_gateup_stacks_integer_sums_are_exact(n):
    """Q5_K gate / up stacks through mq_mul_mat_id_q4k, the gate/up node and the layer's own gate/up launch: products
    exact by construction, the polynomial SiLU a fixed fp32 sequence, so the hidden rows are compared bit for bit.
    384 tokens over 12 experts: the expert-grouped GEMM with its third MFMA chain (the fp32 update there is fused,
    still exact on these operands)."""
    import torch
    from densecore_amd import ops
    Ex, Hx, Ix, Kx, silu = 12, 2048, 512, 4, 1
    ge = exact_q5k_experts("ex5-g", Ex, Ix, Hx, 2.0 ** -17, 2.0 ** -17)
    ue = exact_q5k_experts("ex5-u", Ex, Ix, Hx, 2.0 ** -15, 2.0 ** -16)
    de = np.stack([synth.q5k_matrix(synth.tensor_seed("ex5-d", e), Hx, Ix) for e in range(Ex)])
    GE, UE, DE = (ops.Q4KWeight.from_ggml(a, c, Q5) for a, c in ((ge, Hx), (ue, Hx), (de, Ix)))
    x = exact_acts(n + 3, (n, Hx))
    logits = synth.normal_f32(synth.tensor_seed("ex5-l", n), (n, Ex))
    ids, _ = orc.route_topk(logits, Kx, 0)
    check = range(n) if n <= 40 else range(0, n, 37)
    L = orc.lib()

    def swiglu_rows(t, k):
        a = expected_q5k(ge[ids[t, k]], Hx, x[t:t + 1]).astype(np.float32)[0]
        b = expected_q5k(ue[ids[t, k]], Hx, x[t:t + 1]).astype(np.float32)[0]
        return a, np.array([L.orc_silu_mul(float(p), float(q), silu) for p, q in zip(a, b)], np.float32)

    want = {(t, k): swiglu_rows(t, k) for t in check for k in range(Kx)}
    gk = ops.mul_mat_id(GE, cu(x), cu(ids)).cpu().numpy()
    node = ops.moe_gateup_swiglu(GE, UE, cu(x), cu(ids), silu).cpu().numpy()
    _, ids2, _ = ops.moe_layer(GE, UE, DE, cu(x), cu(logits), Kx, silu=silu)
    assert np.array_equal(ids2.cpu().numpy(), ids)
    layer_hidden = ops.debug_moe_hidden((n, Kx, Ix)).cpu().numpy() if n < 256 else None   # wide: the rows stay in tile order
    for (t, k), (g_want, h_want) in want.items():
        assert np.array_equal(gk[t, k], g_want), f"mul_mat_id t{t} k{k}"
        assert np.array_equal(node[t, k].view(np.uint32), h_want.view(np.uint32)), f"gate/up node t{t} k{k}"
        if layer_hidden is not None:
            assert np.array_equal(layer_hidden[t, k].view(np.uint32), h_want.view(np.uint32)), f"layer hidden rows t{t} k{k}"
    for w in (GE, UE, DE):
        w.free()
