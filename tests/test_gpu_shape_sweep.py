"""Small and awkward shapes at many widths against the CPU restatement: one to 257 weight rows (less than a row tile,
one more than a row tile, no multiple of four), one to 64 super-blocks per row (a single stage, an odd count, more than
LDS holds), the four weight types, 1..100 activation rows -- whatever kernel the combination selects, to the path's
1e-4 (the oracle's row m depends on activation row m alone, so one oracle product of 100 rows serves every width)."""
import numpy as np
import pytest

from densecore_amd import synth
from oracle import binding as orc
from tests._parity import assert_fp32_parity

pytestmark = pytest.mark.gpu

TYPES = {
    12: (synth.q4k_matrix, orc.quantize_rows_q8k, orc.mul_mat_q4k_q8k, lambda w, c, q: orc.dot_magnitude_f64(w, c, q)),
    13: (synth.q5k_matrix, orc.quantize_rows_q8k, orc.mul_mat_q5k_q8k, lambda w, c, q: orc.q5k_dot_dequant_f64(w, c, q, magnitude=True)),
    14: (synth.q6k_matrix, orc.quantize_rows_q8k, orc.mul_mat_q6k_q8k, lambda w, c, q: orc.q6k_dot_dequant_f64(w, c, q, magnitude=True)),
    8: (synth.q80_matrix, orc.quantize_rows_q80, orc.mul_mat_q80_q80, lambda w, c, q: orc.q80_dot_dequant_f64(w, c, q, magnitude=True)),
}
WIDTHS = (1, 2, 3, 4, 5, 8, 9, 16, 17, 33, 49, 65, 100)


@pytest.mark.parametrize("wtype", [12, 13, 14, 8])
@pytest.mark.parametrize("cols", [256, 768, 4352, 16384])
def test_awkward_shapes_against_the_oracle(cols, wtype):
    import torch
    from densecore_amd import ops
    make, quant, mul, magnitude = TYPES[wtype]
    x = synth.normal_f32(synth.tensor_seed("shp-x", cols), (100, cols))
    xd = torch.from_numpy(x).cuda()
    q = quant(x)
    for rows in (1, 5, 17, 100, 257):
        w = make(synth.tensor_seed("shp-w", rows, cols, wtype), rows, cols)
        W = ops.Q4KWeight.from_ggml(w, cols, ggml_type=wtype)
        ref = mul(w, cols, q)
        mag = magnitude(w, cols, q[:8])       # (a per-row scale of the first rows is enough for the floor)
        mag = np.broadcast_to(mag.max(axis=0, keepdims=True), ref.shape)
        for n in WIDTHS:
            got = ops.mul_mat(W, xd[:n]).cpu().numpy()
            assert_fp32_parity(got, ref[:n], mag[:n], f"type {wtype} {rows}x{cols} n={n}")
        W.free()


# (experts, top_k, hidden, inter, shared expert, gate projection of the shared expert)
MOE_CONFIGS = [(1, 1, 256, 256, False, False), (2, 2, 256, 512, True, True), (3, 3, 768, 256, False, False),
               (9, 8, 512, 768, True, False), (300, 2, 256, 256, True, True), (600, 4, 256, 256, False, False)]


@pytest.mark.parametrize("E,K,H,I,shared,gated", MOE_CONFIGS)
def test_awkward_moe_configurations_against_the_oracle(E, K, H, I, shared, gated):
    """One expert, top_k equal to the expert count, a single super-block per row, more experts than the token-major
    kernels take (512), a shared expert without its gate: the layer at twelve widths from 1 to 300 tokens against the
    CPU restatement (one oracle run of 300 tokens serves every width: a token's row depends on that token alone)."""
    import torch
    from densecore_amd import ops
    tag = ("shp-moe", E, K, H, I)
    stack = lambda name, r, c, cnt: np.stack([synth.q4k_matrix(synth.tensor_seed(*tag, name, e), r, c) for e in range(cnt)])
    ge, ue, de = stack("g", I, H, E), stack("u", I, H, E), stack("d", H, I, E)
    GE, UE, DE = ops.Q4KWeight.from_ggml(ge, H), ops.Q4KWeight.from_ggml(ue, H), ops.Q4KWeight.from_ggml(de, I)
    sh_cpu = sh_gpu = None
    if shared:
        sg, su, sd = (synth.q4k_matrix(synth.tensor_seed(*tag, nm), r, c) for nm, r, c in (("sg", I, H), ("su", I, H), ("sd", H, I)))
        gi = synth.normal_f32(synth.tensor_seed(*tag, "gi"), (H,)) * np.float32(0.02) if gated else None
        sh_cpu = (sg, su, sd, gi)
        sh_gpu = (ops.Q4KWeight.from_ggml(sg, H), ops.Q4KWeight.from_ggml(su, H), ops.Q4KWeight.from_ggml(sd, I),
                  torch.from_numpy(gi).cuda() if gated else None)
    N = 300
    x = synth.normal_f32(synth.tensor_seed(*tag, "x"), (N, H))
    logits = synth.normal_f32(synth.tensor_seed(*tag, "l"), (N, E))
    xd, ld = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    ref = orc.moe_layer(ge, ue, de, H, I, K, x, logits, shared=sh_cpu, silu=orc.SILU_FAST)
    scale = np.abs(ref["y"]).max()
    for n in (1, 2, 3, 5, 8, 9, 16, 17, 40, 70, 200, N):
        y, ids, w = ops.moe_layer(GE, UE, DE, xd[:n], ld[:n], K, shared=sh_gpu, silu=ops.SILU_FAST)
        assert np.array_equal(ids.cpu().numpy(), ref["ids"][:n]), f"ids n={n}"
        assert np.allclose(w.cpu().numpy(), ref["weights"][:n], rtol=3e-6, atol=1e-9), f"weights n={n}"
        err = np.abs(y.cpu().numpy() - ref["y"][:n]).max(axis=1) / scale
        # (a last-bit difference in a hidden row can move a code of the down product's quantizer: a few tokens)
        assert err.max() <= 1e-3 and (err > 1e-4).sum() <= max(1, n // 50), f"n={n}: {err.max():.3e}"
    for t in (GE, UE, DE) + (tuple(sh_gpu[:3]) if shared else ()):
        t.free()
