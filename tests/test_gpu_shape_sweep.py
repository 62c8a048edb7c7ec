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
