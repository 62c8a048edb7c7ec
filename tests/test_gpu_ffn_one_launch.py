"""mq_ffn_swiglu_q4k as one persistent launch (up to 8 rows of Q4_K weights) against the one-node entry points.

The persistent kernel splits every row tile over as many wavefronts as the one-node launches do and keeps their
summation orders, so its output equals mq_swiglu_mul_mat_q4k followed by mq_mul_mat_q4k bit for bit; those two are
checked against the CPU restatement in tests/test_gpu_ffn_moe.py and tests/test_gpu_parity.py.  The shapes below
cover every way a workgroup's eight wavefronts can be dealt out: one to eight wavefronts per row tile (including
counts that leave wavefronts idle), more and fewer row tiles than workgroups, odd numbers of super-blocks.
"""
import numpy as np
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    from densecore_amd import ops as o
    assert torch.cuda.is_available()
    return o


def _weights(ops, tag, hidden, inter):
    seeds = [synth.tensor_seed(tag, nm) for nm in "gud"]
    return [ops.Q4KWeight.synthetic(s, r, c) for s, (r, c) in zip(seeds, ((inter, hidden), (inter, hidden), (hidden, inter)))]


def _check(ops, G, U, D, x, silu):
    import torch
    y = ops.ffn_swiglu(G, U, D, x, silu)
    h = ops.swiglu_mul_mat(G, U, x, silu)
    want = ops.mul_mat(D, h)
    torch.cuda.synchronize()
    ops.stream_synchronize()
    assert torch.isfinite(y).all()
    assert torch.equal(y, want), f"max |diff| {(y - want).abs().max().item():.3e}"


SHAPES = [
    # hidden, inter: wavefronts per row tile (gate/up, down)
    (256, 256),      # 1, 1: every wavefront owns a row tile
    (512, 768),      # 2, 3: three wavefronts per row tile leave two idle
    (1024, 1792),    # 4, 7
    (2048, 1280),    # 8, 5
    (1536, 4096),    # 6, 8
    (1792, 4864),    # 7, 1: more gate/up row tiles than workgroups; 19 super-blocks per down row (odd)
    (4096, 14336),   # 2, 8: the dense FFN of the benchmark
]


@pytest.mark.parametrize("hidden,inter", SHAPES)
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_bitwise_equal_to_the_one_node_launches(ops, hidden, inter, n):
    import torch
    G, U, D = _weights(ops, f"ffn1-{hidden}-{inter}", hidden, inter)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("ffn1-x", n), (n, hidden))).cuda()
    _check(ops, G, U, D, x, 2)
    for w in (G, U, D):
        w.free()


@pytest.mark.parametrize("silu", [0, 1])
def test_other_silu_orders(ops, silu):
    import torch
    G, U, D = _weights(ops, "ffn1-silu", 1024, 2048)
    x = torch.from_numpy(synth.normal_f32(5, (4, 1024))).cuda()
    _check(ops, G, U, D, x, silu)
    for w in (G, U, D):
        w.free()


def test_repeated_calls_shrinking_and_growing_widths(ops):
    """The workgroups' LDS and the exchange buffer are re-used: rows left by a wider call must not leak into a
    narrower one, and zero rows / large magnitudes take the quantizer's special paths inside the kernel."""
    import torch
    G, U, D = _weights(ops, "ffn1-rep", 2048, 5632)
    for n, scale in [(8, 1.0), (1, 100.0), (5, 1e-3), (2, 1.0), (8, 3.0)]:
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("ffn1-rep-x", n), (n, 2048))).cuda() * scale
        x[n // 2].zero_()
        _check(ops, G, U, D, x, 2)
    for w in (G, U, D):
        w.free()


def test_graph_replays(ops):
    import torch
    G, U, D = _weights(ops, "ffn1-graph", 1024, 3072)
    x = torch.from_numpy(synth.normal_f32(9, (3, 1024))).cuda()
    want = ops.mul_mat(D, ops.swiglu_mul_mat(G, U, x, 2)).clone()
    ops.ffn_swiglu(G, U, D, x, 2)   # workspaces grow outside the capture
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            y = ops.ffn_swiglu(G, U, D, x, 2)
    for rep in range(3):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), f"replay {rep}"
        assert torch.equal(ops.ffn_swiglu(G, U, D, x, 2), want)   # eager launches between the replays
        torch.cuda.synchronize()
    ops.stream_synchronize()
    for w in (G, U, D):
        w.free()


def test_against_cpu_restatement_end_to_end(ops):
    import torch
    from oracle import binding as orc
    hidden, inter, n = 512, 1024, 3
    g, u, d = (synth.q4k_matrix(synth.tensor_seed("ffn1-orc", nm), r, c) for nm, r, c in
               (("g", inter, hidden), ("u", inter, hidden), ("d", hidden, inter)))
    G, U, D = ops.Q4KWeight.from_ggml(g, hidden), ops.Q4KWeight.from_ggml(u, hidden), ops.Q4KWeight.from_ggml(d, inter)
    x = synth.normal_f32(11, (n, hidden))
    y = ops.ffn_swiglu(G, U, D, torch.from_numpy(x).cuda(), 2).cpu().numpy()
    ref = orc.ffn_swiglu(g, u, d, hidden, inter, x, orc.ORDER_DOTPROD, 2)
    # a 1-ulp difference before the re-quantization can flip a Q8_K code: the end-to-end bound of the dense FFN
    assert np.max(np.abs(y - ref)) <= 2e-3 * np.max(np.abs(ref))
    for w in (G, U, D):
        w.free()
