"""The library's workspaces are one set per process.  Three rules keep that safe:
  * a call on another stream is ordered behind the previous call's device work (no two calls overlap on the device);
  * a workspace that has to grow after a HIP-graph capture is retired, not freed: the graph's replays stay valid;
  * the host-pointer entry point holds the library lock from its first staging copy to its last, so threads cannot
    interleave their copies."""
import threading

import numpy as np
import pytest

from densecore_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    from densecore_amd import _lib, ops
    assert torch.cuda.is_available()
    return torch, _lib, ops


def test_calls_on_two_streams_do_not_share_the_workspace_at_the_same_time(env):
    torch, _lib, ops = env
    rows, cols, n = 4096, 14336, 8      # the quantize + product pair through the global workspace
    W = ops.Q4KWeight.synthetic(61, rows, cols)
    xs = [torch.from_numpy(synth.normal_f32(6100 + i, (n, cols))).cuda() for i in range(6)]
    want = [ops.mul_mat(W, x).clone() for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.empty((n, rows), dtype=torch.float32, device="cuda") for _ in xs]
    for rep in range(5):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        for i, x in enumerate(xs):  # alternate streams, never synchronise in between
            with torch.cuda.stream(streams[i & 1]):
                ops.mul_mat(W, x, outs[i])
        torch.cuda.synchronize()
        for i in range(len(xs)):
            assert torch.equal(outs[i], want[i]), f"rep {rep}, call {i}"


def test_a_workspace_that_grows_after_a_capture_leaves_the_graph_valid(env):
    torch, _lib, ops = env
    small = ops.Q4KWeight.synthetic(62, 512, 1024)
    xs = torch.from_numpy(synth.normal_f32(6200, (6, 1024))).cuda()
    want = ops.mul_mat(small, xs).clone()
    side = torch.cuda.Stream()
    out = torch.empty_like(want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.mul_mat(small, xs, out)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    # a far larger activation set: every workspace of the product has to grow
    big = ops.Q4KWeight.synthetic(63, 256, 65536)
    xb = torch.from_numpy(synth.normal_f32(6201, (16, 65536))).cuda()
    yb = ops.mul_mat(big, xb)
    torch.cuda.synchronize()
    assert torch.isfinite(yb).all()
    for _ in range(3):  # the graph still launches on the addresses it captured
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
    # filler that lands where a freed workspace would have been reused, then replay again
    junk = [torch.full((1 << 20,), float("nan"), device="cuda") for _ in range(8)]
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    del junk


def test_host_entry_point_from_several_threads(env):
    torch, _lib, ops = env
    import ctypes as C
    rows, cols, m = 768, 2048, 3
    W = ops.Q4KWeight.synthetic(64, rows, cols)
    xs = [synth.normal_f32(6300 + i, (m, cols)) for i in range(4)]
    want = [ops.mul_mat(W, torch.from_numpy(x).cuda()).cpu().numpy() for x in xs]
    errors = []

    def worker(i):
        y = np.zeros((m, rows), np.float32)
        for _ in range(25):
            y[:] = 0
            rc = _lib.lib().mq_mul_mat_q4k_host(W._h, C.c_void_p(xs[i].ctypes.data), m, cols, C.c_void_p(y.ctypes.data), rows)
            if rc != 0 or not np.array_equal(y.view(np.uint32), want[i].view(np.uint32)):
                errors.append((i, rc))
                return

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_skeleton_mode_launches_nothing_that_computes_and_restores(env):
    """mq_debug_set_skeleton: while it is on, a product call queues an empty kernel of the same shape (the output stays as
    it was); switched off again the same call computes, and the switch reports its previous setting."""
    import torch
    from densecore_amd import _lib, ops, synth
    L = _lib.lib()
    w = ops.Q4KWeight.synthetic(synth.tensor_seed("skel-w"), 512, 1024)
    x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("skel-x"), (3, 1024))).cuda()
    want = ops.mul_mat(w, x).clone()
    out = torch.full_like(want, 7.0)
    assert L.mq_debug_set_skeleton(1) == 0
    try:
        ops.mul_mat(w, x, out=out)
        torch.cuda.synchronize()
        assert torch.all(out == 7.0)
    finally:
        assert L.mq_debug_set_skeleton(0) == 1
    ops.mul_mat(w, x, out=out)
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    w.free()
