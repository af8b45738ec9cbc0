"""Stream order and HIP graph replay of the kernel launchers: everything the library enqueues goes to the
caller's current stream, and none of it (no allocation, no memset, no host synchronisation inside the C ABI)
stands in the way of capturing it."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(seed, N=640, D=256, V=5000):
    g = torch.Generator().manual_seed(seed)
    e = torch.randn((N, D), generator=g).to(torch.bfloat16)
    c = (torch.randn((V, D), generator=g) * 0.08).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g)
    return e, c, t


def test_operator_on_a_side_stream_matches_the_default_stream():
    """Inputs are produced on a side stream right before the operator runs there: were a kernel enqueued on
    another stream it would race with the fills.  The result must be bit-identical (the kernels are
    deterministic) to the run on the default stream."""
    from cut_cross_entropy import linear_cross_entropy

    e, c, t = _inputs(21)

    def run():
        ed = torch.empty_like(e, device=DEV)
        cd = torch.empty_like(c, device=DEV)
        big = torch.empty((64, 1 << 20), device=DEV)
        for _ in range(4):
            big.normal_()  # keeps the stream busy so that a launch on another stream would run ahead
        ed.copy_(e, non_blocking=False)
        cd.copy_(c, non_blocking=False)
        ed.requires_grad_(True)
        cd.requires_grad_(True)
        loss, lse = linear_cross_entropy(ed, cd, t.to(DEV), softcap=20.0, return_lse=True, filter_eps=None)
        loss.backward()
        return loss.detach(), lse.detach(), ed.grad, cd.grad

    want = run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=DEV)
    with torch.cuda.stream(side):
        got = run()
    side.synchronize()
    for g, w in zip(got, want):
        assert torch.equal(g, w)


@pytest.mark.parametrize("filter_eps", [2.0**-12, None])
def test_launchers_replay_in_a_hip_graph(filter_eps):
    """LSE, indexed dot and backward launchers captured once and replayed on new contents of the same
    buffers, with eager work and synchronisation between the replays; every replay equals the eager call."""
    from cut_cross_entropy.cce_backward import cce_backward_kernel
    from cut_cross_entropy.cce_lse_forward import cce_lse_forward_kernel
    from cut_cross_entropy.indexed_dot import indexed_neg_dot_forward_kernel
    from cut_cross_entropy.utils import TensorInfo

    e0, c0, t0 = _inputs(30)
    e = e0.to(DEV)
    c = c0.to(DEV)
    t = t0.to(DEV)
    do = torch.full((e.size(0),), 1.0 / e.size(0), device=DEV)
    info = TensorInfo(torch.bfloat16, True)

    def step():
        lse = cce_lse_forward_kernel(e, c, softcap=25.0)
        nd = indexed_neg_dot_forward_kernel(e, c, t, softcap=25.0, out_dtype=torch.float32)
        de, dc, _ = cce_backward_kernel(do, None, e, info, c, info, None, None, lse, None, 25.0, filter_eps,
                                        targets=t)
        return lse, nd, de, dc

    step()  # loads the library, sets kernel attributes and warms the GEMM workspaces outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for seed in (31, 32, 33):
        en, cn, tn = _inputs(seed)
        e.copy_(en)
        c.copy_(cn)
        t.copy_(tn)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in out]
        want = step()
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w), seed
