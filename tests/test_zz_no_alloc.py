"""cce_lse_forward_static (the entry point that allocates nothing: its split-vocabulary partials live in a
static device array) against cce_lse_forward with a caller's workspace, through the C ABI: identical
kernels, so the results must be bit-identical.  Two calls in a row share the array; the second is smaller,
so stale partials of the first lie beyond and between what it writes."""

import pytest
import torch

from _util import make_inputs

pytestmark = pytest.mark.gpu


def _lib():
    from cut_cross_entropy import _hip

    return _hip.load()


def _run_both(lib, dev, N, V, D, dtype, softcap, has_bias, invalid_frac, seed):
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=seed, bias=has_bias, invalid_frac=invalid_frac)
    ed, cd = e.to(dev), c.to(dev)
    bd = bias.to(dev) if bias is not None else None
    valids = None
    B = N
    if invalid_frac > 0:
        valids = torch.nonzero(t != -100).flatten().to(torch.int32).to(dev)
        B = valids.numel()
    code = 0 if dtype == torch.bfloat16 else 1
    stream = torch.cuda.current_stream().cuda_stream
    n_stat = lib.cce_tile_stat_elems(B, V)

    def outputs():
        return (torch.full((B,), float("nan"), dtype=torch.float32, device=dev),
                torch.full((V,), float("nan"), dtype=torch.float32, device=dev),
                torch.full((n_stat,), float("nan"), dtype=torch.float32, device=dev))

    lse_a, la_a, tm_a = outputs()
    ws_bytes = lib.cce_lse_forward_workspace_bytes(B, V, D)
    ws = torch.empty((ws_bytes // 8 + 1,), dtype=torch.int64, device=dev)
    st = lib.cce_lse_forward(
        ed.data_ptr(), cd.data_ptr(), bd.data_ptr() if bd is not None else None,
        valids.data_ptr() if valids is not None else None,
        lse_a.data_ptr(), la_a.data_ptr(), tm_a.data_ptr(), ws.data_ptr(), ws.numel() * 8,
        N, B, V, D, ed.stride(0), cd.stride(0), cd.stride(1), softcap or 0.0, code, stream)
    assert st == 0, lib.cce_error_string(st)

    lse_b, la_b, tm_b = outputs()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    st = lib.cce_lse_forward_static(
        ed.data_ptr(), cd.data_ptr(), bd.data_ptr() if bd is not None else None,
        valids.data_ptr() if valids is not None else None,
        lse_b.data_ptr(), la_b.data_ptr(), tm_b.data_ptr(),
        N, B, V, D, ed.stride(0), cd.stride(0), cd.stride(1), softcap or 0.0, code, stream)
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    return (lse_a, tm_a, la_a), (lse_b, tm_b, la_b), (e, c, bias, t, valids)


def test_static_scratch_matches_workspace_entry_on_two_calls_in_a_row():
    from oracle import dense_lce

    lib = _lib()
    dev = torch.device("cuda:0")
    # first call: several vocabulary spans per row block; second: fewer rows, fewer classes, another option set
    cases = [
        dict(N=1536, V=20000, D=256, dtype=torch.bfloat16, softcap=30.0, has_bias=False, invalid_frac=0.0, seed=11),
        dict(N=300, V=1000, D=72, dtype=torch.float16, softcap=None, has_bias=True, invalid_frac=0.2, seed=12),
    ]
    for case in cases:
        print("case", case, flush=True)
        (lse_a, tm_a, la_a), (lse_b, tm_b, la_b), (e, c, bias, t, valids) = _run_both(lib, dev, **case)
        assert torch.isfinite(lse_b).all()
        assert torch.equal(lse_a, lse_b), "lse differs between the two entry points"
        assert torch.equal(tm_a, tm_b), "tile statistic differs between the two entry points"
        # the column average is summed with float atomics in no fixed order: equal up to rounding
        assert torch.allclose(la_a, la_b, atol=1e-4, rtol=1e-4)
        rows = e if valids is None else e[valids.cpu().long()]
        want = dense_lce.dense_lse(rows, c, bias, case["softcap"], compute_dtype=torch.float64)
        assert torch.allclose(lse_b.cpu().double(), want, rtol=1e-3, atol=1e-3)


def test_static_scratch_rejects_shapes_beyond_its_size():
    from cut_cross_entropy import _hip

    lib = _lib()
    dev = torch.device("cuda:0")
    x = torch.zeros((64,), dtype=torch.float32, device=dev)
    B, V, D = 1 << 22, 4096, 64  # 4 M rows: the partials alone need 32 MB or more
    assert lib.cce_lse_forward_workspace_bytes(B, V, D) > _hip.STATIC_SCRATCH_BYTES
    # refused on the host before anything is launched: the pointers are never dereferenced
    st = lib.cce_lse_forward_static(x.data_ptr(), x.data_ptr(), None, None, x.data_ptr(), None, None,
                                    B, B, V, D, D, D, 1, 0.0, 0, torch.cuda.current_stream().cuda_stream)
    assert st == 10005
    assert b"static" in lib.cce_error_string(st)


def test_static_entry_replays_in_a_hip_graph_after_init():
    """The set-up call resolves the device's scratch array, so that a FIRST call of the entry point may fall inside a
    graph capture; every replay, on new contents and with eager work in between, must equal the eager workspace entry."""
    lib = _lib()
    dev = torch.device("cuda:0")
    assert lib.cce_lse_forward_static_init() == 0
    N, V, D = 640, 5000, 128
    g = torch.Generator().manual_seed(21)
    e = torch.empty((N, D), dtype=torch.bfloat16, device=dev)
    c = torch.empty((V, D), dtype=torch.bfloat16, device=dev)
    lse_graph = torch.empty((N,), dtype=torch.float32, device=dev)
    tm_graph = torch.empty((lib.cce_tile_stat_elems(N, V),), dtype=torch.float32, device=dev)

    def refill():
        e.copy_(torch.randn((N, D), generator=g).to(torch.bfloat16))
        c.copy_((torch.randn((V, D), generator=g) * 0.05).to(torch.bfloat16))

    refill()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = lib.cce_lse_forward_static(
            e.data_ptr(), c.data_ptr(), None, None, lse_graph.data_ptr(), None, tm_graph.data_ptr(),
            N, N, V, D, e.stride(0), c.stride(0), c.stride(1), 30.0, 0, torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.cce_error_string(st)
    ws_bytes = lib.cce_lse_forward_workspace_bytes(N, V, D)
    ws = torch.empty((ws_bytes // 8 + 1,), dtype=torch.int64, device=dev)
    for rep in range(3):
        print("replay", rep, flush=True)
        refill()
        lse_graph.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        lse_eager = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
        tm_eager = torch.empty_like(tm_graph)
        st = lib.cce_lse_forward(
            e.data_ptr(), c.data_ptr(), None, None, lse_eager.data_ptr(), None, tm_eager.data_ptr(),
            ws.data_ptr(), ws.numel() * 8, N, N, V, D, e.stride(0), c.stride(0), c.stride(1), 30.0, 0,
            torch.cuda.current_stream().cuda_stream)
        assert st == 0, lib.cce_error_string(st)
        torch.cuda.synchronize()
        assert torch.isfinite(lse_graph).all()
        assert torch.equal(lse_graph, lse_eager)
        assert torch.equal(tm_graph, tm_eager)
