"""Parity of the three HIP kernels, called through the C ABI, against the CPU oracle."""

import pytest
import torch

from _util import IGNORE_INDEX, assert_no_worse, autograd_grads, make_inputs

pytestmark = pytest.mark.gpu

SHAPES = [(256, 512, 128), (255, 507, 128), (255, 507, 123), (300, 1000, 72), (64, 130, 64)]


def _lib():
    from cut_cross_entropy import _hip

    return _hip.load()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_lse_forward_abi(dtype, softcap, has_bias, shape):
    """cce_lse_forward vs logsumexp of the dense logits (reference tests/test_cce_lse.py:23-63)."""
    from oracle import dense_lce

    N, V, D = shape
    e, c, _, bias = make_inputs(N, V, D, dtype, seed=1, bias=has_bias)
    gt = dense_lce.dense_lse(e, c, bias, softcap, compute_dtype=torch.float64)
    ref = dense_lce.dense_lse(e, c, bias, softcap, compute_dtype=dtype)

    lib = _lib()
    dev = torch.device("cuda:0")
    ed, cd = e.to(dev), c.to(dev)
    bd = bias.to(dev) if bias is not None else None
    lse = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    la = torch.empty((V,), dtype=torch.float32, device=dev)
    tm = torch.empty((lib.cce_tile_stat_elems(N, V),), dtype=torch.float32, device=dev)
    ws_bytes = lib.cce_lse_forward_workspace_bytes(N, V, D)
    ws = torch.empty((ws_bytes // 8 + 1,), dtype=torch.int64, device=dev)
    st = lib.cce_lse_forward(
        ed.data_ptr(), cd.data_ptr(), bd.data_ptr() if bd is not None else None, None,
        lse.data_ptr(), la.data_ptr(), tm.data_ptr(), ws.data_ptr(), ws.numel() * 8,
        N, N, V, D, ed.stride(0), cd.stride(0), cd.stride(1),
        softcap or 0.0, 0 if dtype == torch.bfloat16 else 1,
        torch.cuda.current_stream().cuda_stream,
    )
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    assert_no_worse(gt, ref, lse, 1e-5 if dtype == torch.float16 else 2e-5, "lse")

    # column average of the (soft-capped) logits
    logits = dense_lce._dense_logits(e, c, bias, softcap, torch.float64)
    assert torch.allclose(la.cpu().double(), logits.mean(0), atol=2e-2, rtol=2e-2)

    # tile statistic: max soft-capped logit per 32-row x 32-class cell
    nr, nc = (N + 31) // 32, (V + 31) // 32
    want = torch.full((nr, nc), float("-inf"), dtype=torch.float64)
    for r in range(nr):
        for cc in range(nc):
            want[r, cc] = logits[r * 32 : (r + 1) * 32, cc * 32 : (cc + 1) * 32].max()
    got = tm.cpu().double().view(nr, nc)
    assert (got >= want - 0.05).all() and (got <= want + 0.05).all()


@pytest.mark.parametrize("softcap", [None, 20.0, 50.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("shape", [(8192, 20011, 128), (8000, 24576, 192)])
def test_lse_forward_spans_of_many_tiles(softcap, has_bias, shape):
    """Thirty-two row blocks leave eight vocabulary spans per row block, each of nine to twelve 256-class tiles: the
    16x16x32 kernel collects the statistic cells of eight tiles in registers before it stores them, so a span of more
    than eight tiles has a full batch and a remainder; the ring runs on across the tiles of a span.  Checked against
    dense fp32 logits formed on the GPU (soft-cap 50 is beyond the fixed-reference range of the epilogue)."""
    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D = shape
    dtype = torch.bfloat16
    e, c, _, bias = make_inputs(N, V, D, dtype, seed=3, bias=has_bias)
    ed, cd = e.to(dev), c.to(dev)
    bd = bias.to(dev) if bias is not None else None
    logits = ed.float() @ cd.float().T
    if bd is not None:
        logits += bd.float()
    if softcap is not None:
        logits = torch.tanh(logits / softcap) * softcap
    want_lse = torch.logsumexp(logits.double(), dim=1)
    lse = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    tm = torch.full((lib.cce_tile_stat_elems(N, V),), float("nan"), dtype=torch.float32, device=dev)
    ws_bytes = lib.cce_lse_forward_workspace_bytes(N, V, D)
    ws = torch.empty((ws_bytes // 8 + 1,), dtype=torch.int64, device=dev)
    st = lib.cce_lse_forward(
        ed.data_ptr(), cd.data_ptr(), bd.data_ptr() if bd is not None else None, None,
        lse.data_ptr(), None, tm.data_ptr(), ws.data_ptr(), ws.numel() * 8,
        N, N, V, D, ed.stride(0), cd.stride(0), cd.stride(1),
        softcap or 0.0, 0, torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    assert torch.allclose(lse.double(), want_lse, atol=2e-4, rtol=2e-5)
    nr, nc = (N + 31) // 32, (V + 31) // 32
    pad = torch.full((nr * 32, nc * 32), float("-inf"), device=dev)
    pad[:N, :V] = logits
    want = pad.view(nr, 32, nc, 32).amax(dim=(1, 3))
    got = tm.view(nr, nc)
    assert torch.isfinite(got).all()
    assert ((got - want).abs() <= 0.05).all()


@pytest.mark.parametrize("softcap", [None, 20.0, 50.0])
@pytest.mark.parametrize("shape,gathered", [((8192, 20011, 128), False), ((1000, 5000, 192), True), ((700, 2304, 256), True)])
def test_lse_forward_column_average_over_spans(softcap, shape, gathered):
    """logit_avg (reference cce_lse_forward.py:95-97: the mean over the rows of the soft-capped logits with bias) on
    the 16x16x32 kernel: a workgroup sums a tile's columns in LDS and hands them over while it works on the next tile,
    so spans of one, several and many tiles, a last tile that is cut by V, a last row block that is cut by B and rows
    gathered through `valids` are all different code.  Two calls in a row: the entry clears the average itself."""
    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D = shape
    e, c, _, bias = make_inputs(N, V, D, torch.bfloat16, seed=5, bias=True)
    ed, cd, bd = e.to(dev), c.to(dev), bias.to(dev)
    if gathered:
        g = torch.Generator().manual_seed(6)
        valids = torch.randperm(N, generator=g)[: N - 37].sort().values.to(torch.int32).to(dev)
    else:
        valids = None
    B = N if valids is None else valids.numel()
    rows = ed if valids is None else ed[valids.long()]
    logits = rows.float() @ cd.float().T + bd.float()
    if softcap is not None:
        logits = torch.tanh(logits / softcap) * softcap
    want_avg = logits.double().mean(0)
    want_lse = torch.logsumexp(logits.double(), dim=1)
    lse = torch.full((B,), float("nan"), dtype=torch.float32, device=dev)
    la = torch.full((V,), float("nan"), dtype=torch.float32, device=dev)
    ws_bytes = lib.cce_lse_forward_workspace_bytes(B, V, D)
    ws = torch.empty((ws_bytes // 8 + 1,), dtype=torch.int64, device=dev)
    for _ in range(2):
        st = lib.cce_lse_forward(
            ed.data_ptr(), cd.data_ptr(), bd.data_ptr(), valids.data_ptr() if valids is not None else None,
            lse.data_ptr(), la.data_ptr(), None, ws.data_ptr(), ws.numel() * 8,
            N, B, V, D, ed.stride(0), cd.stride(0), cd.stride(1),
            softcap or 0.0, 0, torch.cuda.current_stream().cuda_stream)
        assert st == 0, lib.cce_error_string(st)
        torch.cuda.synchronize()
        assert torch.allclose(lse.double(), want_lse, atol=2e-4, rtol=2e-5)
        assert torch.allclose(la.double(), want_avg, atol=2e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("shape", [(256, 512, 128), (255, 507, 123), (100, 300, 520)])
def test_indexed_neg_dot_abi(dtype, softcap, has_bias, shape):
    """cce_indexed_neg_dot vs the explicit gather-dot (reference tests/test_cce_indexed_dot.py:11-66).
    D = 520 > 256 with a bias checks that the bias is subtracted exactly once."""
    from oracle import dense_lce

    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=2, bias=has_bias)
    gt = dense_lce.dense_indexed_neg_dot(e, c, t, bias, softcap, torch.float64)
    lib = _lib()
    dev = torch.device("cuda:0")
    ed, cd, td = e.to(dev), c.to(dev), t.to(dev)
    bd = bias.to(dev) if bias is not None else None
    out = torch.full((N,), float("nan"), dtype=torch.float32, device=dev)
    st = lib.cce_indexed_neg_dot(
        ed.data_ptr(), cd.data_ptr(), td.data_ptr(), bd.data_ptr() if bd is not None else None, None,
        out.data_ptr(), N, N, V, D, ed.stride(0), cd.stride(0), cd.stride(1), 0, 0,
        softcap or 0.0, 0 if dtype == torch.bfloat16 else 1, torch.cuda.current_stream().cuda_stream,
    )
    assert st == 0
    torch.cuda.synchronize()
    # products are exact in fp32, only the summation order differs
    assert torch.allclose(out.cpu().double(), gt, atol=1e-5, rtol=1e-5)


def _run_backward_abi(e, c, t, bias, valids, lse, d_out, d_lse, softcap, shift, grad_scale, filter_eps,
                      fp32_accum, dtype, order=None):
    lib = _lib()
    dev = torch.device("cuda:0")
    N, D = e.shape
    V = c.shape[0]
    ed, cd, td = e.to(dev), c.to(dev), t.to(dev)
    bd = bias.to(dev) if bias is not None else None
    vd = valids.to(dev) if valids is not None else None
    B = valids.numel() if valids is not None else N
    lsed = lse.float().to(dev)
    dod = d_out.float().to(dev).contiguous()
    dld = d_lse.float().to(dev).contiguous() if d_lse is not None else None
    od = order.to(dev) if order is not None else None
    gdt = torch.float32 if fp32_accum else dtype
    de = torch.zeros((N, D), dtype=gdt, device=dev)
    # d_c need not be initialised: the kernel writes every element, zeros where nothing survived the filter
    dc = torch.full((V, D), float("nan"), dtype=gdt, device=dev)
    db = torch.zeros((V,), dtype=torch.float32, device=dev) if bias is not None else None
    counters = torch.zeros((4,), dtype=torch.int64, device=dev)
    ws = torch.empty((lib.cce_backward_workspace_bytes(B, V, D) // 8 + 1,), dtype=torch.int64, device=dev)
    p = lambda x: x.data_ptr() if x is not None else None
    st = lib.cce_backward(
        p(ed), p(cd), p(bd), p(lsed), p(dod), 1 if dod.numel() == 1 else 0, p(dld),
        p(vd), p(od), p(td), None, p(de), p(dc), p(db), p(ws), ws.numel() * 8, p(counters),
        N, B, V, D, ed.stride(0), cd.stride(0), cd.stride(1),
        grad_scale, -1.0 if filter_eps is None else filter_eps, 1, 1,
        1 if fp32_accum else 0, 1 if fp32_accum else 0, shift, 0,
        softcap or 0.0, 0 if dtype == torch.bfloat16 else 1, torch.cuda.current_stream().cuda_stream,
    )
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    return de.cpu(), dc.cpu(), (db.cpu() if db is not None else None), counters.cpu()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("with_dlse", [False, True])
@pytest.mark.parametrize("shape", [(256, 512, 128), (255, 507, 123), (200, 700, 72)])
def test_backward_abi_exact(dtype, softcap, has_bias, with_dlse, shape):
    """cce_backward without filtering, fp32 accumulation, vs the closed-form dense gradients."""
    from oracle import dense_lce

    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=3, bias=has_bias, invalid_frac=0.2)
    valids = dense_lce.build_flat_valids(t, IGNORE_INDEX, 0)
    g = torch.Generator().manual_seed(7)
    d_out = torch.randn((N,), generator=g)
    d_lse = torch.randn((N,), generator=g) * 0.1 if with_dlse else None
    rows = valids.long()
    lse = dense_lce.dense_lse(e[rows], c, bias, softcap, torch.float64)

    gt = dense_lce.dense_grads(e, c, t, valids, d_out * 0.5, d_lse, bias, softcap, 0, torch.float64)
    ref = autograd_grads(e, c, t, valids, d_out * 0.5, d_lse, bias, softcap, 0, dtype)
    de, dc, db, counters = _run_backward_abi(e, c, t, bias, valids, lse, d_out, d_lse, softcap, 0, 0.5,
                                             None, True, dtype)
    # 1e-2 relative per element (bf16 rounding of dz) plus a small absolute floor
    tol, rel = 2e-3, 1e-2
    assert_no_worse(gt[0], ref[0], de, tol, "dE", rel)
    assert_no_worse(gt[1], ref[1], dc, tol, "dC", rel)
    if has_bias:
        assert_no_worse(gt[2], ref[2], db, tol, "dBias", rel)
    # ignored rows get exactly zero gradient
    ignored = torch.ones(N, dtype=torch.bool)
    ignored[rows] = False
    assert (de[ignored] == 0).all()
    # without filtering every 32 x 32 sub-tile is recomputed and enters both products
    nt = ((valids.numel() + 31) // 32) * ((V + 31) // 32)
    assert counters.tolist() == [nt, nt, nt, nt]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("with_dlse", [False, True])
@pytest.mark.parametrize("shape", [(256, 512, 128), (255, 507, 64), (700, 1300, 192)])
def test_backward_dz_abi(dtype, softcap, has_bias, with_dlse, shape):
    """cce_backward_dz on two vocabulary chunks: the products of the dz it writes (formed here in
    fp64) must be the closed-form dense gradients; rows past the valid ones and padding columns are
    never written."""
    from oracle import dense_lce

    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=5, bias=has_bias, invalid_frac=0.2)
    valids = dense_lce.build_flat_valids(t, IGNORE_INDEX, 0)
    B = valids.numel()
    g = torch.Generator().manual_seed(11)
    d_out = torch.randn((N,), generator=g)
    d_lse = torch.randn((N,), generator=g) * 0.1 if with_dlse else None
    rows = valids.long()
    lse = dense_lce.dense_lse(e[rows], c, bias, softcap, torch.float64)
    gt = dense_lce.dense_grads(e, c, t, valids, d_out * 0.5, d_lse, bias, softcap, 0, torch.float64)
    ref = autograd_grads(e, c, t, valids, d_out * 0.5, d_lse, bias, softcap, 0, dtype)

    ed, cd, td, vd = e.to(dev), c.to(dev), t.to(dev), valids.to(dev)
    bd = bias.to(dev) if bias is not None else None
    lsed, dod = lse.float().to(dev), d_out.float().to(dev)
    dld = d_lse.float().to(dev) if d_lse is not None else None
    p = lambda x: x.data_ptr() if x is not None else None
    split = (V // 2) // 8 * 8 + 8  # second chunk starts at a multiple of 8 that is not a tile boundary
    dz_full = torch.zeros((B, V), dtype=torch.float64)
    for v0, v1 in ((0, split), (split, V)):
        n = v1 - v0
        ldz = (n + 7) // 8 * 8 + 8  # one spare block of padding: must stay untouched
        dz = torch.full((B + 3, ldz), 7.0, dtype=dtype, device=dev)
        st = lib.cce_backward_dz(
            p(ed), cd[v0:v1].data_ptr(), (bd.data_ptr() + 2 * v0) if bd is not None else None,
            p(lsed), p(dod), 0, p(dld), p(vd), p(td), p(dz), ldz, 0,
            N, B, n, D, ed.stride(0), cd.stride(0), cd.stride(1),
            0.5, 0, v0, softcap or 0.0, 0 if dtype == torch.bfloat16 else 1,
            torch.cuda.current_stream().cuda_stream)
        assert st == 0, lib.cce_error_string(st)
        torch.cuda.synchronize()
        dzc = dz.cpu()
        assert (dzc[B:] == 7.0).all() and (dzc[:, n:] == 7.0).all()
        dz_full[:, v0:v1] = dzc[:B, :n].double()
    de = torch.zeros((N, D), dtype=torch.float64)
    de[rows] = dz_full @ c.double()
    dc = dz_full.t() @ e[rows].double()
    tol, rel = 2e-3, 1e-2
    assert_no_worse(gt[0], ref[0], de, tol, "dE", rel)
    assert_no_worse(gt[1], ref[1], dc, tol, "dC", rel)
    if has_bias:
        assert_no_worse(gt[2], ref[2], dz_full.sum(0), tol, "dBias", rel)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("fp32_out", [False, True])
@pytest.mark.parametrize("shape,dz_budget", [((256, 512, 128), 0), ((255, 507, 64), 0), ((700, 1300, 192), 0),
                                             ((300, 1100, 320), 1 << 30), ((520, 2100, 576), 520 * 768 * 2),
                                             ((1500, 300, 128), 0), ((1500, 300, 128), 1 << 30),
                                             ((2100, 500, 320), 768 * 512 * 2), ((900, 130, 64), 0)])
def test_backward_dense_abi(dtype, softcap, has_bias, fp32_out, shape, dz_budget):
    """cce_backward_dense (dz chunks + hand-written dE / dC products, one call) vs the closed-form dense
    gradients: several chunks (smallest workspace), one chunk (large workspace), ragged rows, classes and
    columns, rows gathered through valids, upstream d_lse.  The last four shapes have more than twice as many
    valid rows as classes: with 16-bit gradients the walk then goes by blocks of rows (five blocks of 256, one
    block, three blocks of 768 less a remainder, three of 256), dC carried between them as a 16-bit pair."""
    from oracle import dense_lce

    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=6, bias=has_bias, invalid_frac=0.2)
    valids = dense_lce.build_flat_valids(t, IGNORE_INDEX, 0)
    B = valids.numel()
    g = torch.Generator().manual_seed(13)
    d_out = torch.randn((N,), generator=g)
    d_lse = torch.randn((N,), generator=g) * 0.1
    rows = valids.long()
    lse = dense_lce.dense_lse(e[rows], c, bias, softcap, torch.float64)
    gt = dense_lce.dense_grads(e, c, t, valids, d_out * 0.5, d_lse, bias, softcap, 0, torch.float64)
    ref = autograd_grads(e, c, t, valids, d_out * 0.5, d_lse, bias, softcap, 0, dtype)

    ed, cd, td, vd = e.to(dev), c.to(dev), t.to(dev), valids.to(dev)
    bd = bias.to(dev) if bias is not None else None
    lsed, dod, dld = lse.float().to(dev), d_out.float().to(dev), d_lse.float().to(dev)
    gdt = torch.float32 if fp32_out else dtype
    de = torch.zeros((N, D), dtype=gdt, device=dev)
    dc = torch.full((V, D), float("nan"), dtype=gdt, device=dev)  # written, not accumulated
    db = torch.zeros((V,), dtype=torch.float32, device=dev) if bias is not None else None
    ws_bytes = lib.cce_backward_dense_workspace_bytes(B, V, D, 0 if fp32_out else 1, dz_budget)
    ws = torch.empty((ws_bytes + 256,), dtype=torch.uint8, device=dev)
    ws_ptr = (ws.data_ptr() + 255) // 256 * 256
    p = lambda x: x.data_ptr() if x is not None else None
    st = lib.cce_backward_dense(
        p(ed), p(cd), p(bd), p(lsed), p(dod), 0, p(dld), p(vd), p(td),
        p(de), p(dc), p(db), ws_ptr, ws_bytes,
        N, B, V, D, ed.stride(0), cd.stride(0), cd.stride(1),
        0.5, 1 if fp32_out else 0, 1 if fp32_out else 0, 0, 0,
        softcap or 0.0, 0 if dtype == torch.bfloat16 else 1, torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    tol, rel = 2e-3, 1e-2
    assert_no_worse(gt[0], ref[0], de.cpu(), tol, "dE", rel)
    assert_no_worse(gt[1], ref[1], dc.cpu(), tol, "dC", rel)
    if has_bias:
        assert_no_worse(gt[2], ref[2], db.cpu(), tol, "dBias", rel)
    ignored = torch.ones(N, dtype=torch.bool)
    ignored[rows] = False
    assert (de.cpu()[ignored] == 0).all()


@pytest.mark.parametrize("dz_budget", [0, 1 << 30])
def test_backward_dense_walks_by_rows_with_an_fp32_dc(dz_budget):
    """More than twice as many rows as classes, a 16-bit d_e and an fp32 d_c: the walk goes by blocks of rows, d_e of a
    block is written once, and the fp32 d_c is written by the first block and added to in place by the others (no
    compensation term is used for it).  Rows taken directly (no valids), a scalar upstream gradient."""
    from oracle import dense_lce

    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D, dtype = 1300, 200, 192, torch.bfloat16
    e, c, t, _ = make_inputs(N, V, D, dtype, seed=11)
    lse = dense_lce.dense_lse(e, c, None, None, torch.float64)
    d_out = torch.full((N,), 1.0 / N)
    gt = dense_lce.dense_grads(e, c, t, None, d_out, None, None, None, 0, torch.float64)
    ed, cd, td = e.to(dev), c.to(dev), t.to(dev)
    lsed = lse.float().to(dev)
    do = torch.full((1,), 1.0 / N, device=dev)
    de = torch.full((N, D), float("nan"), dtype=dtype, device=dev)          # written whole
    dc = torch.full((V, D), float("nan"), dtype=torch.float32, device=dev)  # written by the first block
    assert lib.cce_backward_dense_fixed_bytes(N, V, D, 1) == (V * D * 2 + 255) // 256 * 256  # the walk by rows
    ws_bytes = lib.cce_backward_dense_workspace_bytes(N, V, D, 1, dz_budget)
    ws = torch.empty((ws_bytes + 256,), dtype=torch.uint8, device=dev)
    st = lib.cce_backward_dense(
        ed.data_ptr(), cd.data_ptr(), None, lsed.data_ptr(), do.data_ptr(), 1, None, None, td.data_ptr(),
        de.data_ptr(), dc.data_ptr(), None, (ws.data_ptr() + 255) // 256 * 256, ws_bytes,
        N, N, V, D, D, D, 1, 1.0, 0, 1, 0, 0, 0.0, 0, torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    assert torch.isfinite(de).all() and torch.isfinite(dc).all()
    assert torch.allclose(de.cpu().double(), gt[0], atol=2e-2 / N, rtol=2e-2)
    assert torch.allclose(dc.cpu().double(), gt[1], atol=2e-2 / N, rtol=2e-2)


def test_backward_dense_ignores_non_finite_values_it_must_not_read():
    """Rows of e that are not valid and the reduction tails of the product tiles must not leak into the
    gradients: an ignored row full of inf / nan (and such a row as row 0, where absent rows used to point)
    leaves every gradient finite."""
    from oracle import dense_lce

    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D, dtype = 203, 333, 64, torch.bfloat16
    e, c, t, _ = make_inputs(N, V, D, dtype, seed=8)
    t[0] = IGNORE_INDEX
    t[77] = IGNORE_INDEX
    e[0] = float("inf")
    e[77] = float("nan")
    valids = dense_lce.build_flat_valids(t, IGNORE_INDEX, 0)
    B = valids.numel()
    rows = valids.long()
    lse = dense_lce.dense_lse(e[rows], c, None, None, torch.float64)
    d_out = torch.ones((N,))
    gt = dense_lce.dense_grads(e[rows], c, t[rows], None, d_out[rows], None, None, None, 0, torch.float64)
    ed, cd, td, vd = e.to(dev), c.to(dev), t.to(dev), valids.to(dev)
    lsed, dod = lse.float().to(dev), d_out.to(dev)
    de = torch.zeros((N, D), dtype=dtype, device=dev)
    dc = torch.zeros((V, D), dtype=dtype, device=dev)
    ws_bytes = lib.cce_backward_dense_workspace_bytes(B, V, D, 1, 0)
    ws = torch.empty((ws_bytes + 256,), dtype=torch.uint8, device=dev)
    st = lib.cce_backward_dense(
        ed.data_ptr(), cd.data_ptr(), None, lsed.data_ptr(), dod.data_ptr(), 0, None, vd.data_ptr(), td.data_ptr(),
        de.data_ptr(), dc.data_ptr(), None, (ws.data_ptr() + 255) // 256 * 256, ws_bytes,
        N, B, V, D, D, D, 1, 1.0, 0, 0, 0, 0, 0.0, 0, torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.cce_error_string(st)
    torch.cuda.synchronize()
    assert torch.isfinite(dc).all() and torch.isfinite(de[vd.long()]).all()
    assert torch.allclose(dc.cpu().double(), gt[1], atol=2e-2, rtol=2e-2)
    assert torch.allclose(de.cpu().double()[rows], gt[0], atol=2e-2, rtol=2e-2)


def test_backward_dz_rejects_layouts_it_cannot_stream():
    lib = _lib()
    dev = torch.device("cuda:0")
    e = torch.zeros((64, 72), dtype=torch.bfloat16, device=dev)  # D % 64 != 0
    c = torch.zeros((128, 72), dtype=torch.bfloat16, device=dev)
    lse = torch.zeros((64,), device=dev)
    t = torch.zeros((64,), dtype=torch.int64, device=dev)
    dz = torch.zeros((64, 128), dtype=torch.bfloat16, device=dev)
    st = lib.cce_backward_dz(e.data_ptr(), c.data_ptr(), None, lse.data_ptr(), lse.data_ptr(), 0, None, None,
                             t.data_ptr(), dz.data_ptr(), 128, 0, 64, 64, 128, 72, 72, 72, 1, 1.0, 0, 0, 0.0, 0,
                             torch.cuda.current_stream().cuda_stream)
    assert st == 10004  # CCE_ERR_MISALIGNED


def test_entry_points_reject_bad_arguments_before_launching():
    """Status codes of the C ABI for arguments it cannot run: nothing is launched, outputs stay untouched."""
    lib = _lib()
    dev = torch.device("cuda:0")
    N, V, D = 64, 128, 64
    e = torch.zeros((N, D), dtype=torch.bfloat16, device=dev)
    c = torch.zeros((V, D), dtype=torch.bfloat16, device=dev)
    lse = torch.full((N,), 3.0, device=dev)
    ws = torch.zeros((lib.cce_lse_forward_workspace_bytes(N, V, D) // 8 + 2,), dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    INVALID, DTYPE, WORKSPACE, MISALIGNED = 10001, 10002, 10003, 10004

    def fwd(e_ptr=e.data_ptr(), c_ptr=c.data_ptr(), lse_ptr=lse.data_ptr(), ws_ptr=ws.data_ptr(), ws_bytes=ws.numel() * 8,
            n=N, b=N, v=V, d=D, dtype=0):
        return lib.cce_lse_forward(e_ptr, c_ptr, None, None, lse_ptr, None, None, ws_ptr, ws_bytes, n, b, v, d,
                                   D, D, 1, 0.0, dtype, stream)

    assert fwd() == 0
    lse.fill_(3.0)
    assert fwd(b=-1) == INVALID and fwd(v=0) == INVALID and fwd(d=0) == INVALID
    assert fwd(b=N + 1) == INVALID  # more rows than e holds and no index vector
    assert fwd(e_ptr=None) == INVALID and fwd(c_ptr=None) == INVALID and fwd(lse_ptr=None) == INVALID
    assert fwd(dtype=7) == DTYPE
    assert fwd(ws_ptr=None) == WORKSPACE and fwd(ws_bytes=8) == WORKSPACE
    assert fwd(ws_ptr=ws.data_ptr() + 4) == MISALIGNED
    assert fwd(b=0) == 0  # nothing to do is not an error
    torch.cuda.synchronize()
    assert (lse == 3.0).all()

    t = torch.zeros((N,), dtype=torch.int64, device=dev)
    de = torch.zeros((N, D), dtype=torch.bfloat16, device=dev)
    bws = torch.zeros((lib.cce_backward_workspace_bytes(N, V, D) // 8 + 2,), dtype=torch.int64, device=dev)

    def bwd(lse_ptr=lse.data_ptr(), t_ptr=t.data_ptr(), v=V, shift=0, dtype=0, ws_bytes=bws.numel() * 8, dc_ptr=None):
        return lib.cce_backward(e.data_ptr(), c.data_ptr(), None, lse_ptr, lse.data_ptr(), 0, None, None, None, t_ptr,
                                None, de.data_ptr(), dc_ptr, None, bws.data_ptr(), ws_bytes, None,
                                N, N, v, D, D, D, 1, 1.0, 2.0**-12, 1, 1, 0, 0, shift, 0, 0.0, dtype, stream)

    assert bwd(lse_ptr=None) == INVALID and bwd(t_ptr=None) == INVALID and bwd(shift=-1) == INVALID
    assert bwd(v=2**31) == INVALID
    assert bwd(dtype=5) == DTYPE
    dc = torch.zeros((V, D), dtype=torch.bfloat16, device=dev)
    assert bwd(dc_ptr=dc.data_ptr(), ws_bytes=0) == WORKSPACE  # a filtered dC needs the survivor bits
    torch.cuda.synchronize()
    assert (de == 0).all() and (dc == 0).all()
    assert lib.cce_error_string(INVALID) and lib.cce_error_string(MISALIGNED) and lib.cce_error_string(DTYPE)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(256, 512, 128), (300, 500, 72), (1000, 130, 264), (33, 64, 8),
                                   (63, 40, 64), (65, 257, 520), (1, 7, 8), (130, 64, 1032)])
def test_backward_products_abi(dtype, shape):
    """cce_backward_products: d_e += dz . c and d_c (+)= dz^T . e[valids] with fp32 results, against the same
    products in fp64 of the same 16-bit inputs (exact up to fp32 accumulation: 1e-5 of the row scale).  Among
    the shapes: reductions shorter than one 64-step stage (no whole stage: the main loop only fetches zeros), one
    step longer than a stage (the partial stage goes first), five column tiles (two groups in the tile order)."""
    lib = _lib()
    dev = torch.device("cuda:0")
    B, M, D = shape
    g = torch.Generator().manual_seed(B + M + D)
    n_rows = B + 37
    ldz = (M + 63) // 64 * 64
    dz = torch.zeros((B, ldz), dtype=dtype)
    dz[:, :M] = (torch.randn((B, M), generator=g) * 0.1).to(dtype)
    c = torch.randn((M, D), generator=g).to(dtype)
    e = torch.randn((n_rows, D), generator=g).to(dtype)
    valids = torch.randperm(n_rows, generator=g)[:B].sort().values.to(torch.int32)
    de0 = torch.randn((B, D), generator=g)
    dc0 = torch.randn((M, D), generator=g)
    want_de = de0.double() + dz[:, :M].double() @ c.double()
    prod_dc = dz[:, :M].double().T @ e[valids.long()].double()
    code = 0 if dtype == torch.bfloat16 else 1
    dzd, cd, ed, vd = dz.to(dev), c.to(dev), e.to(dev), valids.to(dev)
    for accumulate in (0, 1):
        ded, dcd = de0.to(dev), dc0.to(dev)
        st = lib.cce_backward_products(dzd.data_ptr(), ldz, cd.data_ptr(), D, ed.data_ptr(), D, vd.data_ptr(),
                                       ded.data_ptr(), D, dcd.data_ptr(), D, accumulate, B, M, D, code,
                                       torch.cuda.current_stream().cuda_stream)
        assert st == 0, lib.cce_error_string(st)
        torch.cuda.synchronize()
        want_dc = prod_dc + (dc0.double() if accumulate else 0.0)
        for got, want in ((ded, want_de), (dcd, want_dc)):
            scale = want.abs().max().item()
            assert (got.cpu().double() - want).abs().max().item() <= 1e-5 * scale
    # one product alone, and the layout checks
    ded = de0.to(dev)
    st = lib.cce_backward_products(dzd.data_ptr(), ldz, cd.data_ptr(), D, None, 0, None, ded.data_ptr(), D, None, 0, 0,
                                   B, M, D, code, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    assert (ded.cpu().double() - want_de).abs().max().item() <= 1e-5 * want_de.abs().max().item()
    st = lib.cce_backward_products(dzd.data_ptr(), M if M % 64 else ldz - 8, cd.data_ptr(), D, None, 0, None,
                                   ded.data_ptr(), D, None, 0, 0, B, M, D, code, torch.cuda.current_stream().cuda_stream)
    assert st != 0  # dz rows shorter than the reduction rounded up to 64
