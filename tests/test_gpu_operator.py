"""Operator-level parity: cut_cross_entropy.linear_cross_entropy (HIP kernels) against the CPU
oracle, with the reference's own accuracy criterion and parameter grid
(reference tests/test_cce_loss_forward.py:44-108, tests/test_cce_loss_backward.py:79-227)."""

import pytest
import torch

from _util import IGNORE_INDEX, assert_no_worse, make_inputs

pytestmark = pytest.mark.gpu

SHAPES = [(256, 512, 128), (252, 507, 128), (252, 507, 123)]
TOL = {torch.float16: 1e-3, torch.bfloat16: 1e-2}


def _oracle_loss(e, c, targets, bias, softcap, shift, reduction, z_loss, compute_dtype, want_grads):
    """Loss (and gradients) of the dense oracle with leaves in ``compute_dtype``; the test
    objective mirrors the reference test: mean of the per-token loss (+ z-loss of the lse)."""
    from oracle import dense_lce

    el = e.detach().to(compute_dtype).requires_grad_(want_grads)
    cl = c.detach().to(compute_dtype).requires_grad_(want_grads)
    bl = bias.detach().to(compute_dtype).requires_grad_(want_grads) if bias is not None else None
    loss, lse = dense_lce.dense_linear_cross_entropy(
        el, cl, targets, bl, IGNORE_INDEX, softcap, reduction, shift, return_lse=z_loss
    )
    out = loss
    if want_grads:
        obj = loss
        if reduction == "sum":
            obj = obj / (targets[..., shift:] != IGNORE_INDEX).count_nonzero()
        obj = obj.mean()
        if z_loss:
            obj = obj + dense_lce.compute_z_loss(lse, targets, shift)
        obj.backward()
        return out.detach(), (el.grad, cl.grad, bl.grad if bl is not None else None)
    return out.detach(), None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [True, False])
@pytest.mark.parametrize("shift", [0, 2])
@pytest.mark.parametrize("invalids", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_loss_forward(dtype, softcap, has_bias, shift, invalids, shape):
    from cut_cross_entropy import linear_cross_entropy

    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=11, bias=has_bias, invalid_frac=0.2 if invalids else 0.0)
    e = e.view(4, -1, D)
    t = t.view(4, -1)
    gt, _ = _oracle_loss(e, c, t, bias, softcap, shift, "none", False, torch.float64, False)
    ref, _ = _oracle_loss(e, c, t, bias, softcap, shift, "none", False, dtype, False)

    dev = torch.device("cuda:0")
    got = linear_cross_entropy(
        e.to(dev), c.to(dev), t.to(dev), bias=bias.to(dev) if has_bias else None,
        softcap=softcap, shift=shift, reduction="none", impl="cce",
    )
    assert got.dtype == torch.float32
    assert got.shape == (4, N // 4 - shift)
    assert_no_worse(gt, ref, got, TOL[dtype], "loss")
    # bit-exact masking: ignored positions are exactly zero
    ign = t[..., shift:] == IGNORE_INDEX
    assert (got.cpu()[ign] == 0).all()


@pytest.mark.parametrize("impl", ["cce", "cce_exact", "cce_kahan_full_c", "cce_kahan_full_e", "cce_kahan"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("shift", [False, True])
@pytest.mark.parametrize("invalids", [False, True])
@pytest.mark.parametrize("reduction", ["none", "mean", "sum"])
@pytest.mark.parametrize("z_loss", [True, False])
@pytest.mark.parametrize("shape", [(256, 512, 128), (252, 507, 123)])
def test_loss_backward(impl, dtype, softcap, has_bias, shift, invalids, reduction, z_loss, shape):
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import compute_z_loss

    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, dtype, seed=12, bias=has_bias, invalid_frac=0.2 if invalids else 0.0)
    e = e.view(4, -1, D)
    t = t.view(4, -1)
    sh = int(shift)
    _, gt = _oracle_loss(e, c, t, bias, softcap, sh, reduction, z_loss, torch.float64, True)
    _, ref = _oracle_loss(e, c, t, bias, softcap, sh, reduction, z_loss, dtype, True)

    dev = torch.device("cuda:0")
    ed = e.to(dev).requires_grad_(True)
    cd = c.to(dev).requires_grad_(True)
    bd = bias.to(dev).requires_grad_(True) if has_bias else None
    td = t.to(dev)
    out = linear_cross_entropy(ed, cd, td, bias=bd, softcap=softcap, shift=shift, reduction=reduction,
                               impl=impl, return_lse=z_loss)
    loss, lse = out if z_loss else (out, None)
    if reduction == "sum":
        loss = loss / (td[..., sh:] != IGNORE_INDEX).count_nonzero()
    loss = loss.mean()
    if z_loss:
        loss = loss + compute_z_loss(lse, td, shift)
    loss.backward()

    assert ed.grad.dtype == dtype and cd.grad.dtype == dtype
    names = ["dE", "dC", "dBias"]
    got = [ed.grad, cd.grad, bd.grad if has_bias else None]
    for name, g_gt, g_ref, g in zip(names, gt, ref, got):
        if g is None:
            continue
        assert_no_worse(g_gt, g_ref, g, TOL[dtype], f"{impl} {name}")


@pytest.mark.parametrize(
    "compute_de,compute_dc,compute_dbias",
    [(True, False, True), (False, True, False), (False, False, True), (True, True, False)],
)
def test_loss_partials(compute_de, compute_dc, compute_dbias):
    """Only the inputs that require a gradient receive one (reference test_loss_partials)."""
    from cut_cross_entropy import linear_cross_entropy

    N, V, D = 256, 512, 128
    e, c, t, bias = make_inputs(N, V, D, torch.bfloat16, seed=13, bias=True)
    dev = torch.device("cuda:0")
    ed = e.view(4, -1, D).to(dev).requires_grad_(compute_de)
    cd = c.to(dev).requires_grad_(compute_dc)
    bd = bias.to(dev).requires_grad_(compute_dbias)
    loss = linear_cross_entropy(ed, cd, t.view(4, -1).to(dev), bias=bd, reduction="mean")
    loss.backward()
    assert (ed.grad is not None) == compute_de
    assert (cd.grad is not None) == compute_dc
    assert (bd.grad is not None) == compute_dbias


@pytest.mark.parametrize("impl", ["cce", "cce_exact", "cce_kahan_full_c"])
def test_all_ignored_batch(impl):
    """mean over zero valid tokens: NaN loss like F.cross_entropy, zero gradients, no exception (no kernel
    runs then, on either backward path, so the gradients must come zeroed from the host)."""
    from cut_cross_entropy import linear_cross_entropy

    dev = torch.device("cuda:0")
    poison = torch.full((1 << 20,), float("nan"), device=dev)  # what the next allocations are likely to reuse
    del poison
    e = torch.randn((2, 8, 64), device=dev, dtype=torch.bfloat16, requires_grad=True)
    c = torch.randn((96, 64), device=dev, dtype=torch.bfloat16, requires_grad=True)
    t = torch.full((2, 8), IGNORE_INDEX, device=dev)
    loss = linear_cross_entropy(e, c, t, impl=impl)
    assert torch.isnan(loss)
    loss.backward()
    assert (e.grad == 0).all() and (c.grad == 0).all()
    none = linear_cross_entropy(e, c, t, reduction="none", impl=impl)
    assert (none == 0).all() and none.shape == (2, 8)


def test_module_and_enum():
    from cut_cross_entropy import LinearCrossEntropy, LinearCrossEntropyImpl, linear_cross_entropy

    e, c, t, _ = make_inputs(128, 256, 64, torch.bfloat16, seed=14)
    dev = torch.device("cuda:0")
    e, c, t = e.to(dev), c.to(dev), t.to(dev)
    a = LinearCrossEntropy(softcap=10.0, impl=LinearCrossEntropyImpl.CCE_EXACT)(e, c, t)
    b = linear_cross_entropy(e, c, t, softcap=10.0, impl="cce_exact")
    assert torch.equal(a, b)
    d = linear_cross_entropy(e, c, t, softcap=10.0, impl="torch_compile")
    assert torch.allclose(a, d, rtol=1e-2, atol=1e-2)


def test_deterministic_forward():
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = make_inputs(512, 1024, 128, torch.bfloat16, seed=15)
    dev = torch.device("cuda:0")
    e, c, t = e.to(dev), c.to(dev), t.to(dev)
    a = linear_cross_entropy(e, c, t, reduction="none")
    b = linear_cross_entropy(e, c, t, reduction="none")
    assert torch.equal(a, b)


@pytest.mark.parametrize("impl", ["cce_exact", "cce_kahan_full_c_full_e"])
@pytest.mark.parametrize("with_valids", [False, True])
def test_unfiltered_backward_takes_the_dense_path(monkeypatch, impl, with_valids):
    """With the filter off the backward runs as dz chunks + dense products (and matches the oracle), also for a
    hidden size that is no multiple of the kernels' stage width: the operator pads e and c with zero columns."""
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    calls = []
    real = bw._dense_backward
    monkeypatch.setattr(bw, "_dense_backward", lambda *a, **k: (calls.append(1), real(*a, **k))[1])

    def run(D):
        e, c, t, _ = make_inputs(384, 1100, D, torch.bfloat16, seed=2, invalid_frac=0.25 if with_valids else 0.0)
        ed = e.cuda().requires_grad_(True)
        cd = c.cuda().requires_grad_(True)
        loss = linear_cross_entropy(ed, cd, t.cuda(), softcap=25.0, impl=impl, shift=1 if with_valids else 0)
        # the gradients are allocated without a fill where the kernels write them whole: give the allocator
        # blocks full of NaN to hand out
        for numel in (e.numel(), c.numel(), 384 * 128, 1100 * 128):
            torch.full((numel,), float("nan"), dtype=torch.bfloat16, device="cuda")
        loss.backward()
        e64 = e.double().requires_grad_(True)
        c64 = c.double().requires_grad_(True)
        want, _ = dense_lce.dense_linear_cross_entropy(e64, c64, t, softcap=25.0, shift=1 if with_valids else 0)
        want.backward()
        assert abs(loss.item() - want.item()) <= 1e-3 * abs(want.item())
        scale = 1.0 / 384
        assert torch.allclose(ed.grad.double().cpu(), e64.grad, atol=2e-2 * scale, rtol=2e-2)
        assert torch.allclose(cd.grad.double().cpu(), c64.grad, atol=2e-2 * scale, rtol=2e-2)

    run(128)
    assert len(calls) == 1
    run(72)
    assert len(calls) == 2


@pytest.mark.parametrize("with_valids", [False, True])
@pytest.mark.parametrize("reduction", ["mean", "none"])
def test_unfiltered_backward_walks_by_rows_where_rows_outnumber_classes(monkeypatch, with_valids, reduction):
    """A vocabulary shard in miniature: five times as many rows as classes.  The unfiltered backward then walks blocks
    of rows with the whole vocabulary each (dE complete per block, dC carried between the blocks as a 16-bit pair); a
    small dz budget makes it several blocks.  Rows indexed directly and through valids (shift, ignored labels), a
    scalar and a per-row upstream gradient."""
    from cut_cross_entropy import _hip
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    N, V, D = 1536, 300, 128
    lib = _hip.load()
    assert lib.cce_backward_dense_fixed_bytes(N, V, D, 1) == (V * D * 2 + 255) // 256 * 256  # by rows: the term of dC
    monkeypatch.setattr(bw, "DENSE_DZ_BYTES", 512 * 512 * 2)  # 512 rows x 512 (padded) classes: three blocks
    monkeypatch.setattr(bw, "DENSE_DZ_MIN_CLASSES", 0)
    e, c, t, _ = make_inputs(N, V, D, torch.bfloat16, seed=5, invalid_frac=0.1 if with_valids else 0.0)
    shift = 1 if with_valids else 0
    g = torch.Generator().manual_seed(3)
    w = torch.rand((N - shift,), generator=g) + 0.5  # reduction "none" returns one loss per row that has a target
    ed, cd = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    e64, c64 = e.double().requires_grad_(True), c.double().requires_grad_(True)
    for numel in (e.numel(), c.numel()):  # blocks full of NaN for the allocator to hand out
        torch.full((numel,), float("nan"), dtype=torch.bfloat16, device="cuda")
    loss = linear_cross_entropy(ed, cd, t.cuda(), softcap=25.0, impl="cce_exact", shift=shift, reduction=reduction)
    want, _ = dense_lce.dense_linear_cross_entropy(e64, c64, t, softcap=25.0, shift=shift, reduction=reduction)
    if reduction == "none":
        loss = (loss * w.cuda()).sum() / N
        want = (want * w.double()).sum() / N
    loss.backward()
    want.backward()
    assert abs(loss.item() - want.item()) <= 1e-3 * abs(want.item())
    scale = 1.0 / N
    assert torch.allclose(ed.grad.double().cpu(), e64.grad, atol=2e-2 * scale, rtol=2e-2)
    assert torch.allclose(cd.grad.double().cpu(), c64.grad, atol=2e-2 * scale, rtol=2e-2)
    # one block (the default budget) gives the same dC up to the rounding of the 16-bit pair
    monkeypatch.setattr(bw, "DENSE_DZ_BYTES", 256 << 20)
    ed2, cd2 = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    loss2 = linear_cross_entropy(ed2, cd2, t.cuda(), softcap=25.0, impl="cce_exact", shift=shift, reduction=reduction)
    if reduction == "none":
        loss2 = (loss2 * w.cuda()).sum() / N
    loss2.backward()
    assert torch.equal(ed2.grad, ed.grad)  # dE of a row does not depend on how the rows are cut into blocks
    assert torch.allclose(cd2.grad.float(), cd.grad.float(), atol=1e-2 * scale, rtol=1e-2)


def test_filtered_backward_runs_dense_when_most_cells_can_survive(monkeypatch):
    """Near-uniform soft-max over few classes: every cell's bound exp(max logit - min lse) is above
    filter_eps, so the backward runs unfiltered (and is then exact) -- from the FIRST step on: the first backward
    of a shape waits for the count of its own flagged cells, every later one uses the count of the backward
    before it, so the same inputs take the same path and give the same bits on every call.  With the switch off
    the ownership kernels run.  Peaked soft-max over many classes: the sparse kernels stay."""
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    calls = []
    real = bw._dense_backward
    monkeypatch.setattr(bw, "_dense_backward", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    bw.reset_backward_path_memory()

    e, c, t, _ = make_inputs(512, 2048, 128, torch.bfloat16, seed=4, planted=False, c_std=0.05)
    ed, cd = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    e64, c64 = e.double().requires_grad_(True), c.double().requires_grad_(True)
    dense_lce.dense_linear_cross_entropy(e64, c64, t)[0].backward()
    first = None
    for step in range(3):
        ed.grad = cd.grad = None
        linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
        torch.cuda.synchronize()
        assert len(calls) == step + 1  # dense from the first step on
        assert torch.allclose(ed.grad.double().cpu(), e64.grad, atol=2e-2 / 512, rtol=2e-2)
        assert torch.allclose(cd.grad.double().cpu(), c64.grad, atol=2e-2 / 512, rtol=2e-2)
        if first is None:
            first = (ed.grad.clone(), cd.grad.clone())
        assert torch.equal(ed.grad, first[0]) and torch.equal(cd.grad, first[1])  # call 1 == call n, bit for bit
    calls.clear()
    calls.append(1)

    monkeypatch.setattr(bw, "DENSE_WHEN_FLAGGED_ABOVE", None)
    ed.grad = cd.grad = None
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    assert len(calls) == 1
    monkeypatch.setattr(bw, "DENSE_WHEN_FLAGGED_ABOVE", 0.17)
    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    assert len(calls) == 1
    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "dense")
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    assert len(calls) == 2
    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "auto")
    # a workspace limit below what the unfiltered path needs here keeps the ownership kernels; above, it does not
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_OPERANDS", 0.0)
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", 64 * 1024)
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    torch.cuda.synchronize()
    assert len(calls) == 2
    # (1 MB would leave room for 896 of the 1024 classes a chunk must hold at least: the ownership kernels again)
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", 1 << 20)
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    torch.cuda.synchronize()
    assert len(calls) == 2
    # the limit is the larger of the byte figure and a multiple of what E and C occupy (here 640 KB): once leaves
    # 512 KB beside the compensation buffer, twice leaves room for the 1 MB of a 1024-class chunk
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", 64 * 1024)
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_OPERANDS", 1.0)
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    torch.cuda.synchronize()
    assert len(calls) == 2
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_OPERANDS", 2.0)
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    torch.cuda.synchronize()
    assert len(calls) == 3
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_OPERANDS", 0.0)
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", 2 << 20)
    ed.grad = cd.grad = None
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    torch.cuda.synchronize()
    assert len(calls) == 4
    # the path the filtered preset took by itself stays inside the limit (dz chunk + compensation buffer + the
    # forward's small vectors), whatever DENSE_DZ_BYTES would have allowed
    extra = torch.cuda.max_memory_allocated() - base - ed.grad.numel() * 2 - cd.grad.numel() * 2
    assert extra <= (2 << 20) + (256 << 10), extra
    monkeypatch.setattr(bw, "DENSE_WORKSPACE_LIMIT_BYTES", None)

    g = torch.Generator().manual_seed(1)
    c2 = (torch.randn((65536, 128), generator=g) * 0.5).to(torch.bfloat16)  # 512 cells per row group, <= 32 hold a target
    t2 = torch.randint(0, 65536, (512,), generator=g)
    e2 = (c2[t2].float() * 4).to(torch.bfloat16)  # each row points at its own class: a peaked soft-max
    ed2, cd2 = e2.cuda().requires_grad_(True), c2.cuda().requires_grad_(True)
    for _ in range(2):
        linear_cross_entropy(ed2, cd2, t2.cuda(), impl="cce").backward()
        torch.cuda.synchronize()
    assert len(calls) == 4


@pytest.mark.parametrize("impl", ["cce", "cce_exact"])
def test_backward_never_waits_for_the_device(impl):
    """No host synchronisation between the entry of backward() and its return (the reference's backward has
    none either, cce.py:166-235): torch's sync debug mode turns any .item() / .cpu() / nonzero into an error."""
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = make_inputs(512, 2048, 128, torch.bfloat16, seed=5, planted=False, c_std=0.05)
    ed, cd, td = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True), t.cuda()
    for _ in range(3):  # first step: new monitor, kernel attributes; later steps: the steady state
        ed.grad = cd.grad = None
        loss = linear_cross_entropy(ed, cd, td, softcap=20.0, impl=impl)
        torch.cuda.synchronize()
        torch.cuda.set_sync_debug_mode("error")
        try:
            loss.backward()
        finally:
            torch.cuda.set_sync_debug_mode("default")
        torch.cuda.synchronize()
    assert torch.isfinite(ed.grad).all() and torch.isfinite(cd.grad).all()


def test_a_width_that_is_no_multiple_of_128_costs_padded_copies_and_nothing_else(monkeypatch):
    """D = 200 runs the direct-to-LDS kernels on copies of e and c padded to 256 columns (one copy each in the
    forward, the padded dC and the slice back in the backward).  The copies are the whole price: the loss path's
    transient memory stays below the padded copies plus the padded gradient, and the results match an aligned run
    of the same numbers."""
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    N, V, D, Dp = 512, 8192, 200, 256
    e, c, t, _ = make_inputs(N, V, D, torch.bfloat16, seed=13, planted=True)
    ed, cd, td = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True), t.cuda()
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    linear_cross_entropy(ed, cd, td, softcap=20.0, impl="cce").backward()
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - base - (ed.grad.numel() + cd.grad.numel()) * 2
    padded = (N + V) * Dp * 2
    assert extra <= 2 * padded + (4 << 20), (extra, padded)  # padded e and c, padded dE and dC, small vectors
    ep = torch.nn.functional.pad(e, (0, Dp - D)).cuda().requires_grad_(True)
    cp = torch.nn.functional.pad(c, (0, Dp - D)).cuda().requires_grad_(True)
    linear_cross_entropy(ep, cp, td, softcap=20.0, impl="cce").backward()
    assert torch.equal(ed.grad, ep.grad[:, :D]) and torch.equal(cd.grad, cp.grad[:, :D])


@pytest.mark.parametrize("impl", ["cce_kahan_full_c", "cce_kahan_full_e"])
def test_one_sided_presets_split_between_the_two_backward_paths(monkeypatch, impl):
    """A preset that filters one gradient only runs the filtered side on the ownership kernels and the unfiltered
    side on the dense path (the reference decides per side inside one kernel, cce_backward.py:211-216): the
    unfiltered side is the exact gradient, the filtered side the filtered one."""
    from cut_cross_entropy import _hip
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    # peaked soft-max: filtering drops most of the plane, so the two sides differ visibly
    e, c, t, _ = make_inputs(512, 4096, 128, torch.bfloat16, seed=8, planted=True)
    ed, cd, td = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True), t.cuda()

    def grads(which):
        ed.grad = cd.grad = None
        timers = {}
        _hip.set_timers(timers)
        try:
            linear_cross_entropy(ed, cd, td, softcap=20.0, impl=which).backward()
        finally:
            _hip.set_timers(None)
        torch.cuda.synchronize()
        return ed.grad.clone(), cd.grad.clone(), sorted(k for k in timers if k.startswith("backward"))

    de_f, dc_f, ran_f = grads("cce")
    de_x, dc_x, ran_x = grads("cce_exact")
    de_m, dc_m, ran_m = grads(impl)
    assert ran_f == ["backward_sparse"] and ran_x == ["backward_dense"]
    assert ran_m == ["backward_dense", "backward_sparse"]
    assert not torch.equal(dc_f, dc_x) and not torch.equal(de_f, de_x)  # the case tells the sides apart
    if impl == "cce_kahan_full_c":  # dC unfiltered, dE filtered
        assert torch.equal(dc_m, dc_x) and torch.equal(de_m, de_f)
    else:
        assert torch.equal(de_m, de_x) and torch.equal(dc_m, dc_f)


def test_accumulate_flags_take_no_fp32_gradient_buffers():
    """accum_e_fp32 / accum_c_fp32 ask the reference for fp32 dE / dC buffers (cce_backward.py:390-394).  The kernels
    here accumulate in fp32 registers and write an element once, so a buffer in the input type holds the same bits
    after the final cast: the flags change neither the result nor the memory."""
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = make_inputs(1024, 16384, 256, torch.bfloat16, seed=9, planted=True)
    ed, cd, td = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True), t.cuda()
    out = {}
    for flags in (False, True):
        ed.grad = cd.grad = None
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        old = bw.FILTERED_BACKWARD_PATH
        bw.FILTERED_BACKWARD_PATH = "sparse"
        try:
            linear_cross_entropy(ed, cd, td, impl="cce", accum_e_fp32=flags, accum_c_fp32=flags).backward()
        finally:
            bw.FILTERED_BACKWARD_PATH = old
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - base
        out[flags] = (ed.grad.clone(), cd.grad.clone(), peak - ed.grad.numel() * 2 - cd.grad.numel() * 2)
    assert torch.equal(out[False][0], out[True][0]) and torch.equal(out[False][1], out[True][1])
    assert out[True][2] <= out[False][2] + (1 << 16)  # no fp32 copy of dC (33 MB here) anywhere


@pytest.mark.parametrize("impl,path", [("cce", "sparse"), ("cce", "dense"), ("cce", "auto"), ("cce_exact", "auto"),
                                       ("cce_kahan_full_c", "auto"), ("cce_kahan_full_e", "auto")])
def test_operator_backward_replays_in_a_hip_graph(monkeypatch, impl, path):
    """loss.backward() of the operator captured in a HIP graph (the forward runs eagerly on the capture stream:
    it reads the number of valid rows on the host, as the reference does) and replayed on new contents of e and
    c: every replay gives the gradients of an eager backward on the same contents."""
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", path)
    e0, c0, t0, _ = make_inputs(384, 3000, 128, torch.bfloat16, seed=6, planted=True)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        ed, cd, td = e0.cuda().requires_grad_(True), c0.cuda().requires_grad_(True), t0.cuda()

        def eager_grads():
            ed.grad = cd.grad = None
            linear_cross_entropy(ed, cd, td, softcap=20.0, impl=impl).backward()
            return ed.grad.clone(), cd.grad.clone()

        eager_grads()  # loads the library, sets kernel attributes outside the capture
        ed.grad = cd.grad = None
        loss = linear_cross_entropy(ed, cd, td, softcap=20.0, impl=impl)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        loss.backward(retain_graph=True)
    de_static, dc_static = ed.grad, cd.grad
    # The saved log-sum-exp belongs to the captured forward, so the replays keep e and c; what a replay must
    # reproduce is the whole backward, into buffers that were overwritten in between.
    with torch.cuda.stream(side):
        ed.grad = cd.grad = None
        linear_cross_entropy(ed, cd, td, softcap=20.0, impl=impl).backward()
        want_de, want_dc = ed.grad.clone(), cd.grad.clone()
    side.synchronize()
    for rep in range(3):
        de_static.fill_(7.0)
        dc_static.fill_(7.0)
        junk = torch.randn((1 << 22,), device="cuda")  # eager work and a synchronisation between the replays
        junk.sum().item()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(de_static, want_de) and torch.equal(dc_static, want_dc), rep


def test_rows_that_do_not_exist_read_as_zeros_in_the_ownership_kernels(monkeypatch):
    """An ignored row of e full of inf sitting in row 0, a number of valid rows and of classes that are not
    multiples of 32: the padding rows of the last row group and class group must read as zeros (a masked load
    in the reference), not as row 0, whose inf times a zero dz would poison the gradients of real rows."""
    from cut_cross_entropy import cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    N, V, D = 200, 1001, 128  # D % 128 == 0: the fast ownership kernels
    e, c, t, _ = make_inputs(N, V, D, torch.bfloat16, seed=7, planted=True)
    t[0] = IGNORE_INDEX
    e[0] = float("inf")
    ed, cd = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    linear_cross_entropy(ed, cd, t.cuda(), impl="cce").backward()
    torch.cuda.synchronize()
    assert torch.isfinite(cd.grad).all(), "dC poisoned by a row that is not part of the batch"
    assert torch.isfinite(ed.grad[1:]).all() and (ed.grad[0] == 0).all()
    e64 = e[1:].double().requires_grad_(True)
    c64 = c.double().requires_grad_(True)
    dense_lce.dense_linear_cross_entropy(e64, c64, t[1:])[0].backward()
    assert torch.allclose(cd.grad.double().cpu(), c64.grad, atol=5e-2 / 199, rtol=5e-2)
    assert torch.allclose(ed.grad[1:].double().cpu(), e64.grad, atol=5e-2 / 199, rtol=5e-2)


@pytest.fixture
def highest_matmul_precision():
    """The fp32 tolerances of the reference hold for exact fp32 products, whatever an earlier test selected."""
    before = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision("highest")
    yield
    torch.set_float32_matmul_precision(before)


@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("shift", [0, 1])
@pytest.mark.parametrize("shape", [(256, 512, 128), (252, 507, 123), (1024, 4096, 256)])
def test_fp32_inputs_match_fp64_oracle(highest_matmul_precision, softcap, has_bias, shift, shape):
    """fp32 inputs (three bf16 parts along a widened reduction axis, fp32 dz, fp32 GEMMs): the
    reference's tolerances for this dtype -- 1e-5 on the loss (tests/test_cce_loss_forward.py:47),
    5e-4 on the gradients (tests/test_cce_loss_backward.py:82) -- against the fp64 dense oracle, with the
    fp32 dense result as the yardstick of the reference's criterion."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    N, V, D = shape
    e, c, t, bias = make_inputs(N, V, D, torch.float32, seed=9, bias=has_bias, invalid_frac=0.2)
    if bias is not None:
        bias = bias * 10  # make the bias matter

    def dense(dtype):
        el = e.detach().clone().to(dtype).requires_grad_(True)
        cl = c.detach().clone().to(dtype).requires_grad_(True)
        bl = bias.detach().clone().to(dtype).requires_grad_(True) if bias is not None else None
        loss, _ = dense_lce.dense_linear_cross_entropy(el, cl, t, bias=bl, softcap=softcap, shift=shift,
                                                       reduction="none")
        (loss * w.to(dtype)[..., shift:]).sum().backward()
        return loss.detach(), el.grad, cl.grad, (bl.grad if bl is not None else None)

    g = torch.Generator().manual_seed(3)
    w = torch.randn((N,), generator=g)
    gt = dense(torch.float64)
    ref = dense(torch.float32)

    ed = e.cuda().requires_grad_(True)
    cd = c.cuda().requires_grad_(True)
    bd = bias.cuda().requires_grad_(True) if bias is not None else None
    loss = linear_cross_entropy(ed, cd, t.cuda(), bias=bd, softcap=softcap, shift=shift, reduction="none")
    assert loss.dtype == torch.float32 and ed.dtype == torch.float32
    (loss * w.cuda()[..., shift:]).sum().backward()
    assert_no_worse(gt[0], ref[0], loss.detach(), 1e-5, "loss")
    assert_no_worse(gt[1], ref[1], ed.grad, 5e-4, "dE")
    assert_no_worse(gt[2], ref[2], cd.grad, 5e-4, "dC")
    if bias is not None:
        assert_no_worse(gt[3], ref[3], bd.grad, 5e-4, "dBias")
    ignored = t == IGNORE_INDEX
    if shift:
        ignored = torch.cat([ignored[shift:], torch.ones(shift, dtype=torch.bool)])
    assert (ed.grad.cpu()[ignored] == 0).all()


@pytest.mark.parametrize("shape", [(1, 33, 8), (1, 40, 8), (2, 33, 8), (1, 63, 8), (1, 33, 16)])
@pytest.mark.parametrize("impl", ["cce", "cce_exact"])
def test_fp32_one_row_peaked_soft_max(highest_matmul_precision, shape, impl):
    """One or two rows, fewer than 64 classes, 8 columns, fp32, each row pointing at its own class: the loss
    -log p_target is close to zero (p_target ~ 0.99) while the log-sum-exp and the target logit it is the
    difference of are ~ 6, and the gradients carry the factor (1 - p_target).  In fp32 both therefore come with an
    ABSOLUTE error of a few ulp of the log-sum-exp (|lse| 2^-23), whatever the implementation: the reference forms
    nll = lse - logit in fp32 as well (cce.py:127-131).  A purely relative bound misreads that as an error (the
    bound of 2e-5 on the loss is missed by 6x at |loss| = 0.01 with an absolute error of 1e-6); the bound here is
    relative to the quantities the result is computed from."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    N, V, D = shape
    g = torch.Generator().manual_seed(104)
    c = torch.randn((V, D), generator=g) * (2.0 / D) ** 0.5
    t = torch.randint(0, V, (N,), generator=g)
    e = 3.0 * c[t] + 0.3 * torch.randn((N, D), generator=g)
    e64, c64 = e.double().requires_grad_(True), c.double().requires_grad_(True)
    want, want_lse = dense_lce.dense_linear_cross_entropy(e64, c64, t, return_lse=True)
    want.backward()
    ed, cd = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    loss, lse = linear_cross_entropy(ed, cd, t.cuda(), impl=impl, return_lse=True)
    loss.backward()
    ulp = 2.0**-23 * want_lse.abs().max().item()
    assert abs(loss.item() - want.item()) <= 1e-5 * abs(want.item()) + 4 * ulp
    assert torch.allclose(lse.cpu().double(), want_lse.detach(), rtol=1e-6, atol=4 * ulp)
    # d nll / d logit = p - onehot is known to 4 ulp of the log-sum-exp; the products scale it by |c| resp. |e|
    for got, ref, other in ((ed.grad, e64.grad, c), (cd.grad, c64.grad, e)):
        bound = 5e-4 * ref.abs().max().item() + 8 * ulp * other.abs().max().item() / N
        assert (got.cpu().double() - ref).abs().max().item() <= bound


def test_fp32_mean_and_lse_and_shard(highest_matmul_precision):
    from cut_cross_entropy import VocabParallelOptions, linear_cross_entropy
    from oracle import dense_lce

    e, c, t, _ = make_inputs(300, 1000, 64, torch.float32, seed=12)
    want, want_lse = dense_lce.dense_linear_cross_entropy(e.double(), c.double(), t, return_lse=True)
    got, got_lse = linear_cross_entropy(e.cuda(), c.cuda(), t.cuda(), return_lse=True)
    assert abs(got.item() - want.item()) <= 1e-5
    assert torch.allclose(got_lse.cpu().double(), want_lse, atol=1e-5, rtol=0)
    # a vocabulary shard: shard-local loss = lse over the shard - target logit (0 for foreign targets)
    s0, s1 = 200, 712
    one = linear_cross_entropy(e.cuda(), c[s0:s1].cuda(), t.cuda(), reduction="none",
                               vocab_parallel_options=VocabParallelOptions(s0, s1))
    logits = e.double() @ c[s0:s1].double().T
    inside = (t >= s0) & (t < s1)
    corr = torch.where(inside, logits.gather(1, (t - s0).clamp(0, s1 - s0 - 1).view(-1, 1)).squeeze(1),
                       torch.zeros(300, dtype=torch.float64))
    assert torch.allclose(one.cpu().double(), torch.logsumexp(logits, 1) - corr, atol=2e-5, rtol=0)


@pytest.mark.parametrize("softcap", [None, 20.0])
def test_fp32_inputs_under_fast_matmul_precision(softcap):
    """``torch.set_float32_matmul_precision("high")`` asks for fast fp32 products (the reference then uses tf32, 10
    mantissa bits): the logits are formed from three 16-bit terms instead of six and must still be far better than
    tf32 would be -- 1e-4 on the per-token loss, 2e-3 on the gradients against the fp64 oracle."""
    from cut_cross_entropy import fp32_path, linear_cross_entropy
    from oracle import dense_lce

    e, c, t, _ = make_inputs(512, 2000, 256, torch.float32, seed=14, invalid_frac=0.1)
    el = e.double().requires_grad_(True)
    cl = c.double().requires_grad_(True)
    want, _ = dense_lce.dense_linear_cross_entropy(el, cl, t, softcap=softcap, reduction="none")
    want.sum().backward()
    before = torch.get_float32_matmul_precision()
    try:
        torch.set_float32_matmul_precision("highest")
        assert fp32_path.n_terms() == 6
        torch.set_float32_matmul_precision("high")
        assert fp32_path.n_terms() == 3
        ed = e.cuda().requires_grad_(True)
        cd = c.cuda().requires_grad_(True)
        got = linear_cross_entropy(ed, cd, t.cuda(), softcap=softcap, reduction="none")
        got.sum().backward()
    finally:
        torch.set_float32_matmul_precision(before)
    assert torch.allclose(got.detach().cpu().double(), want.detach(), atol=1e-4, rtol=0)
    assert torch.allclose(ed.grad.cpu().double(), el.grad, atol=2e-3, rtol=2e-3)
    assert torch.allclose(cd.grad.cpu().double(), cl.grad, atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("ignore_index", [0, 7, 10**6])
def test_custom_ignore_index(ignore_index):
    """An ignore value that is itself a class index (or far outside the vocabulary): those rows drop out of loss
    and gradients, every other row is unaffected (reference: the ignore_index argument, cce.py:286-290)."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    e, c, t, _ = make_inputs(300, 500, 64, torch.bfloat16, seed=15)
    t[::5] = ignore_index
    el, cl = e.double().requires_grad_(True), c.double().requires_grad_(True)
    want, _ = dense_lce.dense_linear_cross_entropy(el, cl, t, ignore_index=ignore_index)
    want.backward()
    ed, cd = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    got = linear_cross_entropy(ed, cd, t.cuda(), ignore_index=ignore_index, impl="cce_exact")
    got.backward()
    assert abs(got.item() - want.item()) <= 1e-3 * abs(want.item())
    assert (ed.grad.cpu()[t == ignore_index] == 0).all()
    assert torch.allclose(ed.grad.cpu().double(), el.grad, atol=1e-2 / 240, rtol=2e-2)
    assert torch.allclose(cd.grad.cpu().double(), cl.grad, atol=1e-2 / 240, rtol=2e-2)


@pytest.mark.parametrize("low", [torch.bfloat16, torch.float16])
def test_autocast_region(low):
    """fp32 parameters inside ``torch.autocast``: the kernels run in the autocast dtype, the loss is fp32 and the
    gradients come back in the dtype of the leaves (reference: custom_fwd / custom_bwd and the manual cast,
    cce.py:50,71-76,165)."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    e, c, t, _ = make_inputs(256, 700, 128, torch.float32, seed=16)
    ed, cd = e.cuda().requires_grad_(True), c.cuda().requires_grad_(True)
    with torch.autocast(device_type="cuda", dtype=low):
        loss = linear_cross_entropy(ed, cd, t.cuda(), impl="cce_exact")
    loss.backward()
    assert loss.dtype == torch.float32 and ed.grad.dtype == torch.float32 and cd.grad.dtype == torch.float32
    el, cl = e.to(low).double().requires_grad_(True), c.to(low).double().requires_grad_(True)
    want, _ = dense_lce.dense_linear_cross_entropy(el, cl, t)
    want.backward()
    tol = 1e-2 if low == torch.bfloat16 else 2e-3
    assert abs(loss.item() - want.item()) <= 1e-3 * abs(want.item())
    assert torch.allclose(ed.grad.cpu().double(), el.grad, atol=tol / 256, rtol=2 * tol)
    assert torch.allclose(cd.grad.cpu().double(), cl.grad, atol=tol / 256, rtol=2 * tol)


def test_int32_targets_and_strided_embeddings():
    """Targets as int32 and embeddings that are a strided view of a wider activation tensor, batch shape
    [2, 3, T]: same loss as with int64 targets and a packed copy, gradients arrive in the view's base."""
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = make_inputs(6 * 40, 300, 64, torch.bfloat16, seed=17, invalid_frac=0.1)
    base = torch.zeros((2, 3, 40, 96), dtype=torch.bfloat16, device="cuda")
    base[..., :64] = e.view(2, 3, 40, 64).cuda()
    base.requires_grad_(True)
    view = base[..., :64]
    assert not view.is_contiguous()
    cd = c.cuda().requires_grad_(True)
    t3 = t.view(2, 3, 40).cuda()
    got = linear_cross_entropy(view, cd, t3.to(torch.int32), reduction="none", shift=1, impl="cce_exact")
    assert got.shape == (2, 3, 39)
    got.sum().backward()
    g_view, g_c = base.grad[..., :64].clone(), cd.grad.clone()
    assert (base.grad[..., 64:] == 0).all()

    packed = view.detach().contiguous().requires_grad_(True)
    cd.grad = None
    want = linear_cross_entropy(packed, cd, t3, reduction="none", shift=1, impl="cce_exact")
    want.sum().backward()
    assert torch.equal(got, want) and torch.equal(g_view, packed.grad) and torch.equal(g_c, cd.grad)


def test_inside_a_compiled_function():
    """Called from a function under ``torch.compile`` the operator is a graph break (it launches through ctypes
    and reads the number of valid rows on the host), not a tracing error; values and gradients equal eager."""
    from cut_cross_entropy import linear_cross_entropy

    e, c, t, _ = make_inputs(128, 300, 64, torch.bfloat16, seed=18, invalid_frac=0.1)
    td = t.cuda()

    def fn(x, w):
        return linear_cross_entropy(x * 2.0, w, td, softcap=10.0, impl="cce_exact") * 0.5

    outs = []
    for f in (fn, torch.compile(fn, backend="aot_eager")):
        x = e.cuda().requires_grad_(True)
        w = c.cuda().requires_grad_(True)
        loss = f(x, w)
        loss.backward()
        outs.append((loss.detach(), x.grad, w.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
