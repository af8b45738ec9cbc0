"""Parity at the benchmark configurations (scaled where the dense oracle would not fit in seconds,
full size for the headline shape), plus the properties that only show at scale: gradient
filtering with the no-recompute shortcut, determinism, class permutation, vocabulary shards."""

import pytest
import torch

from _util import IGNORE_INDEX

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _gen(N, D, V, seed=0, e_std=1.0, c_std=0.02, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    e = (torch.randn((N, D), generator=g) * e_std).to(dtype)
    c = (torch.randn((V, D), generator=g) * c_std).to(dtype)
    t = torch.randint(0, V, (N,), generator=g)
    return e, c, t, g


def _oracle_on_gpu(e, c, t, valids, d_out, d_lse, softcap, shift=0, bias=None, filter_eps=None):
    """Dense fp32 oracle evaluated with torch on the GPU, row-chunked: LSE and gradients.

    With ``filter_eps`` the gradient filter is restated exactly as specified: the plane of
    (valid row, class) is cut into 32 x 32 sub-tiles and a sub-tile whose every |p - onehot| is
    below ``filter_eps`` contributes nothing (reference rule, cce_backward.py:211-216, at this
    build's tile size).  The inputs of these tests keep |p - onehot| far from the threshold, so
    the kept set does not depend on rounding."""
    from oracle import dense_lce

    N, D = e.shape
    V = c.shape[0]
    rows = torch.arange(N, device=e.device) if valids is None else valids.long()
    lse = torch.cat([dense_lce.dense_lse(e[r], c, bias, softcap, torch.float32) for r in rows.split(2048)])
    if filter_eps is None:
        de, dc, db = dense_lce.dense_grads(e, c, t, valids, d_out, d_lse, bias, softcap, shift, torch.float32, chunk=1024)
        return lse, de, dc, db
    assert bias is None and d_lse is None
    cc = c.float()
    de = torch.zeros((N, D), dtype=torch.float32, device=e.device)
    dc = torch.zeros((V, D), dtype=torch.float32, device=e.device)
    Vp = (V + 31) // 32 * 32
    for s0 in range(0, rows.numel(), 1024):
        r = rows[s0 : s0 + 1024]
        ee = e[r].float()
        z = ee @ cc.T
        sl = dense_lce.softcapping(z, softcap) if softcap is not None else z
        p = torch.exp(sl - lse[s0 : s0 + 1024, None])
        tt = t[r + shift]
        y = torch.zeros_like(p)
        y.scatter_(1, tt.view(-1, 1), 1.0)
        f = (p - y).abs()
        n = r.numel()
        npad = (n + 31) // 32 * 32
        fp = torch.zeros((npad, Vp), device=e.device)
        fp[:n, :V] = f
        keep = fp.view(npad // 32, 32, Vp // 32, 32).amax(dim=(1, 3)) >= filter_eps
        keep = keep[:, None, :, None].expand(-1, 32, -1, 32).reshape(npad, Vp)[:n, :V]
        g = d_out[r + shift].view(-1, 1) if d_out.numel() > 1 else d_out.reshape(())
        dz = (p - y) * g
        if softcap is not None:
            dz = dz * (1 - (sl / softcap) ** 2)
        dz = dz * keep
        de.index_add_(0, r, dz @ cc)
        dc += dz.T @ ee
    return lse, de, dc, None


def _rel_err(got, want):
    scale = want.abs().max().item()
    return (got.float() - want.float()).abs().max().item() / max(scale, 1e-30)


def _reference_gradients(e, c, t, valids, d_out, d_lse, softcap, shift=0, filter_eps=None, margin=1e-2, lse=None):
    """What the per-element criterion needs, evaluated with torch on the GPU in row chunks:

    gt    dE, dC of the dense fp32 oracle (with the filter rule of 32 x 32 sub-tiles when ``filter_eps``)
    ref   the same algorithm in the 16-bit input type: logits from a 16-bit matmul, soft-max in fp32, dz rounded
          to 16 bits, 16-bit products (the "naive low-precision implementation" the reference's tests hold
          results against, tests/test_cce_loss_backward.py:12-76)
    amb   for every element, the sum of |dz| |operand| over the sub-tiles whose largest |p - onehot| lies within
          ``margin`` of filter_eps: rounding may put such a sub-tile on either side of the threshold, and this is
          exactly how far an element can move when it does (zero for elements no such sub-tile touches)
    """
    from oracle import dense_lce

    N, D = e.shape
    V = c.shape[0]
    dev = e.device
    rows = torch.arange(N, device=dev) if valids is None else valids.long()
    if lse is None:  # (a vocabulary shard passes the log-sum-exp of the whole vocabulary)
        lse = torch.cat([dense_lce.dense_lse(e[r], c, None, softcap, torch.float32) for r in rows.split(2048)])
    cc = c.float()
    out = {k: torch.zeros((N, D), dtype=torch.float32, device=dev) for k in ("de_gt", "de_ref", "de_amb")}
    out.update({k: torch.zeros((V, D), dtype=torch.float32, device=dev) for k in ("dc_gt", "dc_ref", "dc_amb")})
    out["lse"] = lse
    Vp = (V + 31) // 32 * 32
    step = 1024
    for s0 in range(0, rows.numel(), step):
        r = rows[s0 : s0 + step]
        n = r.numel()
        ee = e[r].float()
        tt = t[r + shift]
        g = d_out[r + shift].view(-1, 1) if d_out.numel() > 1 else d_out.reshape(1, 1)
        h = d_lse[r + shift].view(-1, 1) if d_lse is not None else None

        def dz_of(z):
            sl = dense_lce.softcapping(z, softcap) if softcap is not None else z
            p = torch.exp(sl - lse[s0 : s0 + n, None])
            y = torch.zeros_like(p)
            inside = (tt >= 0) & (tt < V)  # a target outside the classes of c matches none of them
            y.scatter_(1, tt.clamp(0, V - 1).view(-1, 1), inside.view(-1, 1).to(p.dtype))
            dz = p * (g + h) - y * g if h is not None else (p - y) * g
            if softcap is not None:
                dz = dz * (1 - (sl / softcap) ** 2)
            return dz, (p - y).abs_()

        dz, f = dz_of(ee @ cc.T)
        dz_lo, _ = dz_of((e[r] @ c.T).float())
        if filter_eps is not None:
            npad = (n + 31) // 32 * 32
            fp = torch.zeros((npad, Vp), device=dev)
            fp[:n, :V] = f
            cell = fp.view(npad // 32, 32, Vp // 32, 32).amax(dim=(1, 3))
            expand = lambda m: m[:, None, :, None].expand(-1, 32, -1, 32).reshape(npad, Vp)[:n, :V]
            keep = expand(cell >= filter_eps)
            amb = expand((cell >= filter_eps * (1 - margin)) & (cell < filter_eps * (1 + margin)))
            dz_amb = dz.abs() * amb
            dz = dz * keep
            dz_lo = dz_lo * keep
            out["de_amb"].index_add_(0, r, dz_amb @ cc.abs())
            out["dc_amb"] += dz_amb.T @ ee.abs()
            del fp, cell, keep, amb, dz_amb
        out["de_gt"].index_add_(0, r, dz @ cc)
        out["dc_gt"] += dz.T @ ee
        dz_lo = dz_lo.to(e.dtype)
        out["de_ref"].index_add_(0, r, (dz_lo @ c).float())
        out["dc_ref"] += (dz_lo.T @ e[r]).float()
        del dz, dz_lo, f
    return out


def _assert_per_element(got, gt, ref, amb, what, rel=1e-2, sigmas=6.0):
    """The reference's criterion per element, |gt - got| <= |gt - ref| + tol (tests/test_cce_loss_forward.py:103-108),
    with ``rel`` |gt| for the 1e-2 relative bound of 16-bit gradients and a ``tol`` that follows the scale of each
    row: ``sigmas`` times the root-mean-square distance between the fp32 and the 16-bit dense result in that
    row (a fixed absolute tolerance would be vacuous for the rows of dC that hold no target, whose entries are
    orders of magnitude below those of the rows that do).  ``amb`` is added where a sub-tile next to the filter
    threshold can go either way."""
    got = got.float()
    noise = (gt - ref).abs()
    tol = sigmas * noise.square().mean(dim=1, keepdim=True).sqrt()
    excess = (got - gt).abs() - noise - rel * gt.abs() - tol - 1.05 * amb
    worst = excess.max()
    if worst.item() > 0:
        i = int(excess.argmax())
        r, col = divmod(i, got.shape[1])
        raise AssertionError(
            f"{what}[{r},{col}]: got {got[r, col].item():.6e}, gt {gt[r, col].item():.6e}, 16-bit {ref[r, col].item():.6e}, "
            f"row tol {tol[r, 0].item():.3e}, ambiguity {amb[r, col].item():.3e}; "
            f"{int((excess > 0).sum())} of {excess.numel()} elements out of bounds")
    assert torch.isfinite(got).all(), f"{what}: non-finite values"


def _check_gradients(ed_grad, cd_grad, refs, what=""):
    D = refs["de_gt"].shape[1]
    _assert_per_element(ed_grad.reshape(-1, D), refs["de_gt"], refs["de_ref"], refs["de_amb"], what + "dE")
    _assert_per_element(cd_grad, refs["dc_gt"], refs["dc_ref"], refs["dc_amb"], what + "dC")


def test_per_element_criterion_has_teeth():
    """The criterion the full-size tests use must fail where a maximum norm would not: a dC whose rows without a
    target (orders of magnitude below the rows with one) are off by 30 %, a dE with one element off by 30 %, a sub-tile dropped that the filter rule keeps."""
    N, D, V = 512, 256, 4096
    e, c, t, _ = _gen(N, D, V, seed=11)
    e, c, t = e.to(DEV), c.to(DEV), t.to(DEV) % 64  # every target in the first 64 classes
    d_out = torch.full((N,), 1.0 / N, device=DEV)
    refs = _reference_gradients(e, c, t, None, d_out, None, None, filter_eps=None)
    _check_gradients(refs["de_gt"].to(torch.bfloat16), refs["dc_gt"].to(torch.bfloat16), refs)  # rounding passes
    bad_dc = refs["dc_gt"].clone()
    bad_dc[64:] *= 1.3
    assert _rel_err(bad_dc, refs["dc_gt"]) <= 1e-2  # the maximum norm does not see it
    with pytest.raises(AssertionError):
        _check_gradients(refs["de_gt"], bad_dc, refs)
    bad_de = refs["de_gt"].clone()
    bad_de[17, int(bad_de[17].abs().argmax())] *= 1.3  # one element of one row
    with pytest.raises(AssertionError):
        _check_gradients(bad_de, refs["dc_gt"], refs)
    # (a threshold every probability of a class that is no target stays far below: no sub-tile is ambiguous)
    filtered = _reference_gradients(e, c, t, None, d_out, None, None, filter_eps=2.0**-8)
    assert filtered["dc_amb"].max().item() == 0 and (filtered["dc_gt"][64:] == 0).all()
    with pytest.raises(AssertionError):  # an unfiltered dC against the filter rule: the dropped sub-tiles show
        _check_gradients(filtered["de_gt"], refs["dc_gt"], filtered)


def test_config1_small_reference_run(monkeypatch):
    """N=4096, D=1024, V=32000, 5 % ignored, mean, seed 0.  Loss against the fp32 oracle on the CPU; gradients per
    element against the dense oracle on the GPU: with the filter rule applied for the ownership kernels, exact
    for the unfiltered path the default impl="cce" switches to at this soft-max (near-uniform: most cells can
    hold a probability above eps) and for impl="cce_exact"."""
    import cut_cross_entropy.cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import _build_flat_valids
    from oracle import dense_lce

    N, D, V = 4096, 1024, 32000
    e, c, t, g = _gen(N, D, V, seed=0)
    t[torch.randperm(N, generator=g)[: int(0.05 * N)]] = IGNORE_INDEX
    want, _ = dense_lce.dense_linear_cross_entropy(e.float(), c.float(), t)

    ed = e.to(DEV).requires_grad_(True)
    cd = c.to(DEV).requires_grad_(True)
    td = t.to(DEV)
    valids = _build_flat_valids(td, IGNORE_INDEX, 0)
    d_out = torch.full((N,), 1.0 / valids.numel(), device=DEV)
    ign = t == IGNORE_INDEX
    for impl, path, eps in (("cce", "sparse", 2.0**-12), ("cce", "dense", None), ("cce_exact", "auto", None)):
        monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", path)
        ed.grad = cd.grad = None
        loss = linear_cross_entropy(ed, cd, td, impl=impl)
        loss.backward()
        assert abs(loss.item() - want.item()) <= 1e-3 * abs(want.item())
        refs = _reference_gradients(e.to(DEV), c.to(DEV), td.clamp_min(0), valids, d_out, None, None, filter_eps=eps)
        _check_gradients(ed.grad, cd.grad, refs, f"{impl}/{path} ")
        assert (ed.grad.cpu()[ign] == 0).all()  # bit-exact masking


def test_config2_full_size_forward_and_backward(monkeypatch):
    """The headline shape at full size against the dense fp32 oracle run with torch on the GPU:
    loss / LSE within 1e-3 relative, dE / dC per element by the reference's criterion with gradient
    filtering on, loss-path memory under 16 MB, and most of the plane skipped unseen."""
    import cut_cross_entropy.cce_backward as bw
    from cut_cross_entropy import cce as cce_mod
    from cut_cross_entropy import linear_cross_entropy

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    N, D, V, softcap = 8192, 2304, 256000, 30.0
    g = torch.Generator(device=DEV).manual_seed(0)
    e = torch.randn((N, D), generator=g, device=DEV).to(torch.bfloat16)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g, device=DEV)
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)

    counters = torch.zeros(4, dtype=torch.int64, device=DEV)
    cce_mod.set_tile_counters(counters)
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    loss, lse = linear_cross_entropy(ed, cd, t, softcap=softcap, impl="cce", return_lse=True)
    loss.backward()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    cce_mod.set_tile_counters(None)
    extra_mb = (peak - ed.grad.numel() * 2 - cd.grad.numel() * 2) / 2**20
    assert extra_mb <= 16.0, extra_mb

    d_out = torch.full((N,), 1.0 / N, device=DEV)
    refs = _reference_gradients(e, c, t, None, d_out, None, softcap, filter_eps=2.0**-12)
    want_lse = refs["lse"]
    assert torch.allclose(lse, want_lse, rtol=1e-3, atol=1e-3)
    from oracle import dense_lce

    want_loss = (want_lse + dense_lce.dense_indexed_neg_dot(e, c, t, None, softcap, torch.float32)).mean()
    assert abs(loss.item() - want_loss.item()) <= 1e-3 * abs(want_loss.item())
    _check_gradients(ed.grad, cd.grad, refs)  # every element of dE and dC, incl. the rows of dC without a target
    total, recomputed, with_de, with_dc = counters.tolist()
    assert total == (N // 32) * (V // 32)
    assert recomputed / total < 0.05 and with_de / total < 0.02 and with_dc == with_de


def test_config2_full_size_one_sided_presets_and_kahan(monkeypatch):
    """The presets that filter one gradient only (cce_kahan_full_c: dC exact, dE filtered; cce_kahan_full_e: the
    other way round) and cce_kahan (both filtered, fp32 accumulation asked for) at the headline shape, every element
    of dE and dC against the dense fp32 oracle with the filter rule on the filtered output only.  cce_kahan must
    also keep the 16 MB of the filtered path: no fp32 copy of dC is taken for the accumulation flags."""
    import cut_cross_entropy.cce_backward as bw
    from cut_cross_entropy import _hip
    from cut_cross_entropy import linear_cross_entropy

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    N, D, V, softcap = 8192, 2304, 256000, 30.0
    g = torch.Generator(device=DEV).manual_seed(0)
    e = torch.randn((N, D), generator=g, device=DEV).to(torch.bfloat16)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g, device=DEV)
    d_out = torch.full((N,), 1.0 / N, device=DEV)
    refs = {True: _reference_gradients(e, c, t, None, d_out, None, softcap, filter_eps=2.0**-12),
            False: _reference_gradients(e, c, t, None, d_out, None, softcap, filter_eps=None)}
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    for impl, e_filtered, c_filtered, want_paths in (
            ("cce_kahan_full_c", True, False, ["backward_dense", "backward_sparse"]),
            ("cce_kahan_full_e", False, True, ["backward_dense", "backward_sparse"]),
            ("cce_kahan", True, True, ["backward_sparse"])):
        print("impl", impl, flush=True)
        ed.grad = cd.grad = None
        timers = {}
        _hip.set_timers(timers)
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        loss = linear_cross_entropy(ed, cd, t, softcap=softcap, impl=impl)
        loss.backward()
        torch.cuda.synchronize()
        _hip.set_timers(None)
        extra_mb = (torch.cuda.max_memory_allocated() - base - ed.grad.numel() * 2 - cd.grad.numel() * 2) / 2**20
        assert sorted(k for k in timers if k.startswith("backward")) == want_paths
        if impl == "cce_kahan":
            assert extra_mb <= 16.0, extra_mb
        re_, rc_ = refs[e_filtered], refs[c_filtered]
        _assert_per_element(ed.grad, re_["de_gt"], re_["de_ref"], re_["de_amb"], impl + " dE")
        _assert_per_element(cd.grad, rc_["dc_gt"], rc_["dc_ref"], rc_["dc_amb"], impl + " dC")


@pytest.mark.parametrize("filter_eps", ["auto", None])
def test_config2_scaled_filter_vs_exact(filter_eps):
    """Near-uniform soft-max: with filtering only the target sub-tiles survive, and the result stays
    within the filter's error bound of the unfiltered one."""
    from cut_cross_entropy import cce as cce_mod
    from cut_cross_entropy import linear_cross_entropy

    N, D, V = 1024, 2304, 32000
    e, c, t, _ = _gen(N, D, V, seed=3, c_std=0.01)  # logit std 0.48: every non-target p is well below eps
    e, c, t = e.to(DEV), c.to(DEV), t.to(DEV)
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    counters = torch.zeros(4, dtype=torch.int64, device=DEV)
    cce_mod.set_tile_counters(counters)
    loss = linear_cross_entropy(ed, cd, t, softcap=30.0, impl="cce", filter_eps=filter_eps, reduction="sum")
    loss.backward()
    torch.cuda.synchronize()
    cce_mod.set_tile_counters(None)
    d_out = torch.ones((N,), device=DEV)
    _, de, dc, _ = _oracle_on_gpu(e, c, t, None, d_out, None, 30.0,
                                  filter_eps=None if filter_eps is None else 2.0**-12)
    assert _rel_err(ed.grad, de) <= 1e-2
    assert _rel_err(cd.grad, dc) <= 1e-2
    total, recomputed, with_de, with_dc = counters.tolist()
    if filter_eps is None:
        assert recomputed == total == with_de == with_dc
    else:
        # a sub-tile survives iff it holds a target (every other |p| is far below eps here)
        want = len({(i // 32, int(tt) // 32) for i, tt in enumerate(t.tolist())})
        # (plus the few sub-tiles where an extreme logit lifts one p above eps)
        assert want <= with_de <= 1.25 * want and with_dc == with_de
        assert recomputed < 0.2 * total


def test_config3_scaled_shift_and_trailing_ignored():
    """Llama-shaped call pattern: [batch, T] with shift=1 and the tail of every row ignored."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    Bt, T, D, V = 4, 512, 1024, 16384
    e, c, t, _ = _gen(Bt * T, D, V, seed=4)
    t = t.view(Bt, T).clone()
    t[:, -32:] = IGNORE_INDEX
    e3 = e.view(Bt, T, D)
    eo = e3.float().requires_grad_(True)
    co = c.float().requires_grad_(True)
    want, _ = dense_lce.dense_linear_cross_entropy(eo, co, t, shift=1)
    want.backward()
    ed = e3.to(DEV).requires_grad_(True)
    cd = c.to(DEV).requires_grad_(True)
    loss = linear_cross_entropy(ed, cd, t.to(DEV), shift=1, impl="cce")
    loss.backward()
    assert abs(loss.item() - want.item()) <= 1e-3 * abs(want.item())
    assert _rel_err(ed.grad.cpu(), eo.grad) <= 1e-2
    assert _rel_err(cd.grad.cpu(), co.grad) <= 1e-2
    # rows whose shifted target is ignored (and the last row of every sequence) get exactly zero
    dead = torch.ones(Bt, T, dtype=torch.bool)
    dead[:, : T - 1] = t[:, 1:] == IGNORE_INDEX
    assert (ed.grad.cpu()[dead] == 0).all()


def test_config4_scaled_kahan_full_zloss_none():
    """Zipf labels, impl=cce_kahan_full_c_full_e (no filtering, fp32 accumulation), z-loss with
    weight 1e-4, reduction none: per-token loss and gradients."""
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import compute_z_loss
    from oracle import dense_lce

    N, D, V, w = 1024, 2048, 16000, 1e-4
    e, c, _, g = _gen(N, D, V, seed=5)
    ranks = torch.arange(1, V + 1, dtype=torch.float64)
    cdf = torch.cumsum(ranks.pow(-1.1), 0)
    cdf /= cdf[-1].clone()
    t = torch.searchsorted(cdf, torch.rand(N, generator=g, dtype=torch.float64)).clamp_max(V - 1)
    eo = e.float().requires_grad_(True)
    co = c.float().requires_grad_(True)
    want, want_lse = dense_lce.dense_linear_cross_entropy(eo, co, t, reduction="none", return_lse=True)
    (want.mean() + w * dense_lce.compute_z_loss(want_lse, t)).backward()
    ed = e.to(DEV).requires_grad_(True)
    cd = c.to(DEV).requires_grad_(True)
    td = t.to(DEV)
    loss, lse = linear_cross_entropy(ed, cd, td, impl="cce_kahan_full_c_full_e", reduction="none", return_lse=True)
    (loss.mean() + w * compute_z_loss(lse, td)).backward()
    assert torch.allclose(loss.cpu(), want.detach(), rtol=1e-3, atol=1e-3)
    assert torch.allclose(lse.cpu(), want_lse.detach(), rtol=1e-3, atol=1e-3)
    assert _rel_err(ed.grad.cpu(), eo.grad) <= 1e-2
    assert _rel_err(cd.grad.cpu(), co.grad) <= 1e-2


def test_config5_scaled_peaked_and_sequential_shards():
    """Rows aligned with their class vector, then the vocabulary cut into 8 shards that are run one
    after another on the one GPU and combined on the host (no collective): LSE, loss, dE and dC
    of the shards recombine to the full-vocabulary result."""
    from cut_cross_entropy import VocabParallelOptions, linear_cross_entropy
    from cut_cross_entropy.vocab_parallel import combine_shards, partition_n_into_range, shard_backward, shard_forward

    N, D, V = 2048, 1024, 19008
    g = torch.Generator().manual_seed(6)
    c = (torch.randn((V, D), generator=g) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g)
    e = (4.0 * c[t].float() + 0.5 * torch.randn((N, D), generator=g)).to(torch.bfloat16)
    e, c, t = e.to(DEV), c.to(DEV), t.to(DEV)

    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    full, full_lse = linear_cross_entropy(ed, cd, t, impl="cce_exact", reduction="none", return_lse=True)
    full.sum().backward()

    corr, lses, bounds = [], [], []
    for rank in range(8):
        s, s_end = partition_n_into_range(V, rank, 8)
        bounds.append((s, s_end))
        cl, ll = shard_forward(e, c[s:s_end], t, VocabParallelOptions(s, s_end))
        corr.append(cl)
        lses.append(ll)
    nll, lse = combine_shards(corr, lses)
    assert torch.allclose(lse, full_lse, rtol=1e-4, atol=1e-4)
    assert torch.allclose(nll, full.detach(), rtol=1e-3, atol=1e-3)
    # rows whose label another shard holds contribute an exact zero
    s0, e0 = bounds[0]
    outside = (t < s0) | (t >= e0)
    assert (corr[0][outside] == 0).all()

    d_out = torch.ones((N,), device=DEV)
    de_sum = torch.zeros((N, D), dtype=torch.float32, device=DEV)
    for (s, s_end) in bounds:
        de, dc, _ = shard_backward(e, c[s:s_end], t, VocabParallelOptions(s, s_end), lse, d_out)
        de_sum += de
        assert _rel_err(dc, cd.grad[s:s_end]) <= 1e-2
    assert _rel_err(de_sum, ed.grad) <= 1e-2

    # the operator itself with shard bounds: shard-local loss = lse_shard - correct_logit
    one = linear_cross_entropy(e, c[s0:e0], t, impl="cce_exact", reduction="none",
                               vocab_parallel_options=VocabParallelOptions(s0, e0))
    assert torch.allclose(one, lses[0] - corr[0], rtol=1e-5, atol=1e-5)


def test_backward_is_deterministic_and_order_invariant():
    """Two runs give bit-identical gradients, and a class permutation (reference vocab_ordering)
    changes nothing but the summation order inside a row group."""
    from cut_cross_entropy.cce_backward import cce_backward_kernel
    from cut_cross_entropy.cce_lse_forward import cce_lse_forward_kernel
    from cut_cross_entropy.utils import TensorInfo

    N, D, V = 512, 256, 4000
    e, c, t, g = _gen(N, D, V, seed=7, c_std=0.05)
    e, c, t = e.to(DEV), c.to(DEV), t.to(DEV)
    lse = cce_lse_forward_kernel(e, c)
    info = TensorInfo(torch.float32, True)
    do = torch.randn((N,), generator=g).to(DEV)

    def run(order):
        return cce_backward_kernel(do, None, e, info, c, info, None, None, lse, None, None, None, targets=t,
                                   vocab_ordering=order, accum_e_fp32=True, accum_c_fp32=True)

    de1, dc1, _ = run(None)
    de2, dc2, _ = run(None)
    assert torch.equal(de1, de2) and torch.equal(dc1, dc2)
    perm = torch.randperm(V, generator=g).to(torch.int32).to(DEV)
    de3, dc3, _ = run(perm)
    assert torch.allclose(de1, de3, rtol=1e-4, atol=1e-5)
    assert torch.allclose(dc1, dc3, rtol=1e-4, atol=1e-5)


def test_dlse_only_gradient():
    """The loss output unused, only the z-loss of the LSE: the gradient arrives through d_lse alone."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    N, D, V = 256, 128, 1000
    e, c, t, _ = _gen(N, D, V, seed=8, c_std=0.1)
    eo = e.float().requires_grad_(True)
    co = c.float().requires_grad_(True)
    _, lse_o = dense_lce.dense_linear_cross_entropy(eo, co, t, return_lse=True)
    lse_o.pow(2).mean().backward()
    ed = e.to(DEV).requires_grad_(True)
    cd = c.to(DEV).requires_grad_(True)
    _, lse = linear_cross_entropy(ed, cd, t.to(DEV), impl="cce_exact", return_lse=True)
    lse.pow(2).mean().backward()
    assert _rel_err(ed.grad.cpu(), eo.grad) <= 1e-2
    assert _rel_err(cd.grad.cpu(), co.grad) <= 1e-2


def test_strided_classifier_and_lse_kernel_logit_avg():
    """A classifier that is a column slice of a wider matrix (row stride != D), and the optional
    column average of the launcher API."""
    from cut_cross_entropy.cce_lse_forward import cce_lse_forward_kernel
    from oracle import dense_lce

    N, D, V = 300, 128, 1000
    e, c_wide, _, _ = _gen(N, D + 64, V, seed=9, c_std=0.1)
    e = e[:, :D].contiguous().to(DEV)
    c = c_wide.to(DEV)[:, :D]
    assert not c.is_contiguous()
    lse, la = cce_lse_forward_kernel(e, c, softcap=20.0, return_logit_avg=True)
    logits = dense_lce._dense_logits(e.cpu(), c.cpu(), None, 20.0, torch.float64)
    assert torch.allclose(lse.cpu().double(), torch.logsumexp(logits, -1), rtol=1e-4, atol=1e-4)
    assert torch.allclose(la.cpu().double(), logits.mean(0), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("impl", ["cce", "cce_exact"])
def test_classifier_beyond_two_to_the_31_elements(impl):
    """A classifier of 2.2e9 elements (4.4 GB of bf16): row offsets into C and dC pass 2^31 both in bytes and in
    elements.  Half of the labels sit in the classes above element offset 2^31, the inputs are peaked on
    their labels so that the sparse kernels run under impl="cce".  Checked against dense fp32 torch."""
    from cut_cross_entropy import linear_cross_entropy

    N, D, V = 512, 8192, 270336
    first_high = (2**31) // D
    assert first_high < V - 1024
    g = torch.Generator(device=DEV).manual_seed(11)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g, device=DEV)
    t[::2] = torch.randint(first_high, V, (N // 2,), generator=g, device=DEV)
    e = (2.0 * c[t].float() + 0.5 * torch.randn((N, D), generator=g, device=DEV)).to(torch.bfloat16)
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    loss, lse = linear_cross_entropy(ed, cd, t, impl=impl, return_lse=True)
    loss.backward()

    d_out = torch.full((N,), 1.0 / N, device=DEV)
    want_lse, de, dc, _ = _oracle_on_gpu(e, c, t, None, d_out, None, None,
                                         filter_eps=2.0**-12 if impl == "cce" else None)
    from oracle import dense_lce

    assert torch.allclose(lse, want_lse, rtol=1e-3, atol=1e-3)
    want_loss = (want_lse + dense_lce.dense_indexed_neg_dot(e, c, t, None, None, torch.float32)).mean()
    assert abs(loss.item() - want_loss.item()) <= 1e-3 * abs(want_loss.item())
    assert _rel_err(ed.grad, de) <= 1e-2
    assert _rel_err(cd.grad[first_high:], dc[first_high:]) <= 1e-2
    assert _rel_err(cd.grad, dc) <= 1e-2


@pytest.mark.parametrize("layout", ["row_gaps", "transposed"])
@pytest.mark.parametrize("impl", ["cce", "cce_exact"])
def test_backward_with_a_classifier_that_is_a_view(layout, impl):
    """c as a column slice of a wider matrix (gaps between rows) and as the transpose of a [D, V] matrix
    (unit stride along the classes): loss and gradients against the dense oracle, gradient in c's shape."""
    from cut_cross_entropy import linear_cross_entropy
    from oracle import dense_lce

    N, D, V = 384, 128, 1500
    e, c, t, _ = _gen(N, D, V, seed=12, c_std=0.1)
    eo = e.float().requires_grad_(True)
    co = c.float().requires_grad_(True)
    want, _ = dense_lce.dense_linear_cross_entropy(eo, co, t, softcap=15.0)
    want.backward()

    ed = e.to(DEV).requires_grad_(True)
    if layout == "row_gaps":
        base = torch.zeros((V, D + 64), dtype=c.dtype, device=DEV)
        base[:, :D] = c.to(DEV)
        base.requires_grad_(True)
        cd = base[:, :D]
    else:
        base = c.to(DEV).t().contiguous().requires_grad_(True)  # [D, V]
        cd = base.t()
    assert not cd.is_contiguous()
    loss = linear_cross_entropy(ed, cd, t.to(DEV), softcap=15.0, impl=impl, filter_eps=None if impl == "cce_exact" else 0.0)
    loss.backward()
    assert abs(loss.item() - want.item()) <= 1e-3 * abs(want.item())
    got_dc = base.grad[:, :D] if layout == "row_gaps" else base.grad.t()
    assert _rel_err(ed.grad.cpu(), eo.grad) <= 1e-2
    assert _rel_err(got_dc.cpu(), co.grad) <= 1e-2
    if layout == "row_gaps":
        assert (base.grad[:, D:] == 0).all()


@pytest.mark.parametrize("style", ["flat", "mixed", "peaked"])
@pytest.mark.parametrize("shape", [(1000, 384, 5000), (256, 2304, 4096), (1024, 128, 8224), (333, 256, 12345),
                                   (2048, 512, 1000), (96, 1152, 2048)])
def test_ownership_kernels_at_many_shapes(monkeypatch, shape, style):
    """The filtered backward pinned to the ownership kernels (no switch to the dense path) on ragged and
    aligned shapes, 5 % of the rows ignored, for a near-uniform soft-max (only target sub-tiles survive), one
    where many probabilities sit around eps, and a peaked one: against the dense oracle with the filter rule
    applied.  A sub-tile whose largest |p - onehot| is within rounding of eps may fall on either side; its
    entries are then below eps, far inside the tolerance."""
    import cut_cross_entropy.cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import _build_flat_valids

    monkeypatch.setattr(bw, "DENSE_WHEN_FLAGGED_ABOVE", None)
    N, D, V = shape
    g = torch.Generator().manual_seed(N + D + V)
    t = torch.randint(0, V, (N,), generator=g)
    if style == "flat":
        e = torch.randn((N, D), generator=g)
        c = torch.randn((V, D), generator=g) * (0.5 / D**0.5)
    elif style == "mixed":
        e = torch.randn((N, D), generator=g)
        c = torch.randn((V, D), generator=g) * (2.0 / D**0.5)
    else:
        c = torch.randn((V, D), generator=g) * (2.0 / D) ** 0.5
        e = 4.0 * c[t] + 0.3 * torch.randn((N, D), generator=g)
    t[torch.randperm(N, generator=g)[: N // 20]] = IGNORE_INDEX
    e, c, t = e.to(torch.bfloat16).to(DEV), c.to(torch.bfloat16).to(DEV), t.to(DEV)
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    linear_cross_entropy(ed, cd, t, impl="cce", reduction="sum").backward()
    valids = _build_flat_valids(t, IGNORE_INDEX, 0)
    _, de, dc, _ = _oracle_on_gpu(e, c, t.clamp_min(0), valids, torch.ones((N,), device=DEV), None, None,
                                  filter_eps=2.0**-12)
    assert _rel_err(ed.grad, de) <= 1e-2
    assert _rel_err(cd.grad, dc) <= 1e-2
    assert (ed.grad[t == IGNORE_INDEX] == 0).all()


def test_config5_full_size_filtered(monkeypatch):
    """E [65536, 3584] peaked on its labels, C [152064, 3584], full vocabulary, gradient filter on: the largest
    configuration at its real size against the dense oracle with the filter rule, evaluated with torch on the
    GPU in row chunks; and the fraction of the plane the backward had to look at."""
    import cut_cross_entropy.cce_backward as bw
    from cut_cross_entropy import cce as cce_mod
    from cut_cross_entropy import linear_cross_entropy

    monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", "sparse")
    N, D, V = 65536, 3584, 152064
    g = torch.Generator(device=DEV).manual_seed(5)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g, device=DEV)
    e = (4.0 * c[t].float() + 0.5 * torch.randn((N, D), generator=g, device=DEV)).to(torch.bfloat16)
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    counters = torch.zeros(4, dtype=torch.int64, device=DEV)
    cce_mod.set_tile_counters(counters)
    loss, lse = linear_cross_entropy(ed, cd, t, impl="cce", return_lse=True)
    loss.backward()
    torch.cuda.synchronize()
    cce_mod.set_tile_counters(None)

    d_out = torch.full((N,), 1.0 / N, device=DEV)
    refs = _reference_gradients(e, c, t, None, d_out, None, None, filter_eps=2.0**-12)
    assert torch.allclose(lse, refs["lse"], rtol=1e-3, atol=1e-3)
    _check_gradients(ed.grad, cd.grad, refs)
    total, recomputed, with_de, with_dc = counters.tolist()
    assert total == (N // 32) * (V // 32)
    assert recomputed / total < 0.02 and with_dc == with_de


def test_config5_shard_leg_at_full_size():
    """The single-GPU vocabulary shard of configuration 5 at its real size: E [65536, 3584] peaked on labels drawn
    over all 152064 classes, the shard C[0:19008] with VocabParallelOptions(0, 19008).  Shard log-sum-exp and
    correct-logit partials against the oracle's vp_shard_partials evaluated with torch on the GPU; shard dC and
    the dE partial, gradient filter on, per element against the dense oracle with the filter rule, given the
    log-sum-exp of the whole vocabulary (computed by the oracle, not by the kernels under test)."""
    from cut_cross_entropy import VocabParallelOptions
    from cut_cross_entropy.vocab_parallel import shard_backward, shard_forward
    from oracle import dense_lce

    N, D, V, start, stop = 65536, 3584, 152064, 0, 19008
    g = torch.Generator(device=DEV).manual_seed(5)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g, device=DEV)
    e = (4.0 * c[t].float() + 0.5 * torch.randn((N, D), generator=g, device=DEV)).to(torch.bfloat16)
    c_shard = c[start:stop]
    opts = VocabParallelOptions(start, stop)
    assert (stop - start) % 256 != 0  # a ragged last tile

    correct, lse_shard = shard_forward(e, c_shard, t, opts)
    want_correct, want_lse = [], []
    for r in torch.arange(N, device=DEV).split(4096):
        cl, ll = dense_lce.vp_shard_partials(e[r], c_shard, t[r], start, stop)
        want_correct.append(cl)
        want_lse.append(ll)
    want_correct, want_lse = torch.cat(want_correct), torch.cat(want_lse)
    assert torch.allclose(lse_shard, want_lse, rtol=1e-3, atol=1e-3)
    assert torch.allclose(correct, want_correct, rtol=1e-3, atol=1e-3)
    outside = (t < start) | (t >= stop)
    assert 0.8 < outside.float().mean().item() < 0.95 and (correct[outside] == 0).all()  # bit-exact zeros

    global_lse = torch.cat([dense_lce.dense_lse(e[r], c, None, None, torch.float32)
                            for r in torch.arange(N, device=DEV).split(2048)])
    d_out = torch.full((N,), 1.0 / N, device=DEV)
    de, dc, _ = shard_backward(e, c_shard, t, opts, global_lse, d_out, filter_eps=2.0**-12, accum_fp32=False)
    refs = _reference_gradients(e, c_shard, t - start, None, d_out, None, None, filter_eps=2.0**-12, lse=global_lse)
    _check_gradients(de, dc, refs, "shard ")
    # rows whose target another shard holds still get their soft-max part of the gradient, and it is small
    assert de[outside].abs().max() < de[~outside].abs().max()


def test_config3_full_size_shift_and_trailing_ignored(monkeypatch):
    """E [4, 4096, 4096], C [128256, 4096], labels with the last 256 of every sequence ignored, shift=1, mean,
    impl="cce", at full size against the dense oracle evaluated with torch on the GPU."""
    import cut_cross_entropy.cce_backward as bw
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import _build_flat_valids
    from oracle import dense_lce

    Bt, T, D, V = 4, 4096, 4096, 128256
    g = torch.Generator(device=DEV).manual_seed(3)
    e = torch.randn((Bt, T, D), generator=g, device=DEV).to(torch.bfloat16)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (Bt, T), generator=g, device=DEV)
    t[:, -256:] = IGNORE_INDEX
    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    valids = _build_flat_valids(t, IGNORE_INDEX, 1)
    assert valids.numel() == Bt * (T - 256 - 1)  # 15356: the last position of a sequence has no next token
    flat_t = t.flatten().clamp_min(0)
    d_out = torch.full((Bt * T,), 1.0 / valids.numel(), device=DEV)
    dead = torch.ones((Bt, T), dtype=torch.bool, device=DEV)
    dead[:, : T - 1] = t[:, 1:] == IGNORE_INDEX
    # 87 % of the cells can hold a probability above eps here, so the operator settles on the unfiltered path;
    # both paths are held to the per-element criterion, each against the oracle with its own rule
    for path, eps in (("dense", None), ("sparse", 2.0**-12)):
        monkeypatch.setattr(bw, "FILTERED_BACKWARD_PATH", path)
        ed.grad = cd.grad = None
        loss, lse = linear_cross_entropy(ed, cd, t, shift=1, impl="cce", return_lse=True)
        loss.backward()
        refs = _reference_gradients(e.view(-1, D), c, flat_t, valids, d_out, None, None, shift=1, filter_eps=eps)
        want_lse = refs["lse"]
        assert lse.shape == (Bt, T - 1)
        full_lse = torch.zeros((Bt * T,), device=DEV)
        full_lse[valids.long() + 1] = want_lse  # batch-shaped, zeros at ignored positions, first position cut off
        assert torch.allclose(lse, full_lse.view(Bt, T)[:, 1:], rtol=1e-3, atol=1e-3)
        nd = dense_lce.dense_indexed_neg_dot(e.view(-1, D)[valids.long()], c, flat_t[valids.long() + 1], None, None,
                                             torch.float32)
        want_loss = (want_lse + nd).mean()
        assert abs(loss.item() - want_loss.item()) <= 1e-3 * abs(want_loss.item())
        _check_gradients(ed.grad, cd.grad, refs, path + " ")
        assert (ed.grad[dead] == 0).all()
        del refs


def test_config4_full_size_kahan_full_zloss_none():
    """E [8192, 2048], C [256000, 2048], Zipf(1.1) labels, impl="cce_kahan_full_c_full_e", reduction none with
    the z-loss of the returned log-sum-exp (weight 1e-4): per-token loss, log-sum-exp and gradients at full size
    against the dense oracle evaluated with torch on the GPU."""
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import compute_z_loss
    from oracle import dense_lce

    N, D, V, w = 8192, 2048, 256000, 1e-4
    g = torch.Generator(device=DEV).manual_seed(4)
    e = torch.randn((N, D), generator=g, device=DEV).to(torch.bfloat16)
    c = (torch.randn((V, D), generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    ranks = torch.arange(1, V + 1, dtype=torch.float64, device=DEV)
    cdf = torch.cumsum(ranks.pow(-1.1), 0)
    cdf /= cdf[-1].clone()
    t = torch.searchsorted(cdf, torch.rand(N, generator=g, dtype=torch.float64, device=DEV)).clamp_max(V - 1)
    assert (t < 100).float().mean() > 0.3  # heavy head: many rows share a class group

    ed = e.clone().requires_grad_(True)
    cd = c.clone().requires_grad_(True)
    loss, lse = linear_cross_entropy(ed, cd, t, impl="cce_kahan_full_c_full_e", reduction="none", return_lse=True)
    (loss.mean() + w * compute_z_loss(lse, t)).backward()

    # d/d nll_i = 1 / N; d/d lse_i = w * 2 lse_i / N
    d_out = torch.full((N,), 1.0 / N, device=DEV)
    want_lse = torch.cat([dense_lce.dense_lse(e[r], c, None, None, torch.float32)
                          for r in torch.arange(N, device=DEV).split(2048)])
    d_lse = w * 2.0 * want_lse / N
    refs = _reference_gradients(e, c, t, None, d_out, d_lse, None)
    want = want_lse + dense_lce.dense_indexed_neg_dot(e, c, t, None, None, torch.float32)
    assert torch.allclose(lse, want_lse, rtol=1e-3, atol=1e-3)
    assert torch.allclose(loss, want, rtol=1e-3, atol=1e-3)
    _check_gradients(ed.grad, cd.grad, refs)
