"""Pins of the CPU oracle (oracle/dense_lce.py): every function is checked against a known
answer of the reference's own tests, a library routine, brute force, or a mathematical identity
chosen so that a dropped term, a wrong sign or a wrong index fails."""

import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

from _util import IGNORE_INDEX, autograd_grads, make_inputs
from oracle import dense_lce


# ---- known-answer test of the reference (tests/test_compute_z_loss.py:8-44) -------------------
@pytest.mark.parametrize("reduction", ["none", "mean", "sum"])
@pytest.mark.parametrize("shift", [False, True])
@pytest.mark.parametrize("invalids", [False, True])
@pytest.mark.parametrize("impl", ["oracle", "package"])
def test_compute_z_loss_known_answer(reduction, invalids, shift, impl):
    if impl == "oracle":
        fn = dense_lce.compute_z_loss
    else:
        from cut_cross_entropy.utils import compute_z_loss as fn
    lse = torch.arange(1, 11, dtype=torch.float64)
    targets = None
    if invalids:
        targets = torch.full((lse.size(0) + int(shift),), IGNORE_INDEX, dtype=torch.int64)
        targets[3] = 1
        targets[5] = 1
    z = fn(lse, shift=shift, targets=targets, reduction=reduction)
    assert z.shape == (lse.shape if reduction == "none" else torch.Size([]))
    if reduction == "mean":
        z = z * (lse.numel() if targets is None else 2)
    want = sum(i**2 for i in range(1, 11)) if targets is None else (4 - int(shift)) ** 2 + (6 - int(shift)) ** 2
    assert torch.isclose(z.sum(), torch.as_tensor(want, dtype=torch.float64))


# ---- exact invariant test of the reference (tests/test_vocab_parallel.py:153-165) -------------
@pytest.mark.parametrize("n", [1023, 2048, 5, 152064])
@pytest.mark.parametrize("world_size", [7, 8, 1])
@pytest.mark.parametrize("impl", ["oracle", "package"])
def test_partition_n_into_range(n, world_size, impl):
    if impl == "oracle":
        fn = dense_lce.partition_n_into_range
    else:
        from cut_cross_entropy.vocab_parallel.utils import partition_n_into_range as fn
    start = 0
    for rank in range(world_size):
        end = start + n // world_size + (1 if rank < (n % world_size) else 0)
        assert fn(n, rank, world_size) == (start, end)
        start = end
    assert end == n


# ---- valids / shift / ignore_index indexing: brute force, bit-exact -----------------------------
def _brute_valids(targets, ignore, shift):
    T = targets.shape[-1]
    flat = targets.reshape(-1, T)
    out = []
    for b in range(flat.shape[0]):
        for t in range(T - shift):
            if flat[b, t + shift] != ignore:
                out.append(b * T + t)
    return out


@pytest.mark.parametrize("shape", [(7,), (3, 9), (2, 3, 5)])
@pytest.mark.parametrize("shift", [0, 1, 2])
@pytest.mark.parametrize("frac", [0.0, 0.3, 1.0])
@pytest.mark.parametrize("impl", ["oracle", "package"])
def test_build_flat_valids_brute_force(shape, shift, frac, impl):
    if impl == "oracle":
        fn = dense_lce.build_flat_valids
    else:
        from cut_cross_entropy.utils import _build_flat_valids as fn
    if shift >= shape[-1]:
        pytest.skip("shift must be below T")
    g = torch.Generator().manual_seed(5)
    t = torch.randint(0, 50, shape, generator=g)
    t[torch.rand(shape, generator=g) < frac] = IGNORE_INDEX
    got = fn(t, IGNORE_INDEX, shift)
    want = _brute_valids(t.numpy(), IGNORE_INDEX, shift)
    if shift == 0 and len(want) == t.numel():
        assert got is None
        return
    assert got.dtype == torch.int32
    assert got.tolist() == want
    # invariants: strictly increasing, and every selected row has a real target at + shift
    assert all(a < b for a, b in zip(want, want[1:]))
    flat = t.reshape(-1)
    assert all(flat[i + shift] != IGNORE_INDEX for i in want)


@pytest.mark.parametrize("impl", ["oracle", "package"])
def test_handle_reduction_none_scatter(impl):
    if impl == "oracle":
        fn = dense_lce.handle_reduction_none
    else:
        from cut_cross_entropy.utils import handle_reduction_none as fn
    valids = torch.tensor([0, 2, 5, 9], dtype=torch.int32)
    loss = torch.tensor([1.0, 2.0, 3.0, 4.0])
    out = fn(torch.Size((3, 4)), valids, 1, loss)
    want = torch.zeros(12)
    for v, l in zip([0, 2, 5, 9], [1.0, 2.0, 3.0, 4.0]):
        want[v + 1] = l
    assert torch.equal(out, want.view(3, 4))
    assert torch.equal(fn(torch.Size((2, 2)), None, 0, loss), loss.view(2, 2))


def test_handle_eps():
    assert dense_lce.handle_eps("auto", torch.bfloat16) == 2.0**-12
    assert dense_lce.handle_eps("auto", torch.float16) == 2.0**-15
    assert dense_lce.handle_eps(None, torch.float16) is None
    assert dense_lce.handle_eps(0.5, torch.float16) == 0.5
    with pytest.raises(RuntimeError):
        dense_lce.handle_eps(1, torch.float16)


# ---- soft-capping and LSE against library routines ------------------------------------------------
def test_softcapping_is_tanh_and_large_cap_is_identity():
    x = torch.linspace(-40, 40, 101, dtype=torch.float64)
    assert np.allclose(dense_lce.softcapping(x, 20.0).numpy(), 20.0 * np.tanh(x.numpy() / 20.0))
    assert torch.allclose(dense_lce.softcapping(x, 1e9), x, atol=1e-6)


@pytest.mark.parametrize("softcap", [None, 20.0])
@pytest.mark.parametrize("has_bias", [False, True])
def test_dense_lse_vs_scipy(softcap, has_bias):
    e, c, _, bias = make_inputs(33, 71, 19, torch.float64, seed=1, bias=has_bias)
    logits = e.numpy() @ c.numpy().T
    if has_bias:
        logits = logits + bias.numpy()
    if softcap is not None:
        logits = softcap * np.tanh(logits / softcap)
    want = scipy.special.logsumexp(logits, axis=-1)
    got = dense_lce.dense_lse(e, c, bias, softcap, torch.float64)
    assert np.allclose(got.numpy(), want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("softcap", [None, 5.0])
def test_dense_indexed_neg_dot_loops(softcap):
    e, c, t, bias = make_inputs(11, 17, 7, torch.float64, seed=2, bias=True)
    got = dense_lce.dense_indexed_neg_dot(e, c, t, bias, softcap, torch.float64)
    for i in range(11):
        dot = sum(float(e[i, d]) * float(c[t[i], d]) for d in range(7))
        v = -dot - float(bias[t[i]])
        if softcap is not None:
            v = softcap * np.tanh(v / softcap)
        assert abs(float(got[i]) - v) < 1e-12


# ---- the loss against F.cross_entropy on the gathered rows -----------------------------------------
@pytest.mark.parametrize("reduction", ["none", "mean", "sum"])
@pytest.mark.parametrize("shift", [0, 1, 3])
@pytest.mark.parametrize("softcap", [None, 10.0])
@pytest.mark.parametrize("invalid_frac", [0.0, 0.25])
def test_dense_loss_vs_f_cross_entropy(reduction, shift, softcap, invalid_frac):
    N, V, D, T = 48, 37, 13, 12
    e, c, t, bias = make_inputs(N, V, D, torch.float64, seed=3, bias=True, invalid_frac=invalid_frac)
    e3, t2 = e.view(N // T, T, D), t.view(N // T, T)
    loss, lse = dense_lce.dense_linear_cross_entropy(e3, c, t2, bias, IGNORE_INDEX, softcap, reduction, shift,
                                                     return_lse=True)
    # textbook formulation: slice, flatten, dense logits, library cross entropy
    es = e3[:, : T - shift].reshape(-1, D) if shift else e3.reshape(-1, D)
    ts = t2[:, shift:].reshape(-1)
    logits = es @ c.T + bias
    if softcap is not None:
        logits = softcap * torch.tanh(logits / softcap)
    want = F.cross_entropy(logits, ts, ignore_index=IGNORE_INDEX, reduction=reduction)
    if reduction == "none":
        want = want.view(N // T, T - shift)
        assert loss.shape == want.shape
    assert torch.allclose(loss, want, rtol=1e-12, atol=1e-12)
    want_lse = torch.logsumexp(logits, -1).view(N // T, T - shift)
    want_lse = torch.where(t2[:, shift:] == IGNORE_INDEX, torch.zeros_like(want_lse), want_lse)
    assert torch.allclose(lse, want_lse, rtol=1e-12, atol=1e-12)


# ---- closed-form gradients: autograd and finite differences -----------------------------------------
@pytest.mark.parametrize("softcap", [None, 4.0])
@pytest.mark.parametrize("with_dlse", [False, True])
@pytest.mark.parametrize("shift", [0, 2])
def test_dense_grads_vs_autograd_and_finite_differences(softcap, with_dlse, shift):
    N, V, D, T = 24, 19, 6, 8
    e, c, t, bias = make_inputs(N, V, D, torch.float64, seed=4, bias=True, invalid_frac=0.2)
    valids = dense_lce.build_flat_valids(t.view(N // T, T), IGNORE_INDEX, shift)
    if valids is None:
        valids = torch.arange(N, dtype=torch.int32)
    g = torch.Generator().manual_seed(9)
    d_out = torch.randn(N, generator=g, dtype=torch.float64)
    d_lse = torch.randn(N, generator=g, dtype=torch.float64) if with_dlse else None
    got = dense_lce.dense_grads(e, c, t, valids, d_out, d_lse, bias, softcap, shift, torch.float64, chunk=7)
    ref = autograd_grads(e, c, t, valids, d_out, d_lse, bias, softcap, shift, torch.float64)
    for a, b in zip(got, ref):
        assert torch.allclose(a, b, rtol=1e-10, atol=1e-12)

    def objective(ee, cc, bb):
        rows = valids.long()
        logits = ee[rows] @ cc.T + bb
        if softcap is not None:
            logits = softcap * torch.tanh(logits / softcap)
        lse = torch.logsumexp(logits, -1)
        nll = lse - logits.gather(1, t[rows + shift].view(-1, 1)).squeeze(1)
        tot = (nll * d_out[rows + shift]).sum()
        if d_lse is not None:
            tot = tot + (lse * d_lse[rows + shift]).sum()
        return tot

    h = 1e-6
    rng = np.random.default_rng(0)
    for which, grad, mat in (("e", got[0], e), ("c", got[1], c), ("b", got[2], bias)):
        for _ in range(6):
            idx = tuple(int(rng.integers(0, s)) for s in mat.shape)
            plus, minus = mat.clone(), mat.clone()
            plus[idx] += h
            minus[idx] -= h
            args_p = {"e": (plus, c, bias), "c": (e, plus, bias), "b": (e, c, plus)}[which]
            args_m = {"e": (minus, c, bias), "c": (e, minus, bias), "b": (e, c, minus)}[which]
            fd = (objective(*args_p) - objective(*args_m)) / (2 * h)
            assert abs(float(fd) - float(grad[idx])) < 1e-6 * max(1.0, abs(float(fd)))


def test_dense_grads_out_of_range_target_has_no_onehot_term():
    e, c, t, _ = make_inputs(8, 10, 4, torch.float64, seed=6)
    t2 = t.clone()
    t2[3] = 10_000  # matches no class: only the soft-max term remains for that row
    d_out = torch.ones(8, dtype=torch.float64)
    de, _, _ = dense_lce.dense_grads(e, c, t2, None, d_out, None, None, None, 0, torch.float64)
    p = torch.softmax(e[3] @ c.T, -1)
    assert torch.allclose(de[3], p @ c, atol=1e-12)


# ---- vocabulary shards recombine to the full result -----------------------------------------------------
@pytest.mark.parametrize("softcap", [None, 8.0])
def test_vp_shard_partials_recombine(softcap):
    N, V, D = 40, 61, 9
    e, c, t, bias = make_inputs(N, V, D, torch.float64, seed=7, bias=True)
    corr, lses = [], []
    for rank in range(4):
        s, e_ = dense_lce.partition_n_into_range(V, rank, 4)
        cl, ll = dense_lce.vp_shard_partials(e, c[s:e_], t, s, e_, bias[s:e_], softcap, torch.float64)
        corr.append(cl)
        lses.append(ll)
    nll, lse = dense_lce.vp_combine(corr, lses)
    want_lse = dense_lce.dense_lse(e, c, bias, softcap, torch.float64)
    want_nll = want_lse + dense_lce.dense_indexed_neg_dot(e, c, t, bias, None, torch.float64) if softcap is None else None
    assert torch.allclose(lse, want_lse, rtol=1e-12)
    full, _ = dense_lce.dense_linear_cross_entropy(e, c, t, bias, IGNORE_INDEX, softcap, "none")
    assert torch.allclose(nll, full, rtol=1e-10, atol=1e-12)
    if want_nll is not None:
        assert torch.allclose(nll, want_nll, rtol=1e-10, atol=1e-12)
