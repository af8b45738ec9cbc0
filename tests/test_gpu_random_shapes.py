"""Seeded sweep over shapes that sit on and next to the kernels' tile boundaries (32-row groups, 128- and
256-wide tiles, 64- and 128-column stages, 8-element vector pieces) with the options drawn at random:
loss, log-sum-exp and gradients of the operator against the dense oracle, same criterion as the grid tests."""

import random

import pytest
import torch

from _util import IGNORE_INDEX, assert_no_worse, make_inputs
from test_gpu_operator import TOL, _oracle_loss

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 31, 32, 33, 63, 64, 65, 255, 256, 257, 300, 511, 513]
CLASSES = [2, 7, 31, 32, 33, 127, 128, 129, 255, 256, 257, 1000, 2049]
WIDTHS = [8, 16, 24, 56, 64, 72, 120, 128, 136, 192, 256, 264, 320, 384]


def _cases(n):
    rng = random.Random(20240607)
    out = []
    for i in range(n):
        batch = rng.choice([1, 1, 2, 3])
        out.append(dict(
            seed=100 + i,
            batch=batch,
            rows=rng.choice(ROWS),
            V=rng.choice(CLASSES),
            D=rng.choice(WIDTHS),
            dtype=rng.choice([torch.bfloat16, torch.bfloat16, torch.float16]),
            softcap=rng.choice([None, None, 5.0, 30.0]),
            bias=rng.random() < 0.3,
            shift=rng.choice([0, 0, 1, 2]),
            invalid=rng.choice([0.0, 0.0, 0.2, 0.9]),
            reduction=rng.choice(["mean", "mean", "sum", "none"]),
            z_loss=rng.random() < 0.3,
            impl=rng.choice(["cce", "cce", "cce_exact", "cce_kahan_full_c"]),
        ))
    return out


def _id(case):
    return "-".join(f"{k}{str(v).replace('torch.', '')}" for k, v in case.items() if k != "seed")


@pytest.mark.parametrize("case", _cases(240), ids=_id)
def test_random_shape(case):
    from cut_cross_entropy import linear_cross_entropy
    from cut_cross_entropy.utils import compute_z_loss

    T, B, V, D, dtype = case["rows"], case["batch"], case["V"], case["D"], case["dtype"]
    shift = min(case["shift"], T - 1)
    e, c, t, bias = make_inputs(B * T, V, D, dtype, seed=case["seed"], bias=case["bias"],
                                invalid_frac=case["invalid"])
    e = e.view(B, T, D)
    t = t.view(B, T)
    softcap, reduction, z_loss = case["softcap"], case["reduction"], case["z_loss"]
    if (t[..., shift:] != IGNORE_INDEX).sum() == 0:
        t[0, shift] = 0  # the empty batch has a test of its own
    gt_loss, gt = _oracle_loss(e, c, t, bias, softcap, shift, reduction, z_loss, torch.float64, True)
    ref_loss, ref = _oracle_loss(e, c, t, bias, softcap, shift, reduction, z_loss, dtype, True)

    dev = torch.device("cuda:0")
    ed = e.to(dev).requires_grad_(True)
    cd = c.to(dev).requires_grad_(True)
    bd = bias.to(dev).requires_grad_(True) if bias is not None else None
    td = t.to(dev)
    out = linear_cross_entropy(ed, cd, td, bias=bd, softcap=softcap, shift=shift, reduction=reduction,
                               impl=case["impl"], return_lse=z_loss)
    loss, lse = out if z_loss else (out, None)
    assert_no_worse(gt_loss, ref_loss, loss.detach(), TOL[dtype], "loss", rel=TOL[dtype])
    obj = loss
    if reduction == "sum":
        obj = obj / (td[..., shift:] != IGNORE_INDEX).count_nonzero()
    obj = obj.mean()
    if z_loss:
        obj = obj + compute_z_loss(lse, td, shift)
    obj.backward()
    for name, g_gt, g_ref, g in zip(["dE", "dC", "dBias"], gt, ref, [ed.grad, cd.grad, bd.grad if bd is not None else None]):
        if g is not None:
            # with a handful of valid rows the gradients are of order one, where one rounding of the 16-bit
            # result alone exceeds the absolute tolerance: allow the same figure relative to the value
            assert_no_worse(g_gt, g_ref, g, TOL[dtype], f"{case['impl']} {name}", rel=TOL[dtype])
    ignored_rows = torch.ones((B, T), dtype=torch.bool)
    ignored_rows[:, : T - shift] = t[:, shift:] == IGNORE_INDEX
    assert (ed.grad.cpu()[ignored_rows] == 0).all()  # rows that do not count get exactly zero
