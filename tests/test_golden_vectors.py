"""The committed vectors of tests/golden/lce_vectors.npz (made by tests/golden/make_vectors.py from the dense oracle
in float64): on the CPU they freeze the oracle, on the GPU the HIP path is held against the same numbers."""

import os

import numpy as np
import pytest
import torch

from _util import IGNORE_INDEX

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lce_vectors.npz")
NAMES = ["plain", "softcap_bias_ignored", "shift_2d", "shift2_softcap_bias"]


def _load(name):
    with np.load(GOLDEN, allow_pickle=False) as z:
        case = {k.split("/", 1)[1]: torch.from_numpy(np.asarray(z[k])) for k in z.files if k.startswith(name + "/")}
    case["softcap"] = float(case["softcap"]) or None
    case["shift"] = int(case["shift"])
    return case


@pytest.mark.parametrize("name", NAMES)
def test_inputs_are_bfloat16_values(name):
    g = _load(name)
    for key in ("e", "c", "bias"):
        if key in g:
            assert torch.equal(g[key], g[key].to(torch.bfloat16).float())


@pytest.mark.parametrize("name", NAMES)
def test_oracle_reproduces_the_vectors(name):
    from oracle import dense_lce

    g = _load(name)
    e = g["e"].double().requires_grad_(True)
    c = g["c"].double().requires_grad_(True)
    bias = g["bias"].double().requires_grad_(True) if "bias" in g else None
    sh = g["shift"]
    loss, lse = dense_lce.dense_linear_cross_entropy(e, c, g["targets"], bias, IGNORE_INDEX, g["softcap"], "none", sh,
                                                     return_lse=True)
    ((loss * g["w_loss"][..., sh:]).sum() + (lse * g["w_lse"][..., sh:]).sum()).backward()
    for got, key in ((loss, "loss"), (lse, "lse"), (e.grad, "d_e"), (c.grad, "d_c")):
        assert torch.allclose(got.detach(), g[key], rtol=1e-12, atol=1e-12), key
    if bias is not None:
        assert torch.allclose(bias.grad, g["d_bias"], rtol=1e-12, atol=1e-12)
    ignored = g["targets"][..., sh:] == IGNORE_INDEX
    assert (g["loss"][ignored] == 0).all() and (g["lse"][ignored] == 0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("impl", ["cce", "cce_exact"])
@pytest.mark.parametrize("name", NAMES)
def test_hip_path_against_the_vectors(name, impl):
    """bf16 inputs (the stored values exactly), loss and log-sum-exp within 1e-3, gradients within 1e-2 of their
    scale (the filter of impl="cce" skips only entries below 2^-12 of it)."""
    from cut_cross_entropy import linear_cross_entropy

    g = _load(name)
    dev = "cuda:0"
    e = g["e"].to(torch.bfloat16).to(dev).requires_grad_(True)
    c = g["c"].to(torch.bfloat16).to(dev).requires_grad_(True)
    bias = g["bias"].to(torch.bfloat16).to(dev).requires_grad_(True) if "bias" in g else None
    sh = g["shift"]
    loss, lse = linear_cross_entropy(e, c, g["targets"].to(dev), bias=bias, softcap=g["softcap"], shift=sh,
                                     reduction="none", return_lse=True, impl=impl)
    ((loss * g["w_loss"].to(dev).float()[..., sh:]).sum() + (lse * g["w_lse"].to(dev).float()[..., sh:]).sum()).backward()
    assert torch.allclose(loss.cpu().double(), g["loss"], rtol=1e-3, atol=1e-3)
    assert torch.allclose(lse.cpu().double(), g["lse"], rtol=1e-3, atol=1e-3)
    ignored = g["targets"][..., sh:] == IGNORE_INDEX
    assert (loss.cpu()[ignored] == 0).all() and (lse.cpu()[ignored] == 0).all()  # bit-exact masking
    pairs = [(e.grad, "d_e"), (c.grad, "d_c")] + ([(bias.grad, "d_bias")] if bias is not None else [])
    for got, key in pairs:
        want = g[key]
        assert (got.cpu().double() - want).abs().max() <= 1e-2 * want.abs().max(), key
