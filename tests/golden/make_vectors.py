"""Writes tests/golden/lce_vectors.npz: small seeded inputs (values exactly representable in bfloat16) and the
loss, log-sum-exp and gradients the dense oracle gives for them in float64.

The vectors come from THIS repository's oracle (oracle/dense_lce.py), whose functions are pinned in
tests/test_oracle_pins.py against closed forms, library routines and the reference's own known-answer test;
nothing of the reference was imported or run to make them.  They freeze the oracle (a later edit that changes
its results fails tests/test_golden_vectors.py on the CPU) and give the GPU tests one fixed set of numbers.

    python tests/golden/make_vectors.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import dense_lce  # noqa: E402

IGNORE = -100
CASES = [
    dict(name="plain", batch=(48,), V=120, D=32, softcap=None, bias=False, shift=0, ignored=0.0),
    dict(name="softcap_bias_ignored", batch=(40,), V=131, D=40, softcap=5.0, bias=True, shift=0, ignored=0.25),
    dict(name="shift_2d", batch=(3, 17), V=97, D=24, softcap=None, bias=False, shift=1, ignored=0.2),
    dict(name="shift2_softcap_bias", batch=(2, 21), V=64, D=48, softcap=12.0, bias=True, shift=2, ignored=0.1),
]


def make_case(spec, seed):
    g = torch.Generator().manual_seed(seed)
    n = int(np.prod(spec["batch"]))
    e = (torch.randn((n, spec["D"]), generator=g) * 0.7).to(torch.bfloat16).double()
    c = (torch.randn((spec["V"], spec["D"]), generator=g) * 0.4).to(torch.bfloat16).double()
    bias = (torch.randn((spec["V"],), generator=g) * 0.5).to(torch.bfloat16).double() if spec["bias"] else None
    t = torch.randint(0, spec["V"], (n,), generator=g)
    t[torch.randperm(n, generator=g)[: int(spec["ignored"] * n)]] = IGNORE
    w_loss = torch.randn((n,), generator=g).double()   # weights of the per-token losses in the test objective
    w_lse = torch.randn((n,), generator=g).double() * 0.1

    e = e.view(*spec["batch"], spec["D"]).requires_grad_(True)
    c.requires_grad_(True)
    if bias is not None:
        bias.requires_grad_(True)
    t = t.view(*spec["batch"])
    sh = spec["shift"]
    loss, lse = dense_lce.dense_linear_cross_entropy(e, c, t, bias, IGNORE, spec["softcap"], "none", sh, return_lse=True)
    wl = w_loss.view(*spec["batch"])[..., sh:]
    wz = w_lse.view(*spec["batch"])[..., sh:]
    ((loss * wl).sum() + (lse * wz).sum()).backward()
    out = dict(e=e.detach(), c=c.detach(), targets=t, w_loss=w_loss.view(*spec["batch"]), w_lse=w_lse.view(*spec["batch"]),
               loss=loss.detach(), lse=lse.detach(), d_e=e.grad, d_c=c.grad)
    if bias is not None:
        out.update(bias=bias.detach(), d_bias=bias.grad)
    return out


def main():
    arrays = {}
    for i, spec in enumerate(CASES):
        for key, value in make_case(spec, 1000 + i).items():
            dtype = np.int64 if key == "targets" else np.float32 if key in ("e", "c", "bias") else np.float64
            arrays[f"{spec['name']}/{key}"] = value.numpy().astype(dtype)
        arrays[f"{spec['name']}/softcap"] = np.float64(spec["softcap"] if spec["softcap"] is not None else 0.0)
        arrays[f"{spec['name']}/shift"] = np.int64(spec["shift"])
    np.savez_compressed(os.path.join(HERE, "lce_vectors.npz"), **arrays)
    print("wrote", len(arrays), "arrays for", len(CASES), "cases")


if __name__ == "__main__":
    main()
