"""``python -m benchmark [--methods cce,torch_compile,baseline] [--test_data gemma2] ...``

Same options, kinds and table as the reference's command line (ref: benchmark/__main__.py:41-133,
README.md:301-311); arguments are parsed with argparse.
"""

import argparse
import dataclasses
import functools
import gc
import pathlib
import time
from typing import Optional

import pandas as pd
import torch
import torch.nn.functional as F

from cut_cross_entropy import linear_cross_entropy
from cut_cross_entropy.constants import IGNORE_INDEX

from . import data, memory

# what each kind times: (forward inside the timed region, backward run at all)
KINDS = {"loss-fw": (True, False), "loss-bw": (False, True), "loss-fw-bw": (True, True)}


def baseline(e, c, targets, softcap: Optional[float] = None, ignore_index: int = IGNORE_INDEX, reduction="mean"):
    """Logits in HBM, then the framework's cross-entropy (ref: benchmark/__main__.py:20-34)."""
    z = e @ c.T
    if softcap is not None:
        z = softcap * torch.tanh(z / softcap)
    return F.cross_entropy(z.float(), targets, reduction=reduction, ignore_index=ignore_index)


def _drop_grads(e, c, *_, **__):
    e.grad = None
    c.grad = None


def _quiesce():
    torch.cuda.synchronize()
    gc.collect()
    torch.cuda.empty_cache()
    time.sleep(0.2)


def _loss_fn(method: str):
    return baseline if method == "baseline" else functools.partial(linear_cross_entropy, impl=method)


def benchmark(methods, test_data, n_iteration, n_rep, dtype, output, kinds, softcap):
    """Repetition 0 of every data set is a warm-up of one iteration and is not reported (unless n_rep is 0)."""
    for kind in kinds:
        if kind not in KINDS:
            raise ValueError(f"Unknown kind {kind=}")
    precision_before = torch.get_float32_matmul_precision()
    torch.set_float32_matmul_precision("high")  # as the reference's benchmark does (benchmark/__main__.py:52)
    try:
        rows = _measure_all(methods, test_data, n_iteration, n_rep, dtype, kinds, softcap)
    finally:
        torch.set_float32_matmul_precision(precision_before)
    table = pd.DataFrame(rows)
    pd.options.display.float_format = "{:.1f}".format
    print(table)
    if output is not None:
        out = pathlib.Path(output)
        out.parent.mkdir(parents=True, exist_ok=True)
        table.to_csv(out)
    return table


def _measure_all(methods, test_data, n_iteration, n_rep, dtype, kinds, softcap):
    rows = []
    for name in test_data:
        make = data.generator(name)
        for rep in range(n_rep + 1):
            reported = rep > 0 or n_rep == 0
            sample = make(dtype=getattr(torch, dtype))
            e = sample.embedding.requires_grad_(True)
            c = sample.classifier.requires_grad_(True)
            cap = sample.softcap if softcap is None else softcap
            for kind in kinds:
                fwd, bwd = KINDS[kind]
                how = dict(forward=fwd, backward=bwd, pre_fn=_drop_grads) if bwd else {}
                for method in methods:
                    stats = memory.Stats.measure(_loss_fn(method), e, c, sample.targets, softcap=cap,
                                                 n_iteration=n_iteration if rep > 0 else 1, **how)
                    if reported:
                        rows.append({"method": method, "kind": kind, **dataclasses.asdict(stats), "test_data": name})
                        _quiesce()
            del sample, e, c
    return rows


def _csv(text: str):
    return [item for item in text.split(",") if item]


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m benchmark")
    ap.add_argument("--methods", type=_csv, default=_csv("cce,torch_compile,baseline,cce_exact"))
    ap.add_argument("--test_data", type=_csv, default=_csv("gemma2"))
    ap.add_argument("--kinds", type=_csv, default=list(KINDS))
    ap.add_argument("--n_iteration", type=int, default=50)
    ap.add_argument("--n_rep", type=int, default=1)
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--softcap", type=float, default=None)
    ap.add_argument("--output", default=None)
    a = ap.parse_args(argv)
    return benchmark(a.methods, a.test_data, a.n_iteration, a.n_rep, a.dtype, a.output, a.kinds, a.softcap)


if __name__ == "__main__":
    main()
