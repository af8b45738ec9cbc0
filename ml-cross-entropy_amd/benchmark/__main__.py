"""``python -m benchmark [--methods cce,torch_compile,baseline] [--test_data gemma2] ...``

Same options, kinds and table as the reference's command line (ref: benchmark/__main__.py:41-133,
README.md:301-311); arguments are parsed with argparse.
"""

import argparse
import functools
import gc
import time
from dataclasses import asdict
from pathlib import Path
from typing import Optional

import pandas as pd
import torch
import torch.nn.functional as F

from cut_cross_entropy import linear_cross_entropy
from cut_cross_entropy.constants import IGNORE_INDEX

from . import data, memory


def baseline(e, c, targets, softcap: Optional[float] = None, ignore_index: int = IGNORE_INDEX, reduction="mean"):
    """Logits in HBM, then the framework's cross-entropy (ref: benchmark/__main__.py:20-34)."""
    logits = e @ c.T
    if softcap is not None:
        logits = torch.tanh(logits / softcap) * softcap
    return F.cross_entropy(logits.float(), targets, ignore_index=ignore_index, reduction=reduction)


def clear_grad_fn(e, c, *args, **kwargs):
    e.grad = c.grad = None


def benchmark(methods, test_data, n_iteration, n_rep, dtype, output, kinds, softcap):
    torch.set_float32_matmul_precision("high")
    dtype = getattr(torch, dtype)
    all_stats = []
    for name in test_data:
        gen = data.generator(name)
        for rep in range(n_rep + 1):
            d = gen(dtype=dtype)
            for kind in kinds:
                e, c, t = d.embedding, d.classifier, d.targets
                kwargs = {"softcap": softcap if softcap is not None else d.softcap}
                e.requires_grad_(True)
                c.requires_grad_(True)
                if kind == "loss-fw":
                    pass
                elif kind in ("loss-bw", "loss-fw-bw"):
                    kwargs["backward"] = True
                    kwargs["forward"] = kind == "loss-fw-bw"
                    kwargs["pre_fn"] = clear_grad_fn
                else:
                    raise ValueError(f"Unknown kind {kind=}")
                for m in methods:
                    f = baseline if m == "baseline" else functools.partial(linear_cross_entropy, impl=m)
                    stats = memory.Stats.measure(f, e, c, t, n_iteration=n_iteration if rep > 0 else 1, **kwargs)
                    if rep > 0 or n_rep == 0:
                        all_stats.append({"method": m, "kind": kind} | asdict(stats) | {"test_data": name})
                        torch.cuda.synchronize()
                        gc.collect()
                        torch.cuda.empty_cache()
                        time.sleep(0.2)
            del d
    frame = pd.DataFrame(all_stats)
    pd.options.display.float_format = "{:.1f}".format
    print(frame)
    if output is not None:
        path = Path(output)
        path.parent.mkdir(parents=True, exist_ok=True)
        frame.to_csv(path)
    return frame


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m benchmark")
    ap.add_argument("--methods", default="cce,torch_compile,baseline,cce_exact")
    ap.add_argument("--test_data", default="gemma2")
    ap.add_argument("--n_iteration", type=int, default=50)
    ap.add_argument("--n_rep", type=int, default=1)
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--output", default=None)
    ap.add_argument("--kinds", default="loss-fw,loss-bw,loss-fw-bw")
    ap.add_argument("--softcap", type=float, default=None)
    a = ap.parse_args(argv)
    return benchmark(a.methods.split(","), a.test_data.split(","), a.n_iteration, a.n_rep, a.dtype, a.output,
                     a.kinds.split(","), a.softcap)


if __name__ == "__main__":
    main()
