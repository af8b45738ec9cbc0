"""Benchmark of the linear-cross-entropy loss path on one MI355X.

One step = forward + backward of ``linear_cross_entropy`` over one batch of synthetic input already
resident in HBM.  Default workload c2: the Gemma-2-2B-shaped head, E [8192, 2304] bf16 ~ N(0,1),
C [256000, 2304] bf16 ~ N(0, 0.02), uniform labels, softcap 30, reduction mean, impl="cce" with gradient
filtering.  ``--workload c1|c3|c4|c5|c5shard`` run the other benchmark configurations; ``--impl`` runs a workload
under another preset (cce_kahan_full_c, cce_kahan_full_e, cce_kahan, cce_exact), ``--dtype fp16|fp32`` and
``--bias`` the same inputs in another input type / with a classifier bias, ``--dense-workspace-mb`` caps the
workspace of the unfiltered backward (memory against time).  Prints one JSON line.

The timing method restates the reference benchmark (benchmark/memory.py:82-112,
benchmark/__main__.py:41-125): warm-up, then per iteration clear the gradients and run loss + backward.
The forward kernel and the backward are also timed one by one with device events recorded around their
launches INSIDE the timed steps.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ml-cross-entropy_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2516.6  # 256 CU x 4096 flop/clk x 2.4 GHz, dense (bf16 and fp16 alike)
PEAK_FP32_TFLOPS = 157.3   # dense fp32 matrix peak
Z_LOSS_WEIGHT = 1e-4

WORKLOADS = {
    # name: N (rows of flattened e), D, V, and what the step does
    "c1": dict(N=4096, D=1024, V=32000, softcap=None, impl="cce", text="5 % of the labels ignored, reduction=mean, impl=cce"),
    "c2": dict(N=8192, D=2304, V=256000, softcap=30.0, impl="cce",
               text="uniform labels, softcap=30.0, reduction=mean, impl=cce, gradient filter on"),
    "c3": dict(N=16384, D=4096, V=128256, softcap=None, impl="cce",
               text="E [4,4096,4096], labels [4,4096] with the last 256 per row ignored, shift=1, reduction=mean, impl=cce"),
    "c4": dict(N=8192, D=2048, V=256000, softcap=None, impl="cce_kahan_full_c_full_e",
               text="Zipf(1.1) labels, impl=cce_kahan_full_c_full_e (no filter), loss = nll + 1e-4 z-loss, reduction=none"),
    "c5": dict(N=65536, D=3584, V=152064, softcap=None, impl="cce",
               text="E = 4 C[label] + N(0,0.5) (peaked soft-max), reduction=mean, impl=cce, gradient filter on"),
    "c5shard": dict(N=65536, D=3584, V=19008, softcap=None, impl="cce",
                    text="the c5 inputs against the vocabulary shard C[0:19008] of 152064 classes, "
                         "VocabParallelOptions(0, 19008), reduction=mean, impl=cce"),
}


def make_workload(name):
    """Inputs on the CPU from one seeded generator in the fixed order E, C, labels (C first where E is
    built from it), rounded to bf16."""
    import torch

    spec = WORKLOADS[name]
    N, D, V = spec["N"], spec["D"], spec["V"]
    g = torch.Generator().manual_seed(0)

    def randn_bf16(rows, cols, std):
        out = torch.empty((rows, cols), dtype=torch.bfloat16)
        for s in range(0, rows, 16384):  # bounded host memory
            n = min(16384, rows - s)
            out[s : s + n] = (torch.randn((n, cols), generator=g) * std).to(torch.bfloat16)
        return out

    w = dict(spec, name=name, shift=0, vocab=V, vp=None)
    if name in ("c5", "c5shard"):
        Vfull = 152064
        c = randn_bf16(Vfull, D, 0.02)
        t = torch.randint(0, Vfull, (N,), generator=g)
        e = torch.empty((N, D), dtype=torch.bfloat16)
        for s in range(0, N, 8192):
            idx = t[s : s + 8192]
            e[s : s + 8192] = (4.0 * c[idx].float() + 0.5 * torch.randn((idx.numel(), D), generator=g)).to(torch.bfloat16)
        if name == "c5shard":
            c = c[:V].contiguous()
            w["vp"] = (0, V)
        w.update(e=e, c=c, t=t, valid=N)
        return w
    e = randn_bf16(N, D, 1.0)
    c = randn_bf16(V, D, 0.02)
    if name == "c4":  # Zipf(s = 1.1) over ranks 1..V by inverse-CDF sampling; rank r -> token r - 1
        ranks = torch.arange(1, V + 1, dtype=torch.float64)
        cdf = torch.cumsum(ranks.pow(-1.1), 0)
        cdf /= cdf[-1].clone()
        t = torch.searchsorted(cdf, torch.rand((N,), generator=g, dtype=torch.float64)).clamp_(max=V - 1)
    else:
        t = torch.randint(0, V, (N,), generator=g)
    valid = N
    if name == "c1":
        t[torch.randperm(N, generator=g)[: int(0.05 * N)]] = -100
        valid = int((t != -100).sum())
    if name == "c3":
        e, t = e.view(4, 4096, D), t.view(4, 4096)
        t[:, -256:] = -100
        w["shift"] = 1
        valid = int((t[:, 1:] != -100).sum())
    w.update(e=e, c=c, t=t, valid=valid)
    return w


def loss_fn(w):
    """The step's forward as a closure over device tensors: returns a scalar loss."""
    from cut_cross_entropy import VocabParallelOptions, linear_cross_entropy
    from cut_cross_entropy.utils import compute_z_loss

    vp = VocabParallelOptions(*w["vp"]) if w["vp"] is not None else None

    def run(e, c, t, bias=None):
        if w["name"] == "c4":
            nll, lse = linear_cross_entropy(e, c, t, bias=bias, reduction="none", return_lse=True, impl=w["impl"])
            return (nll + Z_LOSS_WEIGHT * compute_z_loss(lse, t, reduction="none")).mean()
        return linear_cross_entropy(e, c, t, bias=bias, softcap=w["softcap"], shift=w["shift"], reduction="mean",
                                    impl=w["impl"], vocab_parallel_options=vp)

    return run


def measured_traffic(workload, source_hash):
    """HBM bytes per launch of the dominant kernel from the committed counter summary, if that summary was
    taken with the very sources the loaded library is built from (else None: a stale figure is no measurement)."""
    import re

    try:
        text = open(os.path.join(ROOT, "profiles", "lse_forward_c2_hbm_traffic.txt")).read()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes=(\S+) workload=(\S+) source_hash=(\S+)", text)
    if m and m.group(2) == workload and m.group(3) == source_hash:
        return float(m.group(1)), "profiles/lse_forward_c2_hbm_traffic.txt"
    return None, None


def cpu_baseline(w, rows):
    """Dense oracle (the reference's torch_compile path restated) on the host cores, fp32,
    forward + backward over the first ``rows`` tokens of the same workload."""
    import torch

    from oracle import dense_lce

    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(threads)
    e2 = w["e"].reshape(-1, w["D"])
    t1 = w["t"].reshape(-1)
    if w["shift"]:
        e2, t1 = e2[: rows], t1[w["shift"] : rows + w["shift"]]
    e = e2[:rows].float().requires_grad_(True)
    c = w["c"].float().requires_grad_(True)
    t = t1[:rows].clone()
    if w["vp"] is not None:
        t[(t < w["vp"][0]) | (t >= w["vp"][1])] = -100  # out-of-shard targets contribute no correct-logit term

    def step():
        e.grad = c.grad = None
        loss, _ = dense_lce.dense_linear_cross_entropy(e, c, t, softcap=w["softcap"])
        loss.backward()
        return loss

    step()
    reps, t0 = 0, time.perf_counter()
    while True:
        step()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > 10.0 or reps >= 40:  # about ten seconds of host work
            break
    valid = int((t != -100).sum()) if w["vp"] is None else rows
    return {
        "value": valid * reps / dt,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {rows} of {w['N']} tokens against the full [{w['V']},{w['D']}] classifier, fp32, "
                  f"dense oracle fwd+bwd (mean loss), {reps} timed reps after 1 warm-up",
    }


def gemm_yardstick(args, w, e2, c):
    """The library's matrix product of the forward's shape, timed with device events like the forward kernel."""
    import torch

    n, d = e2.shape
    v = c.shape[0]
    out = torch.empty((n, v), dtype=e2.dtype, device=e2.device)
    for _ in range(args.warmup):
        torch.mm(e2, c.t(), out=out)
    torch.cuda.synchronize()
    evs = []
    for _ in range(args.steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        torch.mm(e2, c.t(), out=out)
        b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    peak = PEAK_FP32_TFLOPS if args.dtype == "fp32" else PEAK_BF16_TFLOPS
    tflops = 2.0 * n * v * d / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "library matrix product E . C^T (yardstick, not the loss path)",
        "config": {"workload": f"{w['name']}: E[{n},{d}] x C[{v},{d}]^T {args.dtype} -> [{n},{v}] {args.dtype}, torch.mm "
                               f"(hipBLASLt / rocBLAS), {w['text']}"},
        "steps": args.steps, "warmup": args.warmup, "ms_per_launch": ms, "tflops": tflops, "frac": tflops / peak,
        "peak": peak, "output_bytes": out.numel() * out.element_size(),
    }))


def forward_launcher(args, w, e2, c):
    """The forward launcher alone (the reference's cce_lse_forward_kernel API), without and with the optional
    average of the logits over the rows, timed with device events."""
    import torch

    from cut_cross_entropy.cce_lse_forward import cce_lse_forward_kernel

    n, d = e2.shape
    v = c.shape[0]
    out = {}
    for name, want in (("lse", False), ("lse_and_logit_avg", True)):
        for _ in range(args.warmup):
            cce_lse_forward_kernel(e2, c, softcap=w["softcap"], return_logit_avg=want)
        torch.cuda.synchronize()
        evs = []
        for _ in range(args.steps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            cce_lse_forward_kernel(e2, c, softcap=w["softcap"], return_logit_avg=want)
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
        out[name] = {"ms_per_call": ms, "tflops": 2.0 * n * v * d / (ms * 1e-3) / 1e12}
    print(json.dumps({
        "metric": "forward launcher alone: lse, and lse with logit_avg (not the loss path)",
        "config": {"workload": f"{w['name']}: E[{n},{d}] x C[{v},{d}] {args.dtype}, softcap={w['softcap']}, all rows valid"},
        "steps": args.steps, "warmup": args.warmup, **out,
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--impl", default=None,
                    help="run the workload under this preset instead of its own (cce, cce_exact, cce_kahan, "
                         "cce_kahan_full_c, cce_kahan_full_e, cce_kahan_full_c_full_e)")
    ap.add_argument("--dtype", default="bf16", choices=("bf16", "fp16", "fp32"),
                    help="input type of e and c (the bf16 values of the workload, converted)")
    ap.add_argument("--bias", action="store_true", help="add a classifier bias ~ N(0, 0.02) that wants a gradient")
    ap.add_argument("--dense-workspace-mb", type=float, default=None,
                    help="cap the workspace of the unfiltered backward (dz chunk + dE compensation buffer) at this "
                         "many MB, for presets that ask for it and for a filtered backward that changes to it")
    ap.add_argument("--zero-data", action="store_true",
                    help="run the workload's shapes on operands of zeros: the kernels do the same work at the clock "
                         "the chip holds when the matrix pipes toggle nothing (what the power limit costs)")
    ap.add_argument("--gemm-yardstick", action="store_true",
                    help="instead of the loss path, time the library's plain matrix product E . C^T of the workload's "
                         "shape and input type (the logits the forward kernel never writes), and print its TFLOP/s")
    ap.add_argument("--forward-launcher", action="store_true",
                    help="instead of the loss path, time the forward launcher alone on the workload's shape, without "
                         "and with its optional logit_avg output")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=256)
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain 1 GiB device copy, the calibration kernel for FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--traffic", type=float, default=None,
                    help="HBM bytes per launch of the dominant kernel of THIS build, measured with rocprofv3 --pmc; "
                         "reported as given; without it the figure of profiles/ is reported if it belongs to this build")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import __graft_entry__

    __graft_entry__.ensure_built()  # loads the library built in the tree; builds it only if there is none
    import torch

    from cut_cross_entropy import _hip
    from cut_cross_entropy import cce as cce_mod
    from cut_cross_entropy import cce_backward as bwd_mod

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = make_workload(args.workload)
    if args.impl is not None:
        w["impl"] = args.impl
        w["text"] += f" [run with impl={args.impl}]"
    if args.dense_workspace_mb is not None:
        limit = int(args.dense_workspace_mb * 2**20)
        # the 16-bit compensation buffer of the gradient the unfiltered backward carries between its launches
        comp = _hip.load().cce_backward_dense_fixed_bytes(w["valid"], w["V"], w["D"], 1)
        bwd_mod.DENSE_WORKSPACE_LIMIT_BYTES = limit
        bwd_mod.DENSE_WORKSPACE_LIMIT_OPERANDS = 0.0
        bwd_mod.DENSE_DZ_BYTES = max(limit - comp, 0)
        bwd_mod.DENSE_DZ_MIN_CLASSES = 0
    in_dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.dtype]
    if args.zero_data:
        w["e"].zero_()
        w["c"].zero_()
        w["text"] += " [operands replaced by zeros]"
    e = w["e"].to(dev).to(in_dtype).requires_grad_(True)
    c = w["c"].to(dev).to(in_dtype).requires_grad_(True)
    t = w["t"].to(dev)
    if args.gemm_yardstick:
        gemm_yardstick(args, w, e.detach().reshape(-1, w["D"]), c.detach())
        return
    if args.forward_launcher:
        forward_launcher(args, w, e.detach().reshape(-1, w["D"]), c.detach())
        return
    bias = None
    if args.bias:
        gb = torch.Generator().manual_seed(1)
        bias = (torch.randn((w["V"],), generator=gb) * 0.02).to(torch.bfloat16).to(dev).to(in_dtype).requires_grad_(True)
    B, N, V, D = w["valid"], w["N"], w["V"], w["D"]
    run = loss_fn(w)
    counters = torch.zeros((4,), dtype=torch.int64, device=dev)

    def step():
        e.grad = None
        c.grad = None
        if bias is not None:
            bias.grad = None
        loss = run(e, c, t, bias)
        loss.backward()
        return loss

    if args.traffic_probe:
        src = torch.empty((1 << 29,), dtype=torch.bfloat16, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps; device events around the kernels of every step ---------------
    timers = {}
    _hip.set_timers(timers)
    cce_mod.set_tile_counters(counters)
    counters.zero_()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    cce_mod.set_tile_counters(None)
    _hip.set_timers(None)
    ms_per_step = dt / args.steps * 1e3
    cnt = [int(x) for x in counters.tolist()]
    k_r, k_e, k_c = (min(cnt[i] / max(cnt[0], 1), 1.0) for i in (1, 2, 3))
    if args.dtype == "fp32":
        k_r = k_e = k_c = 1.0  # the fp32 path is unfiltered and keeps no counters
    # per step: a launcher may be called more than once in a step (the fp32 path walks the vocabulary in chunks)
    kernel_ms = {name: sum(a.elapsed_time(b) for a, b in evs) / args.steps for name, evs in timers.items()}

    # ---- loss-path peak memory (allocator peak minus the returned gradients) --------------------
    e.grad = c.grad = None
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    step()
    torch.cuda.synchronize()
    peak_bytes = torch.cuda.max_memory_allocated() - base
    grads = e.grad.numel() * e.grad.element_size() + c.grad.numel() * c.grad.element_size()
    if bias is not None:
        grads += bias.grad.numel() * bias.grad.element_size()
    extra_mb = (peak_bytes - grads) / 2**20

    traffic, traffic_source = args.traffic, "--traffic" if args.traffic is not None else None
    if traffic is None:
        traffic, traffic_source = measured_traffic(w["name"], _hip.load().cce_source_hash().decode())

    peak = PEAK_FP32_TFLOPS if args.dtype == "fp32" else PEAK_BF16_TFLOPS
    fwd_ms = kernel_ms["forward_fp32"] if args.dtype == "fp32" else kernel_ms["lse_forward"]
    fwd_flops = 2.0 * B * V * D
    fwd_tflops = fwd_flops / (fwd_ms * 1e-3) / 1e12
    bwd_parts = [n for n in ("backward_sparse", "backward_dense", "backward_fp32") if n in kernel_ms]
    bwd_name = "+".join(bwd_parts)
    bwd_ms = sum(kernel_ms[n] for n in bwd_parts)
    bwd_flops = 2.0 * B * V * D * (k_r + k_e + k_c)

    f_alg = 2.0 * B * V * D * (1.0 + k_r + k_e + k_c)
    f_dense = 8.0 * B * V * D
    out = {
        "metric": "fwd+bwd tokens/s",
        "value": B / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {
            "workload": f"{w['name']}: E[{N},{D}] {args.dtype}, C[{V},{D}] {args.dtype} N(0,0.02), {w['text']}"
                        f"{', classifier bias' if args.bias else ''}, fwd+bwd",
            "valid_tokens": B,
            "impl": w["impl"],
            "dense_workspace_limit_mb": None if bwd_mod.DENSE_WORKSPACE_LIMIT_BYTES is None
            else max(bwd_mod.DENSE_WORKSPACE_LIMIT_BYTES,
                     bwd_mod.DENSE_WORKSPACE_LIMIT_OPERANDS * (B * D + V * D) * in_dtype.itemsize) / 2**20,
        },
        "loss": float(loss),
        "loss_path_peak_mb": extra_mb,
        "kept_tiles": {"k_recompute": k_r, "k_dE": k_e, "k_dC": k_c, "tiles": cnt[0] // max(args.steps, 1)},
        "fwd_bwd_tflops_alg": f_alg / (ms_per_step * 1e-3) / 1e12,
        "fwd_bwd_frac_alg": f_alg / (ms_per_step * 1e-3) / 1e12 / peak,
        "fwd_bwd_frac_dense_equiv": f_dense / (ms_per_step * 1e-3) / 1e12 / peak,
        "roofline": {
            "kernel": ("the fp32 forward (three-way bf16 split of e and c, lse_forward16_kernel per vocabulary chunk, merge)"
                       if args.dtype == "fp32" else
                       "lse_forward16_kernel (fused E.C^T + softcap + online log-sum-exp)")
                      + ", device events around its launches inside the timed steps",
            "bound": "mfma",
            "achieved": fwd_tflops,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": fwd_tflops / peak,
            "ms_per_launch": fwd_ms,
            "traffic": traffic,
            "traffic_source": traffic_source,
        },
        "backward": {
            "path": bwd_name,
            "ms": bwd_ms,
            "tflops_alg": bwd_flops / (bwd_ms * 1e-3) / 1e12,
            "frac_alg": bwd_flops / (bwd_ms * 1e-3) / 1e12 / peak,
            "parts_ms": {n: kernel_ms[n] for n in bwd_parts},
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
