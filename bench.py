"""Benchmark of the linear-cross-entropy loss path on one MI355X.

One step = forward + backward of ``linear_cross_entropy`` (impl="cce", gradient filtering on)
over one batch of synthetic input already resident in HBM.  Workload: the Gemma-2-2B-shaped
head, E [8192, 2304] bf16 ~ N(0,1), C [256000, 2304] bf16 ~ N(0, 0.02), uniform labels,
softcap 30, reduction mean.  Prints one JSON line.

The timing method restates the reference benchmark (benchmark/memory.py:82-112,
benchmark/__main__.py:41-125): warm-up, then per iteration clear the gradients and run
loss + backward between device-side time stamps.
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

PEAK_BF16_TFLOPS = 2516.6  # 256 CU x 4096 flop/clk x 2.4 GHz, dense
# HBM bytes per launch of lse_forward_kernel at workload c2, from two rocprofv3 --pmc runs (FETCH_SIZE x 2.0
# + WRITE_SIZE x 1.0, factors from a 1 GiB copy in the same runs; summary in profiles/).  A counter cannot be
# read from inside this script, so the figure of the last profiled build is reported unless --traffic is given.
MEASURED_TRAFFIC_BYTES = {"c2": 1.446e10}


def make_workload(name, device):
    import torch

    g = torch.Generator().manual_seed(0)
    if name == "c2":
        N, D, V, softcap = 8192, 2304, 256000, 30.0
    elif name == "c1":
        N, D, V, softcap = 4096, 1024, 32000, None
    else:
        raise ValueError(name)
    e = torch.randn((N, D), generator=g).to(torch.bfloat16)
    c = torch.empty((V, D), dtype=torch.bfloat16)
    chunk = 32000
    for s in range(0, V, chunk):  # bounded host memory
        c[s : s + chunk] = (torch.randn((min(chunk, V - s), D), generator=g) * 0.02).to(torch.bfloat16)
    t = torch.randint(0, V, (N,), generator=g)
    if name == "c1":
        idx = torch.randperm(N, generator=g)[: int(0.05 * N)]
        t[idx] = -100
    return dict(name=name, N=N, D=D, V=V, softcap=softcap, e=e, c=c, t=t)


def cpu_baseline(w, rows):
    """Dense oracle (the reference's torch_compile path restated) on the host cores, fp32,
    forward + backward over the first ``rows`` tokens of the same workload."""
    import torch

    from oracle import dense_lce

    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(threads)
    e = w["e"][:rows].float().requires_grad_(True)
    c = w["c"].float().requires_grad_(True)
    t = w["t"][:rows]

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
        if dt > 12.0 or reps >= 5:
            break
    valid = int((t != -100).sum())
    return {
        "value": valid * reps / dt,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {rows} of {w['N']} tokens against the full [{w['V']},{w['D']}] classifier, fp32, "
                  f"dense oracle fwd+bwd, {reps} timed reps after 1 warm-up",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=256)
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain 1 GiB device copy, the calibration kernel for FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--traffic", type=float, default=None,
                    help="HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc (reported as given)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import __graft_entry__

    __graft_entry__.ensure_built()  # loads the library built in the tree; builds it only if there is none
    import torch

    from cut_cross_entropy import _hip, linear_cross_entropy
    from cut_cross_entropy import cce as cce_mod

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = make_workload(args.workload, dev)
    e = w["e"].to(dev).requires_grad_(True)
    c = w["c"].to(dev).requires_grad_(True)
    t = w["t"].to(dev)
    B = int((w["t"] != -100).sum())
    N, V, D = w["N"], w["V"], w["D"]

    counters = torch.zeros((4,), dtype=torch.int64, device=dev)

    def step():
        e.grad = None
        c.grad = None
        loss = linear_cross_entropy(e, c, t, softcap=w["softcap"], reduction="mean", impl="cce")
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

    # ---- timed region: exactly K steps -------------------------------------------------------
    cce_mod.set_tile_counters(counters)
    counters.zero_()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    cce_mod.set_tile_counters(None)
    ms_per_step = dt / args.steps * 1e3
    cnt = [int(x) for x in counters.tolist()]
    k_r, k_e, k_c = (cnt[i] / max(cnt[0], 1) for i in (1, 2, 3))

    # ---- loss-path peak memory (allocator peak minus the returned gradients) --------------------
    e.grad = c.grad = None
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    step()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    grads = e.grad.numel() * e.grad.element_size() + c.grad.numel() * c.grad.element_size()
    extra_mb = (peak - grads) / 2**20

    # ---- dominant kernel (fused matmul + LSE) timed alone with device events -----------------
    lib = _hip.load()
    ed, cd = e.detach(), c.detach()
    lse = torch.empty((B,), dtype=torch.float32, device=dev)
    tm = torch.empty((lib.cce_tile_stat_elems(B, V),), dtype=torch.float32, device=dev)
    ws = torch.empty((lib.cce_lse_forward_workspace_bytes(B, V, D) // 8 + 1,), dtype=torch.int64, device=dev)
    valids = None
    if B != N:
        valids = torch.nonzero(t != -100).squeeze(1).to(torch.int32)
    stream = torch.cuda.current_stream().cuda_stream

    def launch_fwd():
        st = lib.cce_lse_forward(
            ed.data_ptr(), cd.data_ptr(), None, valids.data_ptr() if valids is not None else None,
            lse.data_ptr(), None, tm.data_ptr(), ws.data_ptr(), ws.numel() * 8,
            N, B, V, D, ed.stride(0), cd.stride(0), cd.stride(1), w["softcap"] or 0.0, 0, stream)
        assert st == 0

    launch_fwd()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in evs:
        a.record()
        launch_fwd()
        b.record()
    torch.cuda.synchronize()
    fwd_ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    fwd_flops = 2.0 * B * V * D
    fwd_tflops = fwd_flops / (fwd_ms * 1e-3) / 1e12

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
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{w['name']}: E[{N},{D}] bf16 N(0,1), C[{V},{D}] bf16 N(0,0.02), uniform labels, "
                        f"softcap={w['softcap']}, reduction=mean, impl=cce, gradient filter on, fwd+bwd",
            "valid_tokens": B,
        },
        "loss": float(loss),
        "loss_path_peak_mb": extra_mb,
        "kept_tiles": {"k_recompute": k_r, "k_dE": k_e, "k_dC": k_c, "tiles": cnt[0] // max(args.steps, 1)},
        "fwd_bwd_tflops_alg": f_alg / (ms_per_step * 1e-3) / 1e12,
        "fwd_bwd_frac_alg": f_alg / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "fwd_bwd_frac_dense_equiv": f_dense / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "roofline": {
            "kernel": "lse_forward_kernel (fused E.C^T + softcap + online log-sum-exp)",
            "bound": "mfma",
            "achieved": fwd_tflops,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": fwd_tflops / PEAK_BF16_TFLOPS,
            "ms_per_launch": fwd_ms,
            "traffic": args.traffic if args.traffic is not None else MEASURED_TRAFFIC_BYTES.get(w["name"]),
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
