#!/usr/bin/env python3
"""Benchmark of the sparse hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-graph] [--no-cpu] [--no-plan] [--all-configs]

A "step" is one launch of the configuration's kernel (default: BASELINE.json's configs[1], fp32 CSR SpMM
2048x512 * 512x256 at 90 % sparsity with lognormal-skewed rows) on inputs that already sit in device memory.
After W untimed steps, exactly K steps are timed between two device synchronisations and between two HIP
events recorded on the launching stream; the K launches are replayed from one HIP graph so that the host's
per-launch cost (Python + ctypes) does not enter the figure (--no-graph launches them one by one instead).
Prints ONE JSON line:
  value / unit      GFLOP/s with the reference's flop formula (2*nnz - M)*N  (SPMM/spmm-esimd-fromfile2.cpp:253)
  roofline          algorithmic bytes (every operand once) / average launch duration, against 8 TB/s HBM
  effective_GBps    the reference's "application bandwidth" convention (every gathered dense row counted,
                    SDDMM/sddmm-esimd-v1.cpp:190), and its fraction of 8 TB/s -- never used as roofline.achieved
  cpu_baseline      the CPU oracle (a port of the reference's scalar loop) timed on this host, 1 core, and the
                    same loop over all cores for reference
  cold_us/warm_us   single launches timed with events after flushing the caches with a 1 GiB fill / back to back
  row_plan          (SpMM on uneven rows) the steps are spmm_csr_f32_planned launches; the plan is built once per matrix
                    before the timed region, like the look at the row lengths; this object gives what building it cost
                    and the time of the same launches in matrix order (--no-plan measures those as the headline)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "dlspm-esimd_amd"))

HBM_PEAK_GBPS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (default 2, the headline)")
    ap.add_argument("--no-graph", action="store_true", help="launch every step from the host instead of one HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-plan", action="store_true", help="SpMM: launch in matrix order, without the row plan")
    ap.add_argument("--all-configs", action="store_true", help="also time the other four configurations (short runs)")
    ap.add_argument("--pmc-calib", action="store_true",
                    help="also run a plain 256 MiB device copy a few times: the known-size kernel that rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings are scaled by")
    return ap.parse_args()


def make_step(dl, torch, c, use_plan=True, info=None):
    """Uploads configuration c and returns (step_fn, output tensor). What a caller does once per matrix happens here,
    outside the timed steps: one look at the row lengths and, for SpMM on uneven rows, the row plan (its build time
    goes to info["plan_build_ms"])."""
    d = lambda a: torch.from_numpy(a).cuda()
    ro, ci = d(c["row_offsets"]), d(c["col_indices"])
    # the caller owns the workspace; the library asks for none at the sizes of the five configurations
    need = dl.workspace_bytes(c["op"], c["M"], c["K"], c["N"], c["nnz"])
    ws = torch.empty(need, dtype=torch.uint8, device="cuda") if need else None
    if c["op"] == dl.OP_SPMM:
        va, B = d(c["values"]), d(c["d0"])
        out = torch.empty((c["M"], c["N"]), dtype=torch.float32, device="cuda")
        longest, _ = dl.csr_row_stats(ro)
        if use_plan and dl.row_plan_advice(c["op"], c["M"], c["K"], c["N"], c["nnz"], longest):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            plan = dl.row_plan(ro)
            if info is not None:
                info["plan_build_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
            return (lambda: dl.spmm(ro, ci, va, B, K=c["K"], out=out, plan=plan)), out
        return (lambda: dl.spmm(ro, ci, va, B, K=c["K"], out=out, workspace=ws)), out
    if c["op"] == dl.OP_SDDMM:
        lhs, rhs = d(c["d0"]), d(c["d1"])
        out = torch.empty((c["nnz"],), dtype=torch.float32, device="cuda")
        return (lambda: dl.sddmm(ro, ci, lhs, rhs, out=out)), out
    Q, Km, V = d(c["d0"]), d(c["d1"]), d(c["d2"])
    out = torch.empty((c["M"], c["N"]), dtype=torch.float32, device="cuda")
    return (lambda: dl.fused(ro, ci, Q, Km, V, c["scale"], out=out, workspace=ws)), out


def time_steps(torch, step, steps, warmup, use_graph):
    """(seconds between the synchronisations, seconds between the HIP events, launch mode) for `steps` steps."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            step()
        stream.synchronize()
        graph = None
        if use_graph:
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    for _ in range(steps):
                        step()
                graph.replay()  # one untimed replay: first-use setup of the graph
                stream.synchronize()
            except Exception as e:  # capture refused: fall back to host launches, and say so
                print(f"[bench] HIP graph capture failed ({e}); launching from the host", file=sys.stderr)
                graph = None
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        if graph is not None:
            graph.replay()
        else:
            for _ in range(steps):
                step()
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    return t1 - t0, e0.elapsed_time(e1) * 1e-3, ("hipgraph" if graph is not None else "host")


def single_launch_us(torch, step, reps, flush):
    """Median / min duration (us) of single launches bracketed by events, optionally after a cache flush."""
    scratch = torch.empty(256 * 1024 * 1024, dtype=torch.float32, device="cuda") if flush else None  # 1 GiB
    ts = []
    for _ in range(reps):
        if flush:
            scratch.fill_(1.0)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        step()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e3)
    ts.sort()
    return ts[len(ts) // 2], ts[0]


def cpu_baseline(dl, c, acct):
    """The oracle's scalar loop (a port of the reference's CPU path) on this host: min of `reps` runs."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle

    def run(omp):
        if c["op"] == dl.OP_SPMM:
            return oracle.spmm(c["row_offsets"], c["col_indices"], c["values"], c["d0"], omp=omp)
        if c["op"] == dl.OP_SDDMM:
            return oracle.sddmm(c["row_offsets"], c["col_indices"], c["d0"], c["d1"], omp=omp)
        return oracle.fused(c["row_offsets"], c["col_indices"], c["d0"], c["d1"], c["d2"], c["scale"], omp=omp)

    def best(omp, budget_s, max_reps):
        t_best, reps, t_all = float("inf"), 0, time.perf_counter()
        while reps < max_reps and (reps < 3 or time.perf_counter() - t_all < budget_s):
            t0 = time.perf_counter()
            run(omp)
            t_best = min(t_best, time.perf_counter() - t0)
            reps += 1
        return t_best, reps

    t1, r1 = best(False, 10.0, 50)
    tn, rn = best(True, 4.0, 50)
    return {
        "value": round(acct["flops"] / t1 / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
        "sample": f"the full {c['name']} workload, min of {r1} runs of oracle_{['spmm_f32', 'sddmm_f32', 'fused_f32'][c['op']]}",
        "ms": round(t1 * 1e3, 3),
        "all_cores": {"value": round(acct["flops"] / tn / 1e9, 3), "cores": oracle.omp_threads(), "ms": round(tn * 1e3, 3),
                      "runs": rn},
    }, run(True)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (output rows are independent, so sharding "
              "would split the rows and replicate the dense operand, with no exchange). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    import dlspm_hip as dl

    if not torch.cuda.is_available():
        print("bench.py needs the MI355X (no CPU fallback exists)", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    dl.lib()

    c = dl.make_config(args.config)
    acct = dl.account(c["op"], c["M"], c["K"], c["N"], c["nnz"])
    info = {}
    step, out = make_step(dl, torch, c, not args.no_plan, info)
    wall_s, evt_s, mode = time_steps(torch, step, args.steps, args.warmup, not args.no_graph)
    per_launch_s = evt_s / args.steps
    warm_med, warm_min = single_launch_us(torch, step, 30, flush=False)
    cold_med, cold_min = single_launch_us(torch, step, 15, flush=True)

    traffic = None
    pmc_path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    if os.path.exists(pmc_path):
        traffic = json.load(open(pmc_path)).get(c["name"], {}).get("traffic_bytes_per_launch")

    result = {
        "metric": "fp32 CSR SpMM GFLOP/s (reference flop formula) + effective GB/s vs 8 TB/s HBM, 1xMI355X"
        if c["op"] == dl.OP_SPMM else f"fp32 {['spmm', 'sddmm', 'fused sddmm->spmm'][c['op']]} GFLOP/s, 1xMI355X",
        "value": round(acct["flops"] / (wall_s / args.steps) / 1e9, 2),
        "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_s / args.steps * 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded generator, seed 1000+cfg)",
        "config": {"workload": c["name"], "op": ["spmm", "sddmm", "fused"][c["op"]], "M": c["M"], "K": c["K"],
                   "N_or_D": c["N"], "nnz": c["nnz"], "launch": mode, "row_plan": "plan_build_ms" in info},
        "roofline": {"bound": "hbm", "achieved": round(acct["algorithmic_bytes"] / per_launch_s / 1e9, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(acct["algorithmic_bytes"] / per_launch_s / 1e9 / HBM_PEAK_GBPS, 5),
                     "traffic": traffic, "algorithmic_bytes": acct["algorithmic_bytes"],
                     "launch_us": round(per_launch_s * 1e6, 3)},
        "effective_GBps": round(acct["effective_bytes"] / per_launch_s / 1e9, 1),
        "effective_fraction": round(acct["effective_bytes"] / per_launch_s / 1e9 / HBM_PEAK_GBPS, 4),
        "effective_bytes": acct["effective_bytes"],
        "warm_us": {"median": round(warm_med, 2), "min": round(warm_min, 2)},
        "cold_us": {"median": round(cold_med, 2), "min": round(cold_min, 2)},
    }

    if "plan_build_ms" in info:
        # the same launches in matrix order (no plan), and what the plan cost once
        plain, _ = make_step(dl, torch, c, False)
        _, ev, _ = time_steps(torch, plain, min(args.steps, 500), min(args.warmup, 50), not args.no_graph)
        result["row_plan"] = {"build_ms_once_per_matrix": info["plan_build_ms"],
                              "launch_us_without_plan": round(ev / min(args.steps, 500) * 1e6, 3)}

    if not args.no_cpu:
        result["cpu_baseline"], ref = cpu_baseline(dl, c, acct)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        num = float(np.linalg.norm(got.astype(np.float64).ravel() - ref.astype(np.float64).ravel()))
        den = float(np.linalg.norm(ref.astype(np.float64).ravel()))
        result["rel_frobenius_vs_cpu"] = float(f"{num / den:.3e}")
    else:
        result["cpu_baseline"] = None

    if args.pmc_calib:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")  # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        result["pmc_calib"] = {"kernel": "torch elementwise copy", "bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4}

    if args.all_configs:
        others = {}
        for cfg in range(1, 6):
            cc = dl.make_config(cfg)
            a = dl.account(cc["op"], cc["M"], cc["K"], cc["N"], cc["nnz"])
            st, _ = make_step(dl, torch, cc)
            _, ev, _ = time_steps(torch, st, 500, 50, not args.no_graph)
            t = ev / 500
            others[cc["name"]] = {"launch_us": round(t * 1e6, 3), "GFLOPs": round(a["flops"] / t / 1e9, 1),
                                  "effective_GBps": round(a["effective_bytes"] / t / 1e9, 1),
                                  "algorithmic_GBps": round(a["algorithmic_bytes"] / t / 1e9, 1)}
        result["all_configs"] = others

    print(json.dumps(result))


if __name__ == "__main__":
    main()
