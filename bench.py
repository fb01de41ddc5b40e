#!/usr/bin/env python3
"""Benchmark of the sparse hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--replays R] [--no-graph] [--no-cpu] [--no-plan]
                    [--headline-only]

A "step" is one launch of the configuration's kernel through the library's named entry point (default:
BASELINE.json's configs[1], fp32 CSR SpMM 2048x512 * 512x256 at 90 % sparsity with lognormal-skewed rows, through
spmm_csr_f32) on inputs that already sit in device memory. After W untimed steps, exactly K steps are captured in one
HIP graph and that graph is replayed R times back to back; every replay is bracketed by two HIP events recorded on
the launching stream (the device is synchronised before the first replay and after the last), and the MEDIAN replay
gives every figure of the line (one clock: value,
ms_per_step and roofline all come from the same event interval; the host's wall time around all replays, per
replay, is reported separately). R is 5 for K >= 1000 and grows for small K so that a 20-step run is not at the mercy of one
replay. --no-graph launches the K steps from the host instead (Python + ctypes per launch enter the figure then).
For K below 1000 a replay's own cost (its start and its drain, about 15 us) is a visible share of K launches of 6 us:
`timing.steady_state_launch_us` then gives the time per launch between a graph of 2 K and a graph of K steps, and
`timing.replay_overhead_us` what is left per replay; `value` and `ms_per_step` stay those of the K-step replay.

Prints ONE JSON line:
  value / unit      GFLOP/s with the reference's flop formula (2*nnz - M)*N  (SPMM/spmm-esimd-fromfile2.cpp:253)
  roofline          algorithmic bytes (every operand once) / median launch duration, against 8 TB/s HBM; `traffic` =
                    HBM-side bytes per launch from the rocprofv3 --pmc runs recorded in profiles/pmc_traffic.json
  effective_GBps    the reference's "application bandwidth" convention (every gathered dense row counted,
                    SDDMM/sddmm-esimd-v1.cpp:190), and its fraction of 8 TB/s -- never used as roofline.achieved
  gather_ceiling    measured in this run: what the device delivers for whole-wave 1 KiB row gathers from an L2-resident
                    table (the access pattern of these kernels), and each configuration's effective GB/s as a fraction
  cpu_baseline      the CPU oracle (a port of the reference's scalar loop) timed on this host, 1 core, and the same
                    loop over all cores; one per configuration in all_configs
  warm_us / cold_us per-launch time back to back (the graph above) and with the caches flushed before every launch:
                    [1 GiB fill -> launch] pairs replayed from one graph, minus the same graph without the launches
  row_plan          (uneven rows) the steps pass the row plan as their workspace (DLSPM_HINT_ROW_PLAN); the plan is built
                    once per matrix, on the device, before the timed region; this object gives what building it costs
                    and the time of the same launches in matrix order (--no-plan measures those as the headline)
  rows_even_hint    (per configuration) the steps pass DLSPM_HINT_ROWS_EVEN: dlspm_workspace_advice said so for the
                    longest row that one look at the row lengths found (dlspm_csr_row_stats), as the C++ drivers do
  all_configs       the same measurement for every benchmark configuration (shorter runs)
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "dlspm-esimd_amd"))

HBM_PEAK_GBPS = 8000.0
OP_NAMES = ["spmm", "sddmm", "fused"]


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (default 2, the headline)")
    ap.add_argument("--replays", type=int, default=0, help="replays of the K-step graph (default: 5, more for small K)")
    ap.add_argument("--no-graph", action="store_true", help="launch every step from the host instead of one HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-plan", action="store_true", help="launch in matrix order, without the row plan")
    ap.add_argument("--headline-only", action="store_true", help="skip the other four configurations")
    return ap.parse_args()


def median(xs):
    s = sorted(xs)
    return s[len(s) // 2]


def make_step(dl, torch, c, use_plan=True, info=None):
    """Uploads configuration c and returns (step_fn, output tensor). What a caller does once per matrix happens here,
    outside the timed steps: one look at the row lengths and, on uneven rows, the row plan (built on the device)."""
    d = lambda a: torch.from_numpy(a).cuda()
    ro, ci = d(c["row_offsets"]), d(c["col_indices"])
    need = dl.workspace_bytes(c["op"], c["M"], c["K"], c["N"], c["nnz"])  # 0 at the sizes of the five configurations
    ws = torch.empty(need, dtype=torch.uint8, device="cuda") if need else None
    longest, _ = dl.csr_row_stats(ro)
    if not need and dl.workspace_advice(c["op"], c["M"], c["K"], c["N"], c["nnz"], longest) == dl.PASS_ROWS_EVEN:
        ws = dl.ROWS_EVEN  # no memory: the hint that no row is much longer than the mean (cfg1, cfg3, cfg4)
        if info is not None:
            info["rows_even"] = True
    plan = None
    if use_plan and dl.row_plan_advice(c["op"], c["M"], c["K"], c["N"], c["nnz"], longest):
        plan = dl.row_plan(ro)
        ws = None
        if info is not None:
            info["row_offsets"] = ro
            info["plan"] = plan
    if c["op"] == dl.OP_SPMM:
        va, B = d(c["values"]), d(c["d0"])
        out = torch.empty((c["M"], c["N"]), dtype=torch.float32, device="cuda")
        return (lambda: dl.spmm(ro, ci, va, B, K=c["K"], out=out, workspace=ws, plan=plan)), out
    if c["op"] == dl.OP_SDDMM:
        lhs, rhs = d(c["d0"]), d(c["d1"])
        out = torch.empty((c["nnz"],), dtype=torch.float32, device="cuda")
        return (lambda: dl.sddmm(ro, ci, lhs, rhs, out=out, workspace=ws, plan=plan)), out
    Q, Km, V = d(c["d0"]), d(c["d1"]), d(c["d2"])
    out = torch.empty((c["M"], c["N"]), dtype=torch.float32, device="cuda")
    return (lambda: dl.fused(ro, ci, Q, Km, V, c["scale"], out=out, workspace=ws, plan=plan)), out


def capture(torch, stream, body):
    """A HIP graph of body(), captured on `stream` (None if the capture is refused)."""
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            body()
        graph.replay()  # one untimed replay: first-use setup of the graph
        stream.synchronize()
        return graph
    except Exception as e:  # capture refused: the caller falls back to host launches, and says so
        print(f"[bench] HIP graph capture failed ({e}); launching from the host", file=sys.stderr)
        return None


def timed_replays(torch, stream, run, replays):
    """`replays` executions of run(), enqueued back to back on `stream`, each between its own pair of HIP events; the
    device is synchronised before the first and after the last, so a replay starts on a device that is at work, as
    every launch but the first of a long run does: ([event seconds per replay], [host wall seconds / replays] * replays)."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(replays)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(replays)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(replays):
        starts[i].record(stream)
        run()
        ends[i].record(stream)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / replays
    return [starts[i].elapsed_time(ends[i]) * 1e-3 for i in range(replays)], [wall] * replays


def time_steps(torch, step, steps, warmup, replays, use_graph, split_overhead=False):
    """{'per_step_s' (median replay), 'wall_per_step_s' (same replay), 'all_us' per replay, 'mode'} for K = `steps`.
    split_overhead (graph mode, small K): a graph of 2 K steps is timed the same way, and the difference of the two
    medians is K steps without what one replay costs by itself ('steady_per_step_s', 'replay_overhead_s'): reported
    beside the K-step figure, never instead of it."""
    stream = torch.cuda.Stream()
    extra = {}
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            step()
        stream.synchronize()
        graph = capture(torch, stream, lambda: [step() for _ in range(steps)]) if use_graph else None
        run = graph.replay if graph is not None else (lambda: [step() for _ in range(steps)])
        ev, wall = timed_replays(torch, stream, run, replays)
        if split_overhead and graph is not None:
            twice = capture(torch, stream, lambda: [step() for _ in range(2 * steps)])
            if twice is not None:
                ev2, _ = timed_replays(torch, stream, twice.replay, replays)
                m1, m2 = sorted(ev)[replays // 2], sorted(ev2)[replays // 2]
                extra = {"steady_per_step_s": (m2 - m1) / steps, "replay_overhead_s": 2 * m1 - m2}
    order = sorted(range(replays), key=lambda i: ev[i])
    mid = order[replays // 2]
    return {"per_step_s": ev[mid] / steps, "wall_per_step_s": wall[mid] / steps,
            "all_us": [round(x / steps * 1e6, 3) for x in ev], "mode": "hipgraph" if graph is not None else "host", **extra}


def cold_launch_us(torch, step, pairs=24, replays=5):
    """Per-launch time with the caches flushed before every launch: a graph of `pairs` [1 GiB fill -> launch] pairs minus
    the graph of the fills alone, both replayed `replays` times (medians). The fill is a kernel (a captured memset
    node would not do), and 1 GiB is four times the 256 MiB Infinity Cache."""
    scratch = torch.empty(256 * 1024 * 1024, dtype=torch.float32, device="cuda")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        scratch.fill_(0.0)
        step()
        stream.synchronize()

        def both():
            for i in range(pairs):
                scratch.fill_(float(i))
                step()

        def fills():
            for i in range(pairs):
                scratch.fill_(float(i))

        g_both, g_fill = capture(torch, stream, both), capture(torch, stream, fills)
        if g_both is None or g_fill is None:
            return None
        t_both, _ = timed_replays(torch, stream, g_both.replay, replays)
        t_fill, _ = timed_replays(torch, stream, g_fill.replay, replays)
    del scratch
    return {"us": round((median(t_both) - median(t_fill)) / pairs * 1e6, 2), "pairs": pairs, "replays": replays,
            "flush_us": round(median(t_fill) / pairs * 1e6, 1)}


def cpu_baseline(dl, c, acct, budget_1core_s, budget_all_s):
    """The oracle's scalar loop (a port of the reference's CPU path) on this host: min of the runs that fit the budget
    (at least 3), on one core and, beside it, over all cores. Returns (object for the JSON line, the oracle's result)."""
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

    t1, r1 = best(False, budget_1core_s, 50)
    tn, rn = best(True, budget_all_s, 50)
    return {
        "value": round(acct["flops"] / t1 / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
        "sample": f"the full {c['name']} workload, min of {r1} runs of oracle_{OP_NAMES[c['op']]}_f32",
        "ms": round(t1 * 1e3, 3),
        "all_cores": {"value": round(acct["flops"] / tn / 1e9, 3), "cores": oracle.omp_threads(), "ms": round(tn * 1e3, 3),
                      "runs": rn},
    }, run(True)


class Probe:
    """libdlspm_probe.so: the gather-ceiling kernel and the plain copy that calibrates the rocprofv3 byte counters."""

    def __init__(self):
        path = os.path.join(ROOT, "dlspm-esimd_amd", "libdlspm_probe.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is missing: build it with `make -C dlspm-esimd_amd probe`")
        self.lib = ctypes.CDLL(path)
        vp = ctypes.c_void_p
        self.lib.dlspm_probe_gather.argtypes = [vp, ctypes.c_uint, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
        self.lib.dlspm_probe_gather.restype = ctypes.c_int
        self.lib.dlspm_probe_copy.argtypes = [vp, vp, ctypes.c_size_t, vp]
        self.lib.dlspm_probe_copy.restype = ctypes.c_int

    def gather_ceiling(self, torch, use_graph=True):
        """TB/s of whole-wave 1 KiB row gathers: random rows of a 512 KiB table (fits every L2: the ceiling the
        configurations are held against), random rows of an 8 MiB table (beyond one L2), consecutive rows."""
        table = torch.rand(8192 * 256, dtype=torch.float32, device="cuda")
        sink = torch.zeros(4, dtype=torch.float32, device="cuda")
        blocks, iters, launches = 1024, 64, 12
        bytes_per_launch = blocks * 4 * iters * 8 * 1024
        stream = torch.cuda.Stream()
        out = {"what": "whole-wave 1 KiB row gathers, 8 rows in flight per wave, 4096 waves x 64 rounds = 2.15 GB per launch; "
                       f"best of 5 replays of a graph of {launches} launches (a ceiling: the most the device was seen to deliver)",
               "unit": "GB/s"}
        with torch.cuda.stream(stream):
            for name, mask, rnd in (("l2_random_rows", 511, 1), ("beyond_l2_random_rows", 8191, 1), ("l2_consecutive_rows", 511, 0)):
                def one():
                    st = self.lib.dlspm_probe_gather(table.data_ptr(), mask, iters, rnd, blocks, sink.data_ptr(),
                                                     torch.cuda.current_stream().cuda_stream)
                    if st != 0:
                        raise RuntimeError(f"dlspm_probe_gather: hip error {st}")
                for _ in range(3):
                    one()
                stream.synchronize()
                g = capture(torch, stream, lambda: [one() for _ in range(launches)]) if use_graph else None
                ev, _ = timed_replays(torch, stream, g.replay if g else (lambda: [one() for _ in range(launches)]), 5)
                out[name] = round(bytes_per_launch / (min(ev) / launches) / 1e9, 1)
        out["value"] = out["l2_random_rows"]
        return out

    def calibration_copy(self, torch, reps=3):
        """A few launches of the 256 MiB copy kernel (dlspm_probe_copy_kernel): reads 256 MiB, writes 256 MiB."""
        n = 64 * 1024 * 1024
        src = torch.ones(n, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(reps):
            st = self.lib.dlspm_probe_copy(src.data_ptr(), dst.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
            if st != 0:
                raise RuntimeError(f"dlspm_probe_copy: hip error {st}")
        torch.cuda.synchronize()
        return {"kernel": "dlspm_probe_copy_kernel", "launches": reps, "bytes_read": n * 4, "bytes_written": n * 4}


def measure(dl, torch, np, c, args, steps, warmup, replays, ceiling_gbps, with_cpu, cpu_budget):
    """Every figure of one configuration."""
    acct = dl.account(c["op"], c["M"], c["K"], c["N"], c["nnz"])
    info = {}
    step, out = make_step(dl, torch, c, not args.no_plan, info)
    t = time_steps(torch, step, steps, warmup, replays, not args.no_graph, split_overhead=steps < 1000)
    s = t["per_step_s"]
    traffic = None
    pmc_path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    if os.path.exists(pmc_path):
        traffic = json.load(open(pmc_path)).get(c["name"], {}).get("traffic_bytes_per_launch")
    eff_gbps = acct["effective_bytes"] / s / 1e9
    r = {
        "workload": c["name"], "op": OP_NAMES[c["op"]], "entry_point": ["spmm_csr_f32", "sddmm_csr_f32", "fused_sddmm_spmm_f32"][c["op"]],
        "M": c["M"], "K": c["K"], "N_or_D": c["N"], "nnz": c["nnz"], "steps": steps, "replays": replays,
        "launch_us": round(s * 1e6, 3), "replay_launch_us": t["all_us"], "host_wall_us_per_step": round(t["wall_per_step_s"] * 1e6, 3),
        "launch": t["mode"], "row_plan": "plan" in info, "rows_even_hint": "rows_even" in info,
        "GFLOPs": round(acct["flops"] / s / 1e9, 2),
        "roofline": {"bound": "hbm", "achieved": round(acct["algorithmic_bytes"] / s / 1e9, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(acct["algorithmic_bytes"] / s / 1e9 / HBM_PEAK_GBPS, 5), "traffic": traffic,
                     "traffic_over_algorithmic": round(traffic / acct["algorithmic_bytes"], 2) if traffic else None,
                     "algorithmic_bytes": acct["algorithmic_bytes"], "launch_us": round(s * 1e6, 3)},
        "effective_GBps": round(eff_gbps, 1), "effective_fraction": round(eff_gbps / HBM_PEAK_GBPS, 4),
        "effective_bytes": acct["effective_bytes"],
        "frac_of_gather_ceiling": round(eff_gbps / ceiling_gbps, 3) if ceiling_gbps else None,
        "warm_us": round(s * 1e6, 3),
    }
    if "steady_per_step_s" in t:
        r["steady_state_launch_us"] = round(t["steady_per_step_s"] * 1e6, 3)
        r["replay_overhead_us"] = round(t["replay_overhead_s"] * 1e6, 2)
    cold = cold_launch_us(torch, step) if not args.no_graph else None
    r["cold_us"] = cold["us"] if cold else None
    r["cold_detail"] = cold
    if "plan" in info:
        # what the plan costs once per matrix (kernels on the stream, no synchronisation), and the same launches without it
        ro, plan = info["row_offsets"], info["plan"]
        build = time_steps(torch, lambda: dl.row_plan(ro, out=plan), 20, 3, 5, not args.no_graph)
        plain, _ = make_step(dl, torch, c, False)
        k = min(steps, 500)
        without = time_steps(torch, plain, k, min(warmup, 50), replays, not args.no_graph)
        r["row_plan_detail"] = {"build_us_once_per_matrix": round(build["per_step_s"] * 1e6, 2),
                                "build": "dlspm_row_plan_build: kernels on the stream, no host copy, no synchronisation",
                                "launch_us_without_plan": round(without["per_step_s"] * 1e6, 3)}
    if with_cpu:
        r["cpu_baseline"], ref = cpu_baseline(dl, c, acct, *cpu_budget)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        num = float(np.linalg.norm(got.astype(np.float64).ravel() - ref.astype(np.float64).ravel()))
        den = float(np.linalg.norm(ref.astype(np.float64).ravel()))
        r["rel_frobenius_vs_cpu"] = float(f"{num / den:.3e}")
    else:
        r["cpu_baseline"] = None
    return r, acct


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
    probe = Probe()
    replays = args.replays if args.replays > 0 else (5 if args.steps >= 1000 else min(101, max(5, -(-4000 // args.steps)) | 1))

    ceiling = probe.gather_ceiling(torch, not args.no_graph)
    c = dl.make_config(args.config)
    head, acct = measure(dl, torch, np, c, args, args.steps, args.warmup, replays, ceiling["value"], not args.no_cpu, (6.0, 3.0))
    s = head["launch_us"] * 1e-6

    result = {
        "metric": "fp32 CSR SpMM GFLOP/s (reference flop formula) + effective GB/s vs 8 TB/s HBM, 1xMI355X"
        if c["op"] == dl.OP_SPMM else f"fp32 {OP_NAMES[c['op']]} GFLOP/s, 1xMI355X",
        "value": head["GFLOPs"], "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(s * 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded generator, seed 1000+cfg)",
        "config": {"workload": c["name"], "op": head["op"], "entry_point": head["entry_point"], "M": c["M"], "K": c["K"],
                   "N_or_D": c["N"], "nnz": c["nnz"], "launch": head["launch"], "row_plan": head["row_plan"]},
        "timing": {"clock": "HIP events on the launching stream around each replay of the K-step graph; median replay",
                   "replays": replays, "replay_launch_us": head["replay_launch_us"],
                   "host_wall_ms_per_step": round(head["host_wall_us_per_step"] * 1e-3, 6),
                   # small K only: what one replay costs beside its K launches (graph of 2 K steps minus graph of K steps)
                   "steady_state_launch_us": head.get("steady_state_launch_us"),
                   "replay_overhead_us": head.get("replay_overhead_us")},
        "roofline": head["roofline"],
        "effective_GBps": head["effective_GBps"], "effective_fraction": head["effective_fraction"],
        "effective_bytes": head["effective_bytes"],
        "gather_ceiling": ceiling, "frac_of_gather_ceiling": head["frac_of_gather_ceiling"],
        "warm_us": head["warm_us"], "cold_us": head["cold_us"], "cold_detail": head["cold_detail"],
        "cpu_baseline": head["cpu_baseline"],
    }
    if "rel_frobenius_vs_cpu" in head:
        result["rel_frobenius_vs_cpu"] = head["rel_frobenius_vs_cpu"]
    if "row_plan_detail" in head:
        result["row_plan"] = head["row_plan_detail"]
    info = dl.device_info()
    result["device"] = {"compute_units": info["compute_units"], "l2_bytes": info["l2_bytes"], "name": torch.cuda.get_device_name(0)}

    if not args.headline_only:
        others = {}
        for cfg in range(1, 6):
            if cfg == args.config:
                others[c["name"]] = {k: v for k, v in head.items() if k not in ("replay_launch_us",)}
                continue
            cc = dl.make_config(cfg)
            k = min(args.steps, 500)
            rr, _ = measure(dl, torch, np, cc, args, k, min(args.warmup, 50), replays, ceiling["value"], not args.no_cpu, (2.5, 1.5))
            others[cc["name"]] = {k2: v for k2, v in rr.items() if k2 not in ("replay_launch_us",)}
        result["all_configs"] = others

    result["pmc_calibration_copy"] = probe.calibration_copy(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
