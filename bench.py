#!/usr/bin/env python3
"""Benchmark of the sparse hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--replays R] [--no-graph] [--no-cpu] [--no-plan]
                    [--headline-only] [--no-cold] [--no-null]

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
  prepared          what the steps pass as (workspace, workspace_bytes): the answer of dlspm_advise to one look at the
                    matrix (dlspm_analyze), as the C++ drivers do -- a row plan for the uneven rows of the headline
                    (DLSPM_HINT_ROW_PLAN; built once per matrix, on the device, before the timed region),
                    DLSPM_HINT_ROWS_EVEN for the even rows of three others. `prepare_us` says what that costs once per
                    matrix (the synchronising analysis, on the host's clock, and the plan build, on the device's);
                    --no-plan measures the launches that pass NULL as the headline
  null_call_us      the same K-step graph with workspace = NULL, 0 (the plain drop-in call), beside launch_us
  host_enqueue_us   what one call costs the host outside a graph (200 calls issued without synchronising, wall time per
                    call): the plain call, the prepared call, and an empty kernel launch (the runtime's own share)
  launch_floor      measured in this run, between the nodes of a HIP graph like the ops: an empty kernel of 256 ...
                    8192 workgroups of 256 threads, and a kernel that only walks the dependent loads every row-block
                    kernel starts with (row offsets -> column indices -> one dense row -> one store) on the grid of the
                    headline's launch: what a launch costs the device before any arithmetic. `floor_us` of every
                    configuration is the empty kernel at that configuration's number of workgroups (interpolated)
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
    ap.add_argument("--no-cold", action="store_true", help="skip the cold-cache leg (kernel traces of the timed graph alone)")
    ap.add_argument("--no-null", action="store_true", help="skip the legs that time the plain call (NULL workspace) and the plan build")
    return ap.parse_args()


def median(xs):
    s = sorted(xs)
    return s[len(s) // 2]


def make_step(dl, torch, c, prepared=True, info=None):
    """Uploads configuration c and returns (step_fn, output tensor). What a caller does once per matrix happens here,
    outside the timed steps: one look at the matrix (dlspm_analyze), the library's answer for this op and width
    (dlspm_advise), and what that answer asks to allocate and build. prepared=False: the plain call, workspace = NULL."""
    d = lambda a: torch.from_numpy(a).cuda()
    ro, ci = d(c["row_offsets"]), d(c["col_indices"])
    prep = None
    if prepared:
        torch.cuda.synchronize()
        walls = []
        for _ in range(6):  # the first call of a process also loads the kernel: reported by itself
            t0 = time.perf_counter()
            mi = dl.analyze(ro, ci, c["K"])
            walls.append((time.perf_counter() - t0) * 1e6)
        prep = dl.prepare(ro, ci, c["K"], c["op"], c["N"], info=mi)
        if info is not None:
            info.update({"row_offsets": ro, "prepared": prep, "matrix_info": mi.as_dict(), "analyze_host_us": median(walls[1:]),
                         "analyze_first_call_us": walls[0]})
    if c["op"] == dl.OP_SPMM:
        va, B = d(c["values"]), d(c["d0"])
        out = torch.empty((c["M"], c["N"]), dtype=torch.float32, device="cuda")
        step = lambda: dl.spmm(ro, ci, va, B, K=c["K"], out=out, plan=prep)
        raw = ("spmm", (c["M"], c["K"], c["N"], c["nnz"], ro, ci, va, B, out))
    elif c["op"] == dl.OP_SDDMM:
        lhs, rhs = d(c["d0"]), d(c["d1"])
        out = torch.empty((c["nnz"],), dtype=torch.float32, device="cuda")
        step = lambda: dl.sddmm(ro, ci, lhs, rhs, out=out, plan=prep)
        raw = ("sddmm", (c["M"], c["K"], c["N"], c["nnz"], ro, ci, lhs, rhs, out))
    else:
        Q, Km, V = d(c["d0"]), d(c["d1"]), d(c["d2"])
        out = torch.empty((c["M"], c["N"]), dtype=torch.float32, device="cuda")
        step = lambda: dl.fused(ro, ci, Q, Km, V, c["scale"], out=out, plan=prep)
        raw = ("fused", (c["M"], c["K"], c["N"], c["nnz"], ro, ci, Q, Km, V, c["scale"], out))
    if info is not None:
        info["raw"] = raw
    return step, out


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
    stream.wait_stream(torch.cuda.current_stream())  # what was enqueued so far (uploads, a plan build) comes first
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
    stream.wait_stream(torch.cuda.current_stream())
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
        ci, sz, st = ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int)
        for name, args in (("spmm", [vp] * 5), ("sddmm", [vp] * 5), ("fused", [vp] * 5 + [ctypes.c_float, vp])):
            f = getattr(self.lib, "dlspm_probe_enqueue_" + name)
            f.restype = ctypes.c_double
            f.argtypes = [vp, ci, ci, ci, ci, ci] + args + [vp, sz, vp, st]
        self.lib.dlspm_probe_enqueue_empty.restype = ctypes.c_double
        self.lib.dlspm_probe_enqueue_empty.argtypes = [ci, vp]
        self.lib.dlspm_probe_floor.restype = ctypes.c_int
        self.lib.dlspm_probe_floor.argtypes = [ci, ci, ci, ci, vp, vp, vp, vp, vp]

    def launch_floor(self, dl, torch, c, use_graph=True, launches=200):
        """Microseconds per launch between the nodes of a graph of `launches`: the empty kernel against the number of
        workgroups, and the chain kernel (depth 0 ... 3) on configuration c's matrix at one workgroup per row."""
        ro, ci = torch.from_numpy(c["row_offsets"]).cuda(), torch.from_numpy(c["col_indices"]).cuda()
        B = torch.zeros((c["K"], 256), dtype=torch.float32, device="cuda")
        C = torch.empty((c["M"], 256), dtype=torch.float32, device="cuda")
        stream = torch.cuda.Stream()

        def timed(workgroups, depth):
            def one():
                st = self.lib.dlspm_probe_floor(workgroups, 256, depth, c["M"], ro.data_ptr(), ci.data_ptr(), B.data_ptr(),
                                                C.data_ptr(), torch.cuda.current_stream().cuda_stream)
                if st != 0:
                    raise RuntimeError(f"dlspm_probe_floor: hip error {st}")
            with torch.cuda.stream(stream):
                stream.wait_stream(torch.cuda.current_stream())
                for _ in range(3):
                    one()
                stream.synchronize()
                g = capture(torch, stream, lambda: [one() for _ in range(launches)]) if use_graph else None
                ev, _ = timed_replays(torch, stream, g.replay if g else (lambda: [one() for _ in range(launches)]), 7)
            return round(median(ev) / launches * 1e6, 2)

        grids = [256, 512, 1024, 2048, 4096, 8192]
        return {"what": f"us per launch between the nodes of a graph of {launches} (median of 7 replays); 256 threads per workgroup",
                "workgroups": grids, "empty_kernel_us": [timed(g, -1) for g in grids],
                "dependent_loads": {"matrix": c["name"], "workgroups": c["M"],
                                    "row_offsets_us": timed(c["M"], 0), "plus_column_indices_us": timed(c["M"], 1),
                                    "plus_one_dense_row_us": timed(c["M"], 2), "plus_store_us": timed(c["M"], 3)}}

    def host_enqueue_us(self, dl, torch, raw, prepared, calls=200, reps=5):
        """Host microseconds per call of the entry point, issued `calls` times without synchronising, outside a graph
        (median of `reps` such runs): the plain call (NULL, 0), the prepared call, and an empty kernel launch."""
        name, a = raw
        fn = ctypes.cast(getattr(dl.lib(), {"spmm": "spmm_csr_f32", "sddmm": "sddmm_csr_f32", "fused": "fused_sddmm_spmm_f32"}[name]),
                         ctypes.c_void_p)
        ptr = lambda t: t.data_ptr() if hasattr(t, "data_ptr") else t
        status = ctypes.c_int(0)
        run = getattr(self.lib, "dlspm_probe_enqueue_" + name)

        def one(ws, size):
            xs = []
            for _ in range(reps):
                torch.cuda.synchronize()
                xs.append(run(fn, calls, *[ptr(x) for x in a], ws, size, None, ctypes.byref(status)))
                torch.cuda.synchronize()
                if status.value != 0:
                    raise RuntimeError(f"{name}: status {status.value} in the host-enqueue leg")
            return round(median(xs), 2)

        def empty():
            xs = []
            for _ in range(reps):
                torch.cuda.synchronize()
                xs.append(self.lib.dlspm_probe_enqueue_empty(calls, None))
                torch.cuda.synchronize()
            return round(median(xs), 2)

        out = {"plain_call": one(None, 0), "empty_kernel_launch": empty(), "calls": calls}
        if prepared is not None:
            out["prepared_call"] = one(prepared.memory.data_ptr() if prepared.memory is not None else None, prepared.size_and_hints)
        return out

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


HINT_NAMES = (("HINT_ROW_PLAN", "DLSPM_HINT_ROW_PLAN"), ("HINT_CUT_PLAN", "DLSPM_HINT_CUT_PLAN"), ("HINT_ROWS_EVEN", "DLSPM_HINT_ROWS_EVEN"),
              ("HINT_BANDED", "DLSPM_HINT_BANDED"), ("HINT_ROWS_SKEWED", "DLSPM_HINT_ROWS_SKEWED"))


def launch_signature(dl, c, prep):
    """What identifies the launch a traffic figure was recorded for: op, lane layout, split and the hints passed."""
    sh = dl.describe_launch(c["op"], c["M"], c["K"], c["N"], c["nnz"], rows_even=bool(prep and prep.call_plan.hints & dl.HINT_ROWS_EVEN))
    hints = "+".join(n for a, n in HINT_NAMES if prep and prep.call_plan.hints & getattr(dl, a)) or "NULL"
    planned = bool(prep and prep.call_plan.build)
    return (f"{OP_NAMES[c['op']]}:vec{sh['vec']}:row-lanes{sh['G']}x{sh['V']}:dot-lanes{sh['G1']}x{sh['DS']}:"
            f"W{sh['W']}:R{1 if planned else sh['R']}:{hints}")


def floor_at(floor, workgroups):
    """The empty-kernel time of the floor table at `workgroups` (linear between its points, flat outside them)."""
    xs, ys = floor["workgroups"], floor["empty_kernel_us"]
    if workgroups <= xs[0]:
        return ys[0]
    for (x0, y0), (x1, y1) in zip(zip(xs, ys), zip(xs[1:], ys[1:])):
        if workgroups <= x1:
            return round(y0 + (y1 - y0) * (workgroups - x0) / (x1 - x0), 2)
    return ys[-1]


def measure(dl, torch, np, c, args, probe, steps, warmup, replays, ceiling_gbps, with_cpu, cpu_budget, floor=None):
    """Every figure of one configuration."""
    acct = dl.account(c["op"], c["M"], c["K"], c["N"], c["nnz"])
    info = {}
    step, out = make_step(dl, torch, c, not args.no_plan, info)
    prep = info.get("prepared")
    t = time_steps(torch, step, steps, warmup, replays, not args.no_graph, split_overhead=steps < 1000)
    s = t["per_step_s"]
    # HBM-side traffic: recorded by rocprofv3 --pmc runs (profiles/pmc_traffic.json), valid for the launch it names only
    traffic, traffic_source = None, None
    signature = launch_signature(dl, c, prep)
    pmc_path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    if os.path.exists(pmc_path):
        rec = json.load(open(pmc_path)).get(c["name"], {})
        if rec.get("launch") == signature:
            traffic = rec.get("traffic_bytes_per_launch")
            traffic_source = f"recorded@{rec.get('commit', '?')} for {rec.get('kernel', '?')}"
        elif rec:
            traffic_source = f"stale: recorded for {rec.get('launch', 'an unnamed launch')}, this run launches {signature}"
    eff_gbps = acct["effective_bytes"] / s / 1e9
    entry = ["spmm_csr_f32", "sddmm_csr_f32", "fused_sddmm_spmm_f32"][c["op"]]
    hints = [n for a, n in HINT_NAMES if prep and prep.call_plan.hints & getattr(dl, a)]
    r = {
        "workload": c["name"], "op": OP_NAMES[c["op"]], "entry_point": entry + "".join(" + " + h for h in hints),
        "M": c["M"], "K": c["K"], "N_or_D": c["N"], "nnz": c["nnz"], "steps": steps, "replays": replays,
        "launch_us": round(s * 1e6, 3), "replay_launch_us": t["all_us"], "host_wall_us_per_step": round(t["wall_per_step_s"] * 1e6, 3),
        "launch": t["mode"], "launch_signature": signature,
        "prepared": {"build": ["nothing", "dlspm_row_plan_build", "dlspm_row_plan_build_cut"][prep.call_plan.build],
                     "workspace_bytes": int(prep.call_plan.bytes), "hints": hints} if prep else None,
        "row_plan": bool(prep and prep.call_plan.build == dl.BUILD_ROW_PLAN),
        "rows_even_hint": bool(prep and prep.call_plan.hints & dl.HINT_ROWS_EVEN),
        "matrix_info": info.get("matrix_info"),
        "GFLOPs": round(acct["flops"] / s / 1e9, 2),
        "roofline": {"bound": "hbm", "achieved": round(acct["algorithmic_bytes"] / s / 1e9, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(acct["algorithmic_bytes"] / s / 1e9 / HBM_PEAK_GBPS, 5), "traffic": traffic,
                     "traffic_source": traffic_source,
                     "traffic_over_algorithmic": round(traffic / acct["algorithmic_bytes"], 2) if traffic else None,
                     "algorithmic_bytes": acct["algorithmic_bytes"], "launch_us": round(s * 1e6, 3)},
        "effective_GBps": round(eff_gbps, 1), "effective_fraction": round(eff_gbps / HBM_PEAK_GBPS, 4),
        "effective_bytes": acct["effective_bytes"],
        "frac_of_gather_ceiling": round(eff_gbps / ceiling_gbps, 3) if ceiling_gbps else None,
        "warm_us": round(s * 1e6, 3),
    }
    if floor is not None:
        # one workgroup per R rows and column tile (a row plan without grouping: one per row)
        shape = dl.describe_launch(c["op"], c["M"], c["K"], c["N"], c["nnz"], rows_even=r["rows_even_hint"])
        rows_each = 1 if prep and prep.call_plan.build else max(shape["R"], 1)
        r["workgroups"] = -(-c["M"] // rows_each) * max(shape["col_tiles"], 1)
        r["floor_us"] = floor_at(floor, r["workgroups"])
    if "steady_per_step_s" in t:
        r["steady_state_launch_us"] = round(t["steady_per_step_s"] * 1e6, 3)
        r["replay_overhead_us"] = round(t["replay_overhead_s"] * 1e6, 2)
    cold = cold_launch_us(torch, step) if not (args.no_graph or args.no_cold) else None
    r["cold_us"] = cold["us"] if cold else None
    r["cold_detail"] = cold
    if not args.no_null:
        # the plain drop-in call (workspace = NULL, 0) in the same kind of graph, and what the preparation costs once per matrix
        k = min(steps, 500)
        if prep is not None and (prep.memory is not None or prep.call_plan.hints):
            plain, _ = make_step(dl, torch, c, False)
            without = time_steps(torch, plain, k, min(warmup, 50), replays, not args.no_graph)
            r["null_call_us"] = round(without["per_step_s"] * 1e6, 3)
        else:
            r["null_call_us"] = r["launch_us"]  # nothing is passed: the timed launches are the plain call
        prepare = {"analyze_host_us": round(info.get("analyze_host_us", 0.0), 1),
                   "analyze_first_call_us": round(info.get("analyze_first_call_us", 0.0), 1),
                   "analyze": "dlspm_analyze: one pass over the CSR structure on the device, synchronises; host wall time, median of "
                              "five calls after the first (which may load the kernel)"}
        if prep is not None and prep.call_plan.build:
            ro, mem = info["row_offsets"], prep.memory
            build_fn = dl.lib().dlspm_row_plan_build if prep.call_plan.build == dl.BUILD_ROW_PLAN else dl.lib().dlspm_row_plan_build_cut
            M = c["M"]

            def build():
                st = build_fn(M, ctypes.c_void_p(ro.data_ptr()), ctypes.c_void_p(mem.data_ptr()), mem.numel() * 4,
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
                if st != 0:
                    raise RuntimeError(f"plan build: status {st}")

            built = time_steps(torch, build, 20, 3, 5, not args.no_graph)
            prepare["build_us"] = round(built["per_step_s"] * 1e6, 2)
            prepare["build"] = "kernels on the stream, no host copy, no synchronisation (capturable); HIP events, graph of 20 builds"
            gain = (r["null_call_us"] - r["launch_us"])
            prepare["launches_until_the_build_pays"] = round(prepare["build_us"] / gain, 1) if gain > 0 else None
            prepare["launches_until_analysis_and_build_pay"] = (round((prepare["build_us"] + prepare["analyze_host_us"]) / gain, 1)
                                                                if gain > 0 else None)
        r["prepare_us"] = prepare
        r["host_enqueue_us"] = probe.host_enqueue_us(dl, torch, info["raw"], prep)
    if r.get("row_plan") and "prepare_us" in r:
        r["row_plan_detail"] = {"build_us_once_per_matrix": r["prepare_us"].get("build_us"),
                                "build": "dlspm_row_plan_build: kernels on the stream, no host copy, no synchronisation",
                                "launch_us_without_plan": r["null_call_us"]}
    if with_cpu:
        r["cpu_baseline"], ref = cpu_baseline(dl, c, acct, *cpu_budget)
        torch.cuda.synchronize()
        step()
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
    floor = probe.launch_floor(dl, torch, c, not args.no_graph)
    head, acct = measure(dl, torch, np, c, args, probe, args.steps, args.warmup, replays, ceiling["value"], not args.no_cpu, (6.0, 3.0), floor)
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
        "launch_floor": floor,
        "warm_us": head["warm_us"], "cold_us": head["cold_us"], "cold_detail": head["cold_detail"],
        "cpu_baseline": head["cpu_baseline"],
    }
    if "rel_frobenius_vs_cpu" in head:
        result["rel_frobenius_vs_cpu"] = head["rel_frobenius_vs_cpu"]
    if "row_plan_detail" in head:
        result["row_plan"] = head["row_plan_detail"]
    for key in ("null_call_us", "prepare_us", "host_enqueue_us", "prepared", "matrix_info", "workgroups", "floor_us"):
        if key in head:
            result[key] = head[key]
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
            rr, _ = measure(dl, torch, np, cc, args, probe, k, min(args.warmup, 50), replays, ceiling["value"], not args.no_cpu, (2.5, 1.5), floor)
            others[cc["name"]] = {k2: v for k2, v in rr.items() if k2 not in ("replay_launch_us",)}
        result["all_configs"] = others

    result["pmc_calibration_copy"] = probe.calibration_copy(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
