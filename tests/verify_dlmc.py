#!/usr/bin/env python3
"""Oracle parity over a directory of real sparsity patterns (.smtx files, the format of the reference's dlmc/ tree).

    python tests/verify_dlmc.py <dir | pack.npz> [--batch-table rn50_batchsizes.txt | --n 256] [--d-sddmm 128] [--d-fused 64]
                                [--ops spmm,sddmm,fused] [--every 1] [--limit 0] [--report out.txt] [--all-schedules]
                                [--time]

For every file below <dir> (or every pattern of a pack written by tests/golden/dlmc/pack_patterns.py): the pattern is
uploaded, values and dense operands are drawn from a seed, each op runs on the GPU through the C ABI the way the C++
drivers call it (one look at the matrix, dlspm_analyze, then what dlspm_advise says: a row plan, a cut plan, workspace
memory, hints or NULL; --all-schedules runs every one of them that applies) and the
result is compared with the CPU oracle (oracle/, the reference's gold loops: SPMM/spmm-esimd-fromfile.cpp:63-83,
SDDMM/sddmm-esimd-fromfile.cpp:18-36, FUSED/fused.cpp:47-89): CSR arrays bit-identical after the call, values within
1e-4 relative Frobenius error. SpMM widths come from a "<layer name>,<batch size>" table where one is given (files whose
layer is not in it are skipped for SpMM, as in SPMM/batch-run-spmm_fromfile:16-46), else --n.

--time: every case is also timed (a HIP graph of 20 launches, replayed; median of 7) with NULL and with what the library
advised, and the geometric means per op are printed: the speed the one look at the matrix buys.

This is the wide net that the fixtures under tests/golden/dlmc/ are a sample of; it needs the dataset, which is not part
of this repository. Exit status 1 if any case fails.
"""
import argparse
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("dlspm-esimd_amd", "oracle"):
    sys.path.insert(0, os.path.join(ROOT, sub))

TOLERANCE = 1e-4


def load_smtx(path):
    """(M, K, row_offsets, col_indices) of an .smtx file: 'M, K, nnz', then the offsets, then the column indices."""
    with open(path) as f:
        head = f.readline().replace(",", " ").split()
        M, K, nnz = int(head[0]), int(head[1]), int(head[2])
        ro = np.array(f.readline().split(), dtype=np.int64)
        ci = np.array(f.read().split(), dtype=np.int64)  # (an empty matrix has no third line)
    if ro.size != M + 1 or ci.size != nnz or ro[0] != 0 or ro[-1] != nnz or (np.diff(ro) < 0).any():
        raise ValueError(f"{path}: not a CSR structure of {M} x {K} with {nnz} nonzeros")
    if nnz and (ci.min() < 0 or ci.max() >= K):
        raise ValueError(f"{path}: column index out of range")
    return M, K, ro.astype(np.int32), ci.astype(np.int32)


def prepared_name(dl, prep):
    cp = prep.call_plan
    if cp.build == dl.BUILD_CUT_PLAN:
        return "cut_plan"
    if cp.build == dl.BUILD_ROW_PLAN:
        return "row_plan_skewed" if cp.hints & dl.HINT_ROWS_SKEWED else "row_plan"
    if cp.hints & dl.HINT_BANDED:
        return "banded_hint"
    if cp.bytes:
        return "workspace"
    return "rows_even_hint" if cp.hints & dl.HINT_ROWS_EVEN else "rows_skewed_hint" if cp.hints & dl.HINT_ROWS_SKEWED else "null"


def schedules(dl, torch, op, M, K, N, nnz, ro_d, ci_d, every):
    """[(name, workspace, plan)]: what the drivers would pass (dlspm_analyze -> dlspm_advise), or every schedule that
    applies."""
    out = []
    need = dl.workspace_bytes(op, M, K, N, nnz)

    def memory():
        return torch.empty(need, dtype=torch.uint8, device="cuda")

    if every:
        out.append(("null", None, None))
        out.append(("rows_even_hint", dl.ROWS_EVEN, None))
        out.append(("rows_skewed_hint", dl.ROWS_SKEWED, None))
        if need:
            out.append(("workspace", memory(), None))
        if M > 0:
            out.append(("row_plan", None, dl.row_plan(ro_d)))
            if dl.row_plan_bytes_for(op, M, N) > 0:
                out.append(("cut_plan", None, dl.cut_plan(ro_d, op, N)))
        return out
    if M == 0:
        return [("null", None, None)]
    prep = dl.prepare(ro_d, ci_d, K, op, N)
    return [(prepared_name(dl, prep), None, prep)]


def graph_us(torch, step, launches=20, replays=7):
    """Microseconds per launch of step() inside a HIP graph of `launches` launches (median of `replays` double replays)."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())  # what was enqueued so far (a plan build, say) comes first
    with torch.cuda.stream(stream):
        for _ in range(3):
            step()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(launches):
                step()
        graph.replay()
        stream.synchronize()
        times = []
        for _ in range(replays):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            graph.replay()
            graph.replay()
            b.record(stream)
            stream.synchronize()
            times.append(a.elapsed_time(b) * 1e3 / (2 * launches))
    return sorted(times)[len(times) // 2]


def check_pattern(dl, torch, oracle, op, M, K, N, ro, ci, ro_d, ci_d, rng, all_schedules, timed=False):
    """Runs op on the pattern (ro, ci: numpy; ro_d, ci_d: the same on the GPU) with seeded operands under the schedules
    that apply and yields (schedule, relative Frobenius error against the oracle, CSR arrays intact, microseconds per
    launch or None, the same with NULL or None)."""
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    nnz = int(ci.size)
    if op == "spmm":
        code = dl.OP_SPMM
        values = rng.standard_normal(nnz, dtype=np.float32)
        B = rng.standard_normal((K, N), dtype=np.float32)
        want = oracle.spmm(ro, ci, values, B, omp=True)
        values_d, B_d = dev(values), dev(B)
        run = lambda ws, plan: dl.spmm(ro_d, ci_d, values_d, B_d, K=K, workspace=ws, plan=plan)
    elif op == "sddmm":
        code = dl.OP_SDDMM
        lhs = rng.standard_normal((M, N), dtype=np.float32)
        rhs = rng.standard_normal((K, N), dtype=np.float32)
        want = oracle.sddmm(ro, ci, lhs, rhs, omp=True)
        lhs_d, rhs_d = dev(lhs), dev(rhs)
        run = lambda ws, plan: dl.sddmm(ro_d, ci_d, lhs_d, rhs_d, workspace=ws, plan=plan)
    elif op == "fused":
        code = dl.OP_FUSED
        Q = rng.standard_normal((M, N), dtype=np.float32)
        Km = rng.standard_normal((K, N), dtype=np.float32)
        V = rng.standard_normal((K, N), dtype=np.float32)
        scale = float(1.0 / np.sqrt(N))
        want = oracle.fused(ro, ci, Q, Km, V, scale, omp=True)
        Q_d, Km_d, V_d = dev(Q), dev(Km), dev(V)
        run = lambda ws, plan: dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, scale, workspace=ws, plan=plan)
    else:
        raise ValueError(f"unknown op {op}")
    null_us = graph_us(torch, lambda: run(None, None)) if timed and nnz > 0 else None
    for schedule, ws, plan in schedules(dl, torch, code, M, K, N, nnz, ro_d, ci_d, all_schedules):
        got = run(ws, plan).cpu().numpy()
        err = oracle.rel_frobenius(got, want)
        intact = np.array_equal(ro_d.cpu().numpy(), ro) and np.array_equal(ci_d.cpu().numpy(), ci)
        us = None
        if null_us is not None:
            us = null_us if schedule == "null" else graph_us(torch, lambda: run(ws, plan))
        yield schedule, err, intact, us, null_us


class Tally:
    """Counts and prints the cases of one run."""

    def __init__(self, report_path):
        self.cases = self.failures = 0
        self.worst = {}
        self.by_schedule = {}
        self.times = {}  # (op, schedule) -> [(microseconds, microseconds with NULL)]
        self.report = open(report_path, "w") if report_path else None

    def add(self, op, schedule, what, err, intact, us=None, null_us=None):
        ok = bool(intact and err <= TOLERANCE)
        if us is not None:
            self.times.setdefault((op, schedule), []).append((us, null_us))
        self.cases += 1
        self.failures += 0 if ok else 1
        self.worst[op] = max(self.worst.get(op, 0.0), err)
        self.by_schedule[(op, schedule)] = self.by_schedule.get((op, schedule), 0) + 1
        line = f"{'PASS' if ok else 'FAIL'} {op} {schedule} {what} rel={err:.3e}{'' if intact else ' CSR arrays changed'}"
        if us is not None:
            line += f" us={us:.2f} null_us={null_us:.2f}"
        if self.report:
            self.report.write(line + "\n")
        if not ok:
            print(line, flush=True)

    def finish(self, name, what):
        if self.report:
            self.report.close()
        print(f"{self.cases} cases over {what}: {self.cases - self.failures} PASS, {self.failures} FAIL")
        print("largest relative Frobenius error per op: " + ", ".join(f"{op} {self.worst[op]:.3e}" for op in sorted(self.worst)))
        print("cases per (op, schedule): " + ", ".join(f"{op}/{s} {n}" for (op, s), n in sorted(self.by_schedule.items())))
        if self.times:
            geomean = lambda xs: float(np.exp(np.mean(np.log(np.maximum(xs, 1e-9)))))
            print("microseconds per launch inside a HIP graph, geometric means (as advised / with NULL / ratio / cases):")
            for op in sorted({o for o, _ in self.times}):
                rows = [t for (o, _), ts in self.times.items() if o == op for t in ts]
                a, n = geomean([t[0] for t in rows]), geomean([t[1] for t in rows])
                print(f"  {op}: {a:.2f} / {n:.2f} / {a / n:.3f} / {len(rows)}")
                for (o, sched), ts in sorted(self.times.items()):
                    if o == op:
                        a, n = geomean([t[0] for t in ts]), geomean([t[1] for t in ts])
                        print(f"    {sched}: {a:.2f} / {n:.2f} / {a / n:.3f} / {len(ts)}")
        ok = self.failures == 0 and self.cases > 0
        print(f"{name} " + ("PASS" if ok else "FAIL"))
        return 0 if ok else 1


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("dir")
    ap.add_argument("--batch-table", default=None, help="'<layer name>,<batch size>' lines: the SpMM width of each layer")
    ap.add_argument("--n", type=int, default=256, help="SpMM width without a table")
    ap.add_argument("--d-sddmm", type=int, default=128)
    ap.add_argument("--d-fused", type=int, default=64)
    ap.add_argument("--ops", default="spmm,sddmm,fused")
    ap.add_argument("--every", type=int, default=1, help="take every n-th file of the sorted list")
    ap.add_argument("--limit", type=int, default=0, help="stop after this many files (0: all)")
    ap.add_argument("--report", default=None, help="write one line per case to this file")
    ap.add_argument("--all-schedules", action="store_true")
    ap.add_argument("--time", action="store_true", help="also time every case against the call with NULL")
    args = ap.parse_args()

    import torch

    import dlspm_hip as dl
    import oracle

    if not torch.cuda.is_available():
        sys.exit("verify_dlmc.py needs the GPU (it checks the HIP kernels, not the oracle)")
    oracle.lib()
    table = None
    if args.batch_table:
        table = {}
        for line in open(args.batch_table):
            key, _, value = line.strip().partition(",")
            if key and value:
                table[key] = int(value)
    pack = None
    if os.path.isfile(args.dir) and args.dir.endswith(".npz"):
        pack = np.load(args.dir)
        files = [str(x) for x in pack["names"]]
    else:
        files = sorted(os.path.join(d, f) for d, _, fs in os.walk(args.dir) for f in fs if f.endswith(".smtx"))
    numbered = list(enumerate(files))[:: max(args.every, 1)]
    files = [f for _, f in numbered]
    if args.limit:
        files, numbered = files[: args.limit], numbered[: args.limit]
    ops = [o for o in args.ops.split(",") if o]
    tally = Tally(args.report)
    skipped = 0
    t0 = last = time.time()
    print(f"{len(files)} files below {args.dir}; ops {ops}; oracle on {oracle.omp_threads()} threads; {dl.version()}", flush=True)
    for index, (slot, path) in enumerate(numbered):
        if pack is not None:
            M, K = (int(x) for x in pack["shapes"][slot])
            ro, ci = pack[f"ro{slot}"].astype(np.int32), pack[f"ci{slot}"].astype(np.int32)
        else:
            M, K, ro, ci = load_smtx(path)
        name = os.path.basename(path)[: -len(".smtx")]
        rng = np.random.default_rng(index)
        ro_d, ci_d = torch.from_numpy(ro).cuda(), torch.from_numpy(ci).cuda()
        for op in ops:
            N = {"sddmm": args.d_sddmm, "fused": args.d_fused}.get(op)
            if op == "spmm":
                N = table.get(name) if table is not None else args.n
                if N is None:
                    skipped += 1
                    continue
            what = f"{path if pack is not None else os.path.relpath(path, args.dir)} M={M} K={K} nnz={ci.size} N={N}"
            for schedule, err, intact, us, null_us in check_pattern(dl, torch, oracle, op, M, K, N, ro, ci, ro_d, ci_d, rng,
                                                                    args.all_schedules, args.time):
                tally.add(op, schedule, what, err, intact, us, null_us)
        if time.time() - last > 30:
            last = time.time()
            print(f"  {index + 1}/{len(files)} files, {tally.cases} cases, {tally.failures} failures, {last - t0:.0f} s", flush=True)
    print(f"{time.time() - t0:.0f} s; {skipped} SpMM cases skipped (layer not in the table)")
    sys.exit(tally.finish("verify_dlmc", f"{len(files)} files"))


if __name__ == "__main__":
    main()
