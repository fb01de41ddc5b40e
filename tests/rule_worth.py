#!/usr/bin/env python3
"""What each launch rule of libdlspm_hip is worth today: every rule is switched off in turn through dlspm_set_tuning and
the same launches are timed again.

    python tests/rule_worth.py [--ops spmm,sddmm,fused] [--quick] [--out table.txt] [--cases cases.txt]

Cases: the five benchmark configurations; the reference's 12-shape benchmark grid (SPMM/spmm-esimd-allbenchs.cpp:252-255)
at density 0.1 with N = D = 32 and 128 (Bernoulli patterns); lognormal row lengths (sigma 1) on 2048 ... 16384 rows; layer
widths between the powers of two (80, 160, 320; SDDMM and the fused op); layer shapes of 64 ... 512 rows as in the reference's dlmc/ tree, three of them under dense rows of 640 ... 3136 floats (SpMM); very long rows in a tall matrix (16384 x 8192 at density 0.2) and in
few rows (256 ... 512 rows of 2048 ... 4096 nonzeros), which is where the rules that add waves per row apply; the three
patterns of tests/golden/dlmc whose longest row holds four compute units' shares of the nonzeros (cut plans). Every case is launched as a driver would (dlspm_analyze ->
dlspm_advise -> allocate -> build), inside a HIP graph of 20 launches (median of 7 double replays). With a rule off the
preparation is repeated, so that sizes and advice follow the changed rules. The launches with all rules on are timed
before and after the others (after one untimed run) and their mean is the reference. One line per rule and op: the geometric mean
of (time with the rule off / time with it on) over all cases, the number of cases whose time moved by more than 3 %, the
geometric mean over those, and the two extremes. A ratio above 1 says the rule earns its place.
Results are also checked: with a rule off the op must still agree with the result it gave with all rules on (1e-5
relative Frobenius: another order of the same sums at most).
"""
import argparse
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("dlspm-esimd_amd", "tests"):
    sys.path.insert(0, os.path.join(ROOT, sub))

GRID = [(1024, 1024), (3072, 1024), (4096, 1024), (2048, 2048), (6144, 2048), (8192, 2048), (4096, 4096), (12288, 4096),
        (16384, 4096), (8192, 8192), (24576, 8192), (32768, 8192)]


def variants(dl):
    v = [(f"rule {name}", {"rules_off": bit}) for name, bit in dl.RULES.items()]
    v += [("streamed results (stream_results = 0)", {"stream_results": 0}),
          ("tile-major column tiles (tile_major = 0)", {"tile_major": 0}),
          ("column-sliced schedule (slices = 0)", {"slices": 0}),
          ("flat schedule (flat = 0)", {"flat": 0}),
          ("plan packing (plan_order = 2: longest first only)", {"plan_order": 2})]
    return v


def cases(dl, quick):
    out = []
    for cfg in range(1, 6):
        c = dl.make_config(cfg)
        out.append((c["name"], c["op"], c["M"], c["K"], c["N"], c["row_offsets"], c["col_indices"]))
    grid = GRID[:6] if quick else GRID
    for (M, K) in grid:
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 100 + M // 1024 + K, M, K, 0.1)
        for width in (32, 128):
            out.append((f"grid {M}x{K} density 0.1 width {width}", None, M, K, width, ro, ci))
    for (M, K, mean) in ((2048, 2048, 100.0), (4096, 1024, 100.0), (8192, 2048, 60.0), (16384, 4096, 100.0)):
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 7, M, K, mean, 1.0)
        out.append((f"lognormal {M}x{K} mean {mean:.0f} sigma 1 width 128", None, M, K, 128, ro, ci))
    for (M, K, mean) in ((64, 576, 400.0), (128, 1152, 200.0), (256, 2304, 200.0), (512, 512, 50.0), (512, 2048, 100.0)):
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 9, M, K, mean, 0.5)
        out.append((f"layer {M}x{K} mean {mean:.0f} sigma 0.5 width 256/128/64", None, M, K, -1, ro, ci))
    for (M, K, density) in ((16, 1152, 0.25), (64, 4608, 0.3), (128, 1152, 0.25)):
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 12, M, K, density)
        out.append((f"few rows {M}x{K} density {density} width 256/128/64", None, M, K, -1, ro, ci))
    for (M, K, mean, width) in ((128, 1152, 120.0, 784), (300, 1152, 115.0, 3136), (1000, 2048, 200.0, 640)):
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 10, M, K, mean, 0.5)
        out.append((f"wide dense rows {M}x{K} mean {mean:.0f} sigma 0.5 width {width}", dl.OP_SPMM, M, K, width, ro, ci))
    for (M, K, mean, sigma) in ((2048, 2048, 100.0, 0.0), (2048, 2048, 100.0, 0.8), (8192, 2048, 60.0, 0.0), (512, 2304, 230.0, 0.8)):
        if sigma > 0:
            ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 14, M, K, mean, sigma)
        else:
            ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 14, M, K, mean / K)
        for width in (80, 160, 320):
            out.append((f"between the powers of two {M}x{K} mean {mean:.0f} sigma {sigma} width {width}", "dots", M, K, width, ro, ci))
    if not quick:
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 11, 16384, 8192, 0.2)
        for width in (32, 128):
            out.append((f"tall, long rows 16384x8192 density 0.2 width {width}", None, 16384, 8192, width, ro, ci))
        for (M, K, density) in ((256, 8192, 0.5), (512, 8192, 0.25)):
            ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 13, M, K, density)
            out.append((f"few long rows {M}x{K} density {density} width 256/128/64", None, M, K, -1, ro, ci))
    from test_cut_plan import DLMC, LONG_ROW_FILES, load_smtx
    for f in LONG_ROW_FILES:
        M, K, ro, ci = load_smtx(os.path.join(DLMC, f))
        out.append((f"dlmc {f[:28]} {M}x{K} width 256/128/64", None, M, K, -1, ro, ci))
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--ops", default="spmm,sddmm,fused")
    ap.add_argument("--quick", action="store_true", help="half of the grid")
    ap.add_argument("--out", default=None)
    ap.add_argument("--cases", default=None, help="also write every case's ratio, one line per (rule, op, case)")
    args = ap.parse_args()
    import torch

    import dlspm_hip as dl
    from verify_dlmc import graph_us

    ops = {"spmm": dl.OP_SPMM, "sddmm": dl.OP_SDDMM, "fused": dl.OP_FUSED}
    want = [o for o in args.ops.split(",") if o]
    rng = np.random.default_rng(1)
    vs = variants(dl)
    ratios = {(v, o): [] for v, _ in vs for o in want}
    names = {(v, o): [] for v, _ in vs for o in want}
    drift = []
    rel = lambda a, b: float(torch.linalg.norm((a - b).double()) / max(float(torch.linalg.norm(b.double())), 1e-30))
    all_cases = cases(dl, args.quick)
    for index, (name, only_op, M, K, width, ro, ci) in enumerate(all_cases):
        ro_d, ci_d = torch.from_numpy(ro).cuda(), torch.from_numpy(ci).cuda()
        nnz = int(ci.size)
        for o in want:
            if only_op == "dots":
                if o == "spmm":
                    continue
            elif only_op is not None and ops[o] != only_op:
                continue
            w = width if width > 0 else {"spmm": 256, "sddmm": 128, "fused": 64}[o]
            if o == "spmm":
                va = torch.from_numpy(rng.standard_normal(nnz, dtype=np.float32)).cuda()
                B = torch.from_numpy(rng.standard_normal((K, w), dtype=np.float32)).cuda()
                out = torch.empty((M, w), dtype=torch.float32, device="cuda")
                call = lambda prep: dl.spmm(ro_d, ci_d, va, B, K=K, out=out, plan=prep)
            elif o == "sddmm":
                lhs = torch.from_numpy(rng.standard_normal((M, w), dtype=np.float32)).cuda()
                rhs = torch.from_numpy(rng.standard_normal((K, w), dtype=np.float32)).cuda()
                out = torch.empty((nnz,), dtype=torch.float32, device="cuda")
                call = lambda prep: dl.sddmm(ro_d, ci_d, lhs, rhs, out=out, plan=prep)
            else:
                Q = torch.from_numpy(rng.standard_normal((M, w), dtype=np.float32)).cuda()
                Km = torch.from_numpy(rng.standard_normal((K, w), dtype=np.float32)).cuda()
                V = torch.from_numpy(rng.standard_normal((K, w), dtype=np.float32)).cuda()
                out = torch.empty((M, w), dtype=torch.float32, device="cuda")
                call = lambda prep: dl.fused(ro_d, ci_d, Q, Km, V, 0.125, out=out, plan=prep)
            info = dl.analyze(ro_d, ci_d, K)
            prep = dl.prepare(ro_d, ci_d, K, ops[o], w, info=info)
            graph_us(torch, lambda: call(prep))  # untimed: the first graph over fresh operands runs slower than the later ones
            base = graph_us(torch, lambda: call(prep))
            call(prep)
            ref = out.clone()
            measured = []
            for vname, fields in vs:
                dl.set_tuning(**fields)
                prep_v = dl.prepare(ro_d, ci_d, K, ops[o], w, info=info)
                t = graph_us(torch, lambda: call(prep_v))
                call(prep_v)
                err = rel(out, ref)
                dl.set_tuning()
                if err > 1e-5:
                    print(f"MISMATCH {name} {o} with {vname} off: {err:.2e}", flush=True)
                    sys.exit(1)
                measured.append((vname, t))
            # the same launches once more at the end: the reference time is the mean of the two, their ratio the noise
            again = graph_us(torch, lambda: call(prep))
            drift.append(again / base)
            for vname, t in measured:
                ratios[(vname, o)].append(t / (0.5 * (base + again)))
                names[(vname, o)].append(name)
        print(f"  {index + 1}/{len(all_cases)} {name}", flush=True)
    geo = lambda xs: float(np.exp(np.mean(np.log(xs)))) if len(xs) else float("nan")
    lines = ["time with the rule off / time with it on; geometric mean over all cases | cases moved by more than 3 % | their mean | "
             "smallest (case) | largest (case)"]
    for vname, _ in vs:
        for o in want:
            r = np.array(ratios[(vname, o)])
            moved = np.abs(r - 1.0) > 0.03
            lo, hi = int(np.argmin(r)), int(np.argmax(r))
            lines.append(f"{vname:52s} {o:5s} {geo(r):.3f} | {int(moved.sum()):2d} of {r.size} | {geo(r[moved]):.3f} | "
                         f"{r[lo]:.2f} ({names[(vname, o)][lo]}) | {r[hi]:.2f} ({names[(vname, o)][hi]})")
    d = np.array(drift)
    lines.append(f"noise: the launches with all rules on, timed before and after the others: ratio {geo(d):.3f} in the geometric mean, "
                 f"{d.min():.2f} ... {d.max():.2f}")
    text = "\n".join(lines)
    print(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text + "\n")
    if args.cases:
        with open(args.cases, "w") as f:
            for (vname, o), rs in ratios.items():
                for r, n in zip(rs, names[(vname, o)]):
                    f.write(f"{vname} | {o} | {n} | {r:.3f}\n")


if __name__ == "__main__":
    main()
