#!/usr/bin/env python3
"""Two rules for calls without memory or plan, each timed on and off where it applies (MI355X):

  * SpMM, finer column tiles of B (DLSPM_RULE_FINER_COLUMN_TILES): few rows at N = 64 ... 1024, and dense rows wider
    than 512 floats on 64 ... 8192 rows (where B exceeds the L2: every XCD on its own tiles);
  * SDDMM, several workgroups per row of a mask of few rows (DLSPM_RULE_ROW_PIECES_FEW_ROWS), 16 ... 384 rows, D = 32 ... 256,
    with the time of the same launch under a cut plan beside it.

    python tests/plain_call_rules_sweep.py [--quick] [--out table.txt]

Patterns: Bernoulli ("even") and lognormal row lengths (sigma 0.8) from the library's own generator. Every case is
checked first (SpMM against the CPU oracle to 1e-4 relative Frobenius; SDDMM with the rule on against the same call with
it off, bit for bit) and then timed inside a HIP graph of 20 launches (median of 7 double replays), after one untimed
graph. One line per case, then geometric means per group of cases.
"""
import argparse
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("dlspm-esimd_amd", "tests", "oracle"):
    sys.path.insert(0, os.path.join(ROOT, sub))


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--quick", action="store_true", help="a third of the cases")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    import torch

    import dlspm_hip as dl
    import oracle
    from verify_dlmc import graph_us

    lines, groups = [], {}

    def say(text):
        print(text, flush=True)
        lines.append(text)

    def pattern(kind, M, K, per_row):
        if kind == "even":
            return dl.make_pattern(dl.PATTERN_BERNOULLI, 5, M, K, per_row / K)
        return dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 7, M, K, float(per_row), 0.8)

    def spmm_case(group, kind, M, K, per_row, N):
        ro_h, ci_h = pattern(kind, M, K, per_row)
        nnz = int(ci_h.size)
        ro, ci = torch.from_numpy(ro_h).cuda(), torch.from_numpy(ci_h).cuda()
        va = torch.randn(nnz, device="cuda")
        B = torch.randn(K, N, device="cuda")
        out = torch.full((M, N), float("nan"), device="cuda")
        call = lambda: dl.spmm(ro, ci, va, B, K=K, out=out)
        on = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz)
        dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
        off = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz)
        dl.set_tuning()
        call()
        if nnz * N < 3e8:
            want = oracle.spmm(ro_h, ci_h, va.cpu().numpy(), B.cpu().numpy(), omp=True)
            assert oracle.rel_frobenius(out.cpu().numpy(), want) <= 1e-4, (kind, M, K, N)
        n = 20 if nnz * N < 1e9 else 5
        graph_us(torch, call, launches=n, replays=2)
        t_on = graph_us(torch, call, launches=n)
        dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
        t_off = graph_us(torch, call, launches=n)
        dl.set_tuning()
        tile = lambda sh: f"{sh['G'] * sh['vec'] * sh['V']} x {sh['col_tiles']}, W{sh['W']} R{sh['R']}"
        say(f"spmm  {kind} {M:5d} x {K:5d} {nnz:8d} nnz longest {int(np.diff(ro_h).max()):5d} N {N:5d}: tiles {tile(off):>18s} -> {tile(on):>18s}   "
            f"off {t_off:8.2f} on {t_on:8.2f} us  {t_on / t_off:.2f}")
        groups.setdefault((f"spmm {group}", kind), []).append((t_off, t_on))

    def sddmm_case(group, kind, M, K, per_row, D, rule="row_pieces_few_rows"):
        ro_h, ci_h = pattern(kind, M, K, per_row)
        nnz = int(ci_h.size)
        ro, ci = torch.from_numpy(ro_h).cuda(), torch.from_numpy(ci_h).cuda()
        lhs, rhs = torch.randn(M, D, device="cuda"), torch.randn(K, D, device="cuda")
        out = torch.full((nnz,), float("nan"), device="cuda")
        call = lambda **kw: dl.sddmm(ro, ci, lhs, rhs, out=out, **kw)
        on = dl.describe_launch(dl.OP_SDDMM, M, K, D, nnz)
        call()
        with_rule = out.clone()
        dl.set_tuning(rules_off=dl.RULES[rule])
        out.fill_(float("nan"))
        call()
        assert torch.equal(out, with_rule), (kind, M, K, D)
        dl.set_tuning()
        graph_us(torch, call)
        t_on = graph_us(torch, call)
        dl.set_tuning(rules_off=dl.RULES[rule])
        t_off = graph_us(torch, call)
        dl.set_tuning()
        plan = dl.cut_plan(ro, dl.OP_SDDMM, D)
        t_cut = graph_us(torch, lambda: call(plan=plan))
        say(f"sddmm {kind} {M:5d} x {K:5d} {nnz:8d} nnz longest {int(np.diff(ro_h).max()):5d} D {D:5d}: {on['col_tiles']:3d} workgroups per row of {on['W']} waves   "
            f"off {t_off:8.2f} on {t_on:8.2f} us  {t_on / t_off:.2f}   cut plan {t_cut:8.2f}")
        groups.setdefault((f"sddmm {group}", kind), []).append((t_off, t_on, t_cut))

    shapes = ((576, 400), (1152, 290), (2304, 230), (4608, 1380))
    few = (16, 64, 128, 192) if not args.quick else (64,)
    for kind in ("even", "logn"):
        for M in few:
            for K, per_row in shapes:
                for N in (64, 128, 256, 512, 1024):
                    spmm_case(f"{M} rows, N = {N}", kind, M, K, per_row, N)
    wide = ((200, 2304, 230, 784), (128, 1152, 290, 784), (1500, 512, 100, 600), (1000, 2048, 200, 640), (300, 1152, 115, 3136),
            (256, 2304, 230, 3136), (1024, 1152, 115, 12544), (2048, 2304, 230, 3136), (4096, 4096, 200, 3136), (2048, 512, 100, 784),
            (256, 64, 13, 3136), (64, 576, 115, 3136), (64, 147, 75, 12544), (512, 4608, 460, 3136), (8192, 4096, 100, 1024))
    for kind in ("even", "logn"):
        for M, K, per_row, N in (wide[::3] if args.quick else wide):
            spmm_case("dense rows wider than 512", kind, M, K, per_row, N)
    for kind in ("even", "logn"):
        for M in few + ((256, 384) if not args.quick else (384,)):
            for K, per_row in shapes:
                for D in (32, 64, 128, 256):
                    sddmm_case(f"{M} rows, D = {D}", kind, M, K, per_row, D)
    say("")
    say("geometric means per group: rule off / on (us), ratio" + "; SDDMM: / under a cut plan")
    for (group, kind), v in groups.items():
        g = lambda j: float(np.exp(np.mean([np.log(x[j]) for x in v])))
        tail = f" / {g(2):.2f}" if len(v[0]) > 2 else ""
        say(f"  {group:34s} {kind}: {g(0):8.2f} / {g(1):8.2f}  {g(1) / g(0):.2f}{tail}   ({len(v)} cases)")
    if args.out:
        with open(args.out, "w") as f:
            f.write("\n".join(lines) + "\n")


if __name__ == "__main__":
    main()
