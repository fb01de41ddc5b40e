#!/usr/bin/env python3
"""SDDMM and the fused op over inner dimensions D = 16 ... 512 in steps of 16 (MI355X): time per launch and per float of a
gathered row, so that the widths no kernel is built for exactly can be read against their neighbours.

    python tests/width_sweep.py [--quick] [--out table.txt]

Per width: the accesses of 32 floats a lane makes per dot product (DS), which kind of kernel runs (exact: D = 32 x DS, no
bounds handling; range: lanes past D masked by the range check of a buffer load; select: by selects), the time of a plain
call, and for SDDMM the same call with DLSPM_RULE_MASK_BY_RANGE and with DLSPM_RULE_EXACT_WIDTH_KERNELS switched off. Shapes:
2048 x 2048 of 100 per row and 8192 x 2048 of 60 per row, Bernoulli and lognormal (sigma 0.8) rows. Every SDDMM result is
checked against the CPU oracle at the first shape (1e-4 relative Frobenius) and, bit for bit, against the same call with
each rule off. us per launch inside a HIP graph of 20 launches (median of 7 double replays).
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
    ap.add_argument("--quick", action="store_true", help="steps of 48 and one shape")
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    import torch

    import dlspm_hip as dl
    import oracle
    from verify_dlmc import graph_us

    lines = []

    def say(text):
        print(text, flush=True)
        lines.append(text)

    shapes = [(2048, 2048, 100, 0.0), (2048, 2048, 100, 0.8), (8192, 2048, 60, 0.0), (8192, 2048, 60, 0.8)]
    widths = list(range(16, 513, 48 if args.quick else 16))
    for index, (M, K, per_row, sigma) in enumerate(shapes[:1] if args.quick else shapes):
        if sigma > 0:
            ro_h, ci_h = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 31, M, K, float(per_row), sigma)
        else:
            ro_h, ci_h = dl.make_pattern(dl.PATTERN_BERNOULLI, 31, M, K, per_row / K)
        nnz = int(ci_h.size)
        ro, ci = torch.from_numpy(ro_h).cuda(), torch.from_numpy(ci_h).cuda()
        say(f"{M} x {K}, {nnz} nonzeros, {'lognormal rows, sigma %.1f' % sigma if sigma > 0 else 'Bernoulli rows'}")
        say("    D  DS  kind    | sddmm us   ns per 1000 gathered floats | range off   exact off | fused us   ns per 1000 floats (two operands)")
        for D in widths:
            lhs = torch.randn(M, D, device="cuda")
            rhs = torch.randn(K, D, device="cuda")
            val = torch.randn(K, D, device="cuda")
            out = torch.full((nnz,), float("nan"), device="cuda")
            fout = torch.empty((M, D), device="cuda")
            call = lambda: dl.sddmm(ro, ci, lhs, rhs, out=out)
            fcall = lambda: dl.fused(ro, ci, lhs, rhs, val, scale=0.125, out=fout)
            sh = dl.describe_launch(dl.OP_SDDMM, M, K, D, nnz)
            ds = sh["DS"]
            kind = "exact" if D == sh["G1"] * sh["vec"] * ds else "range" if (D % 4 == 0 and 1 <= ds <= 16 and sh["G1"] == 8) else "select"
            call()
            got = out.clone()
            if index == 0:
                want = oracle.sddmm(ro_h, ci_h, lhs.cpu().numpy(), rhs.cpu().numpy(), omp=True)
                assert oracle.rel_frobenius(got.cpu().numpy(), want) <= 1e-4, D
            graph_us(torch, call, replays=2)
            t = graph_us(torch, call)
            off = {}
            for rule in ("mask_by_range", "exact_width_kernels"):
                dl.set_tuning(rules_off=dl.RULES[rule])
                try:
                    out.fill_(float("nan"))
                    call()
                    assert torch.equal(out, got), (D, rule)
                    off[rule] = graph_us(torch, call)
                finally:
                    dl.set_tuning()
            graph_us(torch, fcall, replays=2)
            tf = graph_us(torch, fcall)
            say(f"  {D:3d}  {ds:2d}  {kind:6s}  | {t:8.2f}   {t * 1e6 / (nnz * D):8.1f}                     | {off['mask_by_range']:8.2f}   {off['exact_width_kernels']:8.2f}  "
                f"| {tf:8.2f}   {tf * 1e6 / (2 * nnz * D):8.1f}")
        say("")
    if args.out:
        with open(args.out, "w") as f:
            f.write("\n".join(lines) + "\n")


if __name__ == "__main__":
    main()
