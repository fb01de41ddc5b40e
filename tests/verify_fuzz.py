#!/usr/bin/env python3
"""Seeded random cases against the CPU oracle: odd shapes and widths, four kinds of row-length distribution, every
schedule, with the library's launch rules overridden at random (dlspm_set_tuning: work split, flat schedule and its
chunk, column slices, tile order and width, plan order, XCD-contiguous row blocks, streamed results, single size rules
switched off, the cut rule's percentages, the number of compute units the rules and plans are sized for).

    python tests/verify_fuzz.py [--cases 1000] [--seed 1] [--report out.txt]

Each case runs all three ops on the GPU through the C ABI under every schedule that applies (NULL, the even-rows hint,
workspace memory, a row plan, a cut plan) and compares with the oracle: CSR arrays bit-identical after the call, values within 1e-4
relative Frobenius error. No tuning value may change a result beyond the summation order, and none may make a launch
fail. The case is printed before it runs. Exit status 1 if any case fails.
"""
import argparse
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from conftest import random_csr  # noqa: E402
from verify_dlmc import Tally, check_pattern  # noqa: E402  (also puts the binding and the oracle on sys.path)

SPLITS = [None, (4, 1), (4, 2), (4, 4), (4, 8), (4, 16), (8, 1), (8, 2), (8, 4), (16, 1)]


def random_tuning(rng):
    """Keyword arguments for dl.set_tuning: each knob left to the library's rule with probability 1/2."""
    t = {}
    pick = lambda values: values[int(rng.integers(0, len(values)))]
    if rng.random() < 0.5:
        s = pick(SPLITS)
        if s is not None:
            t["split"] = s
    if rng.random() < 0.5:
        t["flat"] = pick([0, 1])
    if rng.random() < 0.3:
        t["flat_chunk"] = pick([64, 256, 1024, 4096])
    if rng.random() < 0.5:
        t["slices"] = pick([0, 2, 3, 4, 7, 16])
    if rng.random() < 0.5:
        t["tile_major"] = pick([0, 1, 2, 3])
    if rng.random() < 0.5:
        t["tile_width"] = pick([512, 256, 128, 64, 32])
    if rng.random() < 0.5:
        t["plan_order"] = pick([0, 1, 2])
    if rng.random() < 0.5:
        t["xcd_contiguous"] = 1
    if rng.random() < 0.5:
        t["stream_results"] = pick([0, 1])
    if rng.random() < 0.5:
        t["rules_off"] = int(rng.integers(0, 2048))
    if rng.random() < 0.3:
        t["cut_piece_pct"], t["cut_longest_pct"] = pick([(100, 150), (75, 100), (50, 75), (25, 30), (200, 150), (10, 10), (1000, 1000)])
    if rng.random() < 0.3:
        t["compute_units"] = pick([8, 32, 64, 128, 304, 1024])
    return t


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--cases", type=int, default=1000)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--report", default=None)
    args = ap.parse_args()

    import torch

    import dlspm_hip as dl
    import oracle

    if not torch.cuda.is_available():
        sys.exit("verify_fuzz.py needs the GPU (it checks the HIP kernels, not the oracle)")
    oracle.lib()
    rng = np.random.default_rng(args.seed)
    tally = Tally(args.report)
    t0 = time.time()
    print(f"{args.cases} random cases, seed {args.seed}; oracle on {oracle.omp_threads()} threads; {dl.version()}", flush=True)
    for case in range(args.cases):
        M = int(rng.choice([1, 2, 7, 63, 64, 65, 200, 700, 2047, 2500, 9000])) + int(rng.integers(0, 5))
        K = int(rng.choice([1, 3, 64, 130, 500, 1500, 2100, 4200, 20000])) + int(rng.integers(0, 5))
        N = int(rng.choice([1, 2, 3, 5, 16, 33, 49, 64, 65, 96, 100, 128, 129, 192, 196, 256, 257, 384, 392, 512, 513, 700, 1030]))
        kind = str(rng.choice(["uniform", "skewed", "empty_rows", "full"]))
        density = float(rng.choice([0.005, 0.02, 0.1, 0.3]))
        if kind == "full" and M * K > 300000:
            kind = "uniform"
        while kind != "full" and M * K * density > 600000:
            density /= 4
        ro, ci = random_csr(rng, M, K, kind, 1.0 if kind == "full" else density)
        tuning = random_tuning(rng)
        what = f"case {case}: M={M} K={K} N={N} {kind} density={density:g} nnz={ci.size} tuning={tuning}"
        print(what, flush=True)
        dl.set_tuning(**tuning)
        ro_d, ci_d = torch.from_numpy(ro).cuda(), torch.from_numpy(ci).cuda()
        for op in ("spmm", "sddmm", "fused"):
            for schedule, err, intact, _, _ in check_pattern(dl, torch, oracle, op, M, K, N, ro, ci, ro_d, ci_d, rng, True):
                tally.add(op, schedule, what, err, intact)
        dl.set_tuning()
    print(f"{time.time() - t0:.0f} s")
    sys.exit(tally.finish("verify_fuzz", f"{args.cases} random problems"))


if __name__ == "__main__":
    main()
