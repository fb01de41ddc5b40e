#!/usr/bin/env python3
"""Oracle parity over the reference's benchmark grid at full size.

    python tests/verify_sweep.py [--max-m 32768] [--fused-max-m 8192] [--ops spmm,sddmm,fused] [--report out.txt]
                                 [--all-schedules]

The grid of SPMM/spmm-esimd-allbenchs2.cpp:252-266 (12 shapes x width {32,128} x density {0.3,0.2,0.1}; the same in
SDDMM/sddmm-esimd-allbench_v4.cpp:241-244), with the seeded Bernoulli patterns the C++ drivers' --sweep uses (same
generator, same seeds). Each op runs on the GPU through the C ABI under the schedule the library advises (or every one,
--all-schedules) and is compared with the CPU oracle: CSR arrays bit-identical after the call, values within 1e-4
relative Frobenius error. tests/test_drivers.py verifies the drivers' own sweep dumps up to 2048 rows; this is the
whole grid (the largest case has 80 million nonzeros; about 3 GB of host memory). Exit status 1 if any case fails.
"""
import argparse
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from verify_dlmc import Tally, check_pattern  # noqa: E402  (also puts the binding and the oracle on sys.path)

SHAPES = [(1024, 1024), (3072, 1024), (4096, 1024), (2048, 2048), (6144, 2048), (8192, 2048), (4096, 4096), (12288, 4096),
          (16384, 4096), (8192, 8192), (24576, 8192), (32768, 8192)]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--max-m", type=int, default=32768)
    ap.add_argument("--fused-max-m", type=int, default=8192, help="the fused driver's sweep stops there")
    ap.add_argument("--ops", default="spmm,sddmm,fused")
    ap.add_argument("--report", default=None)
    ap.add_argument("--all-schedules", action="store_true")
    args = ap.parse_args()

    import torch

    import dlspm_hip as dl
    import oracle

    if not torch.cuda.is_available():
        sys.exit("verify_sweep.py needs the GPU (it checks the HIP kernels, not the oracle)")
    oracle.lib()
    ops = [o for o in args.ops.split(",") if o]
    tally = Tally(args.report)
    t0 = time.time()
    index = 0
    print(f"grid of {len(SHAPES)} shapes x 2 widths x 3 densities; ops {ops}; oracle on {oracle.omp_threads()} threads; {dl.version()}",
          flush=True)
    for N in (32, 128):
        for M, K in SHAPES:
            for density in (0.3, 0.2, 0.1):
                seed = 7000 + index  # the drivers number the cases of the unrestricted grid the same way
                index += 1
                if M > args.max_m:
                    continue
                ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, seed, M, K, density)
                ro_d, ci_d = torch.from_numpy(ro).cuda(), torch.from_numpy(ci).cuda()
                rng = np.random.default_rng(seed)
                for op in ops:
                    if op == "fused" and M > args.fused_max_m:
                        continue
                    what = f"M={M} K={K} N={N} density={density} nnz={ci.size}"
                    for schedule, err, intact, _, _ in check_pattern(dl, torch, oracle, op, M, K, N, ro, ci, ro_d, ci_d, rng, args.all_schedules):
                        tally.add(op, schedule, what, err, intact)
                print(f"  {M} x {K}, N = {N}, density {density}: {tally.cases} cases, {tally.failures} failures, {time.time() - t0:.0f} s",
                      flush=True)
    print(f"{time.time() - t0:.0f} s")
    sys.exit(tally.finish("verify_sweep", "the grid"))


if __name__ == "__main__":
    main()
