#!/usr/bin/env python3
"""Packs sparsity patterns (.smtx files: "M, K, nnz", the row offsets, the column indices) into one compressed .npz that
tests/verify_dlmc.py reads in place of a directory -- the form in which a selection of the reference's dlmc/ tree travels
to a machine that does not hold the data set.

    python tests/golden/dlmc/pack_patterns.py <dir> <out.npz> [--min-nnz 20000] [--long-rows 1.5] [--compute-units 256]

--long-rows x keeps only the patterns whose longest row holds more than x times one compute unit's share of the nonzeros
(nnz / compute units): the matrices a cut plan (dlspm_row_plan_build_cut) is for.
"""
import argparse
import os

import numpy as np


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("dir")
    ap.add_argument("out")
    ap.add_argument("--min-nnz", type=int, default=0)
    ap.add_argument("--long-rows", type=float, default=0.0)
    ap.add_argument("--compute-units", type=int, default=256)
    args = ap.parse_args()
    arrays, names, shapes = {}, [], []
    files = sorted(os.path.join(d, f) for d, _, fs in os.walk(args.dir) for f in fs if f.endswith(".smtx"))
    for path in files:
        with open(path) as f:
            M, K, nnz = (int(x) for x in f.readline().replace(",", " ").split())
            if nnz < args.min_nnz:
                continue
            ro = np.array(f.readline().split(), dtype=np.int32)
            if args.long_rows > 0:
                share = -(-nnz // args.compute_units)
                if ro.size < 2 or np.diff(ro).max() <= args.long_rows * share:
                    continue
            ci = np.array(f.read().split(), dtype=np.uint16 if K <= 65535 else np.int32)
        slot = len(names)
        arrays[f"ro{slot}"], arrays[f"ci{slot}"] = ro, ci
        names.append(os.path.relpath(path, args.dir))
        shapes.append((M, K))
    np.savez_compressed(args.out, names=np.array(names), shapes=np.array(shapes, dtype=np.int64).reshape(-1, 2), **arrays)
    print(f"{len(names)} of {len(files)} patterns packed into {args.out}")


if __name__ == "__main__":
    main()
