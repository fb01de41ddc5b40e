"""Writes the golden fixtures tests/golden/fused_ref_M*_K*_N*.npz.

Run in the authoring container only (it needs the reference tree, through the checker objects that
`make -C oracle ref` compiles from the reference's FUSED/fused.cpp into oracle/_ref/):

    python tests/golden/make_golden.py

Each fixture holds seeded inputs and what the REFERENCE's own functions returned for them:
    sddmm        Sddmm          (FUSED/fused.cpp:47-65, double accumulate)
    spmm_f64acc  Spmm           (FUSED/fused.cpp:67-89, double accumulate) applied to `sddmm` as the values
    spmm_f32     SpmmEsimdCPU   (FUSED/fused.cpp:218-303) applied to `values`; per output element this is the
                                same fp32 operation sequence as the float-accumulating Spmm of
                                SPMM/spmm-esimd-fromfile.cpp:63-83
    fused_emul   FusedEsimdCPU  (FUSED/fused.cpp:93-216), the fp32 emulation of the fused kernel
Every row has at least one nonzero: the two emulation functions read past an empty row's end.
The fixtures are data only; no reference source is stored.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import oracle  # noqa: E402

GOLDEN_SHAPES = {(64, 128, 32), (96, 80, 64), (37, 53, 16)}


def make_inputs(M, K, D, seed):
    rng = np.random.default_rng(seed)
    lens = np.clip(rng.binomial(K, 0.15, size=M), 1, K)
    lens[0] = min(K, 32)  # an exact multiple of the reference's 32-wide chunk
    lens[1] = min(K, 33)
    lens[2] = 1
    ro = np.zeros(M + 1, dtype=np.int32)
    ro[1:] = np.cumsum(lens)
    ci = np.concatenate([np.sort(rng.choice(K, size=int(k), replace=False)) for k in lens]).astype(np.int32)
    return dict(
        row_offsets=ro, col_indices=ci,
        values=rng.uniform(-1, 1, ci.size).astype(np.float32),
        c=rng.normal(0, 1, (M, D)).astype(np.float32),
        b=rng.normal(0, 1, (K, D)).astype(np.float32),
        d=rng.uniform(-1, 1, (K, D)).astype(np.float32),
    )


def main():
    builds = [r for r in oracle.ref_builds() if (r.M, r.K, r.D) in GOLDEN_SHAPES]
    if len(builds) != len(GOLDEN_SHAPES):
        raise SystemExit("oracle/_ref is incomplete: run `make -C oracle ref` where /root/reference is mounted")
    for ref in builds:
        x = make_inputs(ref.M, ref.K, ref.D, seed=ref.M * 1000 + ref.D)
        sddmm = ref.sddmm(x["row_offsets"], x["col_indices"], x["c"], x["b"])
        out = dict(
            x,
            sddmm=sddmm,
            spmm_f64acc=ref.spmm_f64acc(x["row_offsets"], x["col_indices"], sddmm, x["d"]),
            spmm_f32=ref.spmm_f32_emul(x["row_offsets"], x["col_indices"], x["values"], x["d"]),
            fused_emul=ref.fused_emul(x["row_offsets"], x["col_indices"], x["c"], x["b"], x["d"]),
        )
        path = os.path.join(HERE, f"fused_ref_M{ref.M}_K{ref.K}_N{ref.D}.npz")
        np.savez_compressed(path, **out)
        print("wrote", os.path.relpath(path, ROOT), os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
