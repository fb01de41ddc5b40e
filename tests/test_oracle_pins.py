"""Pins the CPU oracle (oracle/dlspm_oracle.c) before anything is checked against it.

Three independent anchors, chosen so that a dropped term, a wrong index or a transposed operand fails:
  1. the golden fixtures under tests/golden/ -- outputs of the REFERENCE's own functions compiled from its
     FUSED/fused.cpp (written by tests/golden/make_golden.py) -- must be reproduced bit for bit;
  2. where oracle/_ref is present (it travels with the tree but is never committed), the same reference
     functions are called live on fresh seeds and larger shapes, again bit for bit;
  3. what the mathematics fixes: closed forms, a float64 dense product, brute force on tiny inputs,
     linearity and nonzero-splitting invariants.
"""
import glob
import os

import numpy as np
import pytest
import scipy.sparse as sp

from conftest import random_csr

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "fused_ref_M*_K*_N*.npz")))


def test_golden_fixtures_exist():
    assert len(GOLDEN) == 3


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_oracle_reproduces_reference_outputs_bit_exact(oracle, path):
    g = np.load(path)
    ro, ci = g["row_offsets"], g["col_indices"]
    sddmm = oracle.sddmm(ro, ci, g["c"], g["b"])
    assert np.array_equal(sddmm, g["sddmm"]), "Sddmm (double accumulate) differs from the reference"
    assert np.array_equal(oracle.spmm(ro, ci, g["sddmm"], g["d"], acc="f64"), g["spmm_f64acc"])
    assert np.array_equal(oracle.spmm(ro, ci, g["values"], g["d"], acc="f32"), g["spmm_f32"]), \
        "float-accumulating Spmm differs from the reference's fp32 sequence"
    # the reference's fused gold is Sddmm followed by Spmm(double): scale = 1 must give exactly that
    O, scores = oracle.fused(ro, ci, g["c"], g["b"], g["d"], 1.0, return_scores=True)
    assert np.array_equal(scores, g["sddmm"])
    assert np.array_equal(O, g["spmm_f64acc"])
    # and the reference's own fp32 emulation of its fused kernel agrees with it to fp32 rounding, as the
    # reference's driver prints (FUSED/fused.cpp:400-413)
    assert oracle.rel_frobenius(g["fused_emul"], O) < 1e-5


def test_oracle_against_live_reference_build(oracle):
    builds = oracle.ref_builds()
    if not builds:
        pytest.skip("oracle/_ref not built here (needs the reference tree); the golden fixtures cover this")
    for ref in builds:
        for seed in (1, 2):
            rng = np.random.default_rng(seed * 100 + ref.D)
            lens = np.clip(rng.binomial(ref.K, min(0.3, 40.0 / ref.K), size=ref.M), 1, ref.K)
            ro = np.zeros(ref.M + 1, dtype=np.int32)
            ro[1:] = np.cumsum(lens)
            ci = np.concatenate([np.sort(rng.choice(ref.K, size=int(k), replace=False)) for k in lens]).astype(np.int32)
            c = rng.normal(0, 1, (ref.M, ref.D)).astype(np.float32)
            b = rng.normal(0, 1, (ref.K, ref.D)).astype(np.float32)
            d = rng.normal(0, 1, (ref.K, ref.D)).astype(np.float32)
            va = rng.uniform(-1, 1, ci.size).astype(np.float32)
            s_ref = ref.sddmm(ro, ci, c, b)
            assert np.array_equal(oracle.sddmm(ro, ci, c, b), s_ref)
            assert np.array_equal(oracle.spmm(ro, ci, s_ref, d, acc="f64"), ref.spmm_f64acc(ro, ci, s_ref, d))
            assert np.array_equal(oracle.spmm(ro, ci, va, d, acc="f32"), ref.spmm_f32_emul(ro, ci, va, d))
            assert np.array_equal(oracle.fused(ro, ci, c, b, d, 1.0), ref.spmm_f64acc(ro, ci, s_ref, d))


# ---- closed forms and textbook routines ----------------------------------------------------------------

def test_spmm_identity_and_single_entry_rows_are_exact(oracle):
    rng = np.random.default_rng(0)
    K, N = 37, 19
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    ro = np.arange(K + 1, dtype=np.int32)
    ci = np.arange(K, dtype=np.int32)
    ones = np.ones(K, dtype=np.float32)
    for acc in ("f32", "f64"):
        assert np.array_equal(oracle.spmm(ro, ci, ones, B, acc=acc), B)  # A = I
    perm = rng.permutation(K).astype(np.int32)
    va = rng.normal(0, 1, K).astype(np.float32)
    expect = va[:, None] * B[perm]  # one product per element, no addition: exact in fp32
    assert np.array_equal(oracle.spmm(ro, perm, va, B, acc="f32"), expect)


def test_spmm_all_ones_rows_give_column_sums_and_empty_rows_give_zero(oracle):
    rng = np.random.default_rng(1)
    K, N = 50, 8
    B = rng.integers(-8, 9, (K, N)).astype(np.float32)  # small integers: every partial sum is exact
    ro = np.array([0, K, K, 2 * K], dtype=np.int32)     # full row, empty row, full row
    ci = np.concatenate([np.arange(K), np.arange(K)]).astype(np.int32)
    C = oracle.spmm(ro, ci, np.ones(2 * K, dtype=np.float32), B)
    assert np.array_equal(C[0], B.sum(axis=0)) and np.array_equal(C[2], B.sum(axis=0))
    assert (C[1] == 0).all()


def brute_spmm(ro, ci, va, B):
    M, N = len(ro) - 1, B.shape[1]
    C = np.zeros((M, N), dtype=np.float64)
    for i in range(M):
        for l in range(ro[i], ro[i + 1]):
            for j in range(N):
                C[i, j] += float(va[l]) * float(B[ci[l], j])
    return C


def test_spmm_brute_force_and_dense_float64(oracle):
    rng = np.random.default_rng(2)
    ro, ci = random_csr(rng, 9, 11, "uniform", 0.4)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (11, 5)).astype(np.float32)  # non-square, so a transposed operand cannot pass
    for acc in ("f32", "f64"):
        assert np.allclose(oracle.spmm(ro, ci, va, B, acc=acc), brute_spmm(ro, ci, va, B), rtol=1e-5, atol=1e-6)
    for (M, K, N, kind) in [(120, 200, 33, "skewed"), (64, 300, 128, "empty_rows")]:
        ro, ci = random_csr(rng, M, K, kind, 0.1)
        va = rng.normal(0, 1, ci.size).astype(np.float32)
        B = rng.normal(0, 1, (K, N)).astype(np.float32)
        A = sp.csr_matrix((va.astype(np.float64), ci, ro), shape=(M, K))
        dense = A @ B.astype(np.float64)
        assert oracle.rel_frobenius(oracle.spmm(ro, ci, va, B, acc="f32"), dense) < 1e-6
        assert oracle.rel_frobenius(oracle.spmm(ro, ci, va, B, acc="f64"), dense) < 1e-7


def test_spmm_linearity_and_nonzero_splitting(oracle):
    rng = np.random.default_rng(3)
    M, K, N = 40, 60, 12
    ro, ci = random_csr(rng, M, K, "uniform", 0.3)
    va = rng.integers(-4, 5, ci.size).astype(np.float32)
    B1 = rng.integers(-4, 5, (K, N)).astype(np.float32)
    B2 = rng.integers(-4, 5, (K, N)).astype(np.float32)
    # integers keep every operation exact, so the invariants hold bit for bit
    assert np.array_equal(oracle.spmm(ro, ci, va, B1 + B2), oracle.spmm(ro, ci, va, B1) + oracle.spmm(ro, ci, va, B2))
    keep = rng.random(ci.size) < 0.5
    parts = []
    for mask in (keep, ~keep):
        lens = np.array([mask[ro[i]:ro[i + 1]].sum() for i in range(M)])
        r2 = np.zeros(M + 1, dtype=np.int32)
        r2[1:] = np.cumsum(lens)
        parts.append(oracle.spmm(r2, ci[mask], va[mask], B1))
    assert np.array_equal(parts[0] + parts[1], oracle.spmm(ro, ci, va, B1))


def test_sddmm_against_dense_float64_and_special_cases(oracle):
    rng = np.random.default_rng(4)
    M, K, D = 30, 47, 21  # all different: a swapped lhs/rhs or a transposed index cannot pass
    lhs = rng.normal(0, 1, (M, D)).astype(np.float32)
    rhs = rng.normal(0, 1, (K, D)).astype(np.float32)
    dense = lhs.astype(np.float64) @ rhs.astype(np.float64).T
    ro, ci = random_csr(rng, M, K, "skewed", 0.2)
    rows = np.repeat(np.arange(M), np.diff(ro))
    got = oracle.sddmm(ro, ci, lhs, rhs)
    assert np.array_equal(got, dense[rows, ci].astype(np.float32)) or oracle.rel_frobenius(got, dense[rows, ci]) < 1e-7
    # full mask = dense GEMM in CSR order
    ro_f = (np.arange(M + 1) * K).astype(np.int32)
    ci_f = np.tile(np.arange(K, dtype=np.int32), M)
    assert oracle.rel_frobenius(oracle.sddmm(ro_f, ci_f, lhs, rhs).reshape(M, K), dense) < 1e-7
    # D = 1: a sampled outer product, one exactly rounded multiplication per slot
    l1, r1 = lhs[:, :1].copy(), rhs[:, :1].copy()
    assert np.array_equal(oracle.sddmm(ro, ci, l1, r1), (l1[rows, 0].astype(np.float64) * r1[ci, 0]).astype(np.float32))
    # a slot's value does not depend on the other slots: dropping every second nonzero keeps the rest
    keep = np.arange(ci.size) % 2 == 0
    lens = np.array([keep[ro[i]:ro[i + 1]].sum() for i in range(M)])
    r2 = np.zeros(M + 1, dtype=np.int32)
    r2[1:] = np.cumsum(lens)
    assert np.array_equal(oracle.sddmm(r2, ci[keep], lhs, rhs), got[keep])


def test_fused_is_the_composition_and_matches_dense_float64(oracle):
    rng = np.random.default_rng(5)
    M, K, D, scale = 33, 41, 16, 0.125
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    V = rng.normal(0, 1, (K, D)).astype(np.float32)
    ro, ci = random_csr(rng, M, K, "empty_rows", 0.3)
    O, scores = oracle.fused(ro, ci, Q, Km, V, scale, return_scores=True)
    s = oracle.sddmm(ro, ci, Q, Km) * np.float32(scale)
    assert np.array_equal(scores, s)
    assert np.array_equal(O, oracle.spmm(ro, ci, s, V, acc="f64"))
    mask = np.zeros((M, K))
    rows = np.repeat(np.arange(M), np.diff(ro))
    mask[rows, ci] = 1.0
    dense = ((Q.astype(np.float64) @ Km.astype(np.float64).T) * mask * scale) @ V.astype(np.float64)
    assert oracle.rel_frobenius(O, dense) < 1e-6
    assert (O[np.diff(ro) == 0] == 0).all()


def test_omp_variants_are_bit_identical(oracle):
    rng = np.random.default_rng(6)
    M, K, D = 200, 150, 24
    ro, ci = random_csr(rng, M, K, "skewed", 0.1)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    X = rng.normal(0, 1, (M, D)).astype(np.float32)
    Y = rng.normal(0, 1, (K, D)).astype(np.float32)
    Z = rng.normal(0, 1, (K, D)).astype(np.float32)
    for acc in ("f32", "f64"):
        assert np.array_equal(oracle.spmm(ro, ci, va, Y, acc=acc), oracle.spmm(ro, ci, va, Y, acc=acc, omp=True))
    assert np.array_equal(oracle.sddmm(ro, ci, X, Y), oracle.sddmm(ro, ci, X, Y, omp=True))
    assert np.array_equal(oracle.fused(ro, ci, X, Y, Z, 0.5), oracle.fused(ro, ci, X, Y, Z, 0.5, omp=True))


def test_csr_check_names_each_failure(oracle):
    """One malformed structure per test of the reference's SanityCheck (SPMM/spmm-esimd-fromfile.cpp:36-61)."""
    ro = np.array([0, 2, 2, 4], dtype=np.int32)
    ci = np.array([0, 3, 1, 2], dtype=np.int32)
    assert oracle.csr_check(3, 4, 4, ro, ci) == 0
    assert oracle.csr_check(1, 2, 3, np.array([0, 3], dtype=np.int32), np.array([0, 1, 1], dtype=np.int32)) == 1
    assert oracle.csr_check(3, 4, 5, ro, ci) == 2
    assert oracle.csr_check(3, 4, 4, np.array([0, 3, 2, 4], dtype=np.int32), ci) == 3
    assert oracle.csr_check(2, 2, 3, np.array([0, 3, 3], dtype=np.int32), np.array([0, 1, 1], dtype=np.int32)) == 4
    assert oracle.csr_check(3, 3, 4, ro, ci) == 5
    assert oracle.csr_check(3, 4, 4, np.array([1, 2, 2, 4], dtype=np.int32), ci) == 6
    assert oracle.csr_check(3, 4, 4, ro, np.array([0, -1, 1, 2], dtype=np.int32)) == 7
