"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on the same seeded inputs.

Bars (BASELINE.json): the CSR structure must come back bit-identical (the library may not touch it), values
within 1e-4 relative Frobenius error of the reference's CPU loops. Sizes here are ones the oracle finishes
in seconds; the five benchmark configurations are checked at full size.
"""
import glob
import os

import numpy as np
import pytest

from conftest import random_csr

pytestmark = pytest.mark.gpu

TOL = 1e-4  # relative Frobenius error, from BASELINE.json's north_star


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def check_csr_untouched(ro_d, ci_d, ro, ci):
    assert np.array_equal(ro_d.cpu().numpy(), ro), "row_offsets changed"
    assert np.array_equal(ci_d.cpu().numpy(), ci), "col_indices changed"


# (M, K, N, kind, density): N picks the lane layout (G = 8/16/32/64, V = 1/2, dword path for N < 4),
# density and kind pick the (W, R) split and exercise shared rows, empty rows and ragged tails.
SPMM_CASES = [
    (1, 1, 1, "full", 1.0),
    (3, 5, 4, "uniform", 0.5),
    (64, 64, 8, "uniform", 0.2),
    (100, 300, 32, "uniform", 0.05),
    (257, 129, 64, "skewed", 0.1),
    (128, 512, 128, "uniform", 0.3),
    (333, 512, 256, "skewed", 0.1),
    (200, 512, 392, "uniform", 0.2),
    (64, 256, 512, "uniform", 0.1),
    (50, 200, 1000, "skewed", 0.05),
    (77, 130, 33, "uniform", 0.1),
    (40, 100, 7, "empty_rows", 0.3),
    (90, 64, 130, "skewed", 0.3),
    (256, 256, 128, "empty_rows", 0.1),
    (64, 128, 256, "empty", 0.0),
    (16, 700, 256, "full", 1.0),
    (5, 2048, 64, "full", 1.0),
    (1000, 64, 16, "uniform", 0.02),
    (700, 512, 256, "skewed", 0.12),
    (1500, 1024, 96, "uniform", 0.1),
    (2000, 300, 40, "empty_rows", 0.4),
    (300, 512, 64, "full", 1.0),
    # widths that are not a multiple of 4: the row's last lane works on the last four floats; 1 to 3: dword path
    (70, 90, 5, "uniform", 0.3),
    (70, 90, 6, "skewed", 0.3),
    (64, 128, 49, "skewed", 0.2),
    (64, 128, 50, "uniform", 0.2),
    (33, 64, 129, "uniform", 0.3),
    (20, 64, 258, "uniform", 0.3),
    (10, 64, 1026, "uniform", 0.3),
    (12, 64, 1030, "skewed", 0.3),
    (50, 80, 2, "uniform", 0.3),
    (50, 80, 3, "empty_rows", 0.3),
    (300, 80, 1, "skewed", 0.3),
]


@pytest.mark.parametrize("M,K,N,kind,density", SPMM_CASES)
def test_spmm_matches_oracle(torch_cuda, dl, oracle, M, K, N, kind, density):
    torch = torch_cuda
    rng = np.random.default_rng(1234 + M * 7 + N)
    ro, ci = random_csr(rng, M, K, kind, density)
    va = rng.uniform(-1, 1, ci.size).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    ref = oracle.spmm(ro, ci, va, B)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")  # poisoned: every element must be written
    dl.spmm(ro_d, ci_d, dev(torch, va), dev(torch, B), K=K, out=C)
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    assert np.isfinite(got).all(), "an output element was not written"
    assert oracle.rel_frobenius(got, ref) <= TOL
    # the reference drivers' own metric: max |diff| (SPMM/spmm-esimd-fromfile2.cpp:266-276)
    assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
    check_csr_untouched(ro_d, ci_d, ro, ci)
    empty = np.diff(ro) == 0
    assert (got[empty] == 0).all(), "rows without nonzeros must be written as exact zeros"


SDDMM_CASES = [
    (1, 1, 1, "full", 1.0),
    (7, 9, 4, "uniform", 0.5),
    (64, 64, 16, "uniform", 0.3),
    (100, 300, 32, "uniform", 0.1),
    (130, 257, 64, "skewed", 0.1),
    (256, 512, 128, "uniform", 0.05),
    (99, 200, 256, "skewed", 0.1),
    (40, 128, 512, "uniform", 0.2),
    (30, 64, 1024, "uniform", 0.3),
    (50, 100, 48, "uniform", 0.2),
    (50, 100, 100, "skewed", 0.2),
    (33, 77, 13, "uniform", 0.3),
    (64, 128, 1, "uniform", 0.3),
    (200, 300, 128, "empty_rows", 0.1),
    (8, 1500, 128, "full", 1.0),
    (20, 40, 0, "uniform", 0.3),
    # inner dimensions that are not a multiple of 4 (the straddling lane reads the last four floats, overlap zeroed)
    (40, 60, 2, "uniform", 0.3),
    (40, 60, 3, "skewed", 0.3),
    (40, 60, 5, "uniform", 0.3),
    (40, 60, 6, "uniform", 0.3),
    (40, 60, 7, "empty_rows", 0.3),
    (40, 60, 17, "uniform", 0.3),
    (40, 60, 33, "skewed", 0.3),
    (40, 60, 49, "uniform", 0.3),
    (40, 60, 63, "uniform", 0.3),
    (40, 60, 65, "uniform", 0.3),
    (40, 60, 130, "skewed", 0.3),
    (40, 60, 257, "uniform", 0.3),
    (30, 60, 513, "uniform", 0.3),
    (20, 60, 1027, "uniform", 0.3),
]


@pytest.mark.parametrize("M,K,D,kind,density", SDDMM_CASES)
def test_sddmm_matches_oracle(torch_cuda, dl, oracle, M, K, D, kind, density):
    torch = torch_cuda
    rng = np.random.default_rng(4321 + M * 5 + D)
    ro, ci = random_csr(rng, M, K, kind, density)
    lhs = rng.normal(0, 1, (M, D)).astype(np.float32)
    rhs = rng.normal(0, 1, (K, D)).astype(np.float32)
    ref = oracle.sddmm(ro, ci, lhs, rhs)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    out = torch.full((ci.size,), float("nan"), dtype=torch.float32, device="cuda")
    dl.sddmm(ro_d, ci_d, dev(torch, lhs), dev(torch, rhs), out=out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.isfinite(got).all(), "a CSR slot was not written"
    assert oracle.rel_frobenius(got, ref) <= TOL
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("D", [20, 68, 80, 96, 100, 132, 160, 192, 200, 224, 300, 320, 384, 500])
@pytest.mark.parametrize("op", ["sddmm", "fused"])
def test_widths_between_the_powers_of_two(torch_cuda, dl, oracle, op, D):
    """Dot products of D floats are gathered in accesses of 32 floats per nonzero: 1, 2, 3, 4, 6, 8, 12 or 16 of them, the last
    ones past D for some or all lanes. Those lanes add nothing, whatever the floats they re-read are: with an infinity
    at the start of some rows of rhs (where such lanes read) and finite floats everywhere else in those columns' products,
    every result is the oracle's -- infinite where the oracle's is, never a NaN out of 0 * inf."""
    torch = torch_cuda
    rng = np.random.default_rng(977 + D)
    M, K = 300, 400
    ro, ci = random_csr(rng, M, K, "uniform", 0.2)
    lhs = rng.normal(0, 1, (M, D)).astype(np.float32)
    rhs = rng.normal(0, 1, (K, D)).astype(np.float32)
    lhs[:, 0] = np.abs(lhs[:, 0]) + 0.5  # a positive first factor: inf * it is +inf, nothing cancels
    hot = rng.random(K) < 0.1
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    for poisoned in (False, True):
        if poisoned:
            rhs[hot, 0] = np.inf
        if op == "sddmm":
            sh = dl.describe_launch(dl.OP_SDDMM, M, K, D, ci.size)
            assert sh["DS"] == (1 if D <= 32 else next(n for n in (2, 3, 4, 6, 8, 12, 16) if D <= 32 * n))
            got = dl.sddmm(ro_d, ci_d, dev(torch, lhs), dev(torch, rhs)).cpu().numpy()
            with np.errstate(invalid="ignore", over="ignore"):
                ref = oracle.sddmm(ro, ci, lhs, rhs)
            assert not np.isnan(got).any()
            inf = np.isinf(ref)
            assert inf.any() == poisoned and np.array_equal(np.isinf(got), inf) and np.array_equal(got[inf], ref[inf])
            assert oracle.rel_frobenius(got[~inf], ref[~inf]) <= TOL
            # the lanes past D are masked by the range of a buffer where D is a multiple of four, by selects otherwise,
            # under a plan like without: the same bits either way
            kinds = [dl.sddmm(ro_d, ci_d, dev(torch, lhs), dev(torch, rhs), plan=p) for p in (dl.row_plan(ro_d), dl.cut_plan(ro_d, dl.OP_SDDMM, D))]
            dl.set_tuning(rules_off=dl.RULES["mask_by_range"])
            try:
                kinds += [dl.sddmm(ro_d, ci_d, dev(torch, lhs), dev(torch, rhs), plan=p) for p in (None, dl.row_plan(ro_d), dl.cut_plan(ro_d, dl.OP_SDDMM, D))]
            finally:
                dl.set_tuning()
            for other in kinds:
                assert np.array_equal(other.cpu().numpy(), got, equal_nan=True)
        elif not poisoned:  # (the fused op would add inf * V rows of both signs: its oracle holds NaN there)
            V = rng.normal(0, 1, (K, D)).astype(np.float32)
            ops = (dev(torch, lhs), dev(torch, rhs), dev(torch, V))
            got = dl.fused(ro_d, ci_d, *ops, scale=0.1)
            assert oracle.rel_frobenius(got.cpu().numpy(), oracle.fused(ro, ci, lhs, rhs, V, scale=0.1)) <= TOL
            # (D = 257 ... 383: the first stage masks by range too; the bits of the kernels that mask by selects, planned or not)
            plans = (None, dl.row_plan(ro_d), dl.cut_plan(ro_d, dl.OP_FUSED, D))
            with_rule = [got] + [dl.fused(ro_d, ci_d, *ops, scale=0.1, plan=p) for p in plans[1:]]
            dl.set_tuning(rules_off=dl.RULES["mask_by_range"])
            try:
                without = [dl.fused(ro_d, ci_d, *ops, scale=0.1, plan=p) for p in plans]
            finally:
                dl.set_tuning()
            for a, b in zip(with_rule, without):
                assert torch.equal(a, b)
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("schedule,M,K,D,density", [("flat", 4096, 8192, 80, 0.07), ("sliced", 2048, 16384, 160, 0.03)])
def test_sddmm_flat_and_sliced_schedules_at_widths_between_the_powers_of_two(torch_cuda, dl, oracle, schedule, M, K, D, density):
    """The kernels of SDDMM's flat schedule (taken by the sizes alone) and of its column-sliced schedule (with workspace)
    mask the lanes past D by the range of a buffer too: the oracle's values, and the bits of the kernels that mask by selects."""
    torch = torch_cuda
    ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 201, M, K, density)
    nnz = ci.size
    lhs = dl.fill("normal", 202, (M, D), 0.0, 1.0)
    rhs = dl.fill("normal", 203, (K, D), 0.0, 1.0)
    ro_d, ci_d, lhs_d, rhs_d = (dev(torch, x) for x in (ro, ci, lhs, rhs))
    if schedule == "flat":
        assert dl.describe_launch(dl.OP_SDDMM, M, K, D, nnz)["flat_chunk"] > 0
        run = lambda: dl.sddmm(ro_d, ci_d, lhs_d, rhs_d)
    else:
        assert dl.describe_slices(dl.OP_SDDMM, M, K, D, nnz)[0] > 1
        ws = torch.empty(dl.workspace_bytes(dl.OP_SDDMM, M, K, D, nnz), dtype=torch.uint8, device="cuda")
        run = lambda: dl.sddmm(ro_d, ci_d, lhs_d, rhs_d, workspace=ws)
    got = run()
    assert oracle.rel_frobenius(got.cpu().numpy(), oracle.sddmm(ro, ci, lhs, rhs, omp=True)) <= TOL
    dl.set_tuning(rules_off=dl.RULES["mask_by_range"])
    try:
        by_selects = run()
    finally:
        dl.set_tuning()
    assert torch.equal(got, by_selects)
    check_csr_untouched(ro_d, ci_d, ro, ci)


def test_sddmm_rhs_beyond_the_window_of_the_range_masked_kernels(torch_cuda, dl, oracle):
    """rhs of 3.4 million rows of 80 floats (1.09 GB) does not fit the 1 GiB buffer whose range check masks the lanes past D: the
    call takes the kernels that mask by selects, with columns from the whole of rhs."""
    torch = torch_cuda
    M, K, D = 96, 3_400_000, 80
    rng = np.random.default_rng(2718)
    lens = rng.integers(40, 90, M)
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens]).astype(np.int32)
    ci[-1] = K - 1  # the last row of rhs is read too
    lhs = rng.normal(0, 1, (M, D)).astype(np.float32)
    gen = torch.Generator(device="cuda").manual_seed(5)
    rhs_d = torch.randn((K, D), dtype=torch.float32, device="cuda", generator=gen)
    used, where = np.unique(ci, return_inverse=True)
    rhs_used = rhs_d[torch.from_numpy(used.astype(np.int64)).cuda()].cpu().numpy()
    ref = oracle.sddmm(ro, where.astype(np.int32), lhs, rhs_used)
    got = dl.sddmm(dev(torch, ro), dev(torch, ci), dev(torch, lhs), rhs_d).cpu().numpy()
    assert oracle.rel_frobenius(got, ref) <= TOL
    del rhs_d
    torch.cuda.empty_cache()


FUSED_CASES = [
    (1, 1, 4, "full", 1.0, 1.0),
    (9, 11, 8, "uniform", 0.5, 1.0),
    (64, 64, 16, "uniform", 0.3, 0.25),
    (100, 300, 32, "uniform", 0.1, 1.0),
    (130, 257, 64, "skewed", 0.1, 0.125),
    (256, 512, 128, "uniform", 0.05, 1.0),
    (99, 200, 256, "skewed", 0.1, 0.0625),
    (40, 128, 512, "uniform", 0.2, 1.0),
    (20, 64, 1024, "uniform", 0.3, 1.0),
    (12, 64, 2048 + 64, "uniform", 0.3, 1.0),
    (50, 100, 48, "uniform", 0.2, 1.0),
    (33, 77, 13, "uniform", 0.3, 0.5),
    (200, 300, 64, "empty_rows", 0.1, 0.125),
    (8, 1500, 64, "full", 1.0, 0.125),
    (64, 128, 64, "empty", 0.0, 1.0),
    (40, 60, 1, "uniform", 0.3, 1.0),
    (40, 60, 2, "uniform", 0.3, 0.5),
    (40, 60, 3, "skewed", 0.3, 1.0),
    (40, 60, 5, "uniform", 0.3, 1.0),
    (40, 60, 7, "empty_rows", 0.3, 0.5),
    (40, 60, 17, "uniform", 0.3, 1.0),
    (40, 60, 49, "skewed", 0.3, 0.125),
    (40, 60, 65, "uniform", 0.3, 1.0),
    (40, 60, 130, "uniform", 0.3, 1.0),
    (40, 60, 257, "skewed", 0.3, 1.0),
    (30, 60, 513, "uniform", 0.3, 1.0),
    (20, 60, 1027, "uniform", 0.3, 1.0),
]


@pytest.mark.parametrize("M,K,D,kind,density,scale", FUSED_CASES)
def test_fused_matches_oracle(torch_cuda, dl, oracle, M, K, D, kind, density, scale):
    torch = torch_cuda
    rng = np.random.default_rng(999 + M * 3 + D)
    ro, ci = random_csr(rng, M, K, kind, density)
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    V = rng.normal(0, 1, (K, D)).astype(np.float32)
    ref = oracle.fused(ro, ci, Q, Km, V, scale)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    O = torch.full((M, D), float("nan"), dtype=torch.float32, device="cuda")
    dl.fused(ro_d, ci_d, dev(torch, Q), dev(torch, Km), dev(torch, V), scale, out=O)
    torch.cuda.synchronize()
    got = O.cpu().numpy()
    assert np.isfinite(got).all(), "an output element was not written"
    assert oracle.rel_frobenius(got, ref) <= TOL
    check_csr_untouched(ro_d, ci_d, ro, ci)
    empty = np.diff(ro) == 0
    assert (got[empty] == 0).all()


GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "fused_ref_M*_K*_N*.npz")))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_kernels_against_the_references_own_outputs(torch_cuda, dl, oracle, path):
    """Directly against what the REFERENCE's functions (compiled from its FUSED/fused.cpp) returned for the fixture's
    inputs: Sddmm, Spmm applied to those scores (= the fused gold, no scale), the fp32 SpMM emulation and the fp32
    fused emulation. No oracle in between."""
    torch = torch_cuda
    z = np.load(path)
    ro, ci = z["row_offsets"], z["col_indices"]
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    K = z["b"].shape[0]
    got = dl.sddmm(ro_d, ci_d, dev(torch, z["c"]), dev(torch, z["b"])).cpu().numpy()
    assert oracle.rel_frobenius(got, z["sddmm"]) <= TOL
    got = dl.spmm(ro_d, ci_d, dev(torch, z["values"]), dev(torch, z["d"]), K=K).cpu().numpy()
    assert oracle.rel_frobenius(got, z["spmm_f32"]) <= TOL
    got = dl.spmm(ro_d, ci_d, dev(torch, z["sddmm"]), dev(torch, z["d"]), K=K).cpu().numpy()
    assert oracle.rel_frobenius(got, z["spmm_f64acc"]) <= TOL
    got = dl.fused(ro_d, ci_d, dev(torch, z["c"]), dev(torch, z["b"]), dev(torch, z["d"]), 1.0).cpu().numpy()
    assert oracle.rel_frobenius(got, z["spmm_f64acc"]) <= TOL   # the reference's gold: Sddmm then Spmm
    assert oracle.rel_frobenius(got, z["fused_emul"]) <= TOL    # and its own fp32 emulation of the fused kernel
    check_csr_untouched(ro_d, ci_d, ro, ci)


def test_fused_equals_unfused_on_gpu(torch_cuda, dl, oracle):
    """fused(Q, K, V, scale) == spmm(sddmm(Q, K) * scale, V), both on the GPU (the reference checks its fused
    emulation against Sddmm -> Spmm the same way, FUSED/fused.cpp:400-413)."""
    torch = torch_cuda
    rng = np.random.default_rng(5)
    M, K, D, scale = 300, 400, 64, 0.125
    ro, ci = random_csr(rng, M, K, "skewed", 0.1)
    Q, Km, V = (dev(torch, rng.normal(0, 1, s).astype(np.float32)) for s in ((M, D), (K, D), (K, D)))
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    scores = dl.sddmm(ro_d, ci_d, Q, Km) * scale
    unfused = dl.spmm(ro_d, ci_d, scores, V, K=K)
    fusedO = dl.fused(ro_d, ci_d, Q, Km, V, scale)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(fusedO.cpu().numpy(), unfused.cpu().numpy()) <= 1e-5


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_benchmark_configs_full_size(torch_cuda, dl, oracle, cfg):
    """The five BASELINE.json configurations at full size against the oracle."""
    torch = torch_cuda
    c = dl.make_config(cfg)
    ro_d, ci_d = dev(torch, c["row_offsets"]), dev(torch, c["col_indices"])
    if c["op"] == dl.OP_SPMM:
        ref = oracle.spmm(c["row_offsets"], c["col_indices"], c["values"], c["d0"], omp=True)
        got = dl.spmm(ro_d, ci_d, dev(torch, c["values"]), dev(torch, c["d0"]), K=c["K"])
    elif c["op"] == dl.OP_SDDMM:
        ref = oracle.sddmm(c["row_offsets"], c["col_indices"], c["d0"], c["d1"], omp=True)
        got = dl.sddmm(ro_d, ci_d, dev(torch, c["d0"]), dev(torch, c["d1"]))
    else:
        ref = oracle.fused(c["row_offsets"], c["col_indices"], c["d0"], c["d1"], c["d2"], c["scale"], omp=True)
        got = dl.fused(ro_d, ci_d, dev(torch, c["d0"]), dev(torch, c["d1"]), dev(torch, c["d2"]), c["scale"])
    torch.cuda.synchronize()
    err = oracle.rel_frobenius(got.cpu().numpy(), ref)
    print(f"cfg{cfg} {c['name']}: nnz={c['nnz']} rel_frobenius={err:.3e}")
    assert err <= TOL
    check_csr_untouched(ro_d, ci_d, c["row_offsets"], c["col_indices"])
    assert dl.csr_check(c["M"], c["K"], ro_d, ci_d) == dl.OK


@pytest.mark.parametrize("off", [1, 2, 3])
def test_misaligned_operands(torch_cuda, dl, oracle, off):
    """Dense operands and outputs that start 4, 8 or 12 bytes off a 16-byte boundary (dwordx4 accesses need only
    dword alignment), all three entry points, widths that are and are not multiples of 4."""
    torch = torch_cuda
    rng = np.random.default_rng(77 + off)

    def shifted(a):
        buf = torch.empty(a.size + off, dtype=torch.float32, device="cuda")
        view = buf[off:].view(*a.shape)
        view.copy_(torch.from_numpy(a))
        assert view.data_ptr() % 16 == 4 * off
        return view

    for N in (64, 50, 48, 80):  # (48, 80: SDDMM reads rhs through a buffer descriptor whose range check masks the lanes past D)
        M, K = 60, 90
        ro, ci = random_csr(rng, M, K, "skewed", 0.2)
        va = rng.uniform(-1, 1, ci.size).astype(np.float32)
        B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        Q = rng.normal(0, 1, (M, N)).astype(np.float32)
        V = rng.normal(0, 1, (K, N)).astype(np.float32)
        ro_d, ci_d = dev(torch, ro), dev(torch, ci)
        C = shifted(np.full((M, N), np.nan, dtype=np.float32))
        dl.spmm(ro_d, ci_d, shifted(va), shifted(B), K=K, out=C)
        assert oracle.rel_frobenius(C.cpu().numpy(), oracle.spmm(ro, ci, va, B)) <= TOL
        out = shifted(np.full(ci.size, np.nan, dtype=np.float32))
        dl.sddmm(ro_d, ci_d, shifted(Q), shifted(B), out=out)
        assert oracle.rel_frobenius(out.cpu().numpy(), oracle.sddmm(ro, ci, Q, B)) <= TOL
        O = shifted(np.full((M, N), np.nan, dtype=np.float32))
        dl.fused(ro_d, ci_d, shifted(Q), shifted(B), shifted(V), 0.5, out=O)
        assert oracle.rel_frobenius(O.cpu().numpy(), oracle.fused(ro, ci, Q, B, V, 0.5)) <= TOL


def test_deterministic(torch_cuda, dl):
    """Two launches on the same inputs give bit-identical outputs (no atomics anywhere)."""
    torch = torch_cuda
    c = dl.make_config(2)
    args = [dev(torch, c[k]) for k in ("row_offsets", "col_indices", "values", "d0")]
    a = dl.spmm(*args, K=c["K"]).clone()
    b = dl.spmm(*args, K=c["K"]).clone()
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_linearity_at_full_size(torch_cuda, dl, oracle):
    """Size-independent property at cfg4's shape: spmm(A, B1 + B2) == spmm(A, B1) + spmm(A, B2) up to rounding."""
    torch = torch_cuda
    c = dl.make_config(4)
    ro, ci, va = (dev(torch, c[k]) for k in ("row_offsets", "col_indices", "values"))
    B1 = dev(torch, c["d0"])
    B2 = torch.flip(B1, dims=[0]).contiguous()
    lhs = dl.spmm(ro, ci, va, (B1 + B2).contiguous(), K=c["K"])
    rhs = dl.spmm(ro, ci, va, B1, K=c["K"]) + dl.spmm(ro, ci, va, B2, K=c["K"])
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(lhs.cpu().numpy(), rhs.cpu().numpy()) <= 1e-5


def test_large_shape_against_oracle(torch_cuda, dl, oracle):
    """The largest shape of the reference's synthetic sweep (SPMM/batch-run-spmm:9-12: M = 32768, K = 8192, N = 128,
    here at its 10 % density) against the multi-threaded oracle: 26.8 M nonzeros."""
    torch = torch_cuda
    M, K, N = 32768, 8192, 128
    ro, ci = dl.make_pattern(dl.PATTERN_UNIFORM_ROWS, 21, M, K, 0.1 * K, 0.0)
    va = dl.fill("uniform", 22, (ci.size,), -1.0, 1.0)
    B = dl.fill("uniform", 23, (K, N), -1.0, 1.0)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    got = dl.spmm(ro_d, ci_d, dev(torch, va), dev(torch, B), K=K)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(got.cpu().numpy(), oracle.spmm(ro, ci, va, B, omp=True)) <= TOL
    check_csr_untouched(ro_d, ci_d, ro, ci)


def test_sddmm_results_beyond_the_l2_are_streamed(torch_cuda, dl, oracle):
    """More results than one and a half L2s hold (here 9.4 million = 38 MB; an MI355X's L2 is 4 MiB) are stored with the
    non-temporal hint; the bits must be those of ordinary stores under every schedule: row blocks, the
    even-rows hint, a row plan, and the flat schedule forced by tuning, all against the multi-threaded oracle and equal
    to each other."""
    torch = torch_cuda
    M, K, D = 8192, 8192, 32
    ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 71, M, K, 0.14)
    info = dl.device_info()
    assert ci.size * 4 > 1.5 * info["l2_bytes"]
    lhs = dl.fill("normal", 72, (M, D), 0.0, 1.0)
    rhs = dl.fill("normal", 73, (K, D), 0.0, 1.0)
    want = oracle.sddmm(ro, ci, lhs, rhs, omp=True)
    ro_d, ci_d, lhs_d, rhs_d = (dev(torch, x) for x in (ro, ci, lhs, rhs))
    first = None
    for name in ("null", "rows_even", "plan", "flat"):
        if name == "flat":
            dl.set_tuning(flat=1)
        got = dl.sddmm(ro_d, ci_d, lhs_d, rhs_d, workspace=dl.ROWS_EVEN if name == "rows_even" else None,
                       plan=dl.row_plan(ro_d) if name == "plan" else None).cpu().numpy()
        dl.set_tuning()
        assert oracle.rel_frobenius(got, want) <= TOL, name
        first = got if first is None else first
        assert np.array_equal(got, first), name
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("sigma", [0.0, 1.5])
def test_flat_schedule_at_its_own_sizes(torch_cuda, dl, oracle, sigma):
    """A matrix large enough (3.4 M nonzeros, 410 per row on average, N = 128) that a call WITH workspace takes the flat
    schedule by the library's own rule: uniform rows and heavily skewed rows (lognormal, sigma 1.5: rows from 0 to 4096
    nonzeros), SpMM and the fused op against the multi-threaded oracle; the same call without workspace must agree."""
    torch = torch_cuda
    M, K, N = 8192, 4096, 128
    if sigma == 0.0:
        ro, ci = dl.make_pattern(dl.PATTERN_UNIFORM_ROWS, 61, M, K, 0.1)
    else:
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 62, M, K, 0.1 * K, sigma)
    nnz = ci.size
    va = dl.fill("uniform", 63, (nnz,), -1.0, 1.0)
    B = dl.fill("uniform", 64, (K, N), -1.0, 1.0)
    Q = dl.fill("normal", 65, (M, N), 0.0, 1.0)
    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz)
    need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, nnz)
    assert sh["flat_chunk"] > 0 and need == sh["flat_units"] * 2 * N * 4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ro_d, ci_d, va_d, B_d, Q_d = (dev(torch, x) for x in (ro, ci, va, B, Q))
    got = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, workspace=ws)
    ref = oracle.spmm(ro, ci, va, B, omp=True)
    assert oracle.rel_frobenius(got.cpu().numpy(), ref) <= TOL
    assert oracle.rel_frobenius(dl.spmm(ro_d, ci_d, va_d, B_d, K=K).cpu().numpy(), ref) <= TOL
    assert (got.cpu().numpy()[np.diff(ro) == 0] == 0).all()

    assert dl.describe_launch(dl.OP_SDDMM, M, K, N, nnz)["flat_chunk"] > 0  # SDDMM: by the size rule alone
    gotS = dl.sddmm(ro_d, ci_d, Q_d, B_d)
    assert oracle.rel_frobenius(gotS.cpu().numpy(), oracle.sddmm(ro, ci, Q, B, omp=True)) <= TOL

    needf = dl.workspace_bytes(dl.OP_FUSED, M, K, N, nnz)
    assert needf > 0
    wsf = torch.empty(needf, dtype=torch.uint8, device="cuda")
    gotO = dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.01, workspace=wsf)
    refO = oracle.fused(ro, ci, Q, B, B, 0.01, omp=True)
    assert oracle.rel_frobenius(gotO.cpu().numpy(), refO) <= TOL
    assert oracle.rel_frobenius(dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.01).cpu().numpy(), refO) <= TOL
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("sigma", [0.0, 1.5])
def test_column_sliced_schedule_at_its_own_sizes(torch_cuda, dl, oracle, sigma):
    """Dense operands of 16 MiB (SpMM, SDDMM) and 32 MiB (fused) at K = 16384, N = D = 256: a call WITH workspace takes
    the column-sliced schedule by the library's own rule (SpMM: 3 slices of each of its two column tiles; SDDMM 8, fused
    12 slices); all three ops against the multi-threaded oracle, on near-uniform and on heavily skewed rows, and the
    same calls without workspace must agree."""
    torch = torch_cuda
    M, K, N = 4096, 16384, 256
    if sigma == 0.0:
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 71, M, K, 0.05)
    else:
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 72, M, K, 0.05 * K, sigma)
    nnz = ci.size
    va = dl.fill("uniform", 73, (nnz,), -1.0, 1.0)
    B = dl.fill("uniform", 74, (K, N), -1.0, 1.0)
    Q = dl.fill("normal", 75, (M, N), 0.0, 1.0)
    ro_d, ci_d, va_d, B_d, Q_d = (dev(torch, x) for x in (ro, ci, va, B, Q))
    assert dl.describe_slices(dl.OP_SPMM, M, K, N, nnz)[0] == 3 and dl.describe_launch(dl.OP_SPMM, M, K, N, nnz, with_workspace=True)["col_tiles"] == 2
    assert dl.describe_slices(dl.OP_SDDMM, M, K, N, nnz)[0] == 8
    assert dl.describe_slices(dl.OP_FUSED, M, K, N, nnz)[0] == 12

    ws = torch.empty(dl.workspace_bytes(dl.OP_SPMM, M, K, N, nnz), dtype=torch.uint8, device="cuda")
    got = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, workspace=ws)
    ref = oracle.spmm(ro, ci, va, B, omp=True)
    assert oracle.rel_frobenius(got.cpu().numpy(), ref) <= TOL
    assert oracle.rel_frobenius(dl.spmm(ro_d, ci_d, va_d, B_d, K=K).cpu().numpy(), ref) <= TOL
    assert (got.cpu().numpy()[np.diff(ro) == 0] == 0).all()

    wss = torch.empty(dl.workspace_bytes(dl.OP_SDDMM, M, K, N, nnz), dtype=torch.uint8, device="cuda")
    gotS = dl.sddmm(ro_d, ci_d, Q_d, B_d, workspace=wss)
    assert torch.equal(gotS, dl.sddmm(ro_d, ci_d, Q_d, B_d))
    assert oracle.rel_frobenius(gotS.cpu().numpy(), oracle.sddmm(ro, ci, Q, B, omp=True)) <= TOL

    wsf = torch.empty(dl.workspace_bytes(dl.OP_FUSED, M, K, N, nnz), dtype=torch.uint8, device="cuda")
    gotO = dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.01, workspace=wsf)
    refO = oracle.fused(ro, ci, Q, B, B, 0.01, omp=True)
    assert oracle.rel_frobenius(gotO.cpu().numpy(), refO) <= TOL
    assert oracle.rel_frobenius(dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.01).cpu().numpy(), refO) <= TOL
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("M,K,N,per_row,tile,tiles", [
    (128, 1152, 256, 200, 64, 4), (64, 576, 512, 100, 64, 8), (16, 576, 500, 100, 32, 16), (128, 1152, 196, 200, 128, 2),
    (5, 300, 50, 40, 32, 2), (1000, 512, 784, 100, 256, 4), (300, 1152, 3140, 100, 128, 25), (130, 2304, 1030, 60, 64, 17),
    (32, 2304, 2048, 230, 128, 16), (700, 4608, 650, 100, 64, 11), (64, 147, 12548, 75, 128, 99), (300, 4608, 500, 300, 64, 8)])
@pytest.mark.parametrize("sigma", [0.0, 0.8])
def test_finer_column_tiles_of_plain_spmm_calls(torch_cuda, dl, oracle, M, K, N, per_row, tile, tiles, sigma):
    """The column tiles a SpMM call without memory takes for few rows and for wide dense rows (row-major tiles of
    32 ... 256 columns; where B exceeds the L2 every XCD on its own tiles of 64 or 128 columns, with 1 ... 3 tiles left
    over that all XCDs share; last tiles of 4, 6 and 10 columns among them):
    NULL and the even-rows hint against the oracle, and against the same call with the rule switched off."""
    torch = torch_cuda
    if sigma == 0.0:
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 171, M, K, per_row / K)
    else:
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 172, M, K, float(per_row), sigma)
    nnz = ci.size
    va = dl.fill("uniform", 173, (nnz,), -1.0, 1.0)
    B = dl.fill("uniform", 174, (K, N), -1.0, 1.0)
    ro_d, ci_d, va_d, B_d = (dev(torch, x) for x in (ro, ci, va, B))
    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz)
    if nnz >= 16 * M:
        assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (tile, tiles)
    ref = oracle.spmm(ro, ci, va, B, omp=True)
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    dl.spmm(ro_d, ci_d, va_d, B_d, K=K, out=out)
    assert oracle.rel_frobenius(out.cpu().numpy(), ref) <= TOL
    out.fill_(float("nan"))
    dl.spmm(ro_d, ci_d, va_d, B_d, K=K, out=out, workspace=dl.ROWS_EVEN)
    assert oracle.rel_frobenius(out.cpu().numpy(), ref) <= TOL
    dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
    try:
        assert dl.describe_launch(dl.OP_SPMM, M, K, N, nnz)["col_tiles"] < tiles
        off = dl.spmm(ro_d, ci_d, va_d, B_d, K=K)
    finally:
        dl.set_tuning()
    assert oracle.rel_frobenius(off.cpu().numpy(), ref) <= TOL
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("M,K,D,per_row,pieces", [
    (128, 1152, 128, 230, 4), (16, 576, 64, 400, 8), (1, 700, 256, 700, 16), (64, 4608, 100, 1400, 8), (192, 2304, 32, 230, 4),
    (7, 300, 16, 140, 4), (100, 512, 128, 60, 1), (193, 2304, 128, 230, 2), (384, 576, 256, 300, 2), (385, 2304, 128, 230, 1)])
@pytest.mark.parametrize("sigma", [0.0, 0.8])
def test_row_pieces_of_plain_sddmm_calls_on_few_rows(torch_cuda, dl, oracle, M, K, D, per_row, pieces, sigma):
    """Few rows: 2, 4, ... 16 workgroups share each row of a SDDMM call without plan or memory (two from three quarters to
    one and a half of the compute units' count of rows). Every result is still
    one nonzero's own dot product: the bits of the same call with the rule switched off, and the oracle's values."""
    torch = torch_cuda
    if sigma == 0.0:
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 181, M, K, per_row / K)
    else:
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 182, M, K, float(per_row), sigma)
    nnz = ci.size
    lhs = dl.fill("normal", 183, (M, D), 0.0, 1.0)
    rhs = dl.fill("normal", 184, (K, D), 0.0, 1.0)
    ro_d, ci_d, lhs_d, rhs_d = (dev(torch, x) for x in (ro, ci, lhs, rhs))
    sh = dl.describe_launch(dl.OP_SDDMM, M, K, D, nnz)
    if sigma == 0.0:
        assert sh["col_tiles"] == pieces and (pieces == 1 or (sh["W"], sh["R"]) == (4, 1))
    out = torch.full((nnz,), float("nan"), dtype=torch.float32, device="cuda")
    dl.sddmm(ro_d, ci_d, lhs_d, rhs_d, out=out)
    assert oracle.rel_frobenius(out.cpu().numpy(), oracle.sddmm(ro, ci, lhs, rhs, omp=True)) <= TOL
    even = dl.sddmm(ro_d, ci_d, lhs_d, rhs_d, workspace=dl.ROWS_EVEN)
    dl.set_tuning(rules_off=dl.RULES["row_pieces_few_rows"])
    try:
        assert dl.describe_launch(dl.OP_SDDMM, M, K, D, nnz)["col_tiles"] == 1
        off = dl.sddmm(ro_d, ci_d, lhs_d, rhs_d)
    finally:
        dl.set_tuning()
    assert torch.equal(out, off) and torch.equal(even, off)
    check_csr_untouched(ro_d, ci_d, ro, ci)


@pytest.mark.parametrize("sigma", [0.0, 1.0])
def test_sliced_column_tiles_on_a_tall_wide_dense_operand(torch_cuda, dl, oracle, sigma):
    """B of 24576 x 392 floats (37 MiB; not even a tile of 128 columns fits twice the L2) under rows of ~130 nonzeros:
    a call WITH workspace works in four column tiles of 128 (the last one 8 columns wide) and cuts each into slices,
    a call without in tiles of 32; both against the multi-threaded oracle, and the integer-exact row lengths."""
    torch = torch_cuda
    M, K, N = 4100, 24576, 392
    if sigma == 0.0:
        ro, ci = dl.make_pattern(dl.PATTERN_BERNOULLI, 81, M, K, 130.0 / K)
    else:
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 82, M, K, 130.0, sigma)
    nnz = ci.size
    assert nnz >= 1 << 19
    va = dl.fill("uniform", 83, (nnz,), -1.0, 1.0)
    B = dl.fill("uniform", 84, (K, N), -1.0, 1.0)
    ro_d, ci_d, va_d, B_d = (dev(torch, x) for x in (ro, ci, va, B))
    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz, with_workspace=True)
    assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (128, 4)
    slices, R = dl.describe_slices(dl.OP_SPMM, M, K, N, nnz)
    assert slices == 4 and R == 2                       # 32 nonzeros per row and slice; 2050 workgroups per (slice, tile)
    assert dl.describe_launch(dl.OP_SPMM, M, K, N, nnz)["col_tiles"] == 13   # without memory: tiles of 32

    ws = torch.empty(dl.workspace_bytes(dl.OP_SPMM, M, K, N, nnz), dtype=torch.uint8, device="cuda")
    got = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, workspace=ws)
    ref = oracle.spmm(ro, ci, va, B, omp=True)
    assert oracle.rel_frobenius(got.cpu().numpy(), ref) <= TOL
    assert oracle.rel_frobenius(dl.spmm(ro_d, ci_d, va_d, B_d, K=K).cpu().numpy(), ref) <= TOL
    assert (got.cpu().numpy()[np.diff(ro) == 0] == 0).all()
    ones_v, ones_B = torch.ones(nnz, device="cuda"), torch.ones(K, N, device="cuda")
    lengths = torch.from_numpy(np.diff(ro).astype(np.float32)).cuda()[:, None].expand(M, N)
    assert torch.equal(dl.spmm(ro_d, ci_d, ones_v, ones_B, K=K, workspace=ws), lengths)
    check_csr_untouched(ro_d, ci_d, ro, ci)


def test_exact_integer_properties_at_large_size(torch_cuda, dl):
    """Size-independent, bit-exact checks on 65536 skewed rows (several million nonzeros), no oracle needed: with small-integer
    operands every fp32 product and sum is exact whatever the summation order, so
      SpMM  with A = 1, B = 1            gives C[i, :] = length of row i,
      SDDMM with lhs = 1, rhs[k, :] = k/D gives out[j] = col_indices[j]   (D a power of two),
      fused with those and V = 1          gives O[i, :] = sum of row i's column indices."""
    torch = torch_cuda
    M, K, D = 65536, 4096, 128
    ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 31, M, K, 64.0, 1.0)
    lens = np.diff(ro).astype(np.int64)
    colsum = np.add.reduceat(np.append(ci.astype(np.int64), 0), ro[:-1])[:M] * (lens > 0)
    assert colsum.max() < 2**24
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    ones_nnz = torch.ones(ci.size, dtype=torch.float32, device="cuda")
    ones_KD = torch.ones(K, D, dtype=torch.float32, device="cuda")
    ones_MD = torch.ones(M, D, dtype=torch.float32, device="cuda")
    ramp = (torch.arange(K, dtype=torch.float32, device="cuda") / D)[:, None].expand(K, D).contiguous()

    C = dl.spmm(ro_d, ci_d, ones_nnz, ones_KD, K=K)
    assert torch.equal(C, torch.from_numpy(lens.astype(np.float32)).cuda()[:, None].expand(M, D))
    out = dl.sddmm(ro_d, ci_d, ones_MD, ramp)
    assert torch.equal(out, ci_d.to(torch.float32))
    O = dl.fused(ro_d, ci_d, ones_MD, ramp, ones_KD, 1.0)
    assert torch.equal(O, torch.from_numpy(colsum.astype(np.float32)).cuda()[:, None].expand(M, D))
    check_csr_untouched(ro_d, ci_d, ro, ci)

    # the same properties through the planned entry points, on rows long enough (200 on average) that the planned SpMM
    # launch really runs in plan order (65536 workgroups, one row each); 16384 rows for the other two ops
    for rows, planned_ops in ((65536, (dl.OP_SPMM,)), (16384, (dl.OP_SPMM, dl.OP_SDDMM, dl.OP_FUSED))):
        ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 32, rows, K, 200.0 if rows == 65536 else 400.0, 1.0)
        lens = np.diff(ro).astype(np.int64)
        colsum = np.add.reduceat(np.append(ci.astype(np.int64), 0), ro[:-1])[:rows] * (lens > 0)
        assert colsum.max() < 2**24
        for op in planned_ops:
            assert dl.row_plan_advice(op, rows, K, D, ci.size, int(lens.max()))
        ro_d, ci_d = dev(torch, ro), dev(torch, ci)
        plan = dl.row_plan(ro_d)
        ones_nnz = torch.ones(ci.size, dtype=torch.float32, device="cuda")
        C = dl.spmm(ro_d, ci_d, ones_nnz, ones_KD, K=K, plan=plan)
        assert torch.equal(C, torch.from_numpy(lens.astype(np.float32)).cuda()[:, None].expand(rows, D))
        out = dl.sddmm(ro_d, ci_d, ones_MD[:rows], ramp, plan=plan)
        assert torch.equal(out, ci_d.to(torch.float32))
        O = dl.fused(ro_d, ci_d, ones_MD[:rows], ramp, ones_KD, 1.0, plan=plan)
        assert torch.equal(O, torch.from_numpy(colsum.astype(np.float32)).cuda()[:, None].expand(rows, D))
        check_csr_untouched(ro_d, ci_d, ro, ci)


def test_row_plan_changes_the_order_of_the_rows_only(torch_cuda, dl, oracle):
    """spmm_csr_f32 with a row plan hands the rows to the workgroups in the plan's order (longest first), one row per four-wave
    workgroup, and must return the bits of spmm_csr_f32 (NULL workspace) in that same shape -- which is the size rule's
    own shape for most of these cases, and the shape forced by the tuning override split = (4, 1) where the rule groups rows and the plan
    ungroups them. The plan itself is a permutation of the rows with each row's own offsets. Short rows, column tiles of a
    B that fits the L2 and widths below 4 ignore the plan and run as without it."""
    torch = torch_cuda
    rng = np.random.default_rng(97)
    cases = [("cfg2", None), ("cfg1", None), ("cfg4", None),
             ("skewed", (2049, 600, 256)), ("empty_rows", (300, 512, 128)), ("skewed", (1, 700, 64)),
             ("skewed", (5000, 2048, 50)), ("uniform", (4096, 1024, 256)), ("skewed", (2048, 512, 3)),
             ("skewed", (600, 512, 784)), ("skewed", (9000, 300, 128)), ("skewed", (1100, 2200, 1024))]
    used = ungrouped = tiled = 0
    for kind, shape in cases:
        if shape is None:
            c = dl.make_config(int(kind[3]))
            ro, ci, va, B, K = c["row_offsets"], c["col_indices"], c["values"], c["d0"], c["K"]
        else:
            M, K, N = shape
            ro, ci = random_csr(rng, M, K, kind, 0.12)
            va = rng.normal(0, 1, ci.size).astype(np.float32)
            B = rng.normal(0, 1, (K, N)).astype(np.float32)
        M, N = ro.size - 1, B.shape[1]
        print(f"row plan case {kind} {M}x{K} N {N} nnz {ci.size}", flush=True)
        ro_d, ci_d, va_d, B_d = (dev(torch, x) for x in (ro, ci, va, B))
        plan = dl.row_plan(ro_d)
        h = plan.cpu().numpy()
        starts, ends, rows = h[:M], h[M:2 * M], h[2 * M:3 * M]
        assert np.array_equal(np.sort(rows), np.arange(M))
        assert np.array_equal(starts, ro[rows]) and np.array_equal(ends, ro[rows + 1])
        lens = ends - starts
        assert (lens[:min(M, 256)][:-1] >= lens[:min(M, 256)][1:]).all()        # the first group: longest first
        if M > 2048:
            assert (lens[2048:][:-1] >= lens[2048:][1:]).all()                   # after the resident part: descending
        sh = dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size)
        want = dl.spmm(ro_d, ci_d, va_d, B_d, K=K).clone()
        # (a planned launch takes the column tiles of a plain call where every XCD works on its own, and not those of few rows)
        dl.set_tuning(split=(4, 1))
        want_one_row_finer = dl.spmm(ro_d, ci_d, va_d, B_d, K=K).clone()
        dl.set_tuning(split=(4, 1), rules_off=dl.RULES["finer_column_tiles"])
        want_one_row = dl.spmm(ro_d, ci_d, va_d, B_d, K=K).clone()
        dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
        # rows unknown: 1 exactly where the planned kernel runs (with the rule on, few rows are advised against a plan that would run)
        planned_runs = dl.row_plan_advice(dl.OP_SPMM, M, K, N, ci.size, -1)
        dl.set_tuning()
        got = torch.full((M, N), float("nan"), device="cuda")
        dl.spmm(ro_d, ci_d, va_d, B_d, K=K, out=got, plan=plan)
        if planned_runs:
            assert torch.equal(got, want_one_row) or torch.equal(got, want_one_row_finer), (kind, shape)
            used += 1
            tiled += int(sh["col_tiles"] > 1)
            if sh["R"] != 1:
                assert not torch.equal(want, want_one_row)   # the two shapes do round differently: the check above means something
                ungrouped += 1
        else:
            assert torch.equal(got, want), (kind, shape)
        assert oracle.rel_frobenius(got.cpu().numpy(), oracle.spmm(ro, ci, va, B)) <= TOL
        check_csr_untouched(ro_d, ci_d, ro, ci)
    # the planned kernel, rows ungrouped by it, column tiles gone through in plan order, and the fall-back
    assert used >= 6 and ungrouped >= 1 and tiled >= 1 and used < len(cases)


def test_row_plan_for_sddmm_and_the_fused_op(torch_cuda, dl, oracle):
    """The same plan drives sddmm_csr_f32 and fused_sddmm_spmm_f32: one row of the mask per four-wave
    workgroup, in plan order. Their results must have the bits of the plain calls in that same shape (the size rule's
    own, or the tuning override split = (4, 1) where the rule groups rows), and agree with the oracle; widths outside 16 < D <= 512 and short
    rows run as without a plan."""
    torch = torch_cuda
    rng = np.random.default_rng(99)
    cases = [("skewed", 2048, 2048, 64, 0.05), ("skewed", 2049, 700, 128, 0.15), ("skewed", 4096, 1024, 40, 0.1),
             ("empty_rows", 3000, 512, 256, 0.3), ("skewed", 1500, 900, 512, 0.2), ("skewed", 2048, 512, 16, 0.1),
             ("skewed", 5000, 600, 100, 0.02), ("skewed", 1024, 1024, 33, 0.1)]
    planned = {dl.OP_SDDMM: 0, dl.OP_FUSED: 0}
    for kind, M, K, D, den in cases:
        ro, ci = random_csr(rng, M, K, kind, den)
        print(f"planned sddmm/fused case {kind} {M}x{K} D {D} nnz {ci.size}", flush=True)
        Q = rng.normal(0, 1, (M, D)).astype(np.float32)
        Km = rng.normal(0, 1, (K, D)).astype(np.float32)
        V = rng.normal(0, 1, (K, D)).astype(np.float32)
        ro_d, ci_d, Q_d, K_d, V_d = (dev(torch, x) for x in (ro, ci, Q, Km, V))
        plan = dl.row_plan(ro_d)
        for op, plain, with_plan in (
                (dl.OP_SDDMM, lambda: dl.sddmm(ro_d, ci_d, Q_d, K_d).clone(), lambda: dl.sddmm(ro_d, ci_d, Q_d, K_d, plan=plan).clone()),
                (dl.OP_FUSED, lambda: dl.fused(ro_d, ci_d, Q_d, K_d, V_d, 0.25).clone(), lambda: dl.fused(ro_d, ci_d, Q_d, K_d, V_d, 0.25, plan=plan).clone())):
            want = plain()
            dl.set_tuning(split=(4, 1))
            want_one_row = plain()
            dl.set_tuning()
            got = with_plan()
            if dl.row_plan_advice(op, M, K, D, ci.size, -1):
                assert torch.equal(got, want_one_row), (kind, M, K, D, op)
                planned[op] += 1
            else:
                assert torch.equal(got, want), (kind, M, K, D, op)
        assert oracle.rel_frobenius(dl.sddmm(ro_d, ci_d, Q_d, K_d, plan=plan).cpu().numpy(), oracle.sddmm(ro, ci, Q, Km)) <= TOL
        assert oracle.rel_frobenius(dl.fused(ro_d, ci_d, Q_d, K_d, V_d, 0.25, plan=plan).cpu().numpy(),
                                    oracle.fused(ro, ci, Q, Km, V, 0.25)) <= TOL
        check_csr_untouched(ro_d, ci_d, ro, ci)
    assert 4 <= planned[dl.OP_SDDMM] < len(cases) and 4 <= planned[dl.OP_FUSED] < len(cases)


def test_stale_row_plan_stays_inside_the_arrays(torch_cuda, dl):
    """A plan built from another matrix of the same height gives wrong values, but its offsets are clamped to the arrays
    of the call: the launch completes and every row of C holds finite numbers or was left alone."""
    torch = torch_cuda
    rng = np.random.default_rng(98)
    M, K, N = 2048, 512, 256
    ro_big, _ = random_csr(rng, M, K, "skewed", 0.3)
    ro, ci = random_csr(rng, M, K, "skewed", 0.05)
    assert ro_big[-1] > ro[-1]
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    stale = dl.row_plan(dev(torch, ro_big))
    ro_d, ci_d, va_d, B_d = (dev(torch, x) for x in (ro, ci, va, B))
    out = torch.zeros(M, N, device="cuda")
    dl.spmm(ro_d, ci_d, va_d, B_d, K=K, out=out, plan=stale)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    with pytest.raises((dl.DlspmError, ValueError)):   # a plan for fewer rows is refused before any launch (binding or library)
        dl.spmm(ro_d, ci_d, va_d, B_d, K=K, out=out, plan=stale[:3 * M - 3])
    # and the right plan right after gives the right bits
    good = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, plan=dl.row_plan(ro_d))
    assert torch.equal(good, dl.spmm(ro_d, ci_d, va_d, B_d, K=K))


def test_calls_can_be_captured_in_a_hip_graph(torch_cuda, dl):
    """All three schedules only enqueue kernels (no memset, no allocation, no synchronisation), so a call may be captured.
    The graph is replayed several times with eager work and synchronisations in between, on changed inputs, and every
    replay must equal the eager result bit for bit."""
    torch = torch_cuda
    rng = np.random.default_rng(91)
    M, K, N = 700, 400, 128
    ro, ci = random_csr(rng, M, K, "skewed", 0.2)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    va = torch.randn(ci.size, device="cuda")
    B = torch.randn(K, N, device="cuda")
    Q = torch.randn(M, N, device="cuda")
    for schedule in ("row-block", "flat", "sliced"):
        if schedule == "flat":
            dl.set_tuning(flat=1, slices=0, flat_chunk=128)
        elif schedule == "sliced":
            dl.set_tuning(slices=3)
        need = max(dl.workspace_bytes(op, M, K, N, ci.size) for op in (dl.OP_SPMM, dl.OP_SDDMM, dl.OP_FUSED))
        assert (need > 0) == (schedule != "row-block")
        ws = torch.empty(need, dtype=torch.uint8, device="cuda") if need else None
        ws_s = ws if schedule == "sliced" else None  # SDDMM uses a workspace under the sliced schedule only
        C = torch.empty(M, N, device="cuda")
        CP = torch.empty(M, N, device="cuda")
        SP = torch.empty(ci.size, device="cuda")
        OP = torch.empty(M, N, device="cuda")
        plan = dl.row_plan(ro_d)
        S = torch.empty(ci.size, device="cuda")
        O = torch.empty(M, N, device="cuda")
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            dl.spmm(ro_d, ci_d, va, B, K=K, out=C, workspace=ws)  # warm-up outside the capture
            stream.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                dl.spmm(ro_d, ci_d, va, B, K=K, out=C, workspace=ws)
                dl.sddmm(ro_d, ci_d, Q, B, out=S, workspace=ws_s)
                dl.fused(ro_d, ci_d, Q, B, B, 0.5, out=O, workspace=ws)
                if schedule == "row-block":   # planned launches are one kernel each too
                    dl.spmm(ro_d, ci_d, va, B, K=K, out=CP, plan=plan)
                    dl.sddmm(ro_d, ci_d, Q, B, out=SP, plan=plan)
                    dl.fused(ro_d, ci_d, Q, B, B, 0.5, out=OP, plan=plan)
        for rep in range(4):
            va.copy_(torch.randn(ci.size, device="cuda"))  # eager work between the replays: new inputs
            B.copy_(torch.randn(K, N, device="cuda"))
            torch.cuda.synchronize()
            for buf in (C, S, O, CP, SP, OP):
                buf.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            if schedule == "row-block":
                assert torch.equal(CP, dl.spmm(ro_d, ci_d, va, B, K=K, plan=plan)), f"replay {rep}, planned SpMM"
                assert torch.equal(SP, dl.sddmm(ro_d, ci_d, Q, B, plan=plan)), f"replay {rep}, planned SDDMM"
                assert torch.equal(OP, dl.fused(ro_d, ci_d, Q, B, B, 0.5, plan=plan)), f"replay {rep}, planned fused"
                assert torch.allclose(CP, C, rtol=1e-4, atol=1e-4) and torch.equal(SP, S) and torch.allclose(OP, O, rtol=1e-4, atol=1e-3)
            got = (C.clone(), S.clone(), O.clone())
            want = (dl.spmm(ro_d, ci_d, va, B, K=K, workspace=ws).clone(), dl.sddmm(ro_d, ci_d, Q, B, workspace=ws_s).clone(),
                    dl.fused(ro_d, ci_d, Q, B, B, 0.5, workspace=ws).clone())
            torch.cuda.synchronize()
            for g, w in zip(got, want):
                assert torch.equal(g, w), f"replay {rep}, schedule {schedule}"


@pytest.mark.parametrize("M", [1500, 6000])
def test_plan_build_and_planned_launches_in_one_hip_graph(torch_cuda, dl, oracle, M):
    """dlspm_row_plan_build is kernels only, so building the plan and launching with it can be captured together: the
    case of a mask whose structure changes from call to call. Each replay follows an in-place change of row_offsets and
    col_indices (same array sizes, other row lengths) and must give the bits of the eager planned calls on the new
    structure, which in turn agree with the oracle. 1500 rows: the build is one launch; 6000: tiles, merges, packing."""
    torch = torch_cuda
    rng = np.random.default_rng(M)
    K, N = 700, 128
    structures = []
    ro0, ci0 = random_csr(rng, M, K, "skewed", 0.25)   # long enough rows that all three ops run one row per workgroup
    for _ in range(3):   # other structures with the same number of nonzeros: the rows' lengths permuted
        perm = rng.permutation(M)
        lens = np.diff(ro0)[perm]
        ro = np.zeros(M + 1, dtype=np.int32)
        ro[1:] = np.cumsum(lens)
        ci = np.concatenate([ci0[ro0[r]:ro0[r + 1]] for r in perm]).astype(np.int32) if ci0.size else ci0
        structures.append((ro, ci))
    ro_d, ci_d = dev(torch, structures[0][0]), dev(torch, structures[0][1])
    nnz = ci_d.numel()
    va = torch.randn(nnz, device="cuda")
    B = torch.randn(K, N, device="cuda")
    Q = torch.randn(M, N, device="cuda")
    plan = torch.zeros(dl.row_plan_bytes(M) // 4, dtype=torch.int32, device="cuda")
    C, S, O = torch.empty(M, N, device="cuda"), torch.empty(nnz, device="cuda"), torch.empty(M, N, device="cuda")
    assert dl.row_plan_advice(dl.OP_SPMM, M, K, N, nnz, -1) and dl.row_plan_advice(dl.OP_FUSED, M, K, N, nnz, -1)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        dl.row_plan(ro_d, out=plan)   # warm-up outside the capture
        dl.spmm(ro_d, ci_d, va, B, K=K, out=C, plan=plan)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            dl.row_plan(ro_d, out=plan)
            dl.spmm(ro_d, ci_d, va, B, K=K, out=C, plan=plan)
            dl.sddmm(ro_d, ci_d, Q, B, out=S, plan=plan)
            dl.fused(ro_d, ci_d, Q, B, B, 0.5, out=O, plan=plan)
    for rep, (ro, ci) in enumerate(structures + structures[:1]):
        ro_d.copy_(dev(torch, ro))
        ci_d.copy_(dev(torch, ci))
        va.copy_(torch.randn(nnz, device="cuda"))
        plan.fill_(-1)   # whatever the last build left must not matter
        for buf in (C, S, O):
            buf.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_plan = plan.clone()
        eager_plan = dl.row_plan(ro_d)
        assert torch.equal(got_plan[:3 * M], eager_plan[:3 * M]), f"replay {rep}: plan"
        assert torch.equal(C, dl.spmm(ro_d, ci_d, va, B, K=K, plan=eager_plan)), f"replay {rep}: SpMM"
        assert torch.equal(S, dl.sddmm(ro_d, ci_d, Q, B, plan=eager_plan)), f"replay {rep}: SDDMM"
        assert torch.equal(O, dl.fused(ro_d, ci_d, Q, B, B, 0.5, plan=eager_plan)), f"replay {rep}: fused"
        assert oracle.rel_frobenius(C.cpu().numpy(), oracle.spmm(ro, ci, va.cpu().numpy(), B.cpu().numpy(), omp=True)) <= TOL
        rows = got_plan[2 * M:3 * M].cpu().numpy()
        assert np.array_equal(np.sort(rows), np.arange(M))


def test_hint_bits_and_the_deprecated_constant(torch_cuda, dl):
    """The even-rows hint as a bit of workspace_bytes (NULL workspace) and as the deprecated pointer constant select the
    same launch and give the same bits; a row plan is passed as the workspace with DLSPM_HINT_ROW_PLAN."""
    import ctypes

    torch = torch_cuda
    rng = np.random.default_rng(5)
    M, K, N = 4096, 1024, 128
    ro, ci = random_csr(rng, M, K, "uniform", 0.2)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    va = torch.randn(ci.size, device="cuda")
    B = torch.randn(K, N, device="cuda")
    assert dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size, rows_even=True)["R"] == 4 != dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size)["R"]
    by_bit = dl.spmm(ro_d, ci_d, va, B, workspace=dl.ROWS_EVEN).clone()
    by_constant = torch.empty_like(by_bit)
    L, vp = dl.lib(), ctypes.c_void_p
    st = L.spmm_csr_f32(M, K, N, ci.size, vp(ro_d.data_ptr()), vp(ci_d.data_ptr()), vp(va.data_ptr()), vp(B.data_ptr()),
                        vp(by_constant.data_ptr()), vp(1), 0, vp(torch.cuda.current_stream().cuda_stream))
    assert st == dl.OK
    plain = dl.spmm(ro_d, ci_d, va, B)
    assert torch.equal(by_bit, by_constant) and not torch.equal(by_bit, plain) and torch.allclose(by_bit, plain, rtol=1e-4, atol=1e-4)
    plan = dl.row_plan(ro_d)
    via_named = dl.spmm(ro_d, ci_d, va, B, plan=plan).clone()
    via_abi = torch.empty_like(via_named)
    st = L.spmm_csr_f32(M, K, N, ci.size, vp(ro_d.data_ptr()), vp(ci_d.data_ptr()), vp(va.data_ptr()), vp(B.data_ptr()),
                        vp(via_abi.data_ptr()), vp(plan.data_ptr()), (plan.numel() * 4) | dl.HINT_ROW_PLAN,
                        vp(torch.cuda.current_stream().cuda_stream))
    assert st == dl.OK and torch.equal(via_named, via_abi) and not torch.equal(via_named, torch.zeros_like(via_named))


def test_streamed_results_have_the_bits_of_ordinary_stores(torch_cuda, dl, oracle):
    """Large results are stored with the non-temporal hint (instructions written out in the kernels); the size rule
    switches it on only for results of megabytes. dlspm_tuning.stream_results forces it for any size: every width from 1
    float (dword stores) over widths that are no multiple of 4 (rows that end inside a cache line, lanes that store the
    same columns twice) to column tiles, empty rows, shared rows, row plans and grouped rows must give the bits of the
    run with ordinary stores, for all three ops."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    cases = [("skewed", 300, 200, 1, 0.1), ("uniform", 257, 100, 3, 0.2), ("empty_rows", 1000, 300, 5, 0.1), ("skewed", 2048, 512, 49, 0.1),
             ("uniform", 700, 256, 64, 0.2), ("skewed", 513, 700, 129, 0.05), ("empty_rows", 2051, 512, 256, 0.1), ("uniform", 64, 147, 1030, 0.3),
             ("skewed", 9000, 256, 33, 0.05), ("full", 40, 300, 196, 1.0)]
    for kind, M, K, N, den in cases:
        ro, ci = random_csr(rng, M, K, kind, den)
        va = rng.normal(0, 1, ci.size).astype(np.float32)
        B = rng.normal(0, 1, (K, N)).astype(np.float32)
        Q = rng.normal(0, 1, (M, N)).astype(np.float32)
        V = rng.normal(0, 1, (K, N)).astype(np.float32)
        ro_d, ci_d, va_d, B_d, Q_d, V_d = (dev(torch, x) for x in (ro, ci, va, B, Q, V))
        plan = dl.row_plan(ro_d)
        runs = {
            "spmm": lambda **kw: dl.spmm(ro_d, ci_d, va_d, B_d, K=K, **kw),
            "sddmm": lambda **kw: dl.sddmm(ro_d, ci_d, Q_d, B_d, **kw),
            "fused": lambda **kw: dl.fused(ro_d, ci_d, Q_d, B_d, V_d, 0.25, **kw),
        }
        for op, run in runs.items():
            for schedule in ({}, {"workspace": dl.ROWS_EVEN}, {"plan": plan}):
                dl.set_tuning(stream_results=0)
                plain = run(**schedule).cpu().numpy()
                dl.set_tuning(stream_results=1)
                streamed = run(**schedule).cpu().numpy()
                dl.set_tuning()
                assert np.array_equal(plain, streamed), (op, kind, M, K, N, list(schedule))
        want = oracle.spmm(ro, ci, va, B, omp=True)
        dl.set_tuning(stream_results=1)
        assert oracle.rel_frobenius(dl.spmm(ro_d, ci_d, va_d, B_d, K=K).cpu().numpy(), want) <= TOL
        dl.set_tuning()
        check_csr_untouched(ro_d, ci_d, ro, ci)


def test_banded_hint(torch_cuda, dl, oracle):
    """DLSPM_HINT_BANDED on a sliding-window mask whose K-side operands exceed one L2, where dlspm_workspace_advice (which
    cannot see the band) recommends column slices: the call runs as row blocks dealt to the XCDs in contiguous runs,
    with or without memory, and returns the bits of the call with NULL for SDDMM and the fused op; SpMM drops its
    L2-sized column tiles (another, equally fixed order of the same sums, so equal to a tile-free launch and within
    tolerance of the oracle). Combined with the even-rows hint it is that hint's launch."""
    torch = torch_cuda
    M = K = 16384
    D = 128
    ro, ci = dl.make_pattern(dl.PATTERN_BAND_RANDOM, 91, M, K, 96, 0)
    lens = np.diff(ro)
    assert lens.max() <= 96 and (np.abs(ci - np.repeat(np.arange(M), lens)) <= 96).all()
    nnz = ci.size
    assert dl.describe_slices(dl.OP_FUSED, M, K, D, nnz)[0] >= 2  # a call with memory (and no hint) would work in column slices
    rng = np.random.default_rng(92)
    Q, Km, V = (rng.standard_normal(s, dtype=np.float32) for s in ((M, D), (K, D), (K, D)))
    va = rng.standard_normal(nnz, dtype=np.float32)
    ro_d, ci_d, Q_d, Km_d, V_d, va_d = (dev(torch, x) for x in (ro, ci, Q, Km, V, va))
    # fused and SDDMM: the same bits as with NULL, with and without memory behind the hint
    for op, run, want in (
        (dl.OP_FUSED, lambda **kw: dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125, **kw), lambda: oracle.fused(ro, ci, Q, Km, V, 0.125, omp=True)),
        (dl.OP_SDDMM, lambda **kw: dl.sddmm(ro_d, ci_d, Q_d, Km_d, **kw), lambda: oracle.sddmm(ro, ci, Q, Km, omp=True)),
    ):
        plain = run().cpu().numpy()
        assert oracle.rel_frobenius(plain, want()) <= TOL
        assert np.array_equal(run(banded=True).cpu().numpy(), plain)
        ws = torch.empty(max(dl.workspace_bytes(op, M, K, D, nnz), 16), dtype=torch.uint8, device="cuda")
        assert np.array_equal(run(banded=True, workspace=ws).cpu().numpy(), plain)
        even = run(workspace=dl.ROWS_EVEN).cpu().numpy()
        assert np.array_equal(run(banded=True, workspace=dl.ROWS_EVEN).cpu().numpy(), even)
    # SpMM: B (8 MiB) would be cut into column tiles; with the hint it is one tile, as tile_major = 0 gives without it
    want = oracle.spmm(ro, ci, va, Km, omp=True)
    hinted = dl.spmm(ro_d, ci_d, va_d, Km_d, banded=True).cpu().numpy()
    assert oracle.rel_frobenius(hinted, want) <= TOL
    dl.set_tuning(tile_major=0)
    untiled = dl.spmm(ro_d, ci_d, va_d, Km_d).cpu().numpy()
    dl.set_tuning()
    assert np.array_equal(hinted, untiled)
    check_csr_untouched(ro_d, ci_d, ro, ci)


def test_xcd_contiguous_row_blocks_give_the_same_bits(torch_cuda, dl, oracle):
    """dlspm_tuning.xcd_contiguous only changes which workgroup works on which row block (each XCD one contiguous run):
    every row is summed as before, so all three ops return the bits of the default order, also where the number of
    row blocks is no multiple of eight, where rows are grouped, and where column tiles switch it off."""
    torch = torch_cuda
    rng = np.random.default_rng(123)
    for kind, M, K, N, den in (("skewed", 2048, 512, 256, 0.1), ("empty_rows", 2051, 700, 64, 0.1), ("uniform", 9, 300, 128, 0.3),
                               ("skewed", 16390, 256, 32, 0.05), ("uniform", 5, 40, 16, 0.5), ("skewed", 1003, 512, 700, 0.1)):
        ro, ci = random_csr(rng, M, K, kind, den)
        va = rng.normal(0, 1, ci.size).astype(np.float32)
        B = rng.normal(0, 1, (K, N)).astype(np.float32)
        Q = rng.normal(0, 1, (M, N)).astype(np.float32)
        ro_d, ci_d, va_d, B_d, Q_d = (dev(torch, x) for x in (ro, ci, va, B, Q))
        print(f"xcd case {kind} {M}x{K} N {N} nnz {ci.size}", flush=True)
        want = (dl.spmm(ro_d, ci_d, va_d, B_d).clone(), dl.sddmm(ro_d, ci_d, Q_d, B_d).clone(), dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.5).clone())
        dl.set_tuning(xcd_contiguous=1)
        got = (dl.spmm(ro_d, ci_d, va_d, B_d).clone(), dl.sddmm(ro_d, ci_d, Q_d, B_d).clone(), dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.5).clone())
        dl.set_tuning()
        for g, w in zip(got, want):
            assert torch.equal(g, w), (kind, M, K, N)
        assert oracle.rel_frobenius(got[0].cpu().numpy(), oracle.spmm(ro, ci, va, B, omp=True)) <= TOL
        check_csr_untouched(ro_d, ci_d, ro, ci)


def test_concurrent_calls_from_two_threads_on_two_streams(torch_cuda, dl, oracle):
    """The library keeps no mutable global state: two host threads, each with its own stream, outputs and workspace."""
    import threading

    torch = torch_cuda
    c = dl.make_config(2)
    ro_d, ci_d, va, B = (dev(torch, c[k]) for k in ("row_offsets", "col_indices", "values", "d0"))
    ref = dl.spmm(ro_d, ci_d, va, B, K=c["K"]).clone()
    torch.cuda.synchronize()
    results, errors = {}, []

    def worker(tid):
        try:
            stream = torch.cuda.Stream()
            out = torch.empty_like(ref)
            with torch.cuda.stream(stream):
                for _ in range(200):
                    dl.spmm(ro_d, ci_d, va, B, K=c["K"], out=out)
                stream.synchronize()
            results[tid] = out
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for out in results.values():
        assert torch.equal(out, ref)


def test_operands_beyond_2_31_elements(torch_cuda, dl):
    """Dense operands of 2.3e9 floats (9.2 GB each): every element offset inside the kernels must be 64-bit. One
    nonzero per row with value 1 makes SpMM a row gather, SDDMM a row-by-row dot product and the fused op a scaled row
    gather, all checked on the device against torch."""
    torch = torch_cuda
    M, K, N = 70001, 64, 32768
    assert M * N > 2**31
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    ci_d = torch.randint(0, K, (M,), dtype=torch.int32, device="cuda", generator=g)
    ro_d = torch.arange(M + 1, dtype=torch.int32, device="cuda")
    ones = torch.ones(M, dtype=torch.float32, device="cuda")
    B = torch.randn(K, N, device="cuda", generator=g)
    C = torch.empty(M, N, device="cuda")
    dl.spmm(ro_d, ci_d, ones, B, K=K, out=C)
    for lo in range(0, M, 10000):  # compare in slices: the gathered reference would be another 9.2 GB
        hi = min(M, lo + 10000)
        assert torch.equal(C[lo:hi], B[ci_d[lo:hi].long()]), f"rows {lo}..{hi}"
    # SDDMM: lhs = C (M x N, 9.2 GB): out[i] = <C[i], B[col_i]> = |B[col_i]|^2
    out = dl.sddmm(ro_d, ci_d, C, B)
    want = (B.double() ** 2).sum(1)[ci_d.long()]
    assert torch.allclose(out.double(), want, rtol=1e-4)
    # fused: O[i] = (<Q[i], B[col_i]> * scale) * V[col_i], Q = C so the score is |B[col_i]|^2 again; O reuses no input
    O = torch.empty(M, N, device="cuda")
    dl.fused(ro_d, ci_d, C, B, B, 1.0 / N, out=O)
    for lo in range(0, M, 10000):
        hi = min(M, lo + 10000)
        ref = (want[lo:hi] / N).float()[:, None] * B[ci_d[lo:hi].long()]
        assert torch.allclose(O[lo:hi], ref, rtol=1e-3, atol=1e-5), f"rows {lo}..{hi}"


def test_csr_row_stats(torch_cuda, dl):
    torch = torch_cuda
    rng = np.random.default_rng(3)
    for (M, K, kind) in [(1, 1, "empty"), (1000, 300, "skewed"), (5000, 64, "empty_rows"), (70000, 40, "uniform")]:
        ro, ci = random_csr(rng, M, K, kind, 0.1)
        lens = np.diff(ro)
        assert dl.csr_row_stats(dev(torch, ro)) == (int(lens.max()), int((lens == 0).sum()))


def test_error_statuses(torch_cuda, dl):
    torch = torch_cuda
    z = torch.zeros(4, dtype=torch.int32, device="cuda")
    f = torch.zeros(16, dtype=torch.float32, device="cuda")
    L = dl.lib()
    assert L.spmm_csr_f32(-1, 1, 1, 0, z.data_ptr(), None, None, None, f.data_ptr(), None, 0, None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(2, 2, 2, 5, z.data_ptr(), z.data_ptr(), f.data_ptr(), f.data_ptr(), f.data_ptr(), None, 0, None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(2, 2, 2, 1, None, z.data_ptr(), f.data_ptr(), f.data_ptr(), f.data_ptr(), None, 0, None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(0, 2, 2, 0, None, None, None, None, None, None, 0, None) == dl.OK
    # malformed CSR structures are caught by the device-side check
    bad_ro = torch.tensor([0, 3, 2, 4], dtype=torch.int32, device="cuda")
    ci = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device="cuda")
    assert dl.csr_check(3, 4, bad_ro, ci) == dl.E_INVALID_CSR
    good_ro = torch.tensor([0, 2, 2, 4], dtype=torch.int32, device="cuda")
    assert dl.csr_check(3, 4, good_ro, ci) == dl.OK
    assert dl.csr_check(3, 3, good_ro, ci) == dl.E_INVALID_CSR  # column 3 >= K
