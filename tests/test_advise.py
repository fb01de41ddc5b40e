"""dlspm_analyze / dlspm_advise: one look at the matrix, one answer.

CPU part: every branch of dlspm_advise on hand-written dlspm_matrix_info records (the call is host only).
GPU part: dlspm_analyze against numpy on seeded patterns; the lead path analyze -> advise -> allocate -> build -> launch
(dl.prepare) on a band, on a matrix with one very long row, on very uneven rows and on even rows, each against the oracle.
"""
import ctypes

import numpy as np
import pytest

from conftest import random_csr

TOL = 1e-4


def info(dl, M, K, nnz, longest, cover=8000, heaviest=1000, empty=0, span=None):
    return dl.MatrixInfo(M, K, nnz, longest, empty, K if span is None else span, cover, heaviest)


def test_advise_branches(dl):
    """Host only. Sizes are those of an MI355X (256 compute units, 4 MiB per L2), which the library assumes without a
    device too."""
    A = dl.advise
    # a band whose K-side operand exceeds one L2: detected, no memory; with the even-rows hint where that holds too
    cp = A(dl.OP_FUSED, 128, info(dl, 16384, 16384, 16384 * 96, 96, cover=1100, heaviest=1010))
    assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_NOTHING, 0, dl.HINT_BANDED | dl.HINT_ROWS_EVEN)
    cp = A(dl.OP_SDDMM, 128, info(dl, 16384, 16384, 16384 * 60, 130, cover=1100, heaviest=1010))
    assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_NOTHING, 0, dl.HINT_BANDED)
    # ... not when the operand fits the L2 anyway, when the eighths are uneven, or when every eighth reaches all columns
    assert not A(dl.OP_SDDMM, 32, info(dl, 16384, 16384, 16384 * 96, 96, cover=1100)).hints & dl.HINT_BANDED
    assert not A(dl.OP_FUSED, 128, info(dl, 16384, 16384, 16384 * 96, 96, cover=1100, heaviest=2000)).hints & dl.HINT_BANDED
    assert not A(dl.OP_FUSED, 128, info(dl, 16384, 16384, 16384 * 96, 96, cover=8000)).hints & dl.HINT_BANDED
    # one row far above a compute unit's share: a cut plan, sized for the op and the width
    cp = A(dl.OP_SPMM, 256, info(dl, 512, 2048, 52428, 963))
    assert (cp.build, cp.hints) == (dl.BUILD_CUT_PLAN, dl.HINT_CUT_PLAN) and cp.bytes == dl.row_plan_bytes_for(dl.OP_SPMM, 512, 256)
    cp = A(dl.OP_SDDMM, 128, info(dl, 512, 2048, 52428, 963))
    assert (cp.build, cp.hints) == (dl.BUILD_CUT_PLAN, dl.HINT_CUT_PLAN) and cp.bytes == dl.row_plan_bytes_for(dl.OP_SDDMM, 512, 128)
    # uneven rows: a plan over whole rows (the headline matrix)
    cp = A(dl.OP_SPMM, 256, info(dl, 2048, 512, 105687, 312))
    assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_ROW_PLAN, dl.row_plan_bytes(2048), dl.HINT_ROW_PLAN)
    # very uneven rows in a mask of 32 rows per compute unit: the plan, with the word that makes SDDMM / fused use it
    for op, D in ((dl.OP_SDDMM, 128), (dl.OP_FUSED, 64)):
        cp = A(op, D, info(dl, 8192, 2048, 8192 * 60, 1500))
        assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_ROW_PLAN, dl.row_plan_bytes(8192), dl.HINT_ROW_PLAN | dl.HINT_ROWS_SKEWED)
        cp = A(op, D, info(dl, 8192, 2048, 8192 * 60, 400))   # uneven, but not that uneven: the fused op's grouped rows win
        assert cp.build == (dl.BUILD_ROW_PLAN if op == dl.OP_SDDMM else dl.BUILD_NOTHING)  # (SDDMM does not group them)
    # even rows: the hint, no memory
    cp = A(dl.OP_SPMM, 392, info(dl, 2048, 512, 2048 * 102, 102))
    assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_NOTHING, 0, dl.HINT_ROWS_EVEN)
    # a K-side operand far beyond the L2 under random columns: the column-sliced schedule's workspace
    cp = A(dl.OP_FUSED, 128, info(dl, 8192, 32768, 8192 * 600, 700))
    assert cp.build == dl.BUILD_NOTHING and cp.hints == 0 and cp.bytes == dl.workspace_bytes(dl.OP_FUSED, 8192, 32768, 128, 8192 * 600) > 0
    # nothing to say
    cp = A(dl.OP_SPMM, 2, info(dl, 300, 300, 3000, 25))     # widths below 4: no planned launch
    assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_NOTHING, 0, 0)
    cp = A(dl.OP_SPMM, 64, info(dl, 0, 0, 0, 0))
    assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_NOTHING, 0, 0)
    # arguments
    # long rows next to each other in a tall matrix of short rows (one eighth of the rows holds 1.6 times its share, the
    # longest row eight times the mean; too many rows and too short for a plan): the word that keeps the size rule from
    # grouping sixteen rows into one workgroup
    for op, width in ((dl.OP_SPMM, 256), (dl.OP_SDDMM, 128), (dl.OP_FUSED, 64)):
        cp = A(op, width, info(dl, 33288, 512, 584680, 389, heaviest=2672))
        assert (cp.build, cp.bytes, cp.hints) == (dl.BUILD_NOTHING, 0, dl.HINT_ROWS_SKEWED), (op, cp.build, cp.bytes, hex(cp.hints))
        assert dl.describe_launch(op, 33288, 512, width, 584680)["R"] == 16
        assert dl.describe_launch(op, 33288, 512, width, 584680, rows_skewed=True)["R"] == (8 if op == dl.OP_FUSED else 4)
        assert not A(op, width, info(dl, 33288, 512, 584680, 389, heaviest=1500)).hints & dl.HINT_ROWS_SKEWED   # lengths independent of the position
        assert not A(op, width, info(dl, 33288, 512, 584680, 100, heaviest=2672)).hints & dl.HINT_ROWS_SKEWED   # no row of eight times the mean
    L = dl.lib()
    assert L.dlspm_describe_launch_rows(dl.OP_SPMM, 64, 64, 64, 64, 4, (ctypes.c_int * 10)()) == dl.E_INVALID_ARG
    mi, out = info(dl, 8, 8, 8, 1), dl.CallPlan()
    assert L.dlspm_advise(7, 64, ctypes.byref(mi), ctypes.byref(out)) == dl.E_INVALID_ARG
    assert L.dlspm_advise(dl.OP_SPMM, 64, None, ctypes.byref(out)) == dl.E_INVALID_ARG
    assert L.dlspm_advise(dl.OP_SPMM, 64, ctypes.byref(mi), None) == dl.E_INVALID_ARG
    assert L.dlspm_analyze(-1, 1, 0, None, None, None, ctypes.byref(mi)) == dl.E_INVALID_ARG
    assert L.dlspm_analyze(4, 4, 2, None, None, None, ctypes.byref(mi)) == dl.E_INVALID_ARG
    assert L.dlspm_analyze(0, 4, 0, None, None, None, ctypes.byref(mi)) == dl.OK and mi.M == 0 and mi.max_row_len == 0


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def numpy_info(ro, ci, K):
    M = ro.size - 1
    lens = np.diff(ro)
    spans, cover, nnz8 = [0], 0, []
    for x in range(8):
        a, b = x * M // 8, (x + 1) * M // 8
        cols = ci[ro[a]:ro[b]]
        if cols.size:
            cover += int(cols.max()) - int(cols.min()) + 1
        nnz8.append(int(ro[b] - ro[a]))
    for i in np.flatnonzero(lens):
        r = ci[ro[i]:ro[i + 1]]
        spans.append(int(r.max()) - int(r.min()) + 1)
    total = sum(nnz8)
    return {"M": M, "K": K, "nnz": int(ro[-1]), "max_row_len": int(lens.max()) if M else 0, "empty_rows": int((lens == 0).sum()),
            "max_col_span": max(spans), "eighths_cover_permille": min(cover * 1000 // K, 8000) if K else 0,
            "eighths_nnz_permille": min(max(nnz8) * 8000 // total, 8000) if total else 0}


@pytest.mark.gpu
def test_analyze_against_numpy(dl):
    import torch

    rng = np.random.default_rng(3)
    cases = [("uniform", 1000, 777, 0.1), ("skewed", 5000, 2048, 0.02), ("empty_rows", 333, 500, 0.3), ("empty", 64, 64, 0.0),
             ("full", 40, 100, 1.0), ("uniform", 7, 5000, 0.5), ("skewed", 100000, 512, 0.02)]
    for kind, M, K, density in cases:
        ro, ci = random_csr(rng, M, K, kind, density)
        print(f"analyze: {kind} {M}x{K} nnz {ci.size}", flush=True)
        got = dl.analyze(dev(torch, ro), dev(torch, ci), K).as_dict()
        assert got == numpy_info(ro, ci, K), (kind, M, K)
    ro, ci = dl.make_pattern(dl.PATTERN_BAND_RANDOM, 91, 4096, 4096, 64, 0)
    got = dl.analyze(dev(torch, ro), dev(torch, ci), 4096).as_dict()
    assert got == numpy_info(ro, ci, 4096) and got["eighths_cover_permille"] <= 1300 and got["max_col_span"] <= 129
    ro, ci = dl.make_pattern(dl.PATTERN_BAND_RANDOM, 91, 4096, 4096, 32, 48)   # a band plus random columns: no band
    assert dl.analyze(dev(torch, ro), dev(torch, ci), 4096).eighths_cover_permille >= 7900


@pytest.mark.gpu
def test_analyze_from_several_threads_at_once(dl):
    """dlspm_analyze keeps the figures of a call in a slot of a static device array for the length of the call: four host
    threads, each on a stream of its own, analyse different matrices a hundred times at once and get their own answers."""
    import threading

    import torch

    rng = np.random.default_rng(11)
    problems = []
    for kind, M, K, density in (("uniform", 900, 700, 0.1), ("skewed", 3000, 1024, 0.03), ("empty_rows", 500, 400, 0.2),
                                ("uniform", 64, 3000, 0.4)):
        ro, ci = random_csr(rng, M, K, kind, density)
        problems.append((dev(torch, ro), dev(torch, ci), K, numpy_info(ro, ci, K)))
    torch.cuda.synchronize()
    wrong = []

    def work(index):
        ro_d, ci_d, K, want = problems[index]
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            for _ in range(100):
                got = dl.analyze(ro_d, ci_d, K).as_dict()
                if got != want:
                    wrong.append((index, got, want))
                    return

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(problems))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not wrong, wrong[:1]


@pytest.mark.gpu
def test_prepared_calls_follow_the_matrix(dl, oracle):
    """analyze -> advise -> allocate -> build -> launch, with no knowledge of the matrix on the caller's side: the
    sliding-window mask gets the banded launch (the bits of the call with DLSPM_HINT_BANDED), the matrix with one very
    long row a cut plan, very uneven rows in a mask of 8192 rows the plan with one row per workgroup (the bits of that
    split), even rows the even-rows hint; every result against the oracle."""
    import torch

    rng = np.random.default_rng(17)
    # 1. the band
    M = K = 16384
    D = 128
    ro, ci = dl.make_pattern(dl.PATTERN_BAND_RANDOM, 91, M, K, 96, 0)
    Q, Km, V = (rng.standard_normal(s, dtype=np.float32) for s in ((M, D), (K, D), (K, D)))
    ro_d, ci_d, Q_d, Km_d, V_d = (dev(torch, x) for x in (ro, ci, Q, Km, V))
    mi = dl.analyze(ro_d, ci_d, K)
    for op in (dl.OP_FUSED, dl.OP_SDDMM):
        prep = dl.prepare(ro_d, ci_d, K, op, D, info=mi)
        assert prep.call_plan.hints & dl.HINT_BANDED and prep.memory is None
    got = dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125, plan=dl.prepare(ro_d, ci_d, K, dl.OP_FUSED, D, info=mi))
    assert torch.equal(got, dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125, banded=True, workspace=dl.ROWS_EVEN))
    assert oracle.rel_frobenius(got.cpu().numpy(), oracle.fused(ro, ci, Q, Km, V, 0.125, omp=True)) <= TOL
    # 2. one row of many shares: a cut plan for all three ops
    M, K = 512, 2048
    lens = np.minimum(K, rng.poisson(90, M))
    lens[100] = 1000
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens]).astype(np.int32)
    va = rng.standard_normal(ci.size, dtype=np.float32)
    B = rng.uniform(-1, 1, (K, 256)).astype(np.float32)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    prep = dl.prepare(ro_d, ci_d, K, dl.OP_SPMM, 256)
    assert prep.call_plan.build == dl.BUILD_CUT_PLAN
    got = dl.spmm(ro_d, ci_d, dev(torch, va), dev(torch, B), K=K, plan=prep).cpu().numpy()
    assert oracle.rel_frobenius(got, oracle.spmm(ro, ci, va, B)) <= TOL
    Q, Km = rng.standard_normal((M, 128), dtype=np.float32), rng.standard_normal((K, 128), dtype=np.float32)
    prep = dl.prepare(ro_d, ci_d, K, dl.OP_SDDMM, 128)
    assert prep.call_plan.build == dl.BUILD_CUT_PLAN
    assert torch.equal(dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, Km), plan=prep), dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, Km)))
    # 3. very uneven rows, 8192 x 2048: the plan with DLSPM_HINT_ROWS_SKEWED runs one row per workgroup
    M, K, D = 8192, 2048, 64
    ro, ci = dl.make_pattern(dl.PATTERN_LOGNORMAL_ROWS, 5, M, K, 60.0, 1.0)
    assert np.diff(ro).max() * M >= 20 * ci.size
    Q, Km, V = (rng.standard_normal(s, dtype=np.float32) for s in ((M, D), (K, D), (K, D)))
    ro_d, ci_d, Q_d, Km_d, V_d = (dev(torch, x) for x in (ro, ci, Q, Km, V))
    assert dl.describe_launch(dl.OP_FUSED, M, K, D, ci.size)["R"] > 1   # the sizes alone group rows
    prep = dl.prepare(ro_d, ci_d, K, dl.OP_FUSED, D)
    assert prep.call_plan.build == dl.BUILD_ROW_PLAN and prep.call_plan.hints == dl.HINT_ROW_PLAN | dl.HINT_ROWS_SKEWED
    got = dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125, plan=prep)
    dl.set_tuning(split=(4, 1))
    one_row = dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125)
    dl.set_tuning()
    assert torch.equal(got, one_row)
    assert oracle.rel_frobenius(got.cpu().numpy(), oracle.fused(ro, ci, Q, Km, V, 0.125, omp=True)) <= TOL
    # without the word the same plan is ignored at this height (the bits of the plain call)
    plain_plan = dl.row_plan(ro_d)
    assert torch.equal(dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125, plan=plain_plan), dl.fused(ro_d, ci_d, Q_d, Km_d, V_d, 0.125))
    # 3b. a tall matrix of short rows whose long rows lie next to each other (an embedding whose frequent tokens come
    # first): no plan, no memory, DLSPM_HINT_ROWS_SKEWED -- four rows per workgroup instead of sixteen
    M, K = 33288, 512
    lens = rng.poisson(12, M)
    lens[:1200] = rng.integers(150, 390, 1200)
    lens = np.minimum(lens, K)
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens]).astype(np.int32)
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    mi = dl.analyze(ro_d, ci_d, K)
    assert mi.eighths_nnz_permille >= 2000 and mi.max_row_len * M >= 8 * ci.size
    va = rng.standard_normal(ci.size, dtype=np.float32)
    for op, width in ((dl.OP_SPMM, 256), (dl.OP_SDDMM, 128), (dl.OP_FUSED, 64)):
        prep = dl.prepare(ro_d, ci_d, K, op, width, info=mi)
        assert prep.memory is None and prep.call_plan.hints == dl.HINT_ROWS_SKEWED
        Q, Km, V = (rng.standard_normal(sh, dtype=np.float32) for sh in ((M, width), (K, width), (K, width)))
        dl.set_tuning(split=(4, 8 if op == dl.OP_FUSED else 4))
        if op == dl.OP_SPMM:
            got, four = dl.spmm(ro_d, ci_d, dev(torch, va), dev(torch, Km), K=K, plan=prep), None
            four = dl.spmm(ro_d, ci_d, dev(torch, va), dev(torch, Km), K=K)
            want = oracle.spmm(ro, ci, va, Km, omp=True)
        elif op == dl.OP_SDDMM:
            got = dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, Km), plan=prep)
            four = dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, Km))
            want = oracle.sddmm(ro, ci, Q, Km, omp=True)
        else:
            got = dl.fused(ro_d, ci_d, dev(torch, Q), dev(torch, Km), dev(torch, V), 0.125, plan=prep)
            four = dl.fused(ro_d, ci_d, dev(torch, Q), dev(torch, Km), dev(torch, V), 0.125)
            want = oracle.fused(ro, ci, Q, Km, V, 0.125, omp=True)
        dl.set_tuning()
        assert torch.equal(got, four), op                     # the bits of four (fused: eight) rows per workgroup
        assert oracle.rel_frobenius(got.cpu().numpy(), want) <= TOL
    # 4. even rows (the 1x1-convolution configuration): the even-rows hint, nothing to allocate
    c = dl.make_config(4)
    ro_d, ci_d = dev(torch, c["row_offsets"]), dev(torch, c["col_indices"])
    prep = dl.prepare(ro_d, ci_d, c["K"], dl.OP_SPMM, c["N"])
    assert prep.memory is None and prep.call_plan.hints == dl.HINT_ROWS_EVEN
    got = dl.spmm(ro_d, ci_d, dev(torch, c["values"]), dev(torch, c["d0"]), K=c["K"], plan=prep)
    assert torch.equal(got, dl.spmm(ro_d, ci_d, dev(torch, c["values"]), dev(torch, c["d0"]), K=c["K"], workspace=dl.ROWS_EVEN))
