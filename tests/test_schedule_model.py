"""Host model of the GPU schedule (tests/schedule_model/schedule_model.cpp).

CPU part: for every workgroup shape the kernels are instantiated for, the modelled work split writes every output
element exactly once, never consumes a partial sum that no wave produced, and agrees with the oracle.
GPU part: with the launch shape the library reports for a problem (dlspm_describe_launch), the model reproduces the
kernels' fp32 operation order, so the GPU output must equal the model's BIT FOR BIT -- a much sharper check than
the 1e-4 tolerance, and one that would expose a dropped, duplicated or reordered nonzero of any size.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from conftest import random_csr

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "schedule_model")
_i = ctypes.POINTER(ctypes.c_int)
_f = ctypes.POINTER(ctypes.c_float)


@pytest.fixture(scope="module")
def model():
    so = os.path.join(HERE, "libschedule_model.so")
    if not os.path.exists(so):
        subprocess.run(["make", "-s", "-C", HERE], check=True)
    L = ctypes.CDLL(so)
    ci = ctypes.c_int
    L.model_spmm.argtypes = [ci, ci, _i, _i, _f, _f, ci, ci, ci, _f, _i]
    L.model_spmm.restype = ci
    L.model_sddmm.argtypes = [ci, ci, _i, _i, _f, _f, ci, ci, ci, _f]
    L.model_sddmm.restype = None
    L.model_fused.argtypes = [ci, ci, _i, _i, _f, _f, _f, ctypes.c_float, ci, ci, ci, ci, ci, ci, _f, _f, _i]
    L.model_fused.restype = ci
    L.model_spmm_flat.argtypes = [ci, ci, _i, _i, _f, _f, ci, ci, _f, _i]
    L.model_spmm_flat.restype = ci
    L.model_fused_flat.argtypes = [ci, ci, _i, _i, _f, _f, _f, ctypes.c_float, ci, ci, ci, ci, ci, _f, _f, _i]
    L.model_fused_flat.restype = ci
    L.model_row_plan.argtypes = [ci, _i, ci, ci, _i]
    L.model_row_plan.restype = None
    return L


def pi(a):
    return a.ctypes.data_as(_i)


def pf(a):
    return a.ctypes.data_as(_f)


def run_spmm(L, ro, ci, va, B, G, W, R):
    M, N = ro.size - 1, B.shape[1]
    C = np.full((M, N), np.nan, dtype=np.float32)
    writes = np.zeros((M, N), dtype=np.int32)
    ci2 = ci if ci.size else np.zeros(1, np.int32)
    va2 = va if va.size else np.zeros(1, np.float32)
    rc = L.model_spmm(M, N, pi(ro), pi(ci2), pf(va2), pf(B), G, W, R, pf(C), pi(writes))
    return rc, C, writes


SPLITS = [(4, 16), (4, 8), (4, 4), (4, 2), (4, 1), (8, 4), (8, 2), (8, 1), (16, 1)]


@pytest.mark.parametrize("kind,density", [("uniform", 0.2), ("skewed", 0.1), ("empty_rows", 0.3), ("full", 1.0), ("empty", 0.0)])
def test_every_split_writes_each_output_once_and_matches_the_oracle(model, oracle, kind, density):
    rng = np.random.default_rng(11)
    M, K, N = 53, 97, 12
    ro, ci = random_csr(rng, M, K, kind, density)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    ref = oracle.spmm(ro, ci, va, B)
    for (W, R) in SPLITS:
        for G in (64, 32, 16, 8):
            rc, C, writes = run_spmm(model, ro, ci, va, B, G, W, R)
            assert rc == 0, f"inconsistent partial sums for W={W} R={R} G={G}"
            assert (writes == 1).all(), f"W={W} R={R} G={G}: an element was written {writes.min()}..{writes.max()} times"
            assert oracle.rel_frobenius(C, ref) < 1e-6


def test_model_sddmm_and_fused_match_the_oracle(model, oracle):
    rng = np.random.default_rng(12)
    M, K = 40, 70
    ro, ci = random_csr(rng, M, K, "skewed", 0.2)
    for (D, vec, G1, DS) in [(128, 4, 8, 4), (64, 4, 8, 2), (16, 4, 4, 1), (48, 4, 8, 2), (1024, 4, 8, 0), (13, 1, 16, 0)]:
        Q = rng.normal(0, 1, (M, D)).astype(np.float32)
        Km = rng.normal(0, 1, (K, D)).astype(np.float32)
        V = rng.normal(0, 1, (K, D)).astype(np.float32)
        out = np.empty(ci.size, dtype=np.float32)
        model.model_sddmm(M, D, pi(ro), pi(ci), pf(Q), pf(Km), vec, G1, DS, pf(out))
        assert oracle.rel_frobenius(out, oracle.sddmm(ro, ci, Q, Km)) < 1e-6
        scores = np.empty(ci.size, dtype=np.float32)
        O = np.full((M, D), np.nan, dtype=np.float32)
        writes = np.zeros((M, D), dtype=np.int32)
        rc = model.model_fused(M, D, pi(ro), pi(ci), pf(Q), pf(Km), pf(V), 0.125, vec, G1, DS, 16, 4, 4, pf(scores), pf(O), pi(writes))
        assert rc == 0 and (writes == 1).all()
        assert oracle.rel_frobenius(O, oracle.fused(ro, ci, Q, Km, V, 0.125)) < 1e-6


def run_spmm_flat(L, ro, ci, va, B, G, chunk):
    M, N = ro.size - 1, B.shape[1]
    C = np.full((M, N), np.nan, dtype=np.float32)
    writes = np.zeros((M, N), dtype=np.int32)
    rc = L.model_spmm_flat(M, N, pi(ro), pi(ci), pf(va), pf(B), G, chunk, pf(C), pi(writes))
    return rc, C, writes


def long_and_empty_rows(rng, M, K, n_long, long_len, short_avg):
    """A few very long rows, runs of hundreds of empty rows, short rows in between."""
    lens = rng.poisson(short_avg, M)
    lens[rng.random(M) < 0.5] = 0
    start = M // 3
    lens[start:start + min(400, M // 2)] = 0  # a run of empty rows longer than the 64-entry offset window
    for i in rng.choice(M, n_long, replace=False):
        lens[i] = long_len
    lens = np.minimum(lens, K)
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens] + [np.zeros(0, np.int64)]).astype(np.int32)
    return ro, ci


@pytest.mark.parametrize("case", ["uniform", "skewed", "empty_rows", "full", "long_and_empty", "one_row", "many_rows"])
def test_flat_schedule_writes_each_output_once_and_matches_the_oracle(model, oracle, case):
    """The flat schedule's row search, offset window and partial-row bookkeeping, index-checked on the CPU, for chunk
    sizes below, at and above the row lengths."""
    rng = np.random.default_rng(13)
    N = 8
    if case == "long_and_empty":
        M, K = 1500, 700
        ro, ci = long_and_empty_rows(rng, M, K, 3, 650, 3)
    elif case == "one_row":
        M, K = 1, 900
        ro, ci = random_csr(rng, M, K, "full", 1.0)
    elif case == "many_rows":
        M, K = 9000, 40  # more rows than two rounds of the 64-ary search cover
        ro, ci = random_csr(rng, M, K, "empty_rows", 0.05)
    else:
        M, K = 150, 300
        ro, ci = random_csr(rng, M, K, case, 0.2 if case != "full" else 1.0)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    ref = oracle.spmm(ro, ci, va, B)
    for chunk in (64, 128, 192, 512, 4096):
        for G in (64, 8):
            rc, C, writes = run_spmm_flat(model, ro, ci, va, B, G, chunk)
            assert rc == 0, f"chunk {chunk} G {G}: model returned {rc}"
            assert (writes == 1).all(), f"chunk {chunk} G {G}: an element was written {writes.min()}..{writes.max()} times"
            assert oracle.rel_frobenius(C, ref) < 1e-6


# ---- GPU: bit-for-bit ---------------------------------------------------------------------------------------------------
def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


GPU_SPMM = [(300, 200, 256, "skewed", 0.15), (128, 512, 128, "uniform", 0.3), (257, 129, 64, "skewed", 0.1),
            (100, 300, 32, "uniform", 0.05), (200, 512, 392, "uniform", 0.2), (90, 64, 130, "skewed", 0.3),
            (1000, 64, 16, "empty_rows", 0.05), (16, 700, 256, "full", 1.0), (4100, 300, 64, "skewed", 0.05),
            (64, 128, 49, "skewed", 0.2), (70, 90, 5, "uniform", 0.3), (10, 64, 1026, "uniform", 0.3),
            (300, 80, 1, "skewed", 0.3), (50, 80, 3, "uniform", 0.3),
            # several column tiles, narrower the taller B is: 256 columns from K > 2048, 128 from K > 4096
            (40, 2100, 600, "skewed", 0.05), (30, 4200, 530, "uniform", 0.02), (700, 4100, 1030, "empty_rows", 0.01),
            # ... down to 64 and 32 columns for a very tall B (no workspace in these calls)
            (2100, 16500, 100, "uniform", 0.005), (2060, 9000, 120, "skewed", 0.01)]


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,kind,density", GPU_SPMM)
def test_gpu_spmm_equals_model_bit_for_bit(model, dl, M, K, N, kind, density):
    import torch

    rng = np.random.default_rng(21 + M + N)
    ro, ci = random_csr(rng, M, K, kind, density)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size)
    rc, C, writes = run_spmm(model, ro, ci, va, B, sh["G"], sh["W"], sh["R"])
    assert rc == 0 and (writes == 1).all()
    got = dl.spmm(dev(torch, ro), dev(torch, ci), dev(torch, va), dev(torch, B), K=K).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), C.view(np.uint32)), \
        f"shape {sh}: {np.count_nonzero(got.view(np.uint32) != C.view(np.uint32))} of {got.size} elements differ in their bits"


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,D,kind,density", [(130, 257, 64, "skewed", 0.1), (256, 512, 128, "uniform", 0.05),
                                                (50, 100, 48, "uniform", 0.2), (64, 64, 16, "uniform", 0.3),
                                                (30, 64, 1024, "uniform", 0.3), (33, 77, 13, "uniform", 0.3),
                                                (40, 60, 49, "skewed", 0.3), (40, 60, 130, "uniform", 0.3),
                                                (30, 60, 513, "uniform", 0.3), (20, 60, 1027, "uniform", 0.3),
                                                (40, 60, 3, "uniform", 0.3), (40, 60, 7, "uniform", 0.3)])
def test_gpu_sddmm_and_fused_equal_model_bit_for_bit(model, dl, M, K, D, kind, density):
    import torch

    rng = np.random.default_rng(31 + M + D)
    ro, ci = random_csr(rng, M, K, kind, density)
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    V = rng.normal(0, 1, (K, D)).astype(np.float32)
    sh = dl.describe_launch(dl.OP_SDDMM, M, K, D, ci.size)
    out = np.empty(ci.size, dtype=np.float32)
    model.model_sddmm(M, D, pi(ro), pi(ci), pf(Q), pf(Km), sh["vec"], sh["G1"], sh["DS"], pf(out))
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    got = dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, Km)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), out.view(np.uint32)), f"sddmm shape {sh}"

    fs = dl.describe_launch(dl.OP_FUSED, M, K, D, ci.size)
    scores = np.empty(ci.size, dtype=np.float32)
    O = np.full((M, D), np.nan, dtype=np.float32)
    writes = np.zeros((M, D), dtype=np.int32)
    rc = model.model_fused(M, D, pi(ro), pi(ci), pf(Q), pf(Km), pf(V), 0.125, fs["vec"], fs["G1"], fs["DS"], fs["G"],
                           fs["W"], fs["R"], pf(scores), pf(O), pi(writes))
    assert rc == 0 and (writes == 1).all()
    gotO = dl.fused(ro_d, ci_d, dev(torch, Q), dev(torch, Km), dev(torch, V), 0.125).cpu().numpy()
    assert np.array_equal(gotO.view(np.uint32), O.view(np.uint32)), f"fused shape {fs}"


@pytest.mark.gpu
@pytest.mark.parametrize("kind,N,density", [("uniform", 128, 0.4), ("uniform", 32, 0.4), ("skewed", 128, 0.4),
                                            ("empty_rows", 64, 0.7)])
def test_gpu_rows_even_hint_equals_model_bit_for_bit(model, dl, kind, N, density):
    """A call that passes ROWS_EVEN on a tall matrix of long rows runs four rows per workgroup (one whole row per wave
    where the rows of a block are even, the nonzero-even split where they are not): the model reproduces both, also
    when the hint is wrong, and the results stay within the parity tolerance of the default call's."""
    import torch

    M, K = 4200, 600
    rng = np.random.default_rng(61 + N)
    ro, ci = random_csr(rng, M, K, kind, density)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    Q = rng.normal(0, 1, (M, N)).astype(np.float32)
    ro_d, ci_d, va_d, B_d, Q_d = (dev(torch, x) for x in (ro, ci, va, B, Q))

    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size, rows_even=True)
    assert (sh["W"], sh["R"]) == (4, 4) and dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size)["R"] < 4
    rc, C, writes = run_spmm(model, ro, ci, va, B, sh["G"], sh["W"], sh["R"])
    assert rc == 0 and (writes == 1).all()
    got = dl.spmm(ro_d, ci_d, va_d, B_d, K=K, workspace=dl.ROWS_EVEN).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), C.view(np.uint32)), f"spmm shape {sh}"
    plain = dl.spmm(ro_d, ci_d, va_d, B_d, K=K).cpu().numpy()
    assert np.linalg.norm(got - plain) <= 1e-5 * np.linalg.norm(plain)

    fs = dl.describe_launch(dl.OP_FUSED, M, K, N, ci.size, rows_even=True)
    assert (fs["W"], fs["R"]) == (4, 4)
    scores = np.empty(ci.size, dtype=np.float32)
    O = np.full((M, N), np.nan, dtype=np.float32)
    writes = np.zeros((M, N), dtype=np.int32)
    rc = model.model_fused(M, N, pi(ro), pi(ci), pf(Q), pf(B), pf(B), 0.125, fs["vec"], fs["G1"], fs["DS"], fs["G"],
                           fs["W"], fs["R"], pf(scores), pf(O), pi(writes))
    assert rc == 0 and (writes == 1).all()
    gotO = dl.fused(ro_d, ci_d, Q_d, B_d, B_d, 0.125, workspace=dl.ROWS_EVEN).cpu().numpy()
    assert np.array_equal(gotO.view(np.uint32), O.view(np.uint32)), f"fused shape {fs}"

    # SDDMM: every slot is one wave-independent dot product, so the hint cannot change a bit
    a = dl.sddmm(ro_d, ci_d, Q_d, B_d, workspace=dl.ROWS_EVEN)
    b = dl.sddmm(ro_d, ci_d, Q_d, B_d)
    assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("cfg", [1, 2, 3, 5])
def test_gpu_benchmark_configs_equal_model_bit_for_bit(model, dl, cfg):
    import torch

    c = dl.make_config(cfg)
    ro, ci = c["row_offsets"], c["col_indices"]
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    sh = dl.describe_launch(c["op"], c["M"], c["K"], c["N"], c["nnz"])
    if c["op"] == dl.OP_SPMM:
        rc, C, writes = run_spmm(model, ro, ci, c["values"], c["d0"], sh["G"], sh["W"], sh["R"])
        got = dl.spmm(ro_d, ci_d, dev(torch, c["values"]), dev(torch, c["d0"]), K=c["K"]).cpu().numpy()
        assert rc == 0 and (writes == 1).all()
        assert np.array_equal(got.view(np.uint32), C.view(np.uint32))
    elif c["op"] == dl.OP_SDDMM:
        out = np.empty(c["nnz"], dtype=np.float32)
        model.model_sddmm(c["M"], c["N"], pi(ro), pi(ci), pf(c["d0"]), pf(c["d1"]), sh["vec"], sh["G1"], sh["DS"], pf(out))
        got = dl.sddmm(ro_d, ci_d, dev(torch, c["d0"]), dev(torch, c["d1"])).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), out.view(np.uint32))
    else:
        scores = np.empty(c["nnz"], dtype=np.float32)
        O = np.full((c["M"], c["N"]), np.nan, dtype=np.float32)
        writes = np.zeros((c["M"], c["N"]), dtype=np.int32)
        rc = model.model_fused(c["M"], c["N"], pi(ro), pi(ci), pf(c["d0"]), pf(c["d1"]), pf(c["d2"]), c["scale"], sh["vec"],
                               sh["G1"], sh["DS"], sh["G"], sh["W"], sh["R"], pf(scores), pf(O), pi(writes))
        got = dl.fused(ro_d, ci_d, dev(torch, c["d0"]), dev(torch, c["d1"]), dev(torch, c["d2"]), c["scale"]).cpu().numpy()
        assert rc == 0 and (writes == 1).all()
        assert np.array_equal(got.view(np.uint32), O.view(np.uint32))


FLAT_GPU = [("uniform", 300, 200, 256, 0, 128), ("skewed", 257, 129, 64, 0, 64), ("long_and_empty", 1500, 700, 128, 3, 256),
            ("long_and_empty", 1500, 700, 49, 3, 512), ("long_and_empty", 5000, 600, 32, 5, 64), ("uniform", 200, 512, 392, 0, 192),
            ("full", 16, 700, 1030, 0, 320), ("empty_rows", 2000, 300, 5, 0, 64), ("skewed", 300, 80, 1, 0, 128)]


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K,N,n_long,chunk", FLAT_GPU)
def test_gpu_flat_spmm_equals_model_bit_for_bit(model, dl, kind, M, K, N, n_long, chunk):
    """The flat schedule (every wave owns `chunk` consecutive nonzeros; partial rows in the workspace, added by a second
    kernel), forced on small matrices and with small chunks so that rows are shared by many waves."""
    import torch

    rng = np.random.default_rng(41 + M + N)
    if kind == "long_and_empty":
        ro, ci = long_and_empty_rows(rng, M, K, n_long, K - 50, 3)
    else:
        ro, ci = random_csr(rng, M, K, kind, 1.0 if kind == "full" else 0.2)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    dl.set_tuning(flat=1, slices=0, flat_chunk=chunk)
    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size, with_workspace=True)
    assert sh["flat_chunk"] == chunk and sh["flat_units"] == -(-ci.size // chunk)
    need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, ci.size)
    assert need == sh["flat_units"] * 2 * N * 4
    rc, C, writes = run_spmm_flat(model, ro, ci, va, B, sh["G"], chunk)
    assert rc == 0 and (writes == 1).all()
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    args = (dev(torch, ro), dev(torch, ci), dev(torch, va), dev(torch, B))
    dl.spmm(*args, K=K, out=out, workspace=ws)
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), C.view(np.uint32)), \
        f"shape {sh}: {np.count_nonzero(got.view(np.uint32) != C.view(np.uint32))} of {got.size} elements differ in their bits"
    # a workspace that is too small is refused, none at all selects the workgroup-per-row-block schedule
    with pytest.raises(dl.DlspmError) as e:
        dl.spmm(*args, K=K, out=out, workspace=ws[: need // 4 - 1])
    assert e.value.status == dl.E_WORKSPACE
    out2 = dl.spmm(*args, K=K).cpu().numpy()
    assert np.linalg.norm(out2 - C) <= 1e-5 * np.linalg.norm(C)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K,D,n_long,chunk", [("uniform", 300, 200, 64, 0, 128), ("long_and_empty", 1500, 700, 128, 3, 256),
                                                      ("skewed", 130, 257, 49, 0, 64), ("long_and_empty", 900, 600, 256, 2, 192),
                                                      ("uniform", 40, 300, 1027, 0, 320), ("empty_rows", 500, 100, 3, 0, 64)])
def test_gpu_flat_fused_equals_model_bit_for_bit(model, dl, kind, M, K, D, n_long, chunk):
    import torch

    rng = np.random.default_rng(51 + M + D)
    if kind == "long_and_empty":
        ro, ci = long_and_empty_rows(rng, M, K, n_long, K - 50, 3)
    else:
        ro, ci = random_csr(rng, M, K, kind, 0.2)
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    V = rng.normal(0, 1, (K, D)).astype(np.float32)
    dl.set_tuning(flat=1, slices=0, flat_chunk=chunk)
    fs = dl.describe_launch(dl.OP_FUSED, M, K, D, ci.size)
    assert fs["flat_chunk"] == chunk
    need = dl.workspace_bytes(dl.OP_FUSED, M, K, D, ci.size)
    assert need == fs["flat_units"] * 2 * D * 4
    scores = np.empty(ci.size, dtype=np.float32)
    O = np.full((M, D), np.nan, dtype=np.float32)
    writes = np.zeros((M, D), dtype=np.int32)
    rc = model.model_fused_flat(M, D, pi(ro), pi(ci), pf(Q), pf(Km), pf(V), 0.125, fs["vec"], fs["G1"], fs["DS"], fs["G"],
                                chunk, pf(scores), pf(O), pi(writes))
    assert rc == 0 and (writes == 1).all()
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    out = torch.full((M, D), float("nan"), dtype=torch.float32, device="cuda")
    dl.fused(dev(torch, ro), dev(torch, ci), dev(torch, Q), dev(torch, Km), dev(torch, V), 0.125, out=out, workspace=ws)
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), O.view(np.uint32)), \
        f"shape {fs}: {np.count_nonzero(got.view(np.uint32) != O.view(np.uint32))} of {got.size} elements differ in their bits"


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K,D,n_long,chunk", [("uniform", 300, 200, 64, 0, 128), ("long_and_empty", 1500, 700, 128, 3, 256),
                                                      ("skewed", 130, 257, 49, 0, 64), ("long_and_empty", 5000, 600, 32, 5, 64),
                                                      ("uniform", 40, 300, 1027, 0, 320), ("empty_rows", 500, 100, 3, 0, 64)])
def test_gpu_flat_sddmm_equals_model_and_the_row_block_schedule_bit_for_bit(model, dl, kind, M, K, D, n_long, chunk):
    """SDDMM's flat schedule changes which wave computes a dot product, not how: both schedules must give the model's bits."""
    import torch

    rng = np.random.default_rng(61 + M + D)
    if kind == "long_and_empty":
        ro, ci = long_and_empty_rows(rng, M, K, n_long, K - 50, 3)
    else:
        ro, ci = random_csr(rng, M, K, kind, 0.2)
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    sh = dl.describe_launch(dl.OP_SDDMM, M, K, D, ci.size)
    assert sh["flat_chunk"] == 0
    ref = np.empty(ci.size, dtype=np.float32)
    model.model_sddmm(M, D, pi(ro), pi(ci), pf(Q), pf(Km), sh["vec"], sh["G1"], sh["DS"], pf(ref))
    args = (dev(torch, ro), dev(torch, ci), dev(torch, Q), dev(torch, Km))
    block = dl.sddmm(*args).cpu().numpy()
    dl.set_tuning(flat=1, slices=0, flat_chunk=chunk)
    assert dl.describe_launch(dl.OP_SDDMM, M, K, D, ci.size)["flat_chunk"] == chunk
    assert dl.workspace_bytes(dl.OP_SDDMM, M, K, D, ci.size) == 0
    out = torch.full((ci.size,), float("nan"), dtype=torch.float32, device="cuda")
    dl.sddmm(*args, out=out)
    flat = out.cpu().numpy()
    assert np.array_equal(flat.view(np.uint32), ref.view(np.uint32))
    assert np.array_equal(block.view(np.uint32), ref.view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_gpu_random_shapes_equal_model_bit_for_bit(model, dl, seed):
    """Forty random (shape, pattern, width, schedule, chunk) draws per seed, all three entry points, bit for bit."""
    import torch

    rng = np.random.default_rng(seed)
    for it in range(40):
        M = int(rng.choice([1, 2, 7, 63, 64, 65, 200, 700, 2500])) + int(rng.integers(0, 5))
        K = int(rng.choice([1, 3, 64, 130, 500, 1500])) + int(rng.integers(0, 5))
        N = int(rng.choice([1, 2, 3, 4, 5, 8, 31, 32, 33, 64, 100, 128, 196, 256, 257, 392, 512, 700, 1030]))
        kind = str(rng.choice(["uniform", "skewed", "empty_rows", "full", "empty"]))
        if kind == "full" and M * K > 300000:
            kind = "uniform"
        density = float(rng.choice([0.02, 0.1, 0.3, 0.7]))
        ro, ci = random_csr(rng, M, K, kind, 1.0 if kind == "full" else density)
        nnz = ci.size
        flat = bool(rng.integers(0, 2)) and nnz > 0
        chunk = int(rng.choice([64, 128, 192, 320, 512, 1024]))
        dl.set_tuning(flat=1 if flat else 0, slices=0, flat_chunk=chunk)
        tag = f"seed {seed} draw {it}: M {M} K {K} N {N} {kind} {density} nnz {nnz} flat {flat} chunk {chunk}"
        print(tag, flush=True)
        va = rng.normal(0, 1, max(nnz, 1)).astype(np.float32)
        B = rng.normal(0, 1, (K, N)).astype(np.float32)
        Q = rng.normal(0, 1, (M, N)).astype(np.float32)
        V = rng.normal(0, 1, (K, N)).astype(np.float32)
        ci2 = ci if nnz else np.zeros(1, np.int32)
        ro_d, ci_d = dev(torch, ro), dev(torch, ci)
        bits = lambda a: np.ascontiguousarray(a).view(np.uint32)

        sh = dl.describe_launch(dl.OP_SPMM, M, K, N, nnz, with_workspace=flat)
        if flat:
            rc, C, writes = run_spmm_flat(model, ro, ci2, va, B, sh["G"], chunk)
        else:
            rc, C, writes = run_spmm(model, ro, ci2, va, B, sh["G"], sh["W"], sh["R"])
        assert rc == 0 and (writes == 1).all(), tag
        need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, nnz)
        ws = torch.full((max(need // 4, 1),), float("nan"), device="cuda") if flat else None
        out = torch.full((M, N), float("nan"), device="cuda")
        dl.spmm(ro_d, ci_d, dev(torch, va)[:nnz], dev(torch, B), K=K, out=out, workspace=ws)
        assert np.array_equal(bits(out.cpu().numpy()), bits(C)), "spmm " + tag

        if nnz:
            sh = dl.describe_launch(dl.OP_SDDMM, M, K, N, nnz)
            ref = np.empty(nnz, np.float32)
            model.model_sddmm(M, N, pi(ro), pi(ci), pf(Q), pf(B), sh["vec"], sh["G1"], sh["DS"], pf(ref))
            o = torch.full((nnz,), float("nan"), device="cuda")
            dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, B), out=o)
            assert np.array_equal(bits(o.cpu().numpy()), bits(ref)), "sddmm " + tag

        fs = dl.describe_launch(dl.OP_FUSED, M, K, N, nnz)
        scores = np.empty(max(nnz, 1), np.float32)
        O = np.full((M, N), np.nan, np.float32)
        writes = np.zeros((M, N), np.int32)
        if flat:
            rc = model.model_fused_flat(M, N, pi(ro), pi(ci2), pf(Q), pf(B), pf(V), 0.25, fs["vec"], fs["G1"], fs["DS"], fs["G"],
                                        chunk, pf(scores), pf(O), pi(writes))
        else:
            rc = model.model_fused(M, N, pi(ro), pi(ci2), pf(Q), pf(B), pf(V), 0.25, fs["vec"], fs["G1"], fs["DS"], fs["G"],
                                   fs["W"], fs["R"], pf(scores), pf(O), pi(writes))
        assert rc == 0 and (writes == 1).all(), tag
        need = dl.workspace_bytes(dl.OP_FUSED, M, K, N, nnz)
        ws = torch.full((max(need // 4, 1),), float("nan"), device="cuda") if flat else None
        out = torch.full((M, N), float("nan"), device="cuda")
        dl.fused(ro_d, ci_d, dev(torch, Q), dev(torch, B), dev(torch, V), 0.25, out=out, workspace=ws)
        assert np.array_equal(bits(out.cpu().numpy()), bits(O)), "fused " + tag


# ---- column-sliced schedule ------------------------------------------------------------------------------------------
def column_slices(ro, ci, K, slices):
    """The sparse matrix cut into `slices` equal column ranges: per range its own CSR row offsets and the mask of the
    nonzeros it keeps (columns ascend inside a row, so each row's share is one run of the row)."""
    M = ro.size - 1
    rows = np.repeat(np.arange(M), np.diff(ro))
    out = []
    for p in range(slices):
        lo, hi = p * K // slices, (p + 1) * K // slices
        keep = (ci >= lo) & (ci < hi)
        rop = np.zeros(M + 1, dtype=np.int32)
        rop[1:] = np.cumsum(np.bincount(rows[keep], minlength=M))
        out.append((rop, keep))
    assert sum(k.sum() for _, k in out) == ci.size
    return out


SLICED_CASES = [("uniform", 300, 512, 128, 3), ("skewed", 1100, 700, 256, 2), ("empty_rows", 500, 300, 392, 4),
                ("long_and_empty", 1500, 700, 128, 5), ("full", 40, 256, 96, 16), ("uniform", 70, 900, 513, 7),
                ("skewed", 90, 4200, 530, 3), ("skewed", 300, 400, 48, 3), ("uniform", 200, 300, 20, 4),
                ("empty_rows", 400, 200, 7, 2)]


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K,N,slices", SLICED_CASES)
def test_gpu_sliced_spmm_equals_model_bit_for_bit(model, dl, oracle, kind, M, K, N, slices):
    """Column-sliced SpMM = the row-block kernel's arithmetic on each column range of the matrix (the model, run on
    that range's own CSR arrays with the split the library reports), the ranges' partial rows added in range order."""
    import torch

    rng = np.random.default_rng(71 + M + N)
    if kind == "long_and_empty":
        ro, ci = long_and_empty_rows(rng, M, K, 3, K - 50, 3)
    else:
        ro, ci = random_csr(rng, M, K, kind, 1.0 if kind == "full" else 0.2)
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    assert dl.describe_slices(dl.OP_SPMM, M, K, N, ci.size)[0] == 0       # far too small for the rule
    dl.set_tuning(slices=slices)
    got_slices, R = dl.describe_slices(dl.OP_SPMM, M, K, N, ci.size)
    assert got_slices == slices and R in (1, 2, 4, 8, 16)
    sh = dl.describe_launch(dl.OP_SPMM, M, K, N, ci.size, with_workspace=True)
    need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, ci.size)
    assert need >= (slices + 1) * M * 4 + slices * M * N * 4

    expect = None
    for rop, keep in column_slices(ro, ci, K, slices):
        rc, part, writes = run_spmm(model, rop, ci[keep], va[keep], B, sh["G"], 4, R)
        assert rc == 0 and (writes == 1).all()
        expect = part if expect is None else expect + part
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    args = (dev(torch, ro), dev(torch, ci), dev(torch, va), dev(torch, B))
    dl.spmm(*args, K=K, out=out, workspace=ws)
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), expect.view(np.uint32)), \
        f"{np.count_nonzero(got.view(np.uint32) != expect.view(np.uint32))} of {got.size} elements differ in their bits"
    ref = oracle.spmm(ro, ci, va, B)
    assert np.linalg.norm(got - ref) <= 1e-5 * max(np.linalg.norm(ref), 1e-30)
    with pytest.raises(dl.DlspmError) as e:
        dl.spmm(*args, K=K, out=out, workspace=ws[: need // 4 - 1])
    assert e.value.status == dl.E_WORKSPACE


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K,D,slices", [("uniform", 300, 512, 128, 3), ("skewed", 700, 600, 256, 2),
                                               ("long_and_empty", 900, 600, 100, 4), ("empty_rows", 200, 300, 512, 5),
                                               ("uniform", 150, 400, 200, 16), ("skewed", 500, 700, 64, 3),
                                               ("uniform", 300, 200, 24, 4)])
def test_gpu_sliced_fused_equals_model_bit_for_bit(model, dl, oracle, kind, M, K, D, slices):
    import torch

    rng = np.random.default_rng(81 + M + D)
    if kind == "long_and_empty":
        ro, ci = long_and_empty_rows(rng, M, K, 2, K - 50, 3)
    else:
        ro, ci = random_csr(rng, M, K, kind, 0.2)
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    V = rng.normal(0, 1, (K, D)).astype(np.float32)
    dl.set_tuning(slices=slices)
    got_slices, R = dl.describe_slices(dl.OP_FUSED, M, K, D, ci.size)
    assert got_slices == slices
    fs = dl.describe_launch(dl.OP_FUSED, M, K, D, ci.size)
    need = dl.workspace_bytes(dl.OP_FUSED, M, K, D, ci.size)

    expect = None
    for rop, keep in column_slices(ro, ci, K, slices):
        cip = ci[keep] if keep.any() else np.zeros(1, np.int32)
        scores = np.empty(max(int(keep.sum()), 1), dtype=np.float32)
        part = np.full((M, D), np.nan, dtype=np.float32)
        writes = np.zeros((M, D), dtype=np.int32)
        rc = model.model_fused(M, D, pi(rop), pi(cip), pf(Q), pf(Km), pf(V), 0.125, fs["vec"], fs["G1"], fs["DS"], fs["G"],
                               4, R, pf(scores), pf(part), pi(writes))
        assert rc == 0 and (writes == 1).all()
        expect = part if expect is None else expect + part
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    out = torch.full((M, D), float("nan"), dtype=torch.float32, device="cuda")
    dl.fused(dev(torch, ro), dev(torch, ci), dev(torch, Q), dev(torch, Km), dev(torch, V), 0.125, out=out, workspace=ws)
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), expect.view(np.uint32)), \
        f"{np.count_nonzero(got.view(np.uint32) != expect.view(np.uint32))} of {got.size} elements differ in their bits"
    ref = oracle.fused(ro, ci, Q, Km, V, 0.125)
    assert np.linalg.norm(got - ref) <= 1e-5 * max(np.linalg.norm(ref), 1e-30)


@pytest.mark.gpu
def test_gpu_sliced_schedule_does_not_need_ascending_columns(dl, oracle):
    """The slice boundaries are found by a search that assumes ascending columns; with any other order they are still
    a partition of every row (a running maximum), so the result stays right."""
    import torch

    rng = np.random.default_rng(91)
    M, K, N = 400, 500, 128
    ro, ci = random_csr(rng, M, K, "skewed", 0.2)
    ci = ci.copy()
    for i in range(M):
        rng.shuffle(ci[ro[i]:ro[i + 1]])
    va = rng.normal(0, 1, ci.size).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    dl.set_tuning(slices=4)
    need = dl.workspace_bytes(dl.OP_SPMM, M, K, N, ci.size)
    ws = torch.empty(need // 4, dtype=torch.float32, device="cuda")
    got = dl.spmm(dev(torch, ro), dev(torch, ci), dev(torch, va), dev(torch, B), K=K, workspace=ws).cpu().numpy()
    ref = oracle.spmm(ro, ci, va, B)
    assert np.linalg.norm(got - ref) <= 1e-5 * np.linalg.norm(ref)
    Q = rng.normal(0, 1, (M, N)).astype(np.float32)
    need = dl.workspace_bytes(dl.OP_FUSED, M, K, N, ci.size)
    ws = torch.empty(need // 4, dtype=torch.float32, device="cuda")
    gotO = dl.fused(dev(torch, ro), dev(torch, ci), dev(torch, Q), dev(torch, B), dev(torch, B), 0.125, workspace=ws).cpu().numpy()
    refO = oracle.fused(ro, ci, Q, B, B, 0.125)
    assert np.linalg.norm(gotO - refO) <= 1e-5 * np.linalg.norm(refO)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K,D,slices", [("uniform", 300, 512, 128, 3), ("skewed", 700, 600, 256, 2),
                                               ("long_and_empty", 900, 600, 100, 4), ("empty_rows", 200, 300, 512, 5),
                                               ("full", 60, 256, 65, 16), ("skewed", 500, 700, 64, 3),
                                               ("uniform", 300, 200, 20, 4)])
def test_gpu_sliced_sddmm_gives_the_same_bits(dl, oracle, kind, M, K, D, slices):
    """Every SDDMM result is one dot product computed by one lane group in a fixed order, whatever the schedule: the
    column-sliced call must reproduce the plain call bit for bit, and leave no slot unwritten."""
    import torch

    rng = np.random.default_rng(95 + M + D)
    if kind == "long_and_empty":
        ro, ci = long_and_empty_rows(rng, M, K, 2, K - 50, 3)
    else:
        ro, ci = random_csr(rng, M, K, kind, 1.0 if kind == "full" else 0.2)
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    args = (dev(torch, ro), dev(torch, ci), dev(torch, Q), dev(torch, Km))
    plain = dl.sddmm(*args)
    assert dl.workspace_bytes(dl.OP_SDDMM, M, K, D, ci.size) == 0
    dl.set_tuning(slices=slices)
    assert dl.describe_slices(dl.OP_SDDMM, M, K, D, ci.size)[0] == slices
    need = dl.workspace_bytes(dl.OP_SDDMM, M, K, D, ci.size)
    assert need >= (slices + 1) * M * 4
    ws = torch.empty(need // 4, dtype=torch.int32, device="cuda")
    out = torch.full((ci.size,), float("nan"), dtype=torch.float32, device="cuda")
    dl.sddmm(*args, out=out, workspace=ws)
    assert torch.equal(out, plain)
    ref = oracle.sddmm(ro, ci, Q, Km)
    assert np.linalg.norm(out.cpu().numpy() - ref) <= 1e-5 * np.linalg.norm(ref)
    with pytest.raises(dl.DlspmError) as e:
        dl.sddmm(*args, out=out, workspace=ws[: need // 4 - 1])
    assert e.value.status == dl.E_WORKSPACE



# ---- row plan: the device build against its sequential definition ---------------------------------------------------
def model_plan(L, ro, bins, order=0):
    M = ro.size - 1
    plan = np.empty(3 * M, dtype=np.int32)
    L.model_row_plan(M, pi(np.ascontiguousarray(ro, dtype=np.int32)), bins, order, pi(plan))
    return plan


def test_model_row_plan_is_a_balanced_permutation(model, dl):
    """CPU: the sequential definition of the plan. Every row once, with its own offsets; the first 2048 positions in
    256 bins whose loads differ far less than in matrix order; rows without nonzeros last in their bins."""
    c = dl.make_config(2)
    ro = c["row_offsets"]
    M = ro.size - 1
    plan = model_plan(model, ro, 256)
    starts, ends, rows = plan[:M], plan[M:2 * M], plan[2 * M:]
    assert np.array_equal(np.sort(rows), np.arange(M))
    assert np.array_equal(starts, ro[rows]) and np.array_equal(ends, ro[rows + 1])
    lens = np.diff(ro)
    packed = np.array([lens[rows[b::256]].sum() for b in range(256)])
    plain = np.array([lens[b::256].sum() for b in range(256)])
    assert packed.max() <= 1.1 * packed.mean() < 0.75 * plain.max()
    # the two simpler orders
    desc = model_plan(model, ro, 256, 2)[2 * M:]
    assert (np.diff(lens[desc]) <= 0).all()
    alt = model_plan(model, ro, 256, 1)[2 * M:]
    assert np.array_equal(alt[:256], desc[:256]) and np.array_equal(alt[256:512], desc[256:512][::-1])
    # rows without nonzeros take what is left, in order
    ro2 = np.zeros(11, dtype=np.int32)
    ro2[1:] = np.cumsum([5, 0, 3, 0, 0, 9, 1, 0, 2, 2])
    assert model_plan(model, ro2, 4)[20:].tolist() == [5, 0, 2, 8, 1, 3, 6, 9, 4, 7]


PLAN_CASES = [("cfg2", 0, 0), ("skewed", 1, 60), ("skewed", 2, 60), ("uniform", 7, 33), ("skewed", 255, 400), ("skewed", 256, 400),
              ("empty_rows", 257, 300), ("skewed", 2047, 512), ("empty_rows", 2048, 700), ("skewed", 2049, 512),
              ("empty", 1500, 64), ("full", 900, 37), ("skewed", 5000, 2048), ("empty_rows", 20000, 256),
              ("skewed", 70001, 128), ("uniform", 300000, 64)]


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,K", PLAN_CASES)
def test_gpu_row_plan_equals_its_sequential_definition(model, dl, kind, M, K):
    """dlspm_row_plan_build builds the plan with kernels (tile sort, merge passes, batched packing); every entry must
    equal the sequential host definition, for every order, from one row to 300000 (one launch up to 2048 rows, tiles
    and merges beyond), with empty rows, equal rows and rows of one length only."""
    import torch

    if kind == "cfg2":
        ro = dl.make_config(2)["row_offsets"]
        M = ro.size - 1
    else:
        ro, _ = random_csr(np.random.default_rng(M + K), M, K, kind, 0.15)
    info = dl.device_info()
    assert info["status"] == dl.OK and info["gfx950"] and info["compute_units"] > 0 and info["l2_bytes"] >= 1 << 20
    bins = min(info["compute_units"], 256)
    ro_d = dev(torch, ro)
    for order in (0, 1, 2):
        dl.set_tuning(plan_order=order)
        plan = torch.full((dl.row_plan_bytes(M) // 4,), -7, dtype=torch.int32, device="cuda")
        dl.row_plan(ro_d, out=plan)
        got = plan.cpu().numpy()[:3 * M]
        want = model_plan(model, ro, bins, order)
        assert np.array_equal(got, want), (kind, M, K, order, np.flatnonzero(got != want)[:10])
    dl.set_tuning()
    assert np.array_equal(ro_d.cpu().numpy(), ro)


@pytest.mark.gpu
@pytest.mark.parametrize("M,longest,seed", [(700, 1 << 21, 1), (2048, (1 << 21) - 1, 2), (640, 3_000_000, 3), (5000, 2_500_000, 4),
                                            (2048, 1 << 20, 5)])
def test_gpu_row_plan_with_very_long_rows(model, dl, M, longest, seed):
    """The plan needs row_offsets only, so rows of millions of nonzeros can be planned without a matrix behind them:
    from 2^21 nonzeros in one row on, the tile sort and the packing work on 64-bit keys instead of 32-bit ones; both
    forms, and the boundary between them, must give the sequential definition."""
    import torch

    rng = np.random.default_rng(seed)
    lens = rng.integers(0, 2000, M)
    heavy = rng.choice(M, size=min(M, 600), replace=False)
    lens[heavy] = rng.integers(longest // 2, longest + 1, heavy.size)
    lens[heavy[0]] = longest
    while lens.sum() >= (1 << 31) - 1:  # row_offsets are 32-bit
        heavy = heavy[: heavy.size // 2]
        lens[:] = np.minimum(lens, 2000)
        lens[heavy] = rng.integers(longest // 2, longest + 1, heavy.size)
        lens[heavy[0]] = longest
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    bins = min(dl.device_info()["compute_units"], 256)
    ro_d = dev(torch, ro)
    for order in (0, 2):
        dl.set_tuning(plan_order=order)
        plan = torch.full((dl.row_plan_bytes(M) // 4,), -7, dtype=torch.int32, device="cuda")
        dl.row_plan(ro_d, out=plan)
        got = plan.cpu().numpy()[:3 * M]
        want = model_plan(model, ro, bins, order)
        assert np.array_equal(got, want), (M, longest, order, np.flatnonzero(got != want)[:10])
    dl.set_tuning()
