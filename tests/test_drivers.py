"""The C++ drivers (dlspm-esimd_amd/bin/{spmm,sddmm,fused}_run): command-line and file error handling on the CPU,
and on the GPU their single-matrix, from-file, batch and sweep runs, whose dumped outputs are checked here against
the CPU oracle (the drivers themselves only cross-check on the device)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import random_csr

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "dlspm-esimd_amd", "bin")


def run(app, *args):
    exe = os.path.join(BIN, app)
    assert os.path.exists(exe), f"{exe} is missing: run `make -C dlspm-esimd_amd drivers`"
    p = subprocess.run([exe, *map(str, args)], capture_output=True, text=True, timeout=300)
    return p.returncode, p.stdout + p.stderr


def write_smtx(path, M, K, ro, ci):
    with open(path, "w") as f:
        f.write(f"{M}, {K}, {len(ci)}\n")
        f.write(" ".join(map(str, ro)) + "\n")
        f.write(" ".join(map(str, ci)) + "\n")


# ---- CPU: the failure paths the reference's drivers have (wrong argc, unopenable file, short file, bad CSR)
@pytest.mark.parametrize("app", ["spmm_run", "sddmm_run", "fused_run"])
def test_usage_and_file_errors(app, tmp_path):
    rc, out = run(app)
    assert rc == 1 and "Usage:" in out and ".smtx" in out
    rc, out = run(app, "only_one_positional.smtx")
    assert rc == 1 and "Usage:" in out
    rc, out = run(app, tmp_path / "missing.smtx", 64)
    assert rc == 1 and "Error opening file!" in out
    (tmp_path / "short.smtx").write_text("4, 4, 5\n0 1 2\n")
    rc, out = run(app, tmp_path / "short.smtx", 64)
    assert rc == 1 and "Something went wrong reading row_offsets" in out
    (tmp_path / "garbled.smtx").write_text("four by four\n")
    rc, out = run(app, tmp_path / "garbled.smtx", 64)
    assert rc == 1 and "Something went wrong readin M, K, nnz" in out
    (tmp_path / "nocols.smtx").write_text("2, 4, 3\n0 2 3\n0 1\n")
    rc, out = run(app, tmp_path / "nocols.smtx", 64)
    assert rc == 1 and "Something went wrong reading column_indices" in out


@pytest.mark.parametrize("text,message", [
    ("2, 2, 3\n0 2 3\n0 1 5\n", "a_column_indices[i] >= KSZ"),
    ("2, 2, 3\n0 2 4\n0 1 1\n", "a_row_offsets[MSZ] != nnz."),
    ("3, 4, 3\n0 2 1 3\n0 1 1\n", "a_row_offsets[i+1] < a_row_offsets[i]"),
    ("1, 2, 3\n0 3\n0 1 1\n", "nnz is larger than matrix."),
    ("2, 2, 3\n0 3 3\n0 1 1\n", "a_row_offsets[i + 1] - a_row_offsets[i] > KSZ"),
])
def test_sanity_check_messages(tmp_path, text, message):
    """Same tests and messages as the reference's SanityCheck (SPMM/spmm-esimd-fromfile2.cpp:36-61)."""
    (tmp_path / "bad.smtx").write_text(text)
    rc, out = run("spmm_run", tmp_path / "bad.smtx", 16)
    assert rc == 1 and message in out


def test_cfg_of_wrong_kind_is_refused():
    rc, out = run("spmm_run", "--cfg", 3)
    assert rc == 1 and "not an SpMM configuration" in out


# ---- GPU -------------------------------------------------------------------------------------------------------------
def load_dump(d):
    meta = json.load(open(os.path.join(d, "meta.json")))
    arr = lambda name, dt: np.fromfile(os.path.join(d, name), dtype=dt)
    return meta, arr


@pytest.mark.gpu
@pytest.mark.parametrize("cfg,app", [(1, "spmm_run"), (2, "spmm_run"), (4, "spmm_run"), (3, "sddmm_run"), (5, "fused_run")])
def test_driver_runs_benchmark_configuration(oracle, dl, tmp_path, cfg, app):
    rc, out = run(app, "--cfg", cfg, "--dump", tmp_path, "--csv", tmp_path / "r.csv", "--cold")
    print(out)
    assert rc == 0 and "PASS" in out and "bit-identical" in out and "GFLOPS:" in out and "Total kernel time was" in out
    meta, arr = load_dump(str(tmp_path))
    c = dl.make_config(cfg)  # the Python binding and the driver share one generator: same data
    ro, ci = arr("row_offsets.i32", np.int32), arr("col_indices.i32", np.int32)
    assert np.array_equal(ro, c["row_offsets"]) and np.array_equal(ci, c["col_indices"])
    M, K, N = meta["M"], meta["K"], meta["N"]
    if meta["op"] == "spmm":
        ref = oracle.spmm(ro, ci, arr("values.f32", np.float32), arr("B.f32", np.float32).reshape(K, N), omp=True)
        got = arr("C.f32", np.float32).reshape(M, N)
    elif meta["op"] == "sddmm":
        ref = oracle.sddmm(ro, ci, arr("lhs.f32", np.float32).reshape(M, N), arr("rhs.f32", np.float32).reshape(K, N), omp=True)
        got = arr("out.f32", np.float32)
    else:
        ref = oracle.fused(ro, ci, arr("Q.f32", np.float32).reshape(M, N), arr("K.f32", np.float32).reshape(K, N),
                           arr("V.f32", np.float32).reshape(K, N), meta["scale"], omp=True)
        got = arr("O.f32", np.float32).reshape(M, N)
    assert oracle.rel_frobenius(got, ref) <= 1e-4
    assert len(open(tmp_path / "r.csv").read().strip().split(",")) >= 6


@pytest.mark.gpu
@pytest.mark.parametrize("app,width", [("spmm_run", 49), ("sddmm_run", 64), ("fused_run", 32)])
def test_driver_from_file_and_batch(oracle, tmp_path, app, width):
    """`./app <file>.smtx <N>` as in the reference, N = 49 being one of the un-padded rn50 batch sizes."""
    rng = np.random.default_rng(3)
    M, K = 128, 300
    ro, ci = random_csr(rng, M, K, "empty_rows", 0.1)
    write_smtx(tmp_path / "a.smtx", M, K, ro, ci)
    dump = tmp_path / "dump"
    dump.mkdir()
    rc, out = run(app, tmp_path / "a.smtx", width, "--dump", dump, "--csv", tmp_path / "f.csv")
    print(out)
    assert rc == 0 and "PASS" in out and f"nnz: {len(ci)}" in out
    meta, arr = load_dump(str(dump))
    assert np.array_equal(arr("row_offsets.i32", np.int32), ro) and np.array_equal(arr("col_indices.i32", np.int32), ci)
    if meta["op"] == "spmm":
        ref = oracle.spmm(ro, ci, arr("values.f32", np.float32), arr("B.f32", np.float32).reshape(K, width))
        got = arr("C.f32", np.float32).reshape(M, width)
        assert len(open(tmp_path / "f.csv").read().strip().split(",")) == 7  # M,N,K,SP,gflops,max_diff,opcount
    elif meta["op"] == "sddmm":
        ref = oracle.sddmm(ro, ci, arr("lhs.f32", np.float32).reshape(M, width), arr("rhs.f32", np.float32).reshape(K, width))
        got = arr("out.f32", np.float32)
    else:
        ref = oracle.fused(ro, ci, arr("Q.f32", np.float32).reshape(M, width), arr("K.f32", np.float32).reshape(K, width),
                           arr("V.f32", np.float32).reshape(K, width), 1.0)
        got = arr("O.f32", np.float32).reshape(M, width)
    assert oracle.rel_frobenius(got, ref) <= 1e-4
    (tmp_path / "list.txt").write_text(f"# two runs of the same pattern\n{tmp_path / 'a.smtx'} 16\n{tmp_path / 'a.smtx'} 128\n")
    rc, out = run(app, "--batch", tmp_path / "list.txt")
    assert rc == 0 and out.count("PASS") == 2


@pytest.mark.gpu
def test_driver_shape_and_small_sweep():
    rc, out = run("spmm_run", "--shape", 512, 256, 64, 0.2, "--seed", 9)
    assert rc == 0 and "PASS" in out and "MSZ = 512 KSZ = 256 NSZ = 64" in out
    rc, out = run("sddmm_run", "--sweep", "--max-m", 1024, "--iters", 5)
    assert rc == 0 and out.count("PASS") == 6  # (1024,1024) x N in {32,128} x density in {0.3,0.2,0.1}


@pytest.mark.gpu
@pytest.mark.parametrize("app,cfg", [("spmm_run", 2), ("sddmm_run", 3), ("fused_run", 5)])
def test_driver_graph_timing(oracle, app, cfg, tmp_path):
    """--graph n: the launch is also captured n times into a HIP graph (row plan or workspace included) and the replay
    timed as a whole; the result is checked and dumped after those replays, and a launch inside the graph does not take
    longer than a launch between its own pair of events."""
    import re

    d = tmp_path / "dump"
    d.mkdir()
    rc, out = run(app, "--cfg", cfg, "--graph", 40, "--dump", d)
    assert rc == 0 and "PASS" in out, out[-800:]
    m = re.search(r"in a HIP graph of 40 launches: ([0-9.]+) ms per launch, GFLOPS: +([0-9.]+)", out)
    assert m, out[-800:]
    single = float(re.search(r"Total kernel time was ([0-9.]+) ms", out).group(1))
    assert 0 < float(m.group(1)) <= single * 1.05
    meta, err = verify_dump(oracle, str(d))
    assert err <= 1e-4


def verify_dump(oracle, d):
    """Relative Frobenius error of one driver dump (inputs and the kernel's output) against the CPU oracle."""
    meta, arr = load_dump(d)
    M, K, N = meta["M"], meta["K"], meta["N"]
    ro, ci = arr("row_offsets.i32", np.int32), arr("col_indices.i32", np.int32)
    assert ro.size == M + 1 and ci.size == meta["nnz"] and ro[-1] == meta["nnz"]
    if meta["op"] == "spmm":
        ref = oracle.spmm(ro, ci, arr("values.f32", np.float32), arr("B.f32", np.float32).reshape(K, N), omp=True)
        got = arr("C.f32", np.float32).reshape(M, N)
    elif meta["op"] == "sddmm":
        ref = oracle.sddmm(ro, ci, arr("lhs.f32", np.float32).reshape(M, N), arr("rhs.f32", np.float32).reshape(K, N), omp=True)
        got = arr("out.f32", np.float32)
    else:
        ref = oracle.fused(ro, ci, arr("Q.f32", np.float32).reshape(M, N), arr("K.f32", np.float32).reshape(K, N),
                           arr("V.f32", np.float32).reshape(K, N), meta["scale"], omp=True)
        got = arr("O.f32", np.float32).reshape(M, N)
    return meta, oracle.rel_frobenius(got, ref)


SWEEP_GRID_2048 = [(M, K, N, sp) for N in (32, 128) for (M, K) in ((1024, 1024), (2048, 2048)) for sp in (0.3, 0.2, 0.1)]


@pytest.mark.gpu
@pytest.mark.parametrize("app", ["spmm_run", "sddmm_run", "fused_run"])
def test_sweep_against_the_oracle_and_csv_columns(oracle, tmp_path, app):
    """The in-process sweep of the reference (grid SPMM/spmm-esimd-allbenchs2.cpp:252-266, CSV rows :221-226 and
    SDDMM/sddmm-esimd-allbench_v4.cpp:204-209) up to 2048 rows: every case's dumped output is verified here against
    the CPU oracle (the drivers' own PASS only compares with an on-device check kernel), and the CSV has the
    reference's columns, one row per case, in grid order."""
    dumps = tmp_path / "dumps"
    rc, out = run(app, "--sweep", "--max-m", 2048, "--iters", 3, "--warmup", 1, "--dump-each", dumps, "--csv", tmp_path / "s.csv")
    assert rc == 0 and out.count("PASS") == len(SWEEP_GRID_2048), out[-3000:]
    rows = [l.split(",") for l in open(tmp_path / "s.csv").read().strip().splitlines()]
    assert len(rows) == len(SWEEP_GRID_2048)
    for i, (M, K, N, sp) in enumerate(SWEEP_GRID_2048):
        meta, err = verify_dump(oracle, str(dumps / f"case_{i:03d}"))
        assert (meta["M"], meta["K"], meta["N"]) == (M, K, N)
        assert err <= 1e-4, (app, i, err)
        row = [float(x) for x in rows[i]]
        density = meta["nnz"] / (M * K)
        assert abs(density - sp) < 0.01
        if app == "spmm_run":    # M,N,K,SP,gflops,max_rel_diff
            assert len(row) == 6 and row[:3] == [M, N, K] and abs(row[3] - density) < 1e-5 and row[4] > 0 and 0 <= row[5] < 1e-3
        elif app == "sddmm_run":  # M,K,N,SP,gflops,calc_bw,max_diff
            assert len(row) == 7 and row[:3] == [M, K, N] and abs(row[3] - density) < 1e-5 and row[4] > 0 and row[5] > 0 and 0 <= row[6] < 1e-3
        else:                     # M,K,N,SP,gflops,max_diff (FUSED/fused-esimd_cb.cpp prints these; it writes no CSV)
            assert len(row) == 6 and row[:3] == [M, K, N] and abs(row[3] - density) < 1e-5 and row[4] > 0 and 0 <= row[5] < 1e-3


@pytest.mark.gpu
def test_vendor_comparator_against_the_oracle(oracle, dl, tmp_path):
    """bin/vendor_compare (rocSPARSE in the role of the reference's cuSPARSE harness, CUSPARSE/spmm_fromfile.cu:175-234,
    CUSPARSE/sddmm_fromfile.cu:200-224) on all five configurations: exit status 0, every rel.diff <= 1e-4, and BOTH
    results -- the library's and rocSPARSE's -- within 1e-4 of the CPU oracle on the same seeded inputs."""
    exe = os.path.join(BIN, "vendor_compare")
    assert os.path.exists(exe), f"{exe} is missing: run `make -C dlspm-esimd_amd drivers`"
    p = subprocess.run([exe, "--iters", "5", "--dump", str(tmp_path)], capture_output=True, text=True, timeout=300)
    out = p.stdout + p.stderr
    print(out)
    assert p.returncode == 0 and "vendor_compare PASS" in out
    diffs = [float(l.split()[4]) for l in out.splitlines() if l.startswith("cfg") and "(best rocSPARSE algorithm" in l]
    assert len(diffs) == 5 and all(0 <= x <= 1e-4 for x in diffs), diffs
    for cfg in range(1, 6):
        c = dl.make_config(cfg)
        if c["op"] == dl.OP_SPMM:
            ref = oracle.spmm(c["row_offsets"], c["col_indices"], c["values"], c["d0"], omp=True)
        elif c["op"] == dl.OP_SDDMM:
            ref = oracle.sddmm(c["row_offsets"], c["col_indices"], c["d0"], c["d1"], omp=True)
        else:
            ref = oracle.fused(c["row_offsets"], c["col_indices"], c["d0"], c["d1"], c["d2"], c["scale"], omp=True)
        for side in ("dlspm", "rocsparse"):
            got = np.fromfile(tmp_path / f"cfg{cfg}_{side}.f32", dtype=np.float32).reshape(ref.shape)
            assert oracle.rel_frobenius(got, ref) <= 1e-4, (cfg, side)
    # a tolerance nothing can meet: the comparator must fail with status 2, not report success
    p = subprocess.run([exe, "--cfg", "1", "--iters", "2", "--tol", "0"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 2 and "vendor_compare FAIL" in p.stdout


DLMC = os.path.join(ROOT, "tests", "golden", "dlmc")
DLMC_CASES = [  # file, un-padded batch size of that layer (dlmc/rn50_batchsizes.txt)
    ("rn50_emp0.96_bottleneck_3_block_group_projection_block_group1.smtx", 3136),
    ("rn50_emp0.98_bottleneck_2_block_group2_3_1.smtx", 784),
    ("rn50_emp0.98_bottleneck_3_block_group3_5_1.smtx", 196),
]


def read_smtx(path):
    with open(path) as f:
        M, K, nnz = (int(x) for x in f.readline().replace(",", " ").split())
        ro = np.array(f.readline().split(), dtype=np.int32)
        ci = np.array(f.readline().split(), dtype=np.int32)
    assert ro.size == M + 1 and ci.size == nnz
    return M, K, ro, ci


@pytest.mark.gpu
@pytest.mark.parametrize("name,width", DLMC_CASES)
def test_real_dlmc_patterns_through_the_drivers_and_the_abi(oracle, dl, tmp_path, name, width):
    """Real pruned-ResNet-50 patterns (skewed rows, empty rows) with the layer's own un-padded batch size, which the
    reference would have to pad to a multiple of 16 (dlmc/rn50_batchsizes_noconv.txt)."""
    import torch

    path = os.path.join(DLMC, name)
    M, K, ro, ci = read_smtx(path)
    # the from-file driver, result dumped and checked against the oracle
    rc, out = run("spmm_run", path, width, "--dump", tmp_path)
    print(out)
    assert rc == 0 and "PASS" in out and f"nnz: {ci.size}" in out
    arr = lambda n, dt: np.fromfile(os.path.join(tmp_path, n), dtype=dt)
    assert np.array_equal(arr("row_offsets.i32", np.int32), ro) and np.array_equal(arr("col_indices.i32", np.int32), ci)
    ref = oracle.spmm(ro, ci, arr("values.f32", np.float32), arr("B.f32", np.float32).reshape(K, width), omp=True)
    assert oracle.rel_frobenius(arr("C.f32", np.float32).reshape(M, width), ref) <= 1e-4
    # the same pattern through the C ABI for SDDMM and the fused op (inner dimension 64)
    rng = np.random.default_rng(5)
    D = 64
    Q = rng.normal(0, 1, (M, D)).astype(np.float32)
    Km = rng.normal(0, 1, (K, D)).astype(np.float32)
    V = rng.normal(0, 1, (K, D)).astype(np.float32)
    d = lambda a: torch.from_numpy(a).cuda()
    ro_d, ci_d = d(ro), d(ci)
    assert dl.csr_check(M, K, ro_d, ci_d) == dl.OK
    got = dl.sddmm(ro_d, ci_d, d(Q), d(Km)).cpu().numpy()
    assert oracle.rel_frobenius(got, oracle.sddmm(ro, ci, Q, Km)) <= 1e-4
    gotO = dl.fused(ro_d, ci_d, d(Q), d(Km), d(V), 0.125).cpu().numpy()
    assert oracle.rel_frobenius(gotO, oracle.fused(ro, ci, Q, Km, V, 0.125)) <= 1e-4
    assert (gotO[np.diff(ro) == 0] == 0).all()


@pytest.mark.gpu
def test_dlmc_batch_list(tmp_path):
    """The reference's shell loop over DLMC files (SPMM/batch-run-spmm_fromfile:34-46) as one --batch run."""
    lines = "".join(f"{os.path.join(DLMC, n)} {w}\n" for n, w in DLMC_CASES)
    (tmp_path / "rn50.txt").write_text("# file batchsize\n" + lines)
    for app in ("spmm_run", "sddmm_run", "fused_run"):
        rc, out = run(app, "--batch", tmp_path / "rn50.txt", "--csv", tmp_path / f"{app}.csv", "--iters", 5)
        assert rc == 0 and out.count("PASS") == 3, out
        assert len(open(tmp_path / f"{app}.csv").read().strip().splitlines()) == 3


MORE_DLMC = [  # file, dense width: the layer's un-padded batch size (rn50) or a width of our choosing (transformer)
    ("rn50_mp0.5_bottleneck_1_block_group_projection_block_group1.smtx", 3136),
    ("rn50_mp0.8_bottleneck_3_block_group1_1_1.smtx", 3136),
    ("rn50_rp0.9_bottleneck_3_block_group1_2_1.smtx", 49),
    ("rn50_vd0.8_initial_conv.smtx", 12544),
    ("rn50_vd0.95_bottleneck_1_block_group1_1_1.smtx", 196),
    ("transformer_l0r0.98_body_encoder_layer_4_self_attention_multihead_attention_q.smtx", 64),
    ("transformer_l0r0.9_body_encoder_layer_1_self_attention_multihead_attention_q.smtx", 128),
    ("transformer_mp0.98_body_encoder_layer_0_self_attention_multihead_attention_q_fully_connected.smtx", 256),
    ("transformer_mp0.9_body_decoder_layer_0_ffn_conv1_fully_connected.smtx", 256),
    ("transformer_rp0.98_body_decoder_layer_4_self_attention_multihead_attention_v_fully_connected.smtx", 100),
    ("transformer_vd0.95_body_encoder_layer_1_self_attention_multihead_attention_v.smtx", 33),
    ("transformer_vd0.98_body_encoder_layer_5_self_attention_multihead_attention_k.smtx", 128),
]


@pytest.mark.gpu
@pytest.mark.parametrize("app", ["spmm_run", "sddmm_run", "fused_run"])
def test_more_dlmc_patterns_through_batch_runs_against_the_oracle(oracle, tmp_path, app):
    """Twelve more real patterns (ResNet-50 and transformer; magnitude, random, variational-dropout and l0 pruning;
    50-98 % sparse; one file without a single nonzero) as one --batch run per driver, every case dumped and verified
    against the CPU oracle. SDDMM and the fused op take the width as the feature dimension, capped at 256."""
    cap = (lambda w: w) if app == "spmm_run" else (lambda w: min(w, 256))
    (tmp_path / "list.txt").write_text("".join(f"{os.path.join(DLMC, n)} {cap(w)}\n" for n, w in MORE_DLMC))
    dumps = tmp_path / "dumps"
    rc, out = run(app, "--batch", tmp_path / "list.txt", "--iters", 3, "--warmup", 1, "--dump-each", dumps)
    assert rc == 0 and out.count("PASS") == len(MORE_DLMC), out[-3000:]
    for i, (name, w) in enumerate(MORE_DLMC):
        M, K, ro, ci = read_smtx(os.path.join(DLMC, name))
        meta, err = verify_dump(oracle, str(dumps / f"case_{i:03d}"))
        assert (meta["M"], meta["K"], meta["N"], meta["nnz"]) == (M, K, cap(w), ci.size)
        assert np.array_equal(np.fromfile(dumps / f"case_{i:03d}" / "col_indices.i32", dtype=np.int32), ci)
        assert err <= 1e-4, (app, name, err)


@pytest.mark.gpu
def test_batch_run_dlmc_script(oracle, tmp_path):
    """host/batch-run-dlmc, the reference's shell loop over a DLMC directory (SPMM/batch-run-spmm_fromfile:16-46):
    layer names looked up in a '<layer>,<batch size>' table, files that the table does not name skipped, one CSV row
    per file; and the fixed-width form. Outputs verified against the oracle through --dump-each."""
    import shutil

    tree = tmp_path / "dlmc" / "rn50" / "magnitude_pruning" / "0.8"
    tree.mkdir(parents=True)
    layers = {  # layer name in the tree -> (fixture, batch size from the table)
        "bottleneck_3_block_group1_1_1": ("rn50_mp0.8_bottleneck_3_block_group1_1_1.smtx", 3136),
        "bottleneck_1_block_group_projection_block_group1": ("rn50_mp0.5_bottleneck_1_block_group_projection_block_group1.smtx", 3136),
        "bottleneck_3_block_group3_5_1": ("rn50_emp0.98_bottleneck_3_block_group3_5_1.smtx", 196),
    }
    for layer, (fixture, _) in layers.items():
        shutil.copy(os.path.join(DLMC, fixture), tree / f"{layer}.smtx")
    shutil.copy(os.path.join(DLMC, "rn50_vd0.8_initial_conv.smtx"), tree / "not_in_the_table.smtx")
    table = tmp_path / "batchsizes.txt"
    table.write_text("".join(f"{layer},{n}\n" for layer, (_, n) in layers.items()))
    script = os.path.join(ROOT, "dlspm-esimd_amd", "host", "batch-run-dlmc")
    dumps = tmp_path / "dumps"
    p = subprocess.run(["bash", script, "spmm_run", str(tmp_path / "dlmc"), str(table), str(tmp_path / "out.csv"),
                        "--iters", "3", "--dump-each", str(dumps)], capture_output=True, text=True, timeout=300)
    out = p.stdout + p.stderr
    assert p.returncode == 0 and "3 files" in out and out.count("PASS") == 3 and "not_in_the_table" not in out, out[-3000:]
    rows = [l.split(",") for l in open(tmp_path / "out.csv").read().strip().splitlines()]
    assert len(rows) == 3 and all(len(r) == 7 for r in rows)  # M,N,K,SP,gflops,max_diff,opcount
    widths = sorted(int(r[1]) for r in rows)
    assert widths == [196, 3136, 3136]
    for i in range(3):
        _, err = verify_dump(oracle, str(dumps / f"case_{i:03d}"))
        assert err <= 1e-4
    # fixed width instead of a table: every file below the directory, the fourth one included
    p = subprocess.run(["bash", script, "sddmm_run", str(tmp_path / "dlmc"), "64", str(tmp_path / "out2.csv"), "--iters", "3"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0 and "4 files" in p.stderr and p.stdout.count("PASS") == 4, p.stdout[-3000:]
    assert len(open(tmp_path / "out2.csv").read().strip().splitlines()) == 4
    # too few arguments: usage and status 2, nothing run
    p = subprocess.run(["bash", script, "spmm_run"], capture_output=True, text=True, timeout=60)
    assert p.returncode == 2 and "batch-run-dlmc <spmm_run|sddmm_run|fused_run>" in p.stdout


@pytest.mark.gpu
def test_drivers_pass_the_workspace_only_for_uneven_rows():
    """3.3 M nonzeros: large enough for the flat schedule. Even rows: the driver passes DLSPM_HINT_ROWS_EVEN and no memory;
    lognormal rows (sigma 1.5): the workspace; in between (sigma 0.2) nothing; all self-check against the on-device
    gold loop."""
    rc, out = run("spmm_run", "--shape", 8192, 4096, 128, 0.1, "--iters", 3)
    assert rc == 0 and "PASS" in out and "even, DLSPM_HINT_ROWS_EVEN passed" in out and "workspace:" not in out, out
    for app in ("sddmm_run", "fused_run"):
        rc, out = run(app, "--shape", 8192, 4096, 128, 0.1, "--iters", 3)
        assert rc == 0 and "PASS" in out and "even, DLSPM_HINT_ROWS_EVEN passed" in out, out
    rc, out = run("spmm_run", "--shape", 8192, 4096, 128, 0.1, "--sigma", 0.2, "--iters", 3, "--no-plan")
    assert rc == 0 and "PASS" in out and "nothing passed" in out and "workspace:" not in out, out
    rc, out = run("sddmm_run", "--shape", 8192, 4096, 128, 0.1, "--sigma", 0.2, "--iters", 3, "--no-plan")
    assert rc == 0 and "PASS" in out and "nothing passed" in out, out
    rc, out = run("spmm_run", "--shape", 8192, 4096, 128, 0.1, "--no-workspace", "--iters", 3)
    assert rc == 0 and "PASS" in out and "rows:" not in out, out
    rc, out = run("spmm_run", "--shape", 8192, 4096, 128, 0.1, "--sigma", 1.5, "--iters", 3, "--no-plan")
    assert rc == 0 and "PASS" in out and "uneven, workspace passed" in out and "workspace:" in out, out
    rc, out = run("spmm_run", "--shape", 8192, 4096, 128, 0.1, "--sigma", 1.5, "--iters", 3)   # SpMM prefers a row plan
    assert rc == 0 and "PASS" in out and "uneven, row plan" in out and "workspace:" not in out, out
    rc, out = run("fused_run", "--shape", 8192, 4096, 128, 0.1, "--sigma", 1.5, "--iters", 3, "--no-plan")
    assert rc == 0 and "PASS" in out and "uneven, workspace passed" in out, out
    for app in ("fused_run", "sddmm_run"):   # all three ops prefer a row plan on uneven rows
        rc, out = run(app, "--shape", 8192, 4096, 128, 0.1, "--sigma", 1.5, "--iters", 3)
        assert rc == 0 and "PASS" in out and "uneven, row plan" in out and "row plan:" in out, out
    rc, out = run("spmm_run", "--shape", 8192, 4096, 128, 0.1, "--workspace", "--iters", 3)
    assert rc == 0 and "PASS" in out and "workspace passed (--workspace)" in out, out


@pytest.mark.gpu
def test_spmm_driver_builds_a_row_plan_for_small_uneven_matrices():
    """The headline configuration (2048 x 512, lognormal rows, one row per workgroup): the driver builds the row plan
    once and launches spmm_csr_f32 with it; with --no-plan, or on even rows, it does not; all self-check."""
    rc, out = run("spmm_run", "--cfg", 2, "--iters", 5)
    assert rc == 0 and "PASS" in out and "row plan:" in out and "uneven, row plan" in out, out
    rc, out = run("spmm_run", "--cfg", 2, "--iters", 5, "--no-plan")
    assert rc == 0 and "PASS" in out and "row plan:" not in out, out
    rc, out = run("spmm_run", "--cfg", 4, "--iters", 5)          # even rows
    assert rc == 0 and "PASS" in out and "row plan:" not in out, out
    plan = lambda text: "row plan:" in text or "cut plan:" in text  # (a row above one and a half shares: handed out in pieces)
    rc, out = run("spmm_run", "--shape", 1024, 1024, 256, 0.1, "--sigma", 0.8, "--iters", 5)
    assert rc == 0 and "PASS" in out and plan(out), out
    rc, out = run("spmm_run", "--shape", 4096, 1024, 256, 0.1, "--sigma", 0.8, "--iters", 5)    # rows ungrouped by the plan
    assert rc == 0 and "PASS" in out and plan(out), out
    rc, out = run("spmm_run", "--shape", 8192, 512, 256, 0.04, "--sigma", 0.8, "--iters", 5)    # short rows: no plan
    assert rc == 0 and "PASS" in out and "row plan:" not in out, out


@pytest.mark.gpu
def test_verify_dlmc_script_on_the_fixtures(tmp_path):
    """tests/verify_dlmc.py is the wide form of the fixture tests above (any directory of .smtx files, every schedule,
    all three ops against the oracle); here it runs over the eighteen fixtures, with a batch-size table for SpMM, and once
    more the way a driver would call (dlspm_analyze -> dlspm_advise), from a pack of the same patterns, with timing."""
    table = tmp_path / "batchsizes.txt"
    names = sorted(f[:-5] for f in os.listdir(DLMC) if f.endswith(".smtx"))
    table.write_text("".join(f"{n},{w}\n" for n, w in zip(names, [49, 196, 64, 256, 33] * 4)))
    report = tmp_path / "report.txt"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "verify_dlmc.py"), DLMC, "--batch-table", str(table),
                        "--all-schedules", "--report", str(report)], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "verify_dlmc PASS" in r.stdout and " 0 FAIL" in r.stdout
    lines = report.read_text().splitlines()
    assert len(lines) >= 18 * 3 * 3 and all(line.startswith("PASS ") for line in lines)
    assert any(" cut_plan " in line for line in lines)
    pack = tmp_path / "patterns.npz"
    subprocess.run([sys.executable, os.path.join(DLMC, "pack_patterns.py"), DLMC, str(pack), "--min-nnz", "20000"], check=True)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "verify_dlmc.py"), str(pack), "--time", "--report", str(report)],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "verify_dlmc PASS" in r.stdout and "geometric means" in r.stdout
    lines = report.read_text().splitlines()   # the four patterns of 20 000 nonzeros and more: three of them with a very long row
    assert len(lines) == 4 * 3 and all(line.startswith("PASS ") and " us=" in line for line in lines)
    assert sum(" cut_plan " in line for line in lines) >= 4


@pytest.mark.gpu
def test_verify_sweep_script_on_the_smallest_shapes(tmp_path):
    """tests/verify_sweep.py checks the reference's whole benchmark grid against the oracle at full size; under pytest
    it runs the shapes of 1024 rows (12 patterns x 3 ops, every schedule)."""
    report = tmp_path / "report.txt"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "verify_sweep.py"), "--max-m", "1024", "--all-schedules",
                        "--report", str(report)], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "verify_sweep PASS" in r.stdout and " 0 FAIL" in r.stdout
    lines = report.read_text().splitlines()
    assert len(lines) >= 6 * 3 * 3 and all(line.startswith("PASS ") for line in lines)


@pytest.mark.gpu
def test_verify_fuzz_script(tmp_path):
    """tests/verify_fuzz.py: random shapes, widths, row-length distributions and tuning overrides, every schedule, all
    three ops against the oracle; 40 problems of it under pytest."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "verify_fuzz.py"), "--cases", "40", "--seed", "11"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "verify_fuzz PASS" in r.stdout and " 0 FAIL" in r.stdout
