"""Cut plans (dlspm_row_plan_build_cut, DLSPM_HINT_CUT_PLAN): rows longer than one and a half times a compute unit's
share of the nonzeros are handed out in pieces.

CPU part: the sequential definition of the cut rule (tests/schedule_model: model_cut_rows) keeps the bounds the plan's
size relies on and partitions every row; the host-only size and advice queries.
GPU part: the plan built on the device equals the host model entry for entry; SpMM, SDDMM and the fused op launched
with it equal the host model of the schedule bit for bit (the row-block model run on the rows and pieces in matrix
order, pieces added in piece order) and the CPU oracle within 1e-4 relative Frobenius error; SDDMM returns the bits
of every other schedule; the CSR arrays are untouched.
"""
import ctypes
import os

import numpy as np
import pytest

from conftest import random_csr

TOL = 1e-4
HERE = os.path.dirname(os.path.abspath(__file__))
DLMC = os.path.join(HERE, "golden", "dlmc")
_i = ctypes.POINTER(ctypes.c_int)
_f = ctypes.POINTER(ctypes.c_float)


@pytest.fixture(scope="module")
def model():
    import subprocess

    so = os.path.join(HERE, "schedule_model", "libschedule_model.so")
    if not os.path.exists(so):
        subprocess.run(["make", "-s", "-C", os.path.dirname(so)], check=True)
    L = ctypes.CDLL(so)
    ci = ctypes.c_int
    L.model_spmm.argtypes = [ci, ci, _i, _i, _f, _f, ci, ci, ci, _f, _i]
    L.model_spmm.restype = ci
    L.model_fused.argtypes = [ci, ci, _i, _i, _f, _f, _f, ctypes.c_float, ci, ci, ci, ci, ci, ci, _f, _f, _i]
    L.model_fused.restype = ci
    L.model_cut_rows.argtypes = [ci, _i, ci, ci, ci, _i, _i, _i, _i]
    L.model_cut_rows.restype = ci
    L.model_row_plan_cut.argtypes = [ci, _i, ci, ci, ci, ci, _i, _i]
    L.model_row_plan_cut.restype = ci
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


def sizes(M, bins, piece_pct=75, longest_pct=100):
    """(entries, most cut rows) of a cut plan of M rows."""
    return M + 2 * -(-bins * 100 // piece_pct), -(-bins * 100 // longest_pct)


def cut_list_offset(M, bins, piece_pct=75, longest_pct=100):
    """Where the list of cut rows lies in a cut plan, in ints (the layout of cut_plan_layout in csrc/plan.hip: 4 x entries
    ints of plan, the sort keys beyond 2048 entries, the virtual rows, then the list)."""
    E, _ = sizes(M, bins, piece_pct, longest_pct)
    at = (4 * E * 4 + 7) // 8 * 8
    if E > 2048:
        at += 2 * E * 8
    at = (at + (3 * E + 1) * 4 + 15) // 16 * 16
    return at // 4


def cut_model(L, ro, bins, order=0, piece_pct=75, longest_pct=100):
    """(plan[4 x entries], cut list, v_off, v_row, v_slot) by the host definition."""
    ro = np.ascontiguousarray(ro, dtype=np.int32)
    M = ro.size - 1
    E, max_cut = sizes(M, bins, piece_pct, longest_pct)
    v_off, v_row, v_slot = np.empty(E + 1, np.int32), np.empty(E, np.int32), np.empty(E, np.int32)
    cut = np.full(4 + 4 * max_cut, -9, np.int32)
    assert L.model_cut_rows(M, pi(ro), bins, piece_pct, longest_pct, pi(v_off), pi(v_row), pi(v_slot), pi(cut)) == 0
    plan = np.empty(4 * E, np.int32)
    cut2 = np.full(4 + 4 * max_cut, -9, np.int32)
    assert L.model_row_plan_cut(M, pi(ro), bins, piece_pct, longest_pct, order, pi(plan), pi(cut2)) == 0
    assert np.array_equal(cut, cut2)
    return plan, cut, v_off, v_row, v_slot


def rows_with_giants(rng, M, K, mean, giants, giant_len):
    lens = np.minimum(K, rng.poisson(mean, M))
    for i in rng.choice(M, size=min(giants, M), replace=False):
        lens[i] = min(K, giant_len)
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens] + [np.zeros(0, np.int64)]).astype(np.int32)
    return ro, ci


ROW_CASES = [
    ("one giant", lambda r: rows_with_giants(r, 512, 2048, 90, 1, 963)),
    ("ten giants", lambda r: rows_with_giants(r, 512, 4096, 60, 10, 2500)),
    ("all in one row", lambda r: rows_with_giants(r, 300, 4096, 0, 1, 4096)),
    ("few rows, all long", lambda r: rows_with_giants(r, 64, 2048, 400, 0, 0)),
    ("nothing to cut", lambda r: rows_with_giants(r, 2048, 512, 50, 0, 0)),
    ("skewed", lambda r: random_csr(r, 1000, 3000, "skewed", 0.01)),
    ("empty rows", lambda r: random_csr(r, 700, 900, "empty_rows", 0.2)),
    ("empty", lambda r: random_csr(r, 100, 50, "empty", 0.0)),
    ("one row", lambda r: rows_with_giants(r, 1, 5000, 0, 1, 5000)),
    ("tall", lambda r: rows_with_giants(r, 5000, 2048, 20, 3, 2048)),
]


@pytest.mark.parametrize("name,make", ROW_CASES, ids=[c[0] for c in ROW_CASES])
@pytest.mark.parametrize("bins,piece_pct,longest_pct", [(256, 75, 100), (256, 100, 150), (64, 75, 100), (7, 100, 150), (256, 50, 100), (256, 33, 40),
                                                        (104, 200, 150), (256, 1000, 10)])
def test_cut_rule_partitions_rows_within_its_bounds(model, name, make, bins, piece_pct, longest_pct):
    """CPU: every row is covered by its virtual rows exactly, in order; only rows above one and a half shares are cut,
    into a power of two (at most 256) of equal pieces of at most one share; no more than M + 2 x bins virtual rows, 2 x bins
    more pieces than cut rows, fewer than bins cut rows (the bounds the plan's size is made of), for any matrix; the plan
    holds every virtual row once, a piece with the range of its whole row and a word that says which piece of how many it is."""
    ro, _ = make(np.random.default_rng(len(name) * 131 + bins))
    M = ro.size - 1
    E, max_cut = sizes(M, bins, piece_pct, longest_pct)
    plan, cut, v_off, v_row, v_slot = cut_model(model, ro, bins, 0, piece_pct, longest_pct)
    nnz = int(ro[-1])
    share = max(1, -(-nnz // bins))
    piece_max = max(1, -(-share * piece_pct // 100))
    longest = max(piece_max, -(-share * longest_pct // 100))
    assert cut[1] == share
    used = cut[2]
    assert M <= used <= E and (v_row[used:] == -1).all() and (v_slot[used:] == -2).all() and (v_off[used:] == ro[-1]).all()
    lens = np.diff(ro)
    vlen = np.diff(v_off)
    e = 0
    pieces = 0
    cut_rows = []
    for i in range(M):
        if lens[i] <= longest:
            assert v_row[e] == i and v_slot[e] == -1 and v_off[e] == ro[i] and vlen[e] == lens[i]
            e += 1
            continue
        need = -(-int(lens[i]) // piece_max)
        assert need >= 2
        c = min(256, 1 << (need - 1).bit_length())  # the smallest power of two of pieces that are short enough
        assert (v_row[e:e + c] == i).all() and v_off[e] == ro[i] and v_off[e + c] == ro[i + 1]
        piece = -(-int(lens[i]) // c)
        assert np.array_equal(vlen[e:e + c], np.clip(lens[i] - piece * np.arange(c), 0, piece))
        assert vlen[e:e + c].sum() == lens[i] and (need > 256 or piece <= piece_max)
        assert np.array_equal(v_slot[e:e + c], np.arange(pieces, pieces + c))
        cut_rows.append((i, pieces, c))
        pieces += c
        e += c
    assert e == used and pieces <= E - M + max_cut and len(cut_rows) <= max_cut and cut[0] == len(cut_rows)
    for j, (i, s, c) in enumerate(cut_rows):
        assert cut[4 + 4 * j:8 + 4 * j].tolist() == [i, s, c, 1]
    assert not cut[4 + 4 * len(cut_rows):].any()
    # the plan: every virtual row once, with its row and slot; a whole row with its own range, a piece with its row's
    starts, ends, rows, words = plan[:E], plan[E:2 * E], plan[2 * E:3 * E], plan[3 * E:]
    key = lambda a, b, c, d: sorted(zip(a.tolist(), b.tolist(), c.tolist(), d.tolist()))
    of_row = {i: (s, c) for (i, s, c) in cut_rows}
    got_starts, got_ends = starts.copy(), ends.copy()
    for p, (word, row) in enumerate(zip(words.tolist(), rows.tolist())):
        if word >= 0:
            first, c = of_row[row]
            k = (word >> 15) & 255
            assert k == (word & 0x7FFF) - first and 1 << ((word >> 23) & 15) == c
            assert (starts[p], ends[p]) == (ro[row], ro[row + 1])
            piece = -(-int(lens[row]) // c)  # what a launch takes from the word: the piece's share of the row's nonzeros
            got_starts[p] = ro[row] + min(int(lens[row]), k * piece)
            got_ends[p] = min(int(ro[row + 1]), got_starts[p] + piece)
    piece_number = np.where(words >= 0, words & 0x7FFF, words)
    assert key(got_starts, got_ends, rows, piece_number) == key(v_off[:-1], v_off[1:], v_row, v_slot)


def test_cut_plan_sizes_and_advice(dl):
    """Host only: the size grows with the width for SpMM and the fused op and not for SDDMM, taller matrices than one
    workgroup cuts get none; the advice asks for a cut plan where the longest row exceeds one and a half shares by enough
    to pay for the second kernel (SDDMM: for hardly anything), and never for even rows."""
    b0 = dl.row_plan_bytes_for(dl.OP_SDDMM, 512, 128)
    assert b0 > 0 and b0 == dl.row_plan_bytes_for(dl.OP_SDDMM, 512, 7)
    b1, b2 = dl.row_plan_bytes_for(dl.OP_SPMM, 512, 128), dl.row_plan_bytes_for(dl.OP_SPMM, 512, 256)
    assert b0 < b1 < b2 and b2 - b1 == (2 * 342 + 256) * 128 * 4   # room for 2 x ceil(256 x 100 / 75) + 256 x 100 / 100 pieces
    assert dl.row_plan_bytes_for(dl.OP_FUSED, 512, 256) == b2
    assert dl.row_plan_bytes_for(dl.OP_SPMM, (1 << 20) + 1, 64) == 0 and dl.row_plan_bytes_for(7, 512, 64) == 0
    assert dl.row_plan_bytes_for(dl.OP_SPMM, 0, 64) == 0
    # 512 x 2048 with 52 000 nonzeros: a share is 204; longest row 963 (the reference's own transformer layer)
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 256, 52000, 963) == 2
    assert dl.row_plan_advice(dl.OP_SDDMM, 512, 2048, 128, 52000, 963) == 2
    assert dl.row_plan_advice(dl.OP_FUSED, 512, 2048, 64, 52000, 963) == 2
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 256, 52000, 310) == 1    # hardly above one and a half shares
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 256, 52000, -1) == 1     # unknown rows: never a cut plan
    assert dl.row_plan_advice(dl.OP_SPMM, 2048, 512, 256, 105687, 312) == 1   # the headline matrix: below one share
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 256, 52000, 110) == 0    # even rows: no plan at all
    assert dl.row_plan_advice(dl.OP_SPMM, 2048, 512, 256, 4999, 100) == 1     # a handful of nonzeros: all start-up, no cut plan
    assert dl.row_plan_advice(dl.OP_SPMM, 2048, 512, 256, 5000, 100) == 2
    assert dl.row_plan_advice(dl.OP_SDDMM, 2048, 512, 128, 2400, 200) == 2
    # the fused op on fewer rows than two per compute unit (eight waves per row, nothing spreads a row): a cut plan where a
    # row is long enough to pay for the kernel that adds its pieces, and a share holds 32 nonzeros
    assert dl.row_plan_advice(dl.OP_FUSED, 64, 2304, 128, 16905, 1654) == 2
    assert dl.row_plan_advice(dl.OP_FUSED, 64, 2304, 64, 16905, 1654) == 2
    assert dl.row_plan_advice(dl.OP_FUSED, 64, 2304, 64, 16905, 1200) == 0
    assert dl.row_plan_advice(dl.OP_FUSED, 8, 4608, 128, 10981, 1435) == 2
    assert dl.row_plan_advice(dl.OP_FUSED, 8, 4608, 64, 10981, 1435) == 0      # below 32 rows: from 10 us on
    assert dl.row_plan_advice(dl.OP_FUSED, 32, 512, 256, 3314, 512) == 0       # a share of 13 nonzeros
    assert dl.row_plan_advice(dl.OP_FUSED, 128, 1152, 64, 29510, 455) == 0
    # dense rows in column tiles (N above 512): the tiles spread a long row already, no cut plan
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 1024, 52000, 2048) == 1
    assert dl.row_plan_advice(dl.OP_SPMM, 1024, 1152, 12544, 119909, 1152) == 1
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 512, 52000, 2048) == 2    # (SDDMM gains from a cut plan at every size)
    # fewer rows than three quarters of the compute units: a call without plan spreads every row over several workgroups by
    # itself (SDDMM: row pieces; SpMM: column tiles of B), so a cut plan is advised only where a row is still too long for
    # one of them -- and never the plan over whole rows, which would undo the spread
    sh = dl.describe_launch(dl.OP_SDDMM, 128, 1152, 128, 29510)
    assert (sh["W"], sh["R"], sh["col_tiles"]) == (4, 1, 4)                    # ([7]: workgroups per row)
    assert dl.row_plan_advice(dl.OP_SDDMM, 128, 1152, 128, 29510, 455) == 0    # a quarter of 455 is below one and a half shares (174)
    assert dl.row_plan_advice(dl.OP_SDDMM, 128, 1152, 128, 29510, 1152) == 2
    assert dl.row_plan_advice(dl.OP_SDDMM, 64, 576, 128, 31919, 547) == 0
    # three quarters to one and a half of the compute units' count of rows (two workgroups per row without plan): judged as
    # whole rows, from a longest row of little more than one and a half shares on; up to two rows per compute unit
    # (eight waves per row) from about two and a half shares on
    assert dl.row_plan_advice(dl.OP_SDDMM, 256, 2304, 128, 118041, 750) == 0
    assert dl.row_plan_advice(dl.OP_SDDMM, 256, 2304, 128, 118041, 900) == 2
    assert dl.row_plan_advice(dl.OP_SDDMM, 384, 2304, 128, 118041, 900) == 2
    assert dl.row_plan_advice(dl.OP_SDDMM, 385, 2304, 128, 118041, 900) == 0
    assert dl.row_plan_advice(dl.OP_SDDMM, 385, 2304, 128, 118041, 1200) == 2
    assert dl.row_plan_advice(dl.OP_SDDMM, 256, 2304, 128, 53000, 800) == 2
    assert dl.row_plan_advice(dl.OP_SPMM, 128, 1152, 256, 29510, 455) == 0
    assert dl.row_plan_advice(dl.OP_SPMM, 128, 1152, 256, 29510, 1152) == 2
    assert dl.row_plan_advice(dl.OP_SPMM, 128, 1152, 128, 29510, 455) == 0
    assert dl.row_plan_advice(dl.OP_SPMM, 128, 1152, 64, 29510, 455) == 0
    assert dl.row_plan_advice(dl.OP_SPMM, 128, 1152, 64, 29510, 1100) == 2
    assert dl.row_plan_advice(dl.OP_SPMM, 128, 1152, 32, 29510, 455) in (0, 1)  # (32 columns: nothing to tile)
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 8192, 32, 52000, 3000) == 2     # (with partial rows: only from a large gain on
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 32, 52000, 700) == 1      # ... and two rows per compute unit)
    assert dl.row_plan_advice(dl.OP_SPMM, 512, 2048, 256, 52000, 500) == 2
    assert dl.row_plan_advice(dl.OP_FUSED, 128, 1152, 64, 29510, 455) in (0, 1)


def load_smtx(path):
    with open(path) as f:
        M, K, nnz = (int(x) for x in f.readline().replace(",", " ").split())
        ro = np.array(f.readline().split(), dtype=np.int32)
        ci = np.array(f.readline().split(), dtype=np.int32)
    assert ro.size == M + 1 and ci.size == nnz
    return M, K, ro, ci


# three patterns of the reference's data set whose longest row holds 3.8 ... 4.7 shares of the nonzeros
LONG_ROW_FILES = ["transformer_mp0.95_body_decoder_layer_5_ffn_conv2_fully_connected.smtx",
                  "rn50_vd0.9_bottleneck_2_block_group2_1_1.smtx",
                  "transformer_mp0.9_body_decoder_layer_0_encdec_attention_multihead_attention_output_transform_fully_connected.smtx"]


def gpu_cases():
    rng = np.random.default_rng(5)
    cases = [("one giant", 2048) + rows_with_giants(rng, 512, 2048, 90, 1, 963),
             ("ten giants", 4096) + rows_with_giants(rng, 700, 4096, 60, 10, 2500),
             ("few rows", 2048) + rows_with_giants(rng, 64, 2048, 400, 0, 0),
             ("2048 rows", 1024) + rows_with_giants(rng, 2048, 1024, 30, 4, 1000),
             ("tall", 2048) + rows_with_giants(rng, 5000, 2048, 20, 3, 2048),
             ("nothing to cut", 512) + random_csr(rng, 1500, 512, "uniform", 0.1),
             ("empty rows", 900) + random_csr(rng, 700, 900, "empty_rows", 0.2)]
    for f in LONG_ROW_FILES:
        M, K, ro, ci = load_smtx(os.path.join(DLMC, f))
        cases.append((f[:24], K, ro, ci))
    return cases


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.gpu
def test_gpu_cut_plan_equals_its_sequential_definition(model, dl):
    import torch

    bins = min(dl.device_info()["compute_units"], 256)
    for name, K, ro, ci in gpu_cases():
        M = ro.size - 1
        print(f"cut plan build: {name} {M}x{K} nnz {ci.size}", flush=True)
        for order, piece_pct, longest_pct in ((0, 75, 100), (2, 100, 150), (0, 50, 100), (0, 25, 30)):
            E, max_cut = sizes(M, bins, piece_pct, longest_pct)
            dl.set_tuning(plan_order=order, cut_piece_pct=piece_pct, cut_longest_pct=longest_pct)
            mem = torch.full(((dl.row_plan_bytes_for(dl.OP_SDDMM, M, 0) + 3) // 4,), -7, dtype=torch.int32, device="cuda")
            cp = dl.cut_plan(dev(torch, ro), dl.OP_SDDMM, 0, out=mem)
            got = cp.memory.cpu().numpy()
            want, cut, *_ = cut_model(model, ro, bins, order, piece_pct, longest_pct)
            assert np.array_equal(got[:4 * E], want), (name, order, np.flatnonzero(got[:4 * E] != want)[:10])
            tail = got[cut_list_offset(M, bins, piece_pct, longest_pct):][:4 + 4 * max_cut]
            assert np.array_equal(tail, cut), (name, order)
        dl.set_tuning()


def combine(per_virtual_row, M, v_row, v_slot, cut, max_cut):
    """Rows of the output from the results of the virtual rows: whole rows as they are, cut rows as the sum of their
    pieces in piece order, starting from zero (fp32, as cut_rows_sum_kernel adds them)."""
    out = np.zeros((M, per_virtual_row.shape[1]), dtype=np.float32)
    whole = np.flatnonzero(v_slot == -1)
    out[v_row[whole]] = per_virtual_row[whole]
    slot_at = {int(s): e for e, s in enumerate(v_slot) if s >= 0}
    for j in range(cut[0]):
        row, first, cnt = cut[4 + 4 * j:7 + 4 * j]
        acc = np.zeros(per_virtual_row.shape[1], dtype=np.float32)
        for k in range(cnt):
            acc = (acc + per_virtual_row[slot_at[first + k]]).astype(np.float32)
        out[row] = acc
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("width,piece_pct,longest_pct", [(256, 75, 100), (128, 75, 100), (64, 100, 150), (49, 75, 100), (392, 100, 150),
                                                         (256, 50, 100), (64, 25, 30), (250, 100, 150), (100, 100, 150), (130, 10, 10)])
def test_gpu_launches_with_a_cut_plan(model, dl, oracle, width, piece_pct, longest_pct):
    """All three ops with DLSPM_HINT_CUT_PLAN against the host model (bit for bit) and the oracle (1e-4); SDDMM also
    against the plain call (bit for bit: pieces write their own CSR slots)."""
    import torch

    bins = min(dl.device_info()["compute_units"], 256)
    rng = np.random.default_rng(width)
    for name, K, ro, ci in gpu_cases():
        M, nnz = ro.size - 1, ci.size
        E, max_cut = sizes(M, bins, piece_pct, longest_pct)
        dl.set_tuning(cut_piece_pct=piece_pct, cut_longest_pct=longest_pct)
        _, cut, v_off, v_row, v_slot = cut_model(model, ro, bins, 0, piece_pct, longest_pct)
        print(f"cut plan launch: {name} {M}x{K} nnz {nnz} width {width}: {cut[0]} rows cut", flush=True)
        ro_d, ci_d = dev(torch, ro), dev(torch, ci)
        va = rng.normal(0, 1, nnz).astype(np.float32)
        B = rng.uniform(-1, 1, (K, width)).astype(np.float32)
        Q = rng.normal(0, 1, (M, width)).astype(np.float32)
        V = rng.normal(0, 1, (K, width)).astype(np.float32)
        # one plan, sized for SpMM / fused at this width, serves all three ops
        cp = dl.cut_plan(ro_d, dl.OP_SPMM, width)
        # SpMM. Widths that one wave covers with lane groups of 16 to 64 (33 ... 512 columns) share a cut row out by columns: every
        # piece sums the whole row, in the lane layout of its share's width; the other widths (and the rule switched off)
        # by nonzeros, with partial rows that a second kernel adds
        sh = dl.describe_launch(dl.OP_SPMM, M, K, width, nnz)
        want = oracle.spmm(ro, ci, va, B)
        by_columns = sh["vec"] == 4 and sh["G"] >= 16 and sh["col_tiles"] == 1
        for shares in (("columns", "nonzeros") if by_columns else ("nonzeros",)):
            dl.set_tuning(cut_piece_pct=piece_pct, cut_longest_pct=longest_pct,
                          rules_off=dl.RULES["cut_rows_by_columns"] if by_columns and shares == "nonzeros" else 0)
            got = dl.spmm(ro_d, ci_d, dev(torch, va), dev(torch, B), K=K, plan=cp).cpu().numpy()
            assert oracle.rel_frobenius(got, want) <= TOL, (name, "spmm", shares)
            if dl.row_plan_advice(dl.OP_SPMM, M, K, width, nnz, -1) and sh["col_tiles"] == 1 and sh["vec"] == 4:
                rc, Cv, _ = run_spmm(model, v_off, ci, va, B, sh["G"], 4, 1)
                assert rc == 0
                expect = combine(Cv, M, v_row, v_slot, cut, max_cut)
                if shares == "columns":
                    whole_rows = {}
                    for j in range(cut[0]):
                        row, _, c = cut[4 + 4 * j:7 + 4 * j]
                        share = max(4, (-(-width // c) + 3) & ~3)
                        lanes = 32 if share > 64 else 16 if share > 32 else 8
                        if lanes not in whole_rows:
                            rc, whole_rows[lanes], _ = run_spmm(model, ro, ci, va, B, lanes, 4, 1)
                            assert rc == 0
                        expect[row] = whole_rows[lanes][row]
                assert np.array_equal(got, expect), (name, "spmm against the model", shares)
        dl.set_tuning(cut_piece_pct=piece_pct, cut_longest_pct=longest_pct)
        # SDDMM: the same bits as the plain call, whatever the plan
        if width <= 512:
            plain = dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, B))
            cutted = dl.sddmm(ro_d, ci_d, dev(torch, Q), dev(torch, B), plan=cp)
            assert torch.equal(plain, cutted), (name, "sddmm")
            assert oracle.rel_frobenius(cutted.cpu().numpy(), oracle.sddmm(ro, ci, Q, B)) <= TOL or nnz == 0
        # fused
        if width <= 512:
            got = dl.fused(ro_d, ci_d, dev(torch, Q), dev(torch, B), dev(torch, V), 0.25, plan=cp).cpu().numpy()
            want = oracle.fused(ro, ci, Q, B, V, 0.25)
            assert oracle.rel_frobenius(got, want) <= TOL or not np.any(want), (name, "fused")
            fs = dl.describe_launch(dl.OP_FUSED, M, K, width, nnz)
            if dl.row_plan_advice(dl.OP_FUSED, M, K, width, nnz, -1):
                Qv = np.zeros((E, width), dtype=np.float32)
                live = v_row >= 0
                Qv[live] = Q[v_row[live]]
                scores = np.empty(max(nnz, 1), dtype=np.float32)
                Ov = np.full((E, width), np.nan, dtype=np.float32)
                writes = np.zeros((E, width), dtype=np.int32)
                ci2 = ci if nnz else np.zeros(1, np.int32)
                rc = model.model_fused(E, width, pi(v_off), pi(ci2), pf(Qv), pf(B), pf(V), 0.25, fs["vec"], fs["G1"], fs["DS"],
                                       fs["G"], 4, 1, pf(scores), pf(Ov), pi(writes))
                assert rc == 0
                assert np.array_equal(got, combine(Ov, M, v_row, v_slot, cut, max_cut)), (name, "fused against the model")
        assert np.array_equal(ro_d.cpu().numpy(), ro) and np.array_equal(ci_d.cpu().numpy(), ci)


@pytest.mark.gpu
def test_gpu_cut_plan_errors_reuse_and_graph(dl, oracle):
    """A plan that is too small for the op and width is refused; a plan built once serves many launches (nothing in it
    or behind it has to be cleared); build and launches can be captured in one HIP graph and replayed on a structure
    that changes between replays."""
    import torch

    rng = np.random.default_rng(9)
    M, K, N = 512, 2048, 256
    ro, ci = rows_with_giants(rng, M, K, 80, 2, 1200)
    nnz = ci.size
    ro_d, ci_d = dev(torch, ro), dev(torch, ci)
    va = dev(torch, rng.normal(0, 1, nnz).astype(np.float32))
    B = dev(torch, rng.uniform(-1, 1, (K, N)).astype(np.float32))
    small = dl.cut_plan(ro_d, dl.OP_SDDMM, 0)
    with pytest.raises(dl.DlspmError) as e:
        dl.spmm(ro_d, ci_d, va, B, K=K, plan=small)
    assert e.value.status == dl.E_WORKSPACE
    vp = ctypes.c_void_p
    st = dl.lib().dlspm_row_plan_build_cut(M, vp(ro_d.data_ptr()), vp(small.memory.data_ptr()), small.memory.numel() * 4 - 4, None)
    assert st == dl.E_WORKSPACE
    cp = dl.cut_plan(ro_d, dl.OP_SPMM, N)
    first = dl.spmm(ro_d, ci_d, va, B, K=K, plan=cp).clone()
    cp.memory[-1000:] = 0x7f7f7f7f  # rubbish where partial rows go: every one that is read is written first
    for _ in range(3):
        assert torch.equal(first, dl.spmm(ro_d, ci_d, va, B, K=K, plan=cp))
    assert oracle.rel_frobenius(first.cpu().numpy(), oracle.spmm(ro, ci, va.cpu().numpy(), B.cpu().numpy())) <= TOL
    # one graph: build the cut plan, then SpMM and SDDMM with it; the structure changes between replays
    lhs = dev(torch, rng.normal(0, 1, (M, 128)).astype(np.float32))
    rhs = dev(torch, rng.normal(0, 1, (K, 128)).astype(np.float32))
    out_c = torch.empty((M, N), dtype=torch.float32, device="cuda")
    out_s = torch.empty((nnz,), dtype=torch.float32, device="cuda")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        dl.cut_plan(ro_d, dl.OP_SPMM, N, out=cp.memory)
        dl.spmm(ro_d, ci_d, va, B, K=K, out=out_c, plan=cp)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            dl.cut_plan(ro_d, dl.OP_SPMM, N, out=cp.memory)
            dl.spmm(ro_d, ci_d, va, B, K=K, out=out_c, plan=cp)
            dl.sddmm(ro_d, ci_d, lhs, rhs, out=out_s, plan=cp)
    for rep in range(3):
        lens = np.diff(ro)
        lens = np.roll(lens, 37 * (rep + 1))          # same nonzeros, other rows
        ro2 = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        ro_d.copy_(torch.from_numpy(ro2))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want_c = dl.spmm(ro_d, ci_d, va, B, K=K, plan=dl.cut_plan(ro_d, dl.OP_SPMM, N))
        want_s = dl.sddmm(ro_d, ci_d, lhs, rhs)
        assert torch.equal(out_c, want_c), f"replay {rep}: SpMM"
        assert torch.equal(out_s, want_s), f"replay {rep}: SDDMM"
        # (columns are no longer sorted inside the new rows, which no kernel requires)
        ref = oracle.spmm(ro2, ci, va.cpu().numpy(), B.cpu().numpy())
        assert oracle.rel_frobenius(out_c.cpu().numpy(), ref) <= TOL
