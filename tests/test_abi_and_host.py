"""CPU-side checks: the C ABI library loads and exports every function include/dlspm_hip.h declares (no
compute call is made without a GPU), and the host-side generators and accounting behave as documented."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dlspm_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?(?:int|size_t|char\s*\*|void)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)


def test_header_declares_the_three_named_entry_points():
    names = declared_functions()
    for required in ("spmm_csr_f32", "sddmm_csr_f32", "fused_sddmm_spmm_f32"):
        assert required in names
    assert len(names) >= 8


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 (no C++ types, no torch types, no HIP headers)."""
    src = tmp_path / "abi.c"
    src.write_text('#include "dlspm_hip.h"\n'
                   "int use(void) { int shape[10]; return dlspm_describe_launch(DLSPM_OP_SPMM, 1, 1, 1, 1, shape)"
                   " + (int)dlspm_workspace_bytes(DLSPM_OP_FUSED, 1, 1, 1, 1)"
                   " + spmm_csr_f32(0, 0, 0, 0, 0, 0, 0, 0, 0, DLSPM_ROWS_EVEN, 0, 0)"
                   " + spmm_csr_f32(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, DLSPM_HINT_ROWS_EVEN | DLSPM_HINT_ROW_PLAN | DLSPM_HINT_BANDED, 0);"
                   " dlspm_tuning t; dlspm_tuning_default(&t); t.split_w = 4; t.split_r = 1; return dlspm_set_tuning(&t); }\n")
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-I", inc, str(src)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_split_rule_and_the_even_rows_hint(dl):
    """Rows per workgroup: one for long rows of unknown evenness, four (a whole row per wave) once the caller says the
    rows are even and the matrix has at least 2048 rows; the hint changes nothing for short rows or for the benchmark
    configurations' sizes but the fourth. Sixteen waves per row: never in the fused op on tall matrices, in SpMM only from
    16384 rows on."""
    for op in (dl.OP_SPMM, dl.OP_SDDMM, dl.OP_FUSED):
        for width in (32, 128, 256):
            nnz = 8192 * 600
            a = dl.describe_launch(op, 8192, 4096, width, nnz)
            b = dl.describe_launch(op, 8192, 4096, width, nnz, rows_even=True)
            # (the fused op groups long rows by itself where Kmat and V together exceed one L2: 2 x 4096 x 256 floats)
            # (SDDMM keeps the hint's groups of four only where the dot products are long too: from 128 floats on)
            assert (a["W"], a["R"]) == ((4, 4) if op == dl.OP_FUSED and width == 256 else (4, 1))
            assert (b["W"], b["R"]) == ((4, 1) if op == dl.OP_SDDMM and width == 32 else (4, 4))
            same = lambda d: {k: v for k, v in d.items() if k not in ("R", "flat_chunk", "flat_units")}
            assert same(a) == same(b)
            # SDDMM needs no memory for its flat schedule and takes it by the sizes alone -- except for rows known to be even
            if op == dl.OP_SDDMM:
                assert a["flat_chunk"] > 0 and b["flat_chunk"] == 0
            else:
                assert (a["flat_chunk"], a["flat_units"]) == (b["flat_chunk"], b["flat_units"])
            # ... nor where rhs exceeds one L2 under rows of a thousand nonzeros and more
            if op == dl.OP_SDDMM:
                flat = lambda K, D, per_row: dl.describe_launch(op, 8192, K, D, 8192 * per_row)["flat_chunk"] > 0
                assert not flat(8192, 256, 2458) and not flat(16384, 128, 1024) and flat(8192, 128, 2458) and flat(8192, 256, 1023)
            # too few rows for 512 workgroups of four rows: unchanged
            assert dl.describe_launch(op, 2048, 4096, width, 2048 * 600, rows_even=True)["R"] == (1 if op == dl.OP_SDDMM and width == 32 else 4)
            assert dl.describe_launch(op, 1536, 4096, width, 1536 * 600, rows_even=True)["R"] == 1
        # short rows are grouped by the size rule already; the hint never makes the groups smaller
        a = dl.describe_launch(op, 65536, 1024, 64, 65536 * 20)
        b = dl.describe_launch(op, 65536, 1024, 64, 65536 * 20, rows_even=True)
        assert a == b and a["R"] == 16
    # the fused op, Kmat and V together beyond one L2 (2 x K x D floats > 4 MiB): long rows four to a workgroup without the hint
    assert dl.describe_launch(dl.OP_FUSED, 8192, 8192, 128, 8192 * 819)["R"] == 4
    assert dl.describe_launch(dl.OP_FUSED, 8192, 4096, 128, 8192 * 410)["R"] == 1      # exactly one L2: only on the hint
    assert dl.describe_launch(dl.OP_FUSED, 8192, 8192, 128, 8192 * 40)["R"] == dl.describe_launch(dl.OP_FUSED, 8192, 1024, 128, 8192 * 40)["R"]  # short rows: the size rule
    assert dl.describe_launch(dl.OP_SDDMM, 8192, 16384, 128, 8192 * 819)["R"] == 1     # SDDMM: its flat schedule instead
    for cfg in ((dl.OP_SPMM, 512, 512, 128, 78848), (dl.OP_SPMM, 2048, 512, 256, 105687),
                (dl.OP_SDDMM, 2048, 2048, 128, 209715), (dl.OP_FUSED, 4096, 4096, 64, 323000)):
        assert dl.describe_launch(*cfg) == dl.describe_launch(*cfg, rows_even=True)
    # where a row of the dense operand takes a whole wave (SpMM from 256 columns on), even rows are grouped from about a
    # hundred nonzeros on: the fourth benchmark configuration (102 per row), not the same rows at N = 128
    cfg4 = (dl.OP_SPMM, 2048, 512, 392, 208896)
    assert dl.describe_launch(*cfg4)["R"] == 1 and dl.describe_launch(*cfg4, rows_even=True)["R"] == 4
    assert dl.describe_launch(dl.OP_SPMM, 2048, 512, 128, 208896, rows_even=True)["R"] == 1
    long_rows = 2000
    assert dl.describe_launch(dl.OP_SPMM, 8192, 8192, 128, 8192 * long_rows)["W"] == 4
    assert dl.describe_launch(dl.OP_SPMM, 24576, 8192, 128, 24576 * long_rows)["W"] == 16
    assert dl.describe_launch(dl.OP_SPMM, 16384, 8192, 128, 16384 * long_rows)["W"] == 4  # sixteen only from 96 rows per compute unit on
    for op in (dl.OP_SDDMM, dl.OP_FUSED):  # the rules that add waves for very long rows are SpMM's alone
        assert dl.describe_launch(op, 24576, 8192, 128, 24576 * long_rows)["W"] == 4
        assert dl.describe_launch(op, 24576, 8192, 128, 24576 * long_rows, rows_even=True)["R"] == 4
        assert dl.describe_launch(op, 300, 8192, 32, 300 * 7000)["W"] == 8  # (eight: few rows of a hundred nonzeros and more)
    # few rows, very long: sixteen waves per row in SpMM, up to one and a half rows per compute unit
    assert dl.describe_launch(dl.OP_SPMM, 300, 8192, 32, 300 * 7000)["W"] == 16
    assert dl.describe_launch(dl.OP_SPMM, 384, 8192, 256, 384 * 2048)["W"] == 16
    assert dl.describe_launch(dl.OP_SPMM, 512, 8192, 256, 512 * 2048)["W"] == 4


def test_split_rule_for_small_matrices(dl):
    """The reference's layer shapes of 64 ... 2048 rows. Fewer rows than two per compute unit: four waves per row, in
    SDDMM and the fused op eight from about a hundred nonzeros per row on, sixteen only for very long rows. The fused op keeps three
    workgroups per compute unit when it groups rows (SDDMM two, SpMM eight). SDDMM and the fused op take a row plan for
    short rows up to eight rows per compute unit; the advice gives SDDMM's grouping up only for a longest row of eight
    times the mean."""
    for op in (dl.OP_SPMM, dl.OP_SDDMM, dl.OP_FUSED):
        width = 256 if op == dl.OP_SPMM else 64
        assert dl.describe_launch(op, 128, 512, width, 128 * 26)["W"] == 4
        assert dl.describe_launch(op, 64, 576, width, 64 * 58)["W"] == 4
        eight = 4 if op == dl.OP_SPMM else 8  # SpMM: only by the rule for very long rows
        sh = dl.describe_launch(op, 256, 2304, width, 256 * 208)
        assert (sh["W"], sh["col_tiles"]) == ((4, 2) if op == dl.OP_SDDMM else (eight, 1))  # SDDMM: two four-wave workgroups per row
        assert dl.describe_launch(op, 511, 2304, width, 511 * 96)["W"] == eight
        assert dl.describe_launch(op, 512, 2304, width, 512 * 208)["W"] == 4
    assert dl.describe_launch(dl.OP_SPMM, 256, 2304, 196, 256 * 461)["W"] == 8
    # few rows in a plain SpMM call: narrower column tiles of B instead of more waves per row (64 rows x 8 tiles of 32)
    sh = dl.describe_launch(dl.OP_SPMM, 64, 4608, 256, 64 * 800)
    assert (sh["W"], sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (4, 32, 8)
    dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
    try:
        assert dl.describe_launch(dl.OP_SPMM, 64, 4608, 256, 64 * 800)["W"] == 16
    finally:
        dl.set_tuning()
    rows_per_workgroup = lambda op, M, avg: dl.describe_launch(op, M, 1024, 64, M * avg)["R"]
    assert [rows_per_workgroup(dl.OP_FUSED, M, 20) for M in (1024, 2048, 3072, 4096, 8192, 16384)] == [1, 2, 4, 4, 8, 16]
    # SDDMM groups rows of unknown lengths only from 128 rows per compute unit on (from 64 at D <= 32)
    assert [rows_per_workgroup(dl.OP_SDDMM, M, 20) for M in (1024, 2048, 4096, 8192, 16384, 32767, 32768)] == [1, 1, 1, 1, 1, 1, 16]
    assert [dl.describe_launch(dl.OP_SDDMM, M, 1024, 32, M * 20)["R"] for M in (8192, 16383, 16384)] == [1, 1, 16]
    assert dl.describe_launch(dl.OP_SDDMM, 8192, 1024, 64, 8192 * 20, rows_even=True)["R"] == 1      # short even rows: no groups either
    assert dl.describe_launch(dl.OP_SDDMM, 8192, 1024, 128, 8192 * 128, rows_even=True)["R"] == 4    # long rows, long dot products
    dl.set_tuning(rules_off=dl.RULES["group_rows"])
    try:
        assert rows_per_workgroup(dl.OP_SDDMM, 32768, 20) == 1
    finally:
        dl.set_tuning()
    assert [rows_per_workgroup(dl.OP_SPMM, M, 20) for M in (1024, 2048, 4096, 8192)] == [1, 1, 2, 4]
    M, K, nnz = 2048, 512, 2048 * 10
    assert dl.row_plan_advice(dl.OP_FUSED, M, K, 64, nnz, 23) == 1  # short rows: any unevenness
    assert dl.row_plan_advice(dl.OP_FUSED, M, K, 64, nnz, 14) == 0  # even
    assert dl.row_plan_advice(dl.OP_SDDMM, M, K, 128, nnz, 52) == 0
    assert dl.row_plan_advice(dl.OP_SDDMM, M, K, 128, nnz, 158) == 1
    assert dl.row_plan_advice(dl.OP_SDDMM, M, K, 128, 2048 * 64, 209) == 1  # rows of 32 and more: as before
    assert dl.row_plan_advice(dl.OP_FUSED, 4096, K, 64, 4096 * 10, 158) == 0  # more rows: short rows stay grouped


def test_finer_column_tiles_for_plain_spmm_calls(dl):
    """A SpMM call without memory or plan does not know how even the rows are: few rows are covered by the widest column
    tile of B that gives two (row, tile) pairs per compute unit; N above 512 is covered in tiles of 256 instead of 512 up
    to eight rows per compute unit, and in tile-major tiles of 64 where B exceeds the L2. Not for rows below 16 nonzeros,
    not with memory or a plan."""
    tile = lambda M, K, N, per_row, **kw: (lambda sh: (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]))(
        dl.describe_launch(dl.OP_SPMM, M, K, N, M * per_row, **kw))
    assert tile(128, 1152, 256, 200) == (64, 4)      # 128 rows x 4 tiles = 512 pairs
    assert tile(128, 1152, 128, 200) == (32, 4)
    assert tile(64, 576, 256, 100) == (32, 8)
    assert tile(64, 576, 512, 100) == (64, 8)
    assert tile(16, 576, 512, 100) == (32, 16)       # never narrower than 32
    assert tile(192, 1152, 256, 200) == (64, 4)      # up to three quarters of a compute unit's count of pairs
    assert tile(193, 1152, 256, 200) == (256, 1)
    assert tile(128, 1152, 196, 200) == (128, 2)     # tiles of 64 would leave a last tile of 4 columns
    assert tile(128, 1152, 100, 200) == (64, 2)      # (64 + 36: more than half full)
    assert tile(128, 1152, 32, 200) == (32, 1)
    assert tile(128, 1152, 256, 15) == (256, 1)      # short rows pay their start once more per tile
    assert tile(128, 1152, 256, 200, with_workspace=True) == (256, 1)
    assert tile(128, 1152, 256, 200, rows_even=True) == (64, 4)   # the hint changes the grouping of rows, not the tiles
    # N above 512
    assert tile(1000, 512, 784, 100) == (256, 4)
    assert tile(2048, 512, 784, 100) == (256, 4)
    assert tile(2049, 512, 784, 100) == (512, 2)
    assert tile(1000, 512, 784, 15) == (512, 2)
    assert tile(64, 256, 3136, 100) == (256, 13)     # 64 x 7 pairs: no longer "few rows"; B of 3.1 MiB fits the L2
    # B beyond the L2 (K x N x 4 > 4 MiB) under N above 512: every XCD on its own tiles, of 128 columns where that gives
    # each XCD two and more, else of 64; eight tiles at least
    assert tile(64, 576, 3136, 100) == (128, 25)
    assert tile(300, 1152, 3136, 100) == (128, 25)
    assert tile(64, 1152, 12544, 100) == (128, 98)
    assert tile(4096, 4096, 3136, 100) == (128, 25)
    assert tile(256, 2304, 1536, 100) == (64, 24) and tile(1024, 4608, 784, 100) == (64, 13) and tile(1024, 4608, 640, 100) == (64, 10)
    assert tile(8192, 16384, 3136, 100) == (64, 49)  # (the widest tile whose slab fits the L2 is narrower here)
    assert tile(2048, 8192, 512, 400) == (64, 8) and tile(2048, 8192, 448, 400) == (128, 4)   # from eight tiles of 64 on
    assert tile(4096, 4096, 3136, 20) == (512, 7)    # rows below 32 nonzeros keep the widest tile, as before
    assert tile(32, 2304, 2048, 230) == (128, 16)    # few rows: two pairs per compute unit, the XCDs on their own tiles as well
    dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
    try:
        assert tile(128, 1152, 256, 200) == (256, 1) and tile(1000, 512, 784, 100) == (512, 2)
        assert tile(300, 1152, 3136, 100) == (512, 7) and tile(4096, 4096, 3136, 100) == (256, 13)
    finally:
        dl.set_tuning()
    # the tuning fields: tile_major = 0 with a width gives row-major tiles of that width
    dl.set_tuning(tile_major=0, tile_width=128)
    try:
        assert tile(4096, 4096, 3136, 100) == (128, 25) and tile(4096, 4096, 100, 100) == (128, 1)
    finally:
        dl.set_tuning()


def test_row_pieces_for_plain_sddmm_calls_on_few_rows(dl):
    """SDDMM without plan or memory on a mask of at most three quarters of the compute units' count of rows: 2^k four-wave
    workgroups share each row, up to two workgroups per compute unit in all, each keeping 32 nonzeros of a mean row or
    more; up to one and a half of that count: two workgroups per row; rows of 128 nonzeros and more on average only."""
    pieces = lambda M, per_row, **kw: (lambda sh: (sh["W"], sh["col_tiles"]))(dl.describe_launch(dl.OP_SDDMM, M, 4608, 128, M * per_row, **kw))
    assert pieces(128, 300) == (4, 4) and pieces(64, 300) == (4, 8) and pieces(32, 300) == (4, 8)   # (8: 37 per workgroup)
    assert pieces(32, 600) == (4, 16) and pieces(1, 4608) == (4, 128) and pieces(192, 300) == (4, 4)
    # up to one and a half of the compute units' count of rows: two workgroups per row; beyond, eight or four waves as before
    assert pieces(193, 300) == (4, 2) and pieces(256, 300) == (4, 2) and pieces(384, 300) == (4, 2) and pieces(385, 300) == (8, 1)
    assert pieces(300, 127) == (8, 1) and pieces(512, 300) == (4, 1)
    assert pieces(128, 127) == (8, 1) and pieces(128, 128) == (4, 4)
    assert pieces(128, 300, rows_even=True) == (4, 4)      # the hint is about the lengths of the rows, not their number
    assert pieces(128, 300, with_workspace=True) == (8, 1)
    dl.set_tuning(rules_off=dl.RULES["row_pieces_few_rows"])
    try:
        assert pieces(128, 300) == (8, 1)
    finally:
        dl.set_tuning()
    dl.set_tuning(split=(4, 1))                            # a forced split is taken as it is
    try:
        assert pieces(128, 300) == (4, 1)
    finally:
        dl.set_tuning()


def test_column_tiles_narrow_with_the_height_of_the_dense_operand(dl):
    """Dense rows wider than 512 floats are covered by several column tiles, worked through one after the other: the
    widest tile whose K x tile slab of B fits 4 MiB."""
    nnz = 4096 * 100
    for K, tile in ((512, 512), (2048, 512), (2049, 256), (4096, 256), (4097, 128), (8193, 64), (1 << 16, 32)):
        dl.set_tuning(rules_off=dl.RULES["finer_column_tiles"])
        try:
            sh = dl.describe_launch(dl.OP_SPMM, 4096, K, 3136, nnz)
        finally:
            dl.set_tuning()
        assert sh["G"] * sh["vec"] * sh["V"] == tile and sh["col_tiles"] == -(-3136 // tile), (K, sh)
        # a call without memory takes tiles of 128 at most here (25 tiles: three to each XCD, one shared): every XCD
        # works on its own tiles of B
        sh = dl.describe_launch(dl.OP_SPMM, 4096, K, 3136, nnz)
        assert sh["G"] * sh["vec"] * sh["V"] == min(tile, 128) and sh["col_tiles"] == -(-3136 // min(tile, 128)), (K, sh)
        sh = dl.describe_launch(dl.OP_SPMM, 4096, K, 3136, nnz, with_workspace=True)
        assert sh["G"] * sh["vec"] * sh["V"] == (max(tile, 128) if K * 128 * 4 <= (8 << 20) else 512)
    # ... with memory and rows long enough for the column-sliced schedule (64 nonzeros per row, half a million in
    # all), tiles of 128 at any height: the slices cut the slab along K
    for n, tiles in ((3136, 25), (1024, 8), (256, 2)):
        sh = dl.describe_launch(dl.OP_SPMM, 8192, 1 << 15, n, 8192 * 300, with_workspace=True)
        assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (128, tiles)
    assert dl.describe_launch(dl.OP_SPMM, 8192, 1 << 15, 1024, 8192 * 63, with_workspace=True)["col_tiles"] == 2
    # the workgroups of one (slice, tile) pair fill the device by themselves: rows per workgroup from M alone
    assert dl.describe_slices(dl.OP_SPMM, 8192, 1 << 15, 1024, 8192 * 300) == (6, 4)
    assert dl.describe_slices(dl.OP_SPMM, 4096, 1 << 16, 3136, 4096 * 131) == (4, 2)
    assert dl.describe_slices(dl.OP_SPMM, 2048, 1 << 17, 512, 2048 * 655) == (16, 1)
    # the same where one wave could cover the whole width, once B exceeds the L2; tiles below 128 columns only for a
    # call without workspace memory (with it the columns of A are sliced instead)
    sh = dl.describe_launch(dl.OP_SPMM, 4096, 8192, 256, nnz)
    assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (128, 2)
    for K, tile in ((16384, 64), (32768, 32), (1 << 16, 32)):
        sh = dl.describe_launch(dl.OP_SPMM, 4096, K, 128, nnz)
        assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (tile, 128 // tile)
        assert dl.describe_launch(dl.OP_SPMM, 4096, K, 128, nnz, with_workspace=True)["col_tiles"] == 1
        assert dl.describe_launch(dl.OP_SPMM, 4096, K, 128, nnz, rows_even=True)["col_tiles"] == 128 // tile
    # not when even the narrowest slab is beyond twice the L2, nor for rows below 32 nonzeros (graph-like shapes):
    # more tiles than needed cost every row its start-up once more
    assert dl.describe_launch(dl.OP_SPMM, 4096, 1 << 17, 128, nnz)["col_tiles"] == 1
    assert dl.describe_launch(dl.OP_SPMM, 4096, 1 << 17, 3136, nnz)["col_tiles"] == 7      # the usual tiles of 512
    assert dl.describe_launch(dl.OP_SPMM, 1 << 18, 32768, 128, (1 << 18) * 8)["col_tiles"] == 1
    assert dl.describe_launch(dl.OP_SPMM, 4096, 32768, 64, nnz)["col_tiles"] == 2
    assert dl.describe_launch(dl.OP_SPMM, 4096, 32768, 32, nnz)["col_tiles"] == 1   # 32 columns: the narrowest tile
    sh = dl.describe_launch(dl.OP_SPMM, 4097, 4096, 512, nnz)
    assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (256, 2)
    sh = dl.describe_launch(dl.OP_SPMM, 4096, 4096, 512, nnz)         # up to sixteen rows per compute unit: the XCDs' own tiles of 64
    assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (64, 8)
    assert dl.describe_launch(dl.OP_SPMM, 4096, 4096, 256, nnz)["col_tiles"] == 1   # 4 MiB: fits
    assert dl.describe_launch(dl.OP_SPMM, 1024, 8192, 256, nnz)["col_tiles"] == 1   # a grid the device holds at once


def test_column_sliced_schedule_rule(dl):
    """Slices of at most 8/3 MiB of gathered dense operand (2 MiB in SDDMM, which writes no partial rows), only when the operand exceeds 4 MiB, the dense rows are wide
    and a row keeps at least 16 nonzeros per slice on average; the workspace then holds the boundaries and the
    partial rows of every slice."""
    M = K = 8192
    nnz = M * 800
    assert dl.describe_slices(dl.OP_FUSED, M, K, 128, nnz)[0] == 3      # Kmat + V: 8 MiB
    assert dl.describe_slices(dl.OP_FUSED, M, K, 256, nnz)[0] == 6      # 16 MiB
    assert dl.describe_slices(dl.OP_FUSED, M, K, 64, nnz)[0] == 0       # 4 MiB of narrow dense rows: left alone
    assert dl.describe_slices(dl.OP_FUSED, M, 4 * K, 64, nnz)[0] == 6   # sparse attention over 32768 keys, D = 64: 16 MiB
    assert dl.describe_slices(dl.OP_FUSED, M, 4 * K, 64, M * 200)[0] == 3   # ... a row keeps 64 nonzeros per slice at D = 64
    assert dl.describe_slices(dl.OP_FUSED, M, 4 * K, 16, nnz)[0] == 0   # D <= 16: not built for it
    assert dl.describe_slices(dl.OP_FUSED, M, K // 2, 128, nnz)[0] == 2 # 4 MiB just fills the L2: in two for long rows
    assert dl.describe_slices(dl.OP_FUSED, M, K // 2, 128, M * 400)[0] == 0  # ... not for 200 nonzeros per slice
    # SpMM cuts a B beyond 4 MiB into column tiles first (8192 x 128 floats here: 4 MiB per tile), and slices the tile
    assert dl.describe_slices(dl.OP_SPMM, M, K, 256, nnz)[0] == 2       # 4 MiB per tile, 400 nonzeros per slice
    assert dl.describe_slices(dl.OP_SPMM, M, K, 256, M * 400)[0] == 0   # ... 200 nonzeros per slice: not at exactly 4 MiB
    assert dl.describe_slices(dl.OP_SPMM, M, K, 128, nnz)[0] == 2       # one tile of 4 MiB
    assert dl.describe_slices(dl.OP_SPMM, M, K, 100, nnz)[0] == 0       # 3.1 MiB: fits
    assert dl.describe_slices(dl.OP_SPMM, M, 2 * K, 256, nnz)[0] == 3   # 16384 x 128 floats per tile: 8 MiB
    assert dl.describe_slices(dl.OP_SPMM, M, 4 * K, 256, nnz)[0] == 6   # taller: tiles of 128 all the same, 16 MiB each
    assert dl.describe_slices(dl.OP_SPMM, M, 1 << 16, 32, nnz)[0] == 3  # narrow dense rows, very tall B: 8 MiB
    assert dl.describe_slices(dl.OP_SPMM, M, 1 << 16, 32, M * 300)[0] == 2  # ... 128 nonzeros per slice at N = 32
    assert dl.describe_slices(dl.OP_SPMM, M, 1 << 20, 3, nnz)[0] == 0   # fewer than four columns: not built for them
    # a row keeps at least max(16, 4096 / width) nonzeros per slice: 16 at 256 columns, 32 in tiles of 128
    assert dl.describe_slices(dl.OP_SPMM, M, 4 * K, 256, M * 140)[0] == 4   # 140 nonzeros per row: four slices of 35
    assert dl.describe_slices(dl.OP_SPMM, M, 4 * K, 256, M * 70)[0] == 2    # 70 per row: two
    assert dl.describe_slices(dl.OP_SPMM, 2 * M, 4 * K, 256, 2 * M * 60)[0] == 3  # below 64 per row: one tile of 256, three slices of 20
    assert dl.describe_slices(dl.OP_SPMM, M, 2 * K, 256, M * 140)[0] == 3   # 8 MiB per tile: three, whatever the rows allow
    assert dl.describe_slices(dl.OP_SPMM, M, 2 * K, 256, M * 70)[0] == 2    # 70 per row: two
    assert dl.describe_slices(dl.OP_SPMM, M, 4 * K, 256, M * 40)[0] == 0    # 40 per row, 0.33 M nonzeros: too small
    assert dl.describe_slices(dl.OP_SPMM, 4 * M, 4 * K, 256, 4 * M * 64)[0] == 2  # 2.1 M nonzeros, 64 per row
    assert dl.describe_slices(dl.OP_SPMM, 4 * M, 4 * K, 256, 4 * M * 30)[0] == 0  # 30 per row: not even two of 16
    assert dl.describe_slices(dl.OP_SPMM, M, 1 << 17, 256, nnz)[0] == 16      # 128 MiB: the most slices there are
    assert dl.describe_slices(dl.OP_SPMM, M, 1 << 17, 256, M * 100)[0] == 3   # ... but a row keeps 32 nonzeros per slice
    assert dl.describe_slices(dl.OP_SDDMM, M, K, 256, nnz)[0] == 4      # rhs: 8 MiB in slices of 2 MiB (no partial rows); only the boundaries need memory
    assert dl.workspace_bytes(dl.OP_SDDMM, M, K, 256, nnz) == -(-5 * M * 4 // 256) * 256
    assert dl.describe_slices(dl.OP_SDDMM, M, K, 100, nnz)[0] == 0 and dl.workspace_bytes(dl.OP_SDDMM, M, K, 100, nnz) == 0
    # fewer than four rows per compute unit (1024 on this device): one slice's workgroups would not fill it
    for op, width in ((dl.OP_SPMM, 256), (dl.OP_SDDMM, 128), (dl.OP_FUSED, 128)):
        assert dl.describe_slices(op, 512, 4 * K, width, 512 * 2048)[0] == 0
        assert dl.describe_slices(op, 1023, 4 * K, width, 1023 * 2048)[0] == 0
        assert dl.describe_slices(op, 1024, 4 * K, width, 1024 * 2048)[0] >= 6
    assert dl.workspace_bytes(dl.OP_SDDMM, 512, 4 * K, 128, 512 * 2048) == 0
    slices, R = dl.describe_slices(dl.OP_FUSED, M, K, 256, nnz)
    assert R == 2                                                       # 133 nonzeros per row and slice
    bounds = -(-(slices + 1) * M * 4 // 256) * 256
    assert dl.workspace_bytes(dl.OP_FUSED, M, K, 256, nnz) == bounds + slices * M * 256 * 4
    # below the sliced rule the flat schedule's size is reported as before
    assert dl.workspace_bytes(dl.OP_SPMM, M, K, 100, nnz) == dl.describe_launch(dl.OP_SPMM, M, K, 100, nnz)["flat_units"] * 2 * 100 * 4


def test_workspace_advice(dl):
    """One host call holds the measured rules for what to pass as `workspace`."""
    M = K = 8192
    nnz = M * 800
    mean = nnz // M
    A = dl.workspace_advice
    # column-sliced schedule (fused, 8 MiB of Kmat and V: four slices): the memory, whatever the rows
    for longest in (-1, mean, 3 * mean, 10 * mean):
        assert A(dl.OP_FUSED, M, K, 128, nnz, longest) == dl.PASS_WORKSPACE
    # two slices (4 MiB, long rows): even rows rather take the hint in SpMM and the fused op, never in SDDMM
    assert dl.describe_slices(dl.OP_SPMM, M, K, 128, nnz)[0] == 2
    assert A(dl.OP_SPMM, M, K, 128, nnz, mean + 10) == dl.PASS_ROWS_EVEN
    assert A(dl.OP_SPMM, M, K, 128, nnz, 3 * mean) == dl.PASS_WORKSPACE
    assert A(dl.OP_SDDMM, M, K, 128, nnz, mean + 10) == dl.PASS_WORKSPACE
    # few rows: no slices, and even rows take the hint (SpMM, 256 x 8192 half full at N = 256: 42.8 us against 48.2 us with memory)
    assert A(dl.OP_SPMM, 256, K, 256, 256 * 4096, 4200) == dl.PASS_ROWS_EVEN
    assert A(dl.OP_SDDMM, 512, K, 128, 512 * 2048, 2150) == dl.PASS_ROWS_EVEN
    assert A(dl.OP_SDDMM, 1024, 4 * K, 128, 1024 * 2048, 2150) == dl.PASS_WORKSPACE
    assert dl.describe_slices(dl.OP_SPMM, M, 4 * K, 256, M * 120)[0] == 3
    assert A(dl.OP_SPMM, M, 4 * K, 256, M * 120, 3 * 120) == dl.PASS_NULL
    assert A(dl.OP_SPMM, M, 4 * K, 256, M * 120, 130) == dl.PASS_ROWS_EVEN
    assert A(dl.OP_SPMM, M, 4 * K, 256, M * 130, 3 * 130) == dl.PASS_WORKSPACE
    assert A(dl.OP_SPMM, M, 1 << 18, 256, M * 120, 3 * 120) == dl.PASS_WORKSPACE   # no tile would fit: the slices
    assert A(dl.OP_FUSED, M, 4 * K, 256, M * 120, 3 * 120) == dl.PASS_WORKSPACE    # the other two ops have no tiles
    # no slices: the memory for rows at least four times the mean where the flat schedule applies, the hint for even rows
    assert A(dl.OP_SPMM, M, 2048, 128, nnz, 4 * mean) == dl.PASS_WORKSPACE
    assert A(dl.OP_SPMM, M, 2048, 128, nnz, 3 * mean) == dl.PASS_NULL
    assert A(dl.OP_SPMM, M, 2048, 128, nnz, -1) == dl.PASS_NULL
    assert A(dl.OP_SPMM, M, 2048, 128, nnz, int(1.5 * mean)) == dl.PASS_ROWS_EVEN
    assert A(dl.OP_SPMM, 2048, 512, 256, 105687, 300) == dl.PASS_NULL      # small and uneven: nothing helps
    assert A(dl.OP_SDDMM, M, 2048, 128, nnz, 10 * mean) == dl.PASS_NULL    # SDDMM's flat schedule needs no memory
    assert A(dl.OP_SPMM, 0, 0, 0, 0, 0) == dl.PASS_NULL and A(7, M, K, 128, nnz, mean) == dl.PASS_NULL


def test_row_plan_host_side(dl):
    """Size, advice and argument checks of the row plan need no GPU."""
    L = dl.lib()
    assert L.dlspm_row_plan_bytes(2048) == 3 * 2048 * 4 and L.dlspm_row_plan_bytes(0) == 0 and L.dlspm_row_plan_bytes(-5) == 0
    A = lambda *a: dl.row_plan_advice(dl.OP_SPMM, *a)
    assert A(2048, 512, 256, 105687, 312)            # the headline configuration: uneven rows, one row per workgroup
    assert A(2048, 512, 256, 105687, -1)             # rows unknown: nothing better to pass
    assert not A(2048, 512, 256, 105687, 60)         # even rows: another order gains nothing
    # where the size rule groups rows per workgroup, a plan ungroups them if they are long enough for that
    assert dl.describe_launch(dl.OP_SPMM, 4096, 1024, 256, 4096 * 100)["R"] == 2 and A(4096, 1024, 256, 4096 * 100, 400)
    assert A(8192, 2048, 128, 8192 * 200, 1400) and A(16384, 512, 256, 16384 * 51, 500) and A(65536, 2048, 128, 65536 * 197, 2000)
    assert not A(32768, 1024, 256, 32768 * 32, 300)  # 32 per row in a tall matrix: grouped rows win
    assert not A(16384, 2048, 32, 16384 * 101, 1000)  # narrow dense rows in a tall matrix
    assert not A(8192, 512, 256, 8192 * 24, 200)     # short rows
    assert A(4096, 512, 32, 4096 * 52, 500)          # ... but any width up to 4096 rows
    assert not A(600, 512, 784, 600 * 60, 300)       # column tiles
    assert not A(2048, 512, 3, 105687, 312)          # fewer than four columns
    assert A(16384, 4096, 128, 16384 * 400, 4000)    # large and uneven: the plan rather than the flat schedule's workspace
    assert dl.workspace_advice(dl.OP_SPMM, 16384, 4096, 128, 16384 * 400, 4000) == dl.PASS_WORKSPACE   # (what is said without a plan)
    assert not A(8192, 16384, 128, 8192 * 800, 8000)  # B of 8 MiB: the column-sliced schedule's workspace first
    assert not A(0, 0, 0, 0, 0)
    # the other two ops: built for 16 < D <= 512
    for op in (dl.OP_SDDMM, dl.OP_FUSED):
        assert dl.row_plan_advice(op, 2048, 2048, 64, 2048 * 100, 500)
        assert dl.row_plan_advice(op, 8192, 2048, 128, 8192 * 200, 2000)
        assert not dl.row_plan_advice(op, 2048, 2048, 64, 2048 * 100, 120)     # even rows
        assert not dl.row_plan_advice(op, 2048, 2048, 16, 2048 * 100, 500)     # D <= 16
        assert not dl.row_plan_advice(op, 2048, 2048, 1024, 2048 * 100, 500)   # D > 512
        # short rows in a tall mask: the fused op groups them, and its groups win; SDDMM runs one row per workgroup up
        # to 128 rows per compute unit, and a plan over such rows only has to beat their given order
        assert bool(dl.row_plan_advice(op, 8192, 2048, 64, 8192 * 20, 200)) == (op == dl.OP_SDDMM)
        assert dl.describe_launch(op, 16384, 2048, 128, 16384 * 60)["R"] == (1 if op == dl.OP_SDDMM else 8)
        assert bool(dl.row_plan_advice(op, 16384, 2048, 128, 16384 * 60, 600)) == (op == dl.OP_SDDMM)
        assert dl.describe_launch(op, 32768, 2048, 128, 32768 * 60)["R"] == 8
        assert not dl.row_plan_advice(op, 32768, 2048, 128, 32768 * 60, 600)   # grouped rows: the grouping wins
        assert dl.row_plan_advice(op, 16384, 4096, 128, 16384 * 400, 4000)     # ... rows the rule runs one per workgroup anyway
    assert not dl.row_plan_advice(dl.OP_FUSED, 8192, 8192, 128, 8192 * 800, 8000)   # Kmat and V of 8 MiB: the slices first
    assert not dl.row_plan_advice(7, 2048, 2048, 64, 2048 * 100, 500)
    bogus = ctypes.c_void_p(256)   # never dereferenced: the checks come first
    plan_of = lambda n: n | dl.HINT_ROW_PLAN   # (a row plan of n bytes as the workspace of the named entry points)
    assert L.sddmm_csr_f32(2, 2, -4, 1, None, None, None, None, None, bogus, plan_of(24), None) == dl.E_INVALID_ARG
    assert L.sddmm_csr_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, bogus, plan_of(23), None) == dl.E_WORKSPACE
    assert L.sddmm_csr_f32(2, 2, 32, 1, None, None, None, None, None, None, 0, None) == dl.E_INVALID_ARG
    assert L.fused_sddmm_spmm_f32(2, 2, 32, 9, None, None, None, None, None, 1.0, None, bogus, plan_of(24), None) == dl.E_INVALID_ARG
    assert L.fused_sddmm_spmm_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, 1.0, bogus, bogus, plan_of(23), None) == dl.E_WORKSPACE
    assert L.fused_sddmm_spmm_f32(2, 2, 32, 1, None, None, None, None, None, 1.0, None, None, 0, None) == dl.E_INVALID_ARG
    assert L.dlspm_row_plan_build(-1, bogus, bogus, 0, None) == dl.E_INVALID_ARG
    assert L.dlspm_row_plan_build(8, None, bogus, 96, None) == dl.E_INVALID_ARG
    assert L.dlspm_row_plan_build(8, bogus, bogus, 95, None) == dl.E_WORKSPACE
    assert L.dlspm_row_plan_build(4096, bogus, bogus, 3 * 4096 * 4, None) == dl.E_WORKSPACE   # beyond 2048 rows: room for the sort
    assert L.dlspm_row_plan_build(0, None, None, 0, None) == dl.OK
    assert L.spmm_csr_f32(-1, 1, 1, 0, None, None, None, None, None, bogus, plan_of(0), None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(2, 2, 2, 5, None, None, None, None, None, bogus, plan_of(24), None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(2, 2, 2, 1, bogus, bogus, bogus, bogus, bogus, bogus, plan_of(23), None) == dl.E_WORKSPACE
    assert L.spmm_csr_f32(2, 2, 2, 1, None, None, None, None, None, None, 0, None) == dl.E_INVALID_ARG


def test_tuning_overrides_go_through_one_call_and_the_environment_is_read_once(dl):
    """dlspm_set_tuning replaces the per-launch getenv knobs: per thread, validated, and visible to the host-only
    queries; the environment only seeds the process default, once, so a later change of it changes nothing."""
    import threading

    base = dl.get_tuning()
    assert base == {"split_w": 0, "split_r": 0, "flat": -1, "flat_chunk": 0, "slices": -1, "tile_major": -1,
                    "tile_width": 0, "plan_order": 0, "xcd_contiguous": 0, "stream_results": -1, "cut_piece_pct": 0,
                    "cut_longest_pct": 0, "rules_off": 0, "compute_units": 0}
    sizes = (dl.OP_SPMM, 8192, 4096, 128, 8192 * 600)
    rule = dl.describe_launch(*sizes)
    assert (rule["W"], rule["R"]) == (4, 1)
    dl.set_tuning(split=(8, 2))
    assert dl.get_tuning()["split_w"] == 8 and (dl.describe_launch(*sizes)["W"], dl.describe_launch(*sizes)["R"]) == (8, 2)
    seen = {}
    th = threading.Thread(target=lambda: seen.update(dl.get_tuning()))   # another thread still follows the rules
    th.start()
    th.join()
    assert seen == base
    dl.set_tuning(split=(5, 3))          # not a shape the kernels are built for: ignored
    assert (dl.describe_launch(*sizes)["W"], dl.describe_launch(*sizes)["R"]) == (4, 1)
    os.environ["DLSPM_SPLIT"] = "16,1"   # the environment was read when the library first looked; not again
    try:
        dl.set_tuning()
        assert dl.get_tuning() == base and dl.describe_launch(*sizes) == rule
    finally:
        del os.environ["DLSPM_SPLIT"]
    dl.set_tuning(tile_width=128, tile_major=1)
    sh = dl.describe_launch(dl.OP_SPMM, 4096, 512, 512, 4096 * 50)
    assert (sh["G"] * sh["vec"] * sh["V"], sh["col_tiles"]) == (128, 4)
    dl.set_tuning()
    for bad in ({"flat": 2}, {"slices": -2}, {"plan_order": 3}, {"tile_major": 5}, {"split": (-1, 0)}, {"flat_chunk": -64},
                {"xcd_contiguous": 2}, {"stream_results": 2}, {"stream_results": -2}, {"rules_off": -1},
                {"rules_off": 2 * max(dl.RULES.values())}):
        with pytest.raises(dl.DlspmError):
            dl.set_tuning(**bad)
    dl.set_tuning(rules_off=sum(dl.RULES.values()))   # every rule off at once is a valid setting
    dl.set_tuning()
    header = open(os.path.join(ROOT, "include", "dlspm_hip.h")).read()
    assert sorted(dl.RULES.values()) == sorted(int(v) for v in re.findall(r"#define DLSPM_RULE_\w+\s+(\d+)", header))
    assert dl.get_tuning() == base
    assert dl.lib().dlspm_get_tuning(None) == dl.E_INVALID_ARG
    src = open(os.path.join(ROOT, "dlspm-esimd_amd", "csrc", "api.hip")).read()
    sources = "".join(open(os.path.join(ROOT, "dlspm-esimd_amd", "csrc", f)).read()
                      for f in os.listdir(os.path.join(ROOT, "dlspm-esimd_amd", "csrc")))
    assert sources.count("getenv(") == 1 and src.count("getenv(") == 1


def test_the_environment_seeds_the_process_default(dl):
    """A fresh process started with DLSPM_SPLIT / DLSPM_FLAT_CHUNK in its environment starts from those overrides (how
    the C++ drivers are swept from a shell)."""
    code = ("import sys; sys.path.insert(0, %r); import dlspm_hip as dl; t = dl.get_tuning(); "
            "print(t['split_w'], t['split_r'], t['flat_chunk'], t['slices'])" % os.path.join(ROOT, "dlspm-esimd_amd"))
    env = dict(os.environ, DLSPM_SPLIT="8,1", DLSPM_FLAT_CHUNK="320", DLSPM_SLICES="0")
    r = subprocess.run(["python", "-c", code], capture_output=True, text=True, env=env)
    assert r.returncode == 0 and r.stdout.split() == ["8", "1", "320", "0"], r.stderr


def test_device_info_and_hints_without_a_gpu(dl):
    """Host-only: without a device the size rules use a whole MI355X's figures and the compute calls that would have
    to launch say DLSPM_E_NO_DEVICE; the hint bits are no part of the workspace size."""
    import torch

    info = dl.device_info()
    if torch.cuda.is_available():
        assert info["status"] == dl.OK and info["gfx950"]
    else:
        assert info == {"status": dl.E_NO_DEVICE, "compute_units": 256, "l2_bytes": 4 << 20, "gfx950": False}
        bogus = ctypes.c_void_p(256)   # never dereferenced: no device, no launch
        L = dl.lib()
        assert L.spmm_csr_f32(2, 2, 2, 1, bogus, bogus, bogus, bogus, bogus, None, 0, None) == dl.E_NO_DEVICE
        assert L.sddmm_csr_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, None, 0, None) == dl.E_NO_DEVICE
        assert L.fused_sddmm_spmm_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, 1.0, bogus, None, 0, None) == dl.E_NO_DEVICE
        assert L.dlspm_row_plan_build(8, bogus, bogus, 96, None) == dl.E_NO_DEVICE
        assert L.dlspm_csr_check(2, 2, 1, bogus, bogus, None) == dl.E_NO_DEVICE
        assert L.spmm_csr_f32_static(2, 2, 2, 1, bogus, bogus, bogus, bogus, bogus, None) == dl.E_NO_DEVICE
    assert "gfx950" in dl.status_string(dl.E_NO_DEVICE)
    L = dl.lib()
    bogus = ctypes.c_void_p(256)
    # a plan hint with too little memory behind it is refused before anything else is looked at; hint bits alone are not a size
    assert L.spmm_csr_f32(2, 2, 2, 1, bogus, bogus, bogus, bogus, bogus, bogus, 23 | dl.HINT_ROW_PLAN, None) == dl.E_WORKSPACE
    assert L.sddmm_csr_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, bogus, 23 | dl.HINT_ROW_PLAN, None) == dl.E_WORKSPACE
    assert L.fused_sddmm_spmm_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, 1.0, bogus, bogus, 23 | dl.HINT_ROW_PLAN, None) == dl.E_WORKSPACE
    assert L.spmm_csr_f32(0, 5, 5, 0, None, None, None, None, None, None, dl.HINT_ROWS_EVEN, None) == dl.OK
    assert dl.row_plan_bytes(2048) == 3 * 2048 * 4 and dl.row_plan_bytes(2049) == 3 * 2049 * 4 + 4 + 2 * 2049 * 8
    # Bits of the hint byte that mean nothing are refused, so a "plenty of scratch" size such as SIZE_MAX cannot turn
    # scratch memory into a row plan; so are a plan of 2^48 bytes and more, both kinds of plan at once, and the
    # deprecated pointer constant together with a size.
    size_max = (1 << 64) - 1
    spmm = lambda ws, size: L.spmm_csr_f32(2, 2, 2, 1, bogus, bogus, bogus, bogus, bogus, ws, size, None)
    sddmm = lambda ws, size: L.sddmm_csr_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, ws, size, None)
    fused = lambda ws, size: L.fused_sddmm_spmm_f32(2, 2, 32, 1, bogus, bogus, bogus, bogus, bogus, 1.0, bogus, ws, size, None)
    for call in (spmm, sddmm, fused):
        assert call(bogus, size_max) == dl.E_INVALID_ARG
        assert call(bogus, 4096 | (1 << 63)) == dl.E_INVALID_ARG
        assert call(bogus, 4096 | (1 << 57)) == dl.E_INVALID_ARG
        assert call(None, dl.HINT_ROWS_EVEN | dl.HINT_ROWS_SKEWED) == dl.E_INVALID_ARG
        assert call(bogus, (1 << 48) | dl.HINT_ROW_PLAN) == dl.E_INVALID_ARG
        assert call(bogus, 4096 | dl.HINT_ROW_PLAN | dl.HINT_CUT_PLAN) == dl.E_INVALID_ARG
        assert call(ctypes.c_void_p(1), 4096) == dl.E_INVALID_ARG
        assert call(bogus, 23 | dl.HINT_CUT_PLAN) in (dl.E_WORKSPACE, dl.E_NO_DEVICE)
    # cut plans: argument checks come before anything touches the device
    assert L.dlspm_row_plan_build_cut(-1, bogus, bogus, 0, None) == dl.E_INVALID_ARG
    assert L.dlspm_row_plan_build_cut((1 << 20) + 1, bogus, bogus, 1 << 40, None) == dl.E_INVALID_ARG
    assert L.dlspm_row_plan_build_cut(8, None, bogus, 1 << 20, None) == dl.E_INVALID_ARG
    assert L.dlspm_row_plan_build_cut(0, None, None, 0, None) == dl.OK


def test_library_exports_every_declared_symbol(dl):
    lib = ctypes.CDLL(dl.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/dlspm_hip.h but not exported"
    assert set(declared_functions()) == set(dl.EXPORTS)
    # ... and nothing else: the rest of the library has hidden visibility
    import shutil
    import subprocess

    if shutil.which("nm"):
        out = subprocess.run(["nm", "-D", "--defined-only", dl.LIB_PATH], capture_output=True, text=True, check=True).stdout
        exported = {line.split()[2] for line in out.splitlines() if len(line.split()) == 3 and line.split()[1] in "TW"}
        assert exported == set(declared_functions()), sorted(exported ^ set(declared_functions()))


def test_host_only_entry_points_answer_without_a_gpu(dl):
    L = dl.lib()
    assert dl.version().startswith("dlspm_hip") and "gfx950" in dl.version()
    assert dl.status_string(dl.OK) == "ok"
    for code in (dl.E_INVALID_ARG, dl.E_WORKSPACE, dl.E_LAUNCH, dl.E_INVALID_CSR, dl.E_NO_DEVICE, -99):
        assert isinstance(dl.status_string(code), str) and dl.status_string(code)
    assert L.dlspm_workspace_bytes(dl.OP_SPMM, 2048, 512, 256, 100000) == 0
    # argument validation happens before any HIP call, so it can be checked here
    assert L.spmm_csr_f32(-1, 1, 1, 0, None, None, None, None, None, None, 0, None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(2, 2, 2, 5, None, None, None, None, None, None, 0, None) == dl.E_INVALID_ARG  # nnz > M*K
    assert L.spmm_csr_f32(2, 2, 2, 1, None, None, None, None, None, None, 0, None) == dl.E_INVALID_ARG  # NULL CSR
    assert L.sddmm_csr_f32(2, 2, -4, 1, None, None, None, None, None, None, 0, None) == dl.E_INVALID_ARG
    assert L.fused_sddmm_spmm_f32(2, 2, 4, 1, None, None, None, None, None, 1.0, None, None, 0, None) == dl.E_INVALID_ARG
    assert L.spmm_csr_f32(0, 5, 5, 0, None, None, None, None, None, None, 0, None) == dl.OK  # empty problem
    assert L.sddmm_csr_f32(5, 5, 4, 0, None, None, None, None, None, None, 0, None) == dl.OK


def test_flat_schedule_rule_and_workspace_size(dl):
    """Host-only: the size rule of the flat schedule and the workspace it asks for (units x 2 x width floats)."""
    dl.set_tuning()
    M, K, nnz = 8192, 4096, 3355443
    sh = dl.describe_launch(dl.OP_SPMM, M, K, 128, nnz)
    assert sh["flat_chunk"] == 512 and sh["flat_units"] == -(-nnz // 512)
    assert dl.workspace_bytes(dl.OP_SPMM, M, K, 128, nnz) == sh["flat_units"] * 2 * 128 * 4
    assert dl.workspace_bytes(dl.OP_FUSED, M, K, 128, nnz) == sh["flat_units"] * 2 * 128 * 4
    assert dl.workspace_bytes(dl.OP_SDDMM, M, K, 128, nnz) == 0               # nothing to combine
    assert dl.describe_launch(dl.OP_SDDMM, M, K, 32, nnz)["flat_chunk"] == 512  # but the schedule is used, any width
    assert dl.workspace_bytes(dl.OP_SPMM, M, K, 64, nnz) == 0                 # narrow dense rows: row-block schedule
    mid = 838860                                                              # below 2 M nonzeros: 256 per wave
    shm = dl.describe_launch(dl.OP_SPMM, 4096, 4096, 256, mid)
    assert shm["flat_chunk"] == 256 and dl.workspace_bytes(dl.OP_SPMM, 4096, 4096, 256, mid) == -(-mid // 256) * 2 * 256 * 4
    assert dl.describe_launch(dl.OP_SDDMM, 4096, 4096, 128, mid)["flat_chunk"] == 0  # SDDMM: only from 2 M nonzeros on
    assert dl.workspace_bytes(dl.OP_SPMM, M, K, 128, (1 << 19) - 1) == 0      # too few nonzeros
    assert dl.workspace_bytes(dl.OP_SPMM, 65536, K, 128, nnz) == 0            # rows too short (51 on average)
    big = 26843545                                                            # the chunk grows to keep ~32768 units
    shb = dl.describe_launch(dl.OP_SPMM, 32768, 8192, 128, big)
    assert shb["flat_chunk"] == 832 and shb["flat_units"] == -(-big // 832)
    for cfg_sizes in [(512, 512, 128, 78643), (2048, 512, 256, 105687), (2048, 512, 392, 208896), (4096, 4096, 64, 324737)]:
        for op in (dl.OP_SPMM, dl.OP_SDDMM, dl.OP_FUSED):
            assert dl.workspace_bytes(op, *cfg_sizes) == 0 and dl.describe_launch(op, *cfg_sizes)["flat_chunk"] == 0
    dl.set_tuning(flat=1, slices=0, flat_chunk=192)
    assert dl.workspace_bytes(dl.OP_SPMM, 100, 50, 7, 1000) == -(-1000 // 192) * 2 * 7 * 4


def test_binding_refuses_host_tensors(dl):
    import torch

    ro = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(TypeError):
        dl.spmm(ro, ro, torch.zeros(3), torch.zeros(2, 2))


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_benchmark_configs_are_as_specified(dl, oracle, cfg):
    c = dl.make_config(cfg)
    again = dl.make_config(cfg)
    for k in ("row_offsets", "col_indices", "values", "d0", "d1", "d2"):
        assert np.array_equal(c[k], again[k]), "generators must be deterministic"
    ro, ci = c["row_offsets"], c["col_indices"]
    assert oracle.csr_check(c["M"], c["K"], c["nnz"], ro, ci) == 0
    lens = np.diff(ro)
    rows = np.repeat(np.arange(c["M"]), lens)
    inside = np.ones(ci.size, dtype=bool)
    inside[ro[:-1][lens > 0]] = False
    assert (np.diff(ci.astype(np.int64), prepend=-1)[inside] > 0).all(), "columns ascend strictly inside each row"
    sparsity = 1.0 - c["nnz"] / (c["M"] * c["K"])
    expect = {1: (0, 512, 512, 128, 0.70), 2: (0, 2048, 512, 256, 0.90), 3: (1, 2048, 2048, 128, 0.95),
              4: (0, 2048, 512, 392, 0.80), 5: (2, 4096, 4096, 64, 0.98)}[cfg]
    assert (c["op"], c["M"], c["K"], c["N"]) == expect[:4]
    assert abs(sparsity - expect[4]) < 0.005
    if cfg == 2:
        assert lens.max() > 4 * lens.mean(), "row lengths must be skewed"
        assert abs(c["values"].std() - 0.02) < 0.001
    if cfg == 4:
        assert (lens == 102).all()
        assert abs((c["d0"] == 0).mean() - 0.5) < 0.01 and c["d0"].min() >= 0
    if cfg == 5:
        assert c["scale"] == 0.125 and lens.max() <= 80
        i = 1000
        band = np.arange(i - 16, i + 16)
        assert np.isin(band, ci[ro[i]:ro[i + 1]]).all(), "the local band of width 32 is present"


def test_accounting_formulas(dl):
    a = dl.account(dl.OP_SPMM, 2048, 512, 256, 104858)
    assert a["flops"] == (2 * 104858 - 2048) * 256                       # SPMM/spmm-esimd-fromfile2.cpp:253
    assert a["algorithmic_bytes"] == 4 * 2049 + 8 * 104858 + 4 * 512 * 256 + 4 * 2048 * 256
    assert a["effective_bytes"] == 4 * 2049 + 8 * 104858 + 4 * 104858 * 256 + 4 * 2048 * 256
    s = dl.account(dl.OP_SDDMM, 2048, 2048, 128, 209715)
    assert s["flops"] == 209715 * (2 * 128 - 1)                          # SDDMM/sddmm-esimd-fromfile.cpp:160
    assert s["algorithmic_bytes"] == 4 * 2049 + 4 * 209715 + 4 * 2048 * 128 * 2 + 4 * 209715
    f = dl.account(dl.OP_FUSED, 4096, 4096, 64, 327680)
    assert f["flops"] == (2 * 327680 - 4096) * 64 + 327680 * (2 * 64 - 1) + 327680
    assert f["algorithmic_bytes"] == 4 * 4097 + 4 * 327680 + 4 * 4096 * 64 + 8 * 4096 * 64 + 4 * 4096 * 64


def test_host_entry_points_over_edge_and_random_sizes():
    """tests/host_fuzz: every host-side entry point (and, where there is no device, the compute entry points, which
    must answer with a status) over edge values and random sizes up to INT_MAX; `make -C tests/host_fuzz san` runs
    the same program against a build of the library with ASan and UBSan on the host side."""
    d = os.path.join(ROOT, "tests", "host_fuzz")
    r = subprocess.run(["make", "-C", d, "run"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "nothing reported" in r.stdout
