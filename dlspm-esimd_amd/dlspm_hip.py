"""ctypes binding of libdlspm_hip.so (the C ABI declared in include/dlspm_hip.h) for the Python tests and the
benchmark. PyTorch is used for device memory and the stream only; every computation happens inside the
library's HIP kernels. There is no fallback: if the shared library is missing or a call fails, an exception
is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdlspm_hip.so")
GEN_LIB_PATH = os.path.join(_HERE, "libdlspm_gen.so")

OK = 0
E_INVALID_ARG = -1
E_WORKSPACE = -2
E_LAUNCH = -3
E_INVALID_CSR = -4
E_NO_DEVICE = -5
E_STATIC_LIMIT = -6

OP_SPMM, OP_SDDMM, OP_FUSED = 0, 1, 2


HINT_ROWS_EVEN = 1 << 62
HINT_ROW_PLAN = 1 << 61
HINT_BANDED = 1 << 60
HINT_CUT_PLAN = 1 << 59
HINT_ROWS_SKEWED = 1 << 58


class _RowsEven:
    """The header's DLSPM_HINT_ROWS_EVEN: passed as `workspace`, it tells the library that no row is much longer than
    the mean (at most 1.5 x nnz / M); it stands for no memory (a NULL workspace with the hint bit in its size)."""

    def __repr__(self):
        return "ROWS_EVEN"


ROWS_EVEN = _RowsEven()


class _RowsSkewed:
    """The header's DLSPM_HINT_ROWS_SKEWED without a plan: passed as `workspace`, it tells the library that long rows lie
    next to each other (what dlspm_advise says where one eighth of the rows holds 1.6 times its share of the nonzeros);
    no memory."""

    def __repr__(self):
        return "ROWS_SKEWED"


ROWS_SKEWED = _RowsSkewed()

EXPORTS = (
    "spmm_csr_f32",
    "sddmm_csr_f32",
    "fused_sddmm_spmm_f32",
    "dlspm_workspace_bytes",
    "dlspm_csr_check",
    "dlspm_describe_launch",
    "dlspm_describe_launch_rows",
    "dlspm_describe_slices",
    "dlspm_workspace_advice",
    "dlspm_csr_row_stats",
    "dlspm_row_plan_bytes",
    "dlspm_row_plan_advice",
    "dlspm_row_plan_build",
    "dlspm_row_plan_bytes_for",
    "dlspm_analyze",
    "dlspm_advise",
    "dlspm_row_plan_build_cut",
    "dlspm_tuning_default",
    "dlspm_set_tuning",
    "dlspm_get_tuning",
    "dlspm_device_info",
    "spmm_csr_f32_static",
    "dlspm_static_scratch_bytes",
    "dlspm_status_string",
    "dlspm_last_hip_error",
    "dlspm_version",
)


class Tuning(ctypes.Structure):
    """dlspm_tuning of include/dlspm_hip.h."""
    _fields_ = [(n, ctypes.c_int) for n in ("split_w", "split_r", "flat", "flat_chunk", "slices", "tile_major",
                                            "tile_width", "plan_order", "xcd_contiguous", "stream_results",
                                            "cut_piece_pct", "cut_longest_pct", "rules_off", "compute_units")]

RULES = {"eight_waves_few_rows": 1, "sixteen_waves_tall_long_rows": 2, "more_waves_few_long_rows": 4, "group_rows": 8,
         "row_aligned_split": 16, "plan_ungroups": 32, "exact_width_kernels": 64, "cut_rows_by_columns": 128,
         "finer_column_tiles": 256, "row_pieces_few_rows": 512, "mask_by_range": 1024}


class MatrixInfo(ctypes.Structure):
    """dlspm_matrix_info of include/dlspm_hip.h."""
    _fields_ = [(n, ctypes.c_int) for n in ("M", "K", "nnz", "max_row_len", "empty_rows", "max_col_span",
                                            "eighths_cover_permille", "eighths_nnz_permille")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


class CallPlan(ctypes.Structure):
    """dlspm_call_plan of include/dlspm_hip.h."""
    _fields_ = [("build", ctypes.c_int), ("bytes", ctypes.c_size_t), ("hints", ctypes.c_size_t)]


BUILD_NOTHING, BUILD_ROW_PLAN, BUILD_CUT_PLAN = 0, 1, 2


class DlspmError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        super().__init__(f"{where}: status {status} ({status_string(status)}), hip error {lib().dlspm_last_hip_error()}")


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded libdlspm_hip.so. Raises if it has not been built (run `make -C dlspm-esimd_amd lib`)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is missing: build it with `make -C {_HERE} lib` (hipcc, gfx950)")
        L = ctypes.CDLL(LIB_PATH)
        vp, ci, cf, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
        L.spmm_csr_f32.argtypes = [ci, ci, ci, ci, vp, vp, vp, vp, vp, vp, sz, vp]
        L.spmm_csr_f32.restype = ci
        L.sddmm_csr_f32.argtypes = [ci, ci, ci, ci, vp, vp, vp, vp, vp, vp, sz, vp]
        L.sddmm_csr_f32.restype = ci
        L.fused_sddmm_spmm_f32.argtypes = [ci, ci, ci, ci, vp, vp, vp, vp, vp, cf, vp, vp, sz, vp]
        L.fused_sddmm_spmm_f32.restype = ci
        L.dlspm_workspace_bytes.argtypes = [ci, ci, ci, ci, ci]
        L.dlspm_workspace_bytes.restype = sz
        L.dlspm_csr_check.argtypes = [ci, ci, ci, vp, vp, vp]
        L.dlspm_csr_check.restype = ci
        L.dlspm_describe_launch.argtypes = [ci, ci, ci, ci, ci, ctypes.POINTER(ci)]
        L.dlspm_describe_launch_rows.argtypes = [ci, ci, ci, ci, ci, ci, ctypes.POINTER(ci)]
        L.dlspm_describe_launch_rows.restype = ci
        L.dlspm_describe_slices.argtypes = [ci, ci, ci, ci, ci, ctypes.POINTER(ci), ctypes.POINTER(ci)]
        L.dlspm_describe_slices.restype = ci
        L.dlspm_workspace_advice.argtypes = [ci, ci, ci, ci, ci, ci]
        L.dlspm_workspace_advice.restype = ci
        L.dlspm_describe_launch.restype = ci
        L.dlspm_csr_row_stats.argtypes = [ci, vp, vp, ctypes.POINTER(ci), ctypes.POINTER(ci)]
        L.dlspm_csr_row_stats.restype = ci
        L.dlspm_row_plan_bytes.argtypes = [ci]
        L.dlspm_row_plan_bytes.restype = sz
        L.dlspm_row_plan_advice.argtypes = [ci, ci, ci, ci, ci, ci]
        L.dlspm_row_plan_advice.restype = ci
        L.dlspm_row_plan_build.argtypes = [ci, vp, vp, sz, vp]
        L.dlspm_row_plan_build.restype = ci
        L.dlspm_row_plan_bytes_for.argtypes = [ci, ci, ci]
        L.dlspm_row_plan_bytes_for.restype = sz
        L.dlspm_row_plan_build_cut.argtypes = [ci, vp, vp, sz, vp]
        L.dlspm_row_plan_build_cut.restype = ci
        L.dlspm_analyze.argtypes = [ci, ci, ci, vp, vp, vp, ctypes.POINTER(MatrixInfo)]
        L.dlspm_analyze.restype = ci
        L.dlspm_advise.argtypes = [ci, ci, ctypes.POINTER(MatrixInfo), ctypes.POINTER(CallPlan)]
        L.dlspm_advise.restype = ci
        L.spmm_csr_f32_static.argtypes = [ci, ci, ci, ci, vp, vp, vp, vp, vp, vp]
        L.spmm_csr_f32_static.restype = ci
        L.dlspm_static_scratch_bytes.restype = sz
        L.dlspm_tuning_default.argtypes = [ctypes.POINTER(Tuning)]
        L.dlspm_tuning_default.restype = None
        L.dlspm_set_tuning.argtypes = [ctypes.POINTER(Tuning)]
        L.dlspm_set_tuning.restype = ci
        L.dlspm_get_tuning.argtypes = [ctypes.POINTER(Tuning)]
        L.dlspm_get_tuning.restype = ci
        L.dlspm_device_info.argtypes = [ctypes.POINTER(ci), ctypes.POINTER(ctypes.c_longlong), ctypes.POINTER(ci)]
        L.dlspm_device_info.restype = ci
        L.dlspm_status_string.argtypes = [ci]
        L.dlspm_status_string.restype = ctypes.c_char_p
        L.dlspm_last_hip_error.restype = ci
        L.dlspm_version.restype = ctypes.c_char_p
        _lib = L
    return _lib


def status_string(status: int) -> str:
    return lib().dlspm_status_string(status).decode()


def version() -> str:
    return lib().dlspm_version().decode()


def set_tuning(**fields) -> None:
    """Overrides of the launch rules for the calling thread (dlspm_set_tuning): split=(W, R), flat, flat_chunk, slices,
    tile_major, tile_width, plan_order, xcd_contiguous, stream_results; fields not named follow the rules. No argument: back to the process default."""
    if not fields:
        st = lib().dlspm_set_tuning(None)
    else:
        t = Tuning()
        lib().dlspm_tuning_default(ctypes.byref(t))
        if "split" in fields:
            t.split_w, t.split_r = fields.pop("split")
        for k, v in fields.items():
            if not hasattr(t, k):
                raise TypeError(f"dlspm_tuning has no field {k}")
            setattr(t, k, int(v))
        st = lib().dlspm_set_tuning(ctypes.byref(t))
    if st != OK:
        raise DlspmError(st, "dlspm_set_tuning")


def get_tuning() -> dict:
    t = Tuning()
    lib().dlspm_get_tuning(ctypes.byref(t))
    return {n: getattr(t, n) for n, _ in Tuning._fields_}


def device_info() -> dict:
    """{'status', 'compute_units', 'l2_bytes', 'gfx950'} of the current device as the library sees it."""
    cu, l2, ok = ctypes.c_int(0), ctypes.c_longlong(0), ctypes.c_int(0)
    st = lib().dlspm_device_info(ctypes.byref(cu), ctypes.byref(l2), ctypes.byref(ok))
    return {"status": st, "compute_units": cu.value, "l2_bytes": l2.value, "gfx950": bool(ok.value)}


def _ptr(t, dtype, name, numel=None):
    """Device pointer of tensor t after checking where it lives, its type, its layout and (numel) that it holds at
    least that many elements: a size mismatch must be a Python exception, not an out-of-bounds access on the device."""
    import torch

    if t is None:
        return None
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous (row-major)")
    if numel is not None and t.numel() < numel:
        raise ValueError(f"{name} holds {t.numel()} elements, the call needs {numel}")
    return ctypes.c_void_p(t.data_ptr()) if t.numel() > 0 else None


def _stream():
    import torch

    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def row_plan_advice(op, M, K, N_or_D, nnz, max_row_len=-1) -> int:
    """Whether a row plan is worth building for op at these sizes (dlspm_row_plan_advice): 0 no, 1 a plan over whole rows
    (row_plan), 2 a plan that cuts the longest rows (cut_plan)."""
    return int(lib().dlspm_row_plan_advice(op, M, K, N_or_D, nnz, max_row_len))


def row_plan_bytes(M: int) -> int:
    return int(lib().dlspm_row_plan_bytes(M))


def row_plan(row_offsets, out=None):
    """The row plan of one matrix (an int32 GPU tensor of row_plan_bytes(M) / 4 entries; the launches read the first
    3 * M) for spmm / sddmm / fused(..., plan=...). Built by kernels on the current stream: no synchronisation.
    `out`: a tensor to build into (callers under graph capture)."""
    import torch

    M = row_offsets.numel() - 1
    need = row_plan_bytes(M) // 4
    plan = out if out is not None else torch.empty((need,), dtype=torch.int32, device=row_offsets.device)
    st = lib().dlspm_row_plan_build(M, _ptr(row_offsets, torch.int32, "row_offsets", M + 1), _ptr(plan, torch.int32, "plan", need),
                                    plan.numel() * 4, _stream())
    if st != OK:
        raise DlspmError(st, "dlspm_row_plan_build")
    return plan


class CutPlan:
    """A row plan that cuts rows longer than one compute unit's share of the nonzeros into pieces (cut_plan()): the
    device memory, and the op and width it has room for."""

    def __init__(self, memory, op, width):
        self.memory, self.op, self.width = memory, op, width


def row_plan_bytes_for(op: int, M: int, width: int) -> int:
    return int(lib().dlspm_row_plan_bytes_for(op, M, width))


def cut_plan(row_offsets, op, width, out=None) -> CutPlan:
    """The cut plan of one matrix for op at dense width `width` (dlspm_row_plan_build_cut into
    dlspm_row_plan_bytes_for(op, M, width) bytes), built by kernels on the current stream. Pass it as plan=... ."""
    import torch

    M = row_offsets.numel() - 1
    need = (row_plan_bytes_for(op, M, width) + 3) // 4
    if need == 0:
        raise ValueError(f"no cut plan for a matrix of {M} rows")
    mem = out if out is not None else torch.empty((need,), dtype=torch.int32, device=row_offsets.device)
    st = lib().dlspm_row_plan_build_cut(M, _ptr(row_offsets, torch.int32, "row_offsets", M + 1), _ptr(mem, torch.int32, "plan", need),
                                        mem.numel() * 4, _stream())
    if st != OK:
        raise DlspmError(st, "dlspm_row_plan_build_cut")
    return CutPlan(mem, op, width)


def analyze(row_offsets, col_indices, K) -> MatrixInfo:
    """dlspm_analyze: one synchronising pass over the CSR structure on the GPU."""
    import torch

    M, nnz = row_offsets.numel() - 1, col_indices.numel()
    info = MatrixInfo()
    st = lib().dlspm_analyze(M, K, nnz, _ptr(row_offsets, torch.int32, "row_offsets", M + 1),
                             _ptr(col_indices, torch.int32, "col_indices"), _stream(), ctypes.byref(info))
    if st != OK:
        raise DlspmError(st, "dlspm_analyze")
    return info


def advise(op, width, info: MatrixInfo) -> CallPlan:
    """dlspm_advise (host only): what to allocate, build and hint for op at this dense width."""
    cp = CallPlan()
    st = lib().dlspm_advise(op, width, ctypes.byref(info), ctypes.byref(cp))
    if st != OK:
        raise DlspmError(st, "dlspm_advise")
    return cp


class Prepared:
    """What dlspm_advise said for one matrix, op and width, allocated and built (prepare()): pass as prepared=... ."""

    def __init__(self, memory, size_and_hints, call_plan):
        self.memory, self.size_and_hints, self.call_plan = memory, size_and_hints, call_plan


def prepare(row_offsets, col_indices, K, op, width, info=None) -> Prepared:
    """The lead path of a caller: dlspm_analyze (unless `info` is given) -> dlspm_advise -> allocate -> build."""
    import torch

    info = info if info is not None else analyze(row_offsets, col_indices, K)
    cp = advise(op, width, info)
    M = row_offsets.numel() - 1
    mem = torch.empty(((cp.bytes + 3) // 4,), dtype=torch.int32, device=row_offsets.device) if cp.bytes else None
    if cp.build == BUILD_ROW_PLAN:
        st = lib().dlspm_row_plan_build(M, _ptr(row_offsets, torch.int32, "row_offsets", M + 1), ctypes.c_void_p(mem.data_ptr()),
                                        mem.numel() * 4, _stream())
    elif cp.build == BUILD_CUT_PLAN:
        st = lib().dlspm_row_plan_build_cut(M, _ptr(row_offsets, torch.int32, "row_offsets", M + 1), ctypes.c_void_p(mem.data_ptr()),
                                            mem.numel() * 4, _stream())
    else:
        st = OK
    if st != OK:
        raise DlspmError(st, "dlspm_row_plan_build")
    return Prepared(mem, (mem.numel() * 4 if mem is not None else 0) | cp.hints, cp)


def _csr_sizes(row_offsets, col_indices):
    if row_offsets.numel() < 1:
        raise ValueError("row_offsets must hold M + 1 >= 1 entries")
    return row_offsets.numel() - 1, col_indices.numel()


def _workspace_args(workspace, plan, M, banded=False):
    """(pointer, size with hint bits) for the pair (workspace, workspace_bytes) of the three compute entry points.
    banded: the caller knows that every row's columns lie in a narrow window that moves with the row (DLSPM_HINT_BANDED)."""
    import torch

    hint = HINT_BANDED if banded else 0
    if isinstance(plan, Prepared):
        if workspace is not None:
            raise ValueError("pass what prepare() returned or a workspace, not both")
        return (ctypes.c_void_p(plan.memory.data_ptr()) if plan.memory is not None else None), plan.size_and_hints | hint
    if isinstance(plan, CutPlan):
        if workspace is not None:
            raise ValueError("pass a row plan or a workspace, not both")
        return _ptr(plan.memory, torch.int32, "plan"), (plan.memory.numel() * 4) | HINT_CUT_PLAN | hint
    if plan is not None:
        if workspace is not None:
            raise ValueError("pass a row plan or a workspace, not both")
        need = row_plan_bytes(M) // 4
        return _ptr(plan, torch.int32, "plan", need), (plan.numel() * 4) | HINT_ROW_PLAN | hint
    pointer, size = _workspace(workspace)
    return pointer, size | hint


def spmm(row_offsets, col_indices, values, B, K=None, out=None, workspace=None, plan=None, banded=False):
    """C = A_csr @ B on the current stream (spmm_csr_f32). row_offsets/col_indices int32, values/B float32, all on
    the GPU. `workspace`: optional GPU tensor of at least workspace_bytes(OP_SPMM, ...) bytes, or ROWS_EVEN.
    `plan`: optional row plan of this matrix (row_plan()), passed as the workspace with DLSPM_HINT_ROW_PLAN.
    `banded`: every row's columns lie in a narrow window that moves with the row (DLSPM_HINT_BANDED)."""
    import torch

    M, nnz = _csr_sizes(row_offsets, col_indices)
    if B.dim() != 2:
        raise ValueError("B must be a K x N matrix")
    Kd, N = B.shape
    K = Kd if K is None else K
    if K > Kd:
        raise ValueError(f"B has {Kd} rows, the matrix has K = {K} columns")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=B.device)
    wp, wb = _workspace_args(workspace, plan, M, banded)
    st = lib().spmm_csr_f32(M, K, N, nnz, _ptr(row_offsets, torch.int32, "row_offsets"),
                            _ptr(col_indices, torch.int32, "col_indices"), _ptr(values, torch.float32, "values", nnz),
                            _ptr(B, torch.float32, "B"), _ptr(out, torch.float32, "C", M * N), wp, wb, _stream())
    if st != OK:
        raise DlspmError(st, "spmm_csr_f32")
    return out


def static_scratch_bytes() -> int:
    """Size of the library-held scratch array that spmm_static() works in (per GPU)."""
    return int(lib().dlspm_static_scratch_bytes())


def spmm_static(row_offsets, col_indices, values, B, K=None, out=None):
    """spmm() through spmm_csr_f32_static: the schedule of a call with workspace, in the library's own static scratch
    array; allocates nothing inside the library. `out` must be given by callers that may not allocate either."""
    import torch

    M, nnz = _csr_sizes(row_offsets, col_indices)
    Kd, N = B.shape
    K = Kd if K is None else K
    if K > Kd:
        raise ValueError(f"B has {Kd} rows, the matrix has K = {K} columns")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=B.device)
    st = lib().spmm_csr_f32_static(M, K, N, nnz, _ptr(row_offsets, torch.int32, "row_offsets"),
                                   _ptr(col_indices, torch.int32, "col_indices"), _ptr(values, torch.float32, "values", nnz),
                                   _ptr(B, torch.float32, "B"), _ptr(out, torch.float32, "C", M * N), _stream())
    if st != OK:
        raise DlspmError(st, "spmm_csr_f32_static")
    return out


def sddmm(row_offsets, col_indices, lhs, rhs, out=None, workspace=None, plan=None, banded=False):
    """out[j] = <lhs[i], rhs[col[j]]> for each CSR slot j of row i, on the current stream (sddmm_csr_f32).
    `workspace`: None, ROWS_EVEN, or a GPU tensor of workspace_bytes(OP_SDDMM, ...) bytes (the slice boundaries of the
    column-sliced schedule; 0 bytes where that schedule does not apply). `plan`: a row plan of the mask instead."""
    import torch

    M, nnz = _csr_sizes(row_offsets, col_indices)
    if lhs.dim() != 2 or rhs.dim() != 2 or lhs.shape[1] != rhs.shape[1]:
        raise ValueError("lhs must be M x D and rhs K x D")
    K, D = rhs.shape
    if lhs.shape[0] < M:
        raise ValueError(f"lhs has {lhs.shape[0]} rows, the mask has {M}")
    if out is None:
        out = torch.empty((nnz,), dtype=torch.float32, device=lhs.device)
    wp, wb = _workspace_args(workspace, plan, M, banded)
    st = lib().sddmm_csr_f32(M, K, D, nnz, _ptr(row_offsets, torch.int32, "row_offsets"),
                             _ptr(col_indices, torch.int32, "col_indices"), _ptr(lhs, torch.float32, "lhs"),
                             _ptr(rhs, torch.float32, "rhs"), _ptr(out, torch.float32, "out", nnz), wp, wb, _stream())
    if st != OK:
        raise DlspmError(st, "sddmm_csr_f32")
    return out


def fused(row_offsets, col_indices, Q, Kmat, V, scale=1.0, out=None, workspace=None, plan=None, banded=False):
    """O = (S .* (Q Kmat^T) * scale) V on the current stream (fused_sddmm_spmm_f32); the scores are never stored.
    `workspace`: optional GPU tensor of at least workspace_bytes(OP_FUSED, ...) bytes, or ROWS_EVEN.
    `plan`: optional row plan of the mask (row_plan()), passed as the workspace with DLSPM_HINT_ROW_PLAN."""
    import torch

    M, nnz = _csr_sizes(row_offsets, col_indices)
    if Q.dim() != 2 or Kmat.dim() != 2 or V.shape != Kmat.shape or Q.shape[1] != Kmat.shape[1]:
        raise ValueError("Q must be M x D, Kmat and V K x D")
    K, D = Kmat.shape
    if Q.shape[0] < M:
        raise ValueError(f"Q has {Q.shape[0]} rows, the mask has {M}")
    if out is None:
        out = torch.empty((M, D), dtype=torch.float32, device=Q.device)
    wp, wb = _workspace_args(workspace, plan, M, banded)
    st = lib().fused_sddmm_spmm_f32(M, K, D, nnz, _ptr(row_offsets, torch.int32, "row_offsets"),
                                    _ptr(col_indices, torch.int32, "col_indices"), _ptr(Q, torch.float32, "Q"),
                                    _ptr(Kmat, torch.float32, "Kmat"), _ptr(V, torch.float32, "V"),
                                    ctypes.c_float(scale), _ptr(out, torch.float32, "O", M * D), wp, wb, _stream())
    if st != OK:
        raise DlspmError(st, "fused_sddmm_spmm_f32")
    return out


def describe_launch(op: int, M: int, K: int, N: int, nnz: int, rows_even: bool = False,
                    with_workspace: bool = False, rows_skewed: bool = False) -> dict:
    """Launch shape the library uses for these sizes: {'vec','G','V','G1','DS','W','R','col_tiles','flat_chunk',
    'flat_units'} (host only). rows_even: for a call that passes ROWS_EVEN; with_workspace: for one that passes
    workspace memory; neither: for one that passes None."""
    out = (ctypes.c_int * 10)()
    passing = PASS_WORKSPACE if with_workspace else PASS_ROWS_EVEN if rows_even else PASS_ROWS_SKEWED if rows_skewed else PASS_NULL
    st = lib().dlspm_describe_launch_rows(op, M, K, N, nnz, passing, out)
    if st != OK:
        raise DlspmError(st, "dlspm_describe_launch")
    return dict(zip(("vec", "G", "V", "G1", "DS", "W", "R", "col_tiles", "flat_chunk", "flat_units"),
                    (int(x) for x in out)))


def describe_slices(op: int, M: int, K: int, N: int, nnz: int) -> tuple:
    """(slices, rows per workgroup) of the column-sliced schedule a call with workspace would use; slices == 0: none."""
    a, b = ctypes.c_int(0), ctypes.c_int(0)
    st = lib().dlspm_describe_slices(op, M, K, N, nnz, ctypes.byref(a), ctypes.byref(b))
    if st != OK:
        raise DlspmError(st, "dlspm_describe_slices")
    return a.value, b.value


PASS_NULL, PASS_ROWS_EVEN, PASS_WORKSPACE, PASS_ROWS_SKEWED = 0, 1, 2, 3


def workspace_advice(op: int, M: int, K: int, N: int, nnz: int, max_row_len: int = -1) -> int:
    """What to pass as `workspace` (PASS_NULL / PASS_ROWS_EVEN / PASS_WORKSPACE) given the longest row (-1: unknown)."""
    return int(lib().dlspm_workspace_advice(op, M, K, N, nnz, max_row_len))


def workspace_bytes(op: int, M: int, K: int, N: int, nnz: int) -> int:
    """Bytes of device workspace the op can use for these sizes (0 = none)."""
    return int(lib().dlspm_workspace_bytes(op, M, K, N, nnz))


def _workspace(ws):
    """(pointer, bytes) of an optional workspace tensor (any dtype, contiguous, on the GPU)."""
    if ws is None:
        return None, 0
    if ws is ROWS_EVEN:
        return None, HINT_ROWS_EVEN
    if ws is ROWS_SKEWED:
        return None, HINT_ROWS_SKEWED
    if not ws.is_cuda or not ws.is_contiguous():
        raise ValueError("workspace must be a contiguous GPU tensor")
    return ctypes.c_void_p(ws.data_ptr()), ws.numel() * ws.element_size()


def csr_row_stats(row_offsets):
    """(longest row, rows without nonzeros) of a CSR structure on the GPU; synchronises the current stream."""
    import torch

    mx, em = ctypes.c_int(0), ctypes.c_int(0)
    st = lib().dlspm_csr_row_stats(row_offsets.numel() - 1, _ptr(row_offsets, torch.int32, "row_offsets"), _stream(),
                                   ctypes.byref(mx), ctypes.byref(em))
    if st != OK:
        raise DlspmError(st, "dlspm_csr_row_stats")
    return mx.value, em.value


def csr_check(M, K, row_offsets, col_indices) -> int:
    """Status of the device-side CSR check (OK or E_INVALID_CSR); synchronises the current stream."""
    import torch

    nnz = col_indices.numel()
    return int(lib().dlspm_csr_check(M, K, nnz, _ptr(row_offsets, torch.int32, "row_offsets"),
                                     _ptr(col_indices, torch.int32, "col_indices"), _stream()))


# ------------------------------------------------------------------------------------------------------
# seeded inputs (libdlspm_gen.so): the same generators the C++ drivers use
# ------------------------------------------------------------------------------------------------------
_gen = None


def gen_lib() -> ctypes.CDLL:
    global _gen
    if _gen is None:
        if not os.path.exists(GEN_LIB_PATH):
            raise FileNotFoundError(f"{GEN_LIB_PATH} is missing: build it with `make -C {_HERE} gen`")
        G = ctypes.CDLL(GEN_LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        G.dlspm_gen_config_create.argtypes = [ci]
        G.dlspm_gen_config_create.restype = vp
        G.dlspm_gen_config_destroy.argtypes = [vp]
        G.dlspm_gen_config_dims.argtypes = [vp, ctypes.POINTER(ci), ctypes.POINTER(ctypes.c_float)]
        G.dlspm_gen_config_name.argtypes = [ci]
        G.dlspm_gen_config_name.restype = ctypes.c_char_p
        for f in ("row_offsets", "col_indices", "values"):
            getattr(G, "dlspm_gen_config_" + f).argtypes = [vp]
            getattr(G, "dlspm_gen_config_" + f).restype = vp
        G.dlspm_gen_config_dense.argtypes = [vp, ci, ctypes.POINTER(ctypes.c_size_t)]
        G.dlspm_gen_config_dense.restype = vp
        G.dlspm_gen_pattern_create.argtypes = [ci, ctypes.c_uint64, ci, ci, ctypes.c_double, ctypes.c_double]
        G.dlspm_gen_pattern_create.restype = vp
        G.dlspm_gen_pattern_destroy.argtypes = [vp]
        G.dlspm_gen_pattern_nnz.argtypes = [vp]
        G.dlspm_gen_pattern_nnz.restype = ci
        G.dlspm_gen_pattern_copy.argtypes = [vp, vp, vp]
        G.dlspm_gen_fill_uniform.argtypes = [ctypes.c_uint64, ctypes.c_size_t, ctypes.c_float, ctypes.c_float, vp]
        G.dlspm_gen_fill_normal.argtypes = [ctypes.c_uint64, ctypes.c_size_t, ctypes.c_float, ctypes.c_float, vp]
        G.dlspm_gen_fill_relu_like.argtypes = [ctypes.c_uint64, ctypes.c_size_t, ctypes.c_double, vp]
        G.dlspm_account.argtypes = [ci] + [ctypes.c_double] * 4 + [ctypes.POINTER(ctypes.c_double)]
        _gen = G
    return _gen


PATTERN_UNIFORM_ROWS, PATTERN_LOGNORMAL_ROWS, PATTERN_BERNOULLI, PATTERN_BAND_RANDOM = 0, 1, 2, 3


def make_pattern(kind: int, seed: int, M: int, K: int, p0: float, p1: float = 0.0):
    """(row_offsets, col_indices) as numpy int32 arrays from one of the seeded pattern generators."""
    import numpy as np

    G = gen_lib()
    h = G.dlspm_gen_pattern_create(kind, seed, M, K, p0, p1)
    if not h:
        raise ValueError(f"unknown pattern kind {kind}")
    try:
        nnz = G.dlspm_gen_pattern_nnz(h)
        ro = np.empty(M + 1, dtype=np.int32)
        ci = np.empty(max(nnz, 1), dtype=np.int32)
        G.dlspm_gen_pattern_copy(h, ro.ctypes.data, ci.ctypes.data)
        return ro, ci[:nnz]
    finally:
        G.dlspm_gen_pattern_destroy(h)


def fill(kind: str, seed: int, shape, a: float = 0.0, b: float = 1.0):
    """Seeded float32 numpy array: kind 'uniform' (a = lo, b = hi), 'normal' (a = mean, b = std), 'relu' (a = p_zero)."""
    import numpy as np

    G = gen_lib()
    out = np.empty(shape, dtype=np.float32)
    if kind == "uniform":
        G.dlspm_gen_fill_uniform(seed, out.size, a, b, out.ctypes.data)
    elif kind == "normal":
        G.dlspm_gen_fill_normal(seed, out.size, a, b, out.ctypes.data)
    elif kind == "relu":
        G.dlspm_gen_fill_relu_like(seed, out.size, a, out.ctypes.data)
    else:
        raise ValueError(kind)
    return out


def make_config(cfg: int) -> dict:
    """Benchmark configuration cfg (1..5) as numpy arrays:
    {'cfg','name','op','M','K','N','nnz','scale','row_offsets','col_indices','values','d0','d1','d2'}."""
    import numpy as np

    G = gen_lib()
    h = G.dlspm_gen_config_create(cfg)
    if not h:
        raise ValueError(f"unknown configuration {cfg}")
    try:
        dims = (ctypes.c_int * 5)()
        scale = ctypes.c_float()
        G.dlspm_gen_config_dims(h, dims, ctypes.byref(scale))
        op, M, K, N, nnz = (int(x) for x in dims)

        def arr(ptr, n, dtype):
            if n == 0 or not ptr:
                return np.empty(0, dtype=dtype)
            ctype = ctypes.c_int if dtype == np.int32 else ctypes.c_float
            return np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(ctype)), shape=(n,)).copy()

        out = {
            "cfg": cfg, "name": G.dlspm_gen_config_name(cfg).decode(), "op": op, "M": M, "K": K, "N": N, "nnz": nnz,
            "scale": float(scale.value),
            "row_offsets": arr(G.dlspm_gen_config_row_offsets(h), M + 1, np.int32),
            "col_indices": arr(G.dlspm_gen_config_col_indices(h), nnz, np.int32),
            "values": arr(G.dlspm_gen_config_values(h), nnz if op == OP_SPMM else 0, np.float32),
        }
        for which in range(3):
            cnt = ctypes.c_size_t()
            p = G.dlspm_gen_config_dense(h, which, ctypes.byref(cnt))
            out[f"d{which}"] = arr(p, int(cnt.value), np.float32)
        rows = {OP_SPMM: (K, None, None), OP_SDDMM: (M, K, None), OP_FUSED: (M, K, K)}[op]
        for which, r in enumerate(rows):
            if r is not None:
                out[f"d{which}"] = out[f"d{which}"].reshape(r, N)
        return out
    finally:
        G.dlspm_gen_config_destroy(h)


def account(op: int, M: int, K: int, N: int, nnz: int) -> dict:
    """{'flops', 'algorithmic_bytes', 'effective_bytes'} for one launch (the reference's flop formulas; bytes as
    every operand once / every gathered dense row counted)."""
    out = (ctypes.c_double * 3)()
    gen_lib().dlspm_account(op, float(M), float(K), float(N), float(nnz), out)
    return {"flops": out[0], "algorithmic_bytes": out[1], "effective_bytes": out[2]}
