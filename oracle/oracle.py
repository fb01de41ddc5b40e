"""ctypes front end of the CPU oracle (oracle/libdlspm_oracle.so) and of the reference-built
checker objects under oracle/_ref/.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the CPU-baseline leg of bench.py.
The library and its host-side wrappers never import this module.

Every function takes and returns numpy arrays (int32 CSR arrays, float32 dense arrays, C order).
"""
from __future__ import annotations

import ctypes
import glob
import os
import re
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdlspm_oracle.so")
_REF_DIR = os.path.join(_HERE, "_ref")

_i32p = ctypes.POINTER(ctypes.c_int)
_f32p = ctypes.POINTER(ctypes.c_float)


def build(with_ref: bool = True) -> None:
    """Compile the oracle (and oracle/_ref when the reference tree is mounted) with oracle/Makefile."""
    target = ["all"] if with_ref else ["libdlspm_oracle.so"]
    subprocess.run(["make", "-s", "-C", _HERE] + target, check=True)


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build(with_ref=False)
        _lib = ctypes.CDLL(_LIB_PATH)
        csr = [_i32p, _i32p]
        for suffix in ("", "_omp"):
            getattr(_lib, "oracle_spmm_f32" + suffix).argtypes = [ctypes.c_int, ctypes.c_int] + csr + [_f32p, _f32p, _f32p]
            getattr(_lib, "oracle_spmm_f64acc" + suffix).argtypes = [ctypes.c_int, ctypes.c_int] + csr + [_f32p, _f32p, _f32p]
            getattr(_lib, "oracle_sddmm_f32" + suffix).argtypes = [ctypes.c_int, ctypes.c_int] + csr + [_f32p, _f32p, _f32p]
            getattr(_lib, "oracle_fused_f32" + suffix).argtypes = (
                [ctypes.c_int, ctypes.c_int] + csr + [_f32p, _f32p, _f32p, ctypes.c_float, _f32p, _f32p])
            for name in ("oracle_spmm_f32", "oracle_spmm_f64acc", "oracle_sddmm_f32", "oracle_fused_f32"):
                getattr(_lib, name + suffix).restype = None
        _lib.oracle_csr_check.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p, _i32p]
        _lib.oracle_csr_check.restype = ctypes.c_int
        _lib.oracle_omp_threads.restype = ctypes.c_int
    return _lib


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _pi(a: np.ndarray):
    return a.ctypes.data_as(_i32p)


def _pf(a: np.ndarray):
    return a.ctypes.data_as(_f32p)


def spmm(row_offsets, col_indices, values, B, *, acc: str = "f32", omp: bool = False) -> np.ndarray:
    """C = A_csr @ B with the reference's float (acc='f32') or double (acc='f64') accumulator."""
    ro, ci, va, B = _i32(row_offsets), _i32(col_indices), _f32(values), _f32(B)
    M, N = ro.size - 1, B.shape[1]
    C = np.empty((M, N), dtype=np.float32)
    name = ("oracle_spmm_f32" if acc == "f32" else "oracle_spmm_f64acc") + ("_omp" if omp else "")
    getattr(lib(), name)(M, N, _pi(ro), _pi(ci), _pf(va), _pf(B), _pf(C))
    return C


def sddmm(row_offsets, col_indices, lhs, rhs, *, omp: bool = False) -> np.ndarray:
    """out[j] = <lhs[i], rhs[col[j]]> for each CSR slot j of row i (double accumulator)."""
    ro, ci, lhs, rhs = _i32(row_offsets), _i32(col_indices), _f32(lhs), _f32(rhs)
    M, D = ro.size - 1, lhs.shape[1]
    out = np.empty(int(ro[-1]), dtype=np.float32)
    getattr(lib(), "oracle_sddmm_f32" + ("_omp" if omp else ""))(M, D, _pi(ro), _pi(ci), _pf(lhs), _pf(rhs), _pf(out))
    return out


def fused(row_offsets, col_indices, Q, Kmat, V, scale: float = 1.0, *, omp: bool = False,
          return_scores: bool = False):
    """O = (S .* (Q Kmat^T) * scale) V, fp32 scores between the two stages."""
    ro, ci, Q, Kmat, V = _i32(row_offsets), _i32(col_indices), _f32(Q), _f32(Kmat), _f32(V)
    M, D = ro.size - 1, Q.shape[1]
    scores = np.empty(max(int(ro[-1]), 1), dtype=np.float32)
    O = np.empty((M, D), dtype=np.float32)
    getattr(lib(), "oracle_fused_f32" + ("_omp" if omp else ""))(
        M, D, _pi(ro), _pi(ci), _pf(Q), _pf(Kmat), _pf(V), ctypes.c_float(scale), _pf(scores), _pf(O))
    return (O, scores[: int(ro[-1])]) if return_scores else O


def csr_check(M: int, K: int, nnz: int, row_offsets, col_indices) -> int:
    ro, ci = _i32(row_offsets), _i32(col_indices)
    if ci.size == 0:
        ci = np.zeros(1, dtype=np.int32)
    return int(lib().oracle_csr_check(M, K, nnz, _pi(ro), _pi(ci)))


def omp_threads() -> int:
    return int(lib().oracle_omp_threads())


# ----------------------------------------------------------------------------------------------
# error metrics used by every parity test
# ----------------------------------------------------------------------------------------------

def rel_frobenius(x, x_ref) -> float:
    """||x - x_ref||_F / ||x_ref||_F in float64 (0 when both are all-zero)."""
    x = np.asarray(x, dtype=np.float64).ravel()
    r = np.asarray(x_ref, dtype=np.float64).ravel()
    den = np.linalg.norm(r)
    num = np.linalg.norm(x - r)
    if den == 0.0:
        return 0.0 if num == 0.0 else float("inf")
    return float(num / den)


# ----------------------------------------------------------------------------------------------
# the reference's own gold loops, compiled from FUSED/fused.cpp at fixed shapes (oracle/_ref)
# ----------------------------------------------------------------------------------------------

class RefFused:
    """One shape-specialised build of the reference's FUSED/fused.cpp (M, K, D fixed at compile time).

    Sddmm            FUSED/fused.cpp:47-65    double accumulate
    Spmm             FUSED/fused.cpp:67-89    double accumulate
    FusedEsimdCPU    FUSED/fused.cpp:93-216   fp32 emulation of the fused kernel's 32-wide chunks
    SpmmEsimdCPU     FUSED/fused.cpp:218-303  fp32 emulation of the SpMM kernel; per output element it
                     performs the same fp32 operation sequence as the float-accumulating Spmm of
                     SPMM/spmm-esimd-fromfile.cpp:63-83
    """

    def __init__(self, path: str):
        m = re.search(r"fused_ref_M(\d+)_K(\d+)_N(\d+)\.so$", path)
        if not m:
            raise ValueError(path)
        self.M, self.K, self.D = (int(g) for g in m.groups())
        self._lib = ctypes.CDLL(path)
        self._sddmm = getattr(self._lib, "_Z5SddmmPKiS0_PKfS2_Pf")
        self._sddmm.argtypes = [_i32p, _i32p, _f32p, _f32p, _f32p]
        self._spmm = getattr(self._lib, "_Z4SpmmPKfPKiS2_S0_Pf")
        self._spmm.argtypes = [_f32p, _i32p, _i32p, _f32p, _f32p]
        self._fused_emul = getattr(self._lib, "_Z13FusedEsimdCPUPKiS0_PKfS2_S2_Pf")
        self._fused_emul.argtypes = [_i32p, _i32p, _f32p, _f32p, _f32p, _f32p]
        self._spmm_emul = getattr(self._lib, "_Z12SpmmEsimdCPUPKfPKiS2_S0_Pf")
        self._spmm_emul.argtypes = [_f32p, _i32p, _i32p, _f32p, _f32p]
        for f in (self._sddmm, self._spmm, self._fused_emul, self._spmm_emul):
            f.restype = None

    def _check(self, ro, dense_rows=None):
        assert ro.size == self.M + 1, "row_offsets does not match the compiled MSZ"

    def sddmm(self, row_offsets, col_indices, c, b) -> np.ndarray:
        ro, ci, c, b = _i32(row_offsets), _i32(col_indices), _f32(c), _f32(b)
        self._check(ro)
        assert c.shape == (self.M, self.D) and b.shape == (self.K, self.D)
        out = np.zeros(max(int(ro[-1]), 1), dtype=np.float32)
        self._sddmm(_pi(ro), _pi(ci), _pf(c), _pf(b), _pf(out))
        return out[: int(ro[-1])]

    def spmm_f64acc(self, row_offsets, col_indices, values, d) -> np.ndarray:
        ro, ci, va, d = _i32(row_offsets), _i32(col_indices), _f32(values), _f32(d)
        self._check(ro)
        assert d.shape == (self.K, self.D)
        e = np.zeros((self.M, self.D), dtype=np.float32)
        self._spmm(_pf(va), _pi(ro), _pi(ci), _pf(d), _pf(e))
        return e

    def spmm_f32_emul(self, row_offsets, col_indices, values, d) -> np.ndarray:
        ro, ci, va, d = _i32(row_offsets), _i32(col_indices), _f32(values), _f32(d)
        self._check(ro)
        assert d.shape == (self.K, self.D)
        e = np.zeros((self.M, self.D), dtype=np.float32)
        self._spmm_emul(_pf(va), _pi(ro), _pi(ci), _pf(d), _pf(e))
        return e

    def fused_emul(self, row_offsets, col_indices, c, b, d) -> np.ndarray:
        ro, ci, c, b, d = _i32(row_offsets), _i32(col_indices), _f32(c), _f32(b), _f32(d)
        self._check(ro)
        e = np.zeros((self.M, self.D), dtype=np.float32)
        self._fused_emul(_pi(ro), _pi(ci), _pf(c), _pf(b), _pf(d), _pf(e))
        return e


def ref_builds() -> list:
    """Every reference build present under oracle/_ref (empty where the reference was never mounted)."""
    return [RefFused(p) for p in sorted(glob.glob(os.path.join(_REF_DIR, "fused_ref_M*_K*_N*.so")))]
