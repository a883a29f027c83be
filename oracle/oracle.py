"""TEST INFRASTRUCTURE -- ctypes access to the CPU oracle and, where it has
been built, to the compiled reference under ``oracle/_ref``.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product never does.

Matrices are numpy arrays holding a column-major window: a 2-D array ``X`` of
shape ``(ld, cols)`` in Fortran order, of which rows ``0..rows-1`` are the
matrix and the rest is padding (what the netlib testers call ``AA``).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_DIR = os.path.join(HERE, "_ref")

ROW_MAJOR, COL_MAJOR = 101, 102
NO_TRANS, TRANS, CONJ_TRANS, ATLAS_CONJ = 111, 112, 113, 114
UPPER, LOWER = 121, 122
NON_UNIT, UNIT = 131, 132
LEFT, RIGHT = 141, 142


class BlockSize(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("MC", "KC", "NC", "MR", "NR")]


def build(with_reference: bool = True) -> None:
    """Compile liboracle.so (and oracle/_ref when the reference tree exists)."""
    target = "all" if with_reference else "liboracle.so"
    subprocess.run(["make", "-s", "-C", HERE, target], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build(with_reference=False)
        L = C.CDLL(ORACLE_SO)
        lng, dbl, flt, vp, i32 = C.c_long, C.c_double, C.c_float, C.c_void_p, C.c_int
        bsp = C.POINTER(BlockSize)
        L.ulm_oracle_gemm_d.argtypes = [lng, lng, lng, dbl, vp, lng, lng, vp, lng, lng, dbl, vp, lng, lng, bsp]
        L.ulm_oracle_gemm_s.argtypes = [lng, lng, lng, flt, vp, lng, lng, vp, lng, lng, flt, vp, lng, lng, bsp]
        L.ulm_oracle_gemm_s_f64.argtypes = [lng, lng, lng, dbl, vp, lng, lng, vp, lng, lng, dbl, vp, lng, lng, bsp]
        L.ulm_oracle_f77_gemm_info.argtypes = [C.c_char, C.c_char] + [i32] * 6
        L.ulm_oracle_cblas_gemm_info.argtypes = [i32] * 9
        L.ulm_oracle_dgemm_f77.argtypes = [C.c_char, C.c_char, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32]
        L.ulm_oracle_sgemm_f77.argtypes = [C.c_char, C.c_char, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32]
        L.ulm_oracle_cblas_dgemm.argtypes = [i32, i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32]
        L.ulm_oracle_cblas_sgemm.argtypes = [i32, i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32]
        L.ulm_oracle_gemm_samples.argtypes = [i32, C.c_char, C.c_char, lng, lng, lng, dbl, vp, lng, vp, lng, dbl,
                                              vp, lng, lng, vp, vp, vp, vp]
        L.ulm_oracle_trsm_d.argtypes = [i32, lng, lng, dbl, i32, vp, lng, lng, vp, lng, lng, bsp]
        L.ulm_oracle_trsm_s.argtypes = [i32, lng, lng, flt, i32, vp, lng, lng, vp, lng, lng, bsp]
        L.ulm_oracle_trsm_s_f64.argtypes = [i32, lng, lng, dbl, i32, vp, lng, lng, vp, lng, lng, bsp]
        L.ulm_oracle_f77_trsm_info.argtypes = [C.c_char] * 4 + [i32] * 4
        L.ulm_oracle_cblas_trsm_info.argtypes = [i32] * 9
        L.ulm_oracle_dtrsm_f77.argtypes = [C.c_char] * 4 + [i32, i32, dbl, vp, i32, vp, i32]
        L.ulm_oracle_strsm_f77.argtypes = [C.c_char] * 4 + [i32, i32, flt, vp, i32, vp, i32]
        L.ulm_oracle_cblas_dtrsm.argtypes = [i32] * 7 + [dbl, vp, i32, vp, i32]
        L.ulm_oracle_cblas_strsm.argtypes = [i32] * 7 + [flt, vp, i32, vp, i32]
        for f in ("ulm_oracle_trsm_d", "ulm_oracle_trsm_s", "ulm_oracle_trsm_s_f64", "ulm_oracle_f77_trsm_info",
                  "ulm_oracle_cblas_trsm_info", "ulm_oracle_dtrsm_f77", "ulm_oracle_strsm_f77",
                  "ulm_oracle_cblas_dtrsm", "ulm_oracle_cblas_strsm"):
            getattr(L, f).restype = C.c_int
        L.ulm_oracle_getrf_d.argtypes = [lng, lng, vp, lng, lng, vp, lng, lng, bsp]
        L.ulm_oracle_getf2_d.argtypes = [lng, lng, vp, lng, lng, vp, lng]
        L.ulm_oracle_laswp_d.argtypes = [lng, vp, lng, lng, lng, lng, vp, lng]
        L.ulm_oracle_dgetrf.argtypes = [i32, i32, i32, vp, i32, vp]
        L.ulm_oracle_dlaswp.argtypes = [i32, vp, i32, i32, i32, vp, i32]
        for suf, sc in (("d", dbl), ("s", flt), ("s_f64", dbl)):
            getattr(L, "ulm_oracle_syrk_" + suf).argtypes = [i32, lng, lng, sc, vp, lng, lng, sc, vp, lng, lng, bsp]
            getattr(L, "ulm_oracle_symm_" + suf).argtypes = [i32, lng, lng, sc, vp, lng, lng, vp, lng, lng, sc, vp, lng,
                                                             lng, bsp]
            getattr(L, "ulm_oracle_trmm_" + suf).argtypes = [i32, lng, lng, sc, i32, vp, lng, lng, vp, lng, lng, bsp]
            getattr(L, "ulm_oracle_syr2k_" + suf).argtypes = [i32, lng, lng, sc, vp, lng, lng, vp, lng, lng, sc, vp,
                                                              lng, lng, bsp]
            for r in ("syrk", "syr2k", "symm", "trmm"):
                getattr(L, f"ulm_oracle_{r}_{suf}").restype = C.c_int
        for suf in ("z", "c"):
            getattr(L, "ulm_oracle_gemm_" + suf).argtypes = [lng, lng, lng, vp, i32, vp, lng, lng, i32, vp, lng, lng, vp, vp,
                                                             lng, lng, bsp]
            getattr(L, "ulm_oracle_gemm_" + suf).restype = C.c_int
        L.ulm_oracle_f77_syrk_info.argtypes = [C.c_char, C.c_char, i32, i32, i32, i32]
        L.ulm_oracle_cblas_syrk_info.argtypes = [i32] * 7
        L.ulm_oracle_f77_symm_info.argtypes = [C.c_char, C.c_char, i32, i32, i32, i32, i32]
        L.ulm_oracle_cblas_symm_info.argtypes = [i32] * 8
        L.ulm_oracle_f77_syr2k_info.argtypes = [C.c_char, C.c_char, i32, i32, i32, i32, i32]
        L.ulm_oracle_cblas_syr2k_info.argtypes = [i32] * 8
        for f in ("ulm_oracle_f77_syrk_info", "ulm_oracle_cblas_syrk_info", "ulm_oracle_f77_symm_info",
                  "ulm_oracle_cblas_symm_info", "ulm_oracle_f77_syr2k_info", "ulm_oracle_cblas_syr2k_info"):
            getattr(L, f).restype = C.c_int
        for f in ("ulm_oracle_getrf_d", "ulm_oracle_getf2_d", "ulm_oracle_dgetrf"):
            getattr(L, f).restype = C.c_int
        L.ulm_oracle_laswp_d.restype = None
        L.ulm_oracle_dlaswp.restype = None
        for f in ("ulm_oracle_gemm_d", "ulm_oracle_gemm_s", "ulm_oracle_gemm_s_f64", "ulm_oracle_f77_gemm_info",
                  "ulm_oracle_cblas_gemm_info", "ulm_oracle_dgemm_f77", "ulm_oracle_sgemm_f77",
                  "ulm_oracle_cblas_dgemm", "ulm_oracle_cblas_sgemm", "ulm_oracle_gemm_samples"):
            getattr(L, f).restype = C.c_int
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def _ch(c):
    return c.encode() if isinstance(c, str) else c


def _strides(trans: bool, ld: int):
    return (ld, 1) if trans else (1, ld)


def is_trans(t: str) -> bool:
    return t.upper() in ("T", "C")


VARIANTS = {
    "d": ("ulm_oracle_gemm_d", np.float64, C.c_double),
    "s": ("ulm_oracle_gemm_s", np.float32, C.c_float),
    "s_f64": ("ulm_oracle_gemm_s_f64", np.float32, C.c_double),
}


def gemm_strided(variant, m, n, k, alpha, A, sa, B, sb, beta, Cm, sc, blocksize=None):
    """ulmBLAS::gemm on element strides; Cm is updated in place."""
    name, dt, _ = VARIANTS[variant]
    assert A.dtype == dt and B.dtype == dt and Cm.dtype == dt
    bs = None
    if blocksize is not None:
        bs = C.pointer(BlockSize(*blocksize))
    rc = getattr(lib(), name)(m, n, k, alpha, _ptr(A), sa[0], sa[1], _ptr(B), sb[0], sb[1], beta, _ptr(Cm),
                              sc[0], sc[1], bs)
    if rc != 0:
        raise RuntimeError(f"{name} failed with {rc}")
    return Cm


def gemm(variant, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, blocksize=None):
    """Column-major C <- alpha op(A) op(B) + beta C, in place in Cm."""
    return gemm_strided(variant, m, n, k, alpha, A, _strides(is_trans(transA), lda), B,
                        _strides(is_trans(transB), ldb), beta, Cm, (1, ldc), blocksize)


def is_conj(t: str) -> bool:
    """'C' (conjugate transpose) and 'R' (conjugate, not transposed): interfaces/blas/F77/gemm.cc:273-274."""
    return t.upper() in ("C", "R")


def _scalar2(x, dtype):
    """A complex scalar as the (re, im) pair the interfaces take by pointer."""
    real = np.float64 if dtype == np.complex128 else np.float32
    return np.array([np.real(x), np.imag(x)], dtype=real)


def cgemm(variant, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, blocksize=None):
    """Complex column-major C <- alpha op(A) op(B) + beta C in place in Cm; variant "z"
    (complex128) or "c" (complex64); transA / transB in N, T, C, R (zgemm_'s
    dispatch, interfaces/blas/F77/gemm.cc:461-505)."""
    dt = np.complex128 if variant == "z" else np.complex64
    for a in (A, B, Cm):
        assert a.dtype == dt and a.flags.f_contiguous
    sa, sb = _strides(is_trans(transA), lda), _strides(is_trans(transB), ldb)
    al, be = _scalar2(alpha, dt), _scalar2(beta, dt)
    rc = getattr(lib(), "ulm_oracle_gemm_" + variant)(m, n, k, _ptr(al), int(is_conj(transA)), _ptr(A), sa[0], sa[1],
                                                      int(is_conj(transB)), _ptr(B), sb[0], sb[1], _ptr(be), _ptr(Cm),
                                                      1, ldc, _bs(blocksize))
    if rc != 0:
        raise RuntimeError(f"complex gemm oracle failed with {rc}")
    return Cm


def cgauge(transA, transB, m, n, k, alpha, A, B, beta, C0):
    """ZMMCH's error scale (test/F77/zblat3.f:2935-3000): with ABS1(z) = |re z| +
    |im z|, ABS1(alpha) sum ABS1(a) ABS1(b) + ABS1(beta) ABS1(c), in float64."""
    abs1 = lambda z: np.abs(np.real(z)).astype(np.float64) + np.abs(np.imag(z)).astype(np.float64)
    a, b = abs1(np.asarray(A)), abs1(np.asarray(B))
    opa = a[:k, :m].T if is_trans(transA) else a[:m, :k]
    opb = b[:n, :k].T if is_trans(transB) else b[:k, :n]
    g = abs1(alpha) * (opa @ opb) if (k > 0 and alpha != 0) else np.zeros((m, n))
    if beta != 0:
        g = g + abs1(beta) * abs1(np.asarray(C0)[:m, :n])
    return g


def f77_info(transA, transB, m, n, k, lda, ldb, ldc) -> int:
    return lib().ulm_oracle_f77_gemm_info(_ch(transA), _ch(transB), m, n, k, lda, ldb, ldc)


def cblas_info(order, transA, transB, m, n, k, lda, ldb, ldc) -> int:
    return lib().ulm_oracle_cblas_gemm_info(order, transA, transB, m, n, k, lda, ldb, ldc)


def dgemm_f77(transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc) -> int:
    return lib().ulm_oracle_dgemm_f77(_ch(transA), _ch(transB), m, n, k, alpha, _ptr(A), lda, _ptr(B), ldb, beta,
                                      _ptr(Cm), ldc)


def sgemm_f77(transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc) -> int:
    return lib().ulm_oracle_sgemm_f77(_ch(transA), _ch(transB), m, n, k, alpha, _ptr(A), lda, _ptr(B), ldb, beta,
                                      _ptr(Cm), ldc)


def cblas_dgemm(order, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc) -> int:
    return lib().ulm_oracle_cblas_dgemm(order, transA, transB, m, n, k, alpha, _ptr(A), lda, _ptr(B), ldb, beta,
                                        _ptr(Cm), ldc)


def cblas_sgemm(order, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc) -> int:
    return lib().ulm_oracle_cblas_sgemm(order, transA, transB, m, n, k, alpha, _ptr(A), lda, _ptr(B), ldb, beta,
                                        _ptr(Cm), ldc)


def samples(variant, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C0, ldc, rows, cols):
    """Values and gauges of sampled elements (rows[s], cols[s]) of the result."""
    vid = {"d": 0, "s": 1, "s_f64": 2}[variant]
    dt = VARIANTS[variant][1]
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    cols = np.ascontiguousarray(cols, dtype=np.int64)
    out = np.empty(rows.shape[0], dtype=dt)
    gauge = np.empty(rows.shape[0], dtype=np.float64)
    rc = lib().ulm_oracle_gemm_samples(vid, _ch(transA), _ch(transB), m, n, k, alpha, _ptr(A), lda, _ptr(B), ldb,
                                       beta, _ptr(C0), ldc, rows.shape[0], _ptr(rows), _ptr(cols), _ptr(out),
                                       _ptr(gauge))
    if rc != 0:
        raise RuntimeError(f"ulm_oracle_gemm_samples failed with {rc}")
    return out, gauge


def gauge(transA, transB, m, n, k, alpha, A, B, beta, C0):
    """|alpha| |op(A)| |op(B)| + |beta| |C|, the error scale of DMMCH
    (test/F77/dblat3.f:2496-2533), on the m x n windows, in float64."""
    a = np.abs(np.asarray(A, dtype=np.float64))
    b = np.abs(np.asarray(B, dtype=np.float64))
    opa = a[:k, :m].T if is_trans(transA) else a[:m, :k]
    opb = b[:n, :k].T if is_trans(transB) else b[:k, :n]
    g = abs(alpha) * (opa @ opb) if (k > 0 and alpha != 0) else np.zeros((m, n))
    if beta != 0:
        g = g + abs(beta) * np.abs(np.asarray(C0, dtype=np.float64)[:m, :n])
    return g


# ---------------------------------------------------------------------------
# triangular solve
# ---------------------------------------------------------------------------

def trsm_strided(variant, lower, m, n, alpha, unit, A, sa, B, sb, blocksize=None):
    """ulmBLAS::trlsm (lower) / trusm on element strides: B <- alpha inv(A) B in place."""
    name, dt, _ = VARIANTS[variant]
    name = name.replace("gemm", "trsm")
    assert A.dtype == dt and B.dtype == dt
    bs = C.pointer(BlockSize(*blocksize)) if blocksize is not None else None
    rc = getattr(lib(), name)(int(lower), m, n, alpha, int(unit), _ptr(A), sa[0], sa[1], _ptr(B), sb[0], sb[1], bs)
    if rc != 0:
        raise RuntimeError(f"{name} failed with {rc}")
    return B


def trsm_dispatch(side, uplo, trans, m, n, lda, ldb):
    """(lower, rows, cols, strides of A, strides of B) the interfaces hand to
    the solver for a column-major call (interfaces/blas/F77/trsm.cc:183-227)."""
    left, low, tr = side.upper() == "L", uplo.upper() == "L", is_trans(trans)
    sa = (lda, 1) if tr else (1, lda)
    if left:
        return (low != tr), m, n, sa, (1, ldb)
    # right: op(A)^T X^T = alpha B^T
    sa = (sa[1], sa[0])
    return (low == tr), n, m, sa, (ldb, 1)


def trsm(variant, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, blocksize=None):
    """Column-major op(A) X = alpha B (side L) or X op(A) = alpha B (side R), in place in B."""
    lower, rows, cols, sa, sb = trsm_dispatch(side, uplo, trans, m, n, lda, ldb)
    return trsm_strided(variant, lower, rows, cols, alpha, diag.upper() == "U", A, sa, B, sb, blocksize)


def f77_trsm_info(side, uplo, trans, diag, m, n, lda, ldb) -> int:
    return lib().ulm_oracle_f77_trsm_info(_ch(side), _ch(uplo), _ch(trans), _ch(diag), m, n, lda, ldb)


def cblas_trsm_info(order, side, uplo, trans, diag, m, n, lda, ldb) -> int:
    return lib().ulm_oracle_cblas_trsm_info(order, side, uplo, trans, diag, m, n, lda, ldb)


def dtrsm_f77(side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb) -> int:
    return lib().ulm_oracle_dtrsm_f77(_ch(side), _ch(uplo), _ch(trans), _ch(diag), m, n, alpha, _ptr(A), lda,
                                      _ptr(B), ldb)


def strsm_f77(side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb) -> int:
    return lib().ulm_oracle_strsm_f77(_ch(side), _ch(uplo), _ch(trans), _ch(diag), m, n, alpha, _ptr(A), lda,
                                      _ptr(B), ldb)


def cblas_dtrsm(order, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb) -> int:
    return lib().ulm_oracle_cblas_dtrsm(order, side, uplo, trans, diag, m, n, alpha, _ptr(A), lda, _ptr(B), ldb)


def cblas_strsm(order, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb) -> int:
    return lib().ulm_oracle_cblas_strsm(order, side, uplo, trans, diag, m, n, alpha, _ptr(A), lda, _ptr(B), ldb)


# ---------------------------------------------------------------------------
# symmetric rank-k update, symmetric product, triangular product: column-major
# calls mapped onto the strided routines the way the interfaces do it
# (interfaces/blas/F77/{syrk,symm,trmm}.cc)
# ---------------------------------------------------------------------------

def _l3(variant, routine):
    return getattr(lib(), f"ulm_oracle_{routine}_{variant}")


def _bs(blocksize):
    return C.pointer(BlockSize(*blocksize)) if blocksize is not None else None


def syrk(variant, uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, blocksize=None):
    """C <- beta C + alpha op(A) op(A)^T on the uplo triangle, in place in Cm."""
    low, tr = uplo.upper() == "L", is_trans(trans)
    sa, sc = ((lda, 1), (ldc, 1)) if tr else ((1, lda), (1, ldc))
    rc = _l3(variant, "syrk")(int(low != tr), n, k, alpha, _ptr(A), sa[0], sa[1], beta, _ptr(Cm), sc[0], sc[1],
                              _bs(blocksize))
    if rc != 0:
        raise RuntimeError(f"syrk oracle failed with {rc}")
    return Cm


def syr2k(variant, uplo, trans, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, blocksize=None):
    """C <- beta C + alpha op(A) op(B)^T + alpha op(B) op(A)^T on the uplo triangle, in place in Cm
    (dispatch of interfaces/blas/F77/syr2k.cc:150-164)."""
    low, tr = uplo.upper() == "L", is_trans(trans)
    sa, sb, sc = ((lda, 1), (ldb, 1), (ldc, 1)) if tr else ((1, lda), (1, ldb), (1, ldc))
    rc = _l3(variant, "syr2k")(int(low != tr), n, k, alpha, _ptr(A), sa[0], sa[1], _ptr(B), sb[0], sb[1], beta,
                               _ptr(Cm), sc[0], sc[1], _bs(blocksize))
    if rc != 0:
        raise RuntimeError(f"syr2k oracle failed with {rc}")
    return Cm


def symm(variant, side, uplo, m, n, alpha, A, lda, B, ldb, beta, Cm, ldc, blocksize=None):
    """C <- beta C + alpha A B (side L) or alpha B A (side R), A symmetric, in place in Cm."""
    low = uplo.upper() == "L"
    if side.upper() == "L":
        args = (int(low), m, n, alpha, _ptr(A), 1, lda, _ptr(B), 1, ldb, beta, _ptr(Cm), 1, ldc)
    else:
        args = (int(not low), n, m, alpha, _ptr(A), lda, 1, _ptr(B), ldb, 1, beta, _ptr(Cm), ldc, 1)
    rc = _l3(variant, "symm")(*args, _bs(blocksize))
    if rc != 0:
        raise RuntimeError(f"symm oracle failed with {rc}")
    return Cm


def trmm(variant, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, blocksize=None):
    """B <- alpha op(A) B (side L) or alpha B op(A) (side R), in place in B."""
    lower, rows, cols, sa, sb = trsm_dispatch(side, uplo, trans, m, n, lda, ldb)
    rc = _l3(variant, "trmm")(int(lower), rows, cols, alpha, int(diag.upper() == "U"), _ptr(A), sa[0], sa[1], _ptr(B),
                              sb[0], sb[1], _bs(blocksize))
    if rc != 0:
        raise RuntimeError(f"trmm oracle failed with {rc}")
    return B


def f77_syrk_info(uplo, trans, n, k, lda, ldc) -> int:
    return lib().ulm_oracle_f77_syrk_info(_ch(uplo), _ch(trans), n, k, lda, ldc)


def cblas_syrk_info(order, uplo, trans, n, k, lda, ldc) -> int:
    return lib().ulm_oracle_cblas_syrk_info(order, uplo, trans, n, k, lda, ldc)


def f77_syr2k_info(uplo, trans, n, k, lda, ldb, ldc) -> int:
    return lib().ulm_oracle_f77_syr2k_info(_ch(uplo), _ch(trans), n, k, lda, ldb, ldc)


def cblas_syr2k_info(order, uplo, trans, n, k, lda, ldb, ldc) -> int:
    return lib().ulm_oracle_cblas_syr2k_info(order, uplo, trans, n, k, lda, ldb, ldc)


def f77_symm_info(side, uplo, m, n, lda, ldb, ldc) -> int:
    return lib().ulm_oracle_f77_symm_info(_ch(side), _ch(uplo), m, n, lda, ldb, ldc)


def cblas_symm_info(order, side, uplo, m, n, lda, ldb, ldc) -> int:
    return lib().ulm_oracle_cblas_symm_info(order, side, uplo, m, n, lda, ldb, ldc)


# ---------------------------------------------------------------------------
# LU factorisation (double)
# ---------------------------------------------------------------------------

def getrf_strided(m, n, A, sa, nb=0, blocksize=None):
    """ulmBLAS::getrf on element strides, in place in A.  Returns (info, piv)."""
    assert A.dtype == np.float64
    piv = np.zeros(max(min(m, n), 1), dtype=np.int32)
    bs = C.pointer(BlockSize(*blocksize)) if blocksize is not None else None
    info = lib().ulm_oracle_getrf_d(m, n, _ptr(A), sa[0], sa[1], _ptr(piv), 1, nb, bs)
    return info, piv[:min(m, n)]


def getf2_strided(m, n, A, sa):
    assert A.dtype == np.float64
    piv = np.zeros(max(min(m, n), 1), dtype=np.int32)
    info = lib().ulm_oracle_getf2_d(m, n, _ptr(A), sa[0], sa[1], _ptr(piv), 1)
    return info, piv[:min(m, n)]


def dgetrf(order, m, n, A, lda):
    """ULMLAPACK(dgetrf) (interfaces/lapack/C/getrf.cc:7-19).  Returns (info, piv)."""
    assert A.dtype == np.float64
    count = min(m, n)
    piv = np.zeros(max(count, 1), dtype=np.int32)
    info = lib().ulm_oracle_dgetrf(order, m, n, _ptr(A), lda, _ptr(piv))
    return info, piv[:count]


def dlaswp(n, A, lda, k1, k2, piv, inc_piv=1):
    """ULMLAPACK(dlaswp) (interfaces/lapack/C/laswp.cc:7-18), in place in A."""
    assert A.dtype == np.float64 and piv.dtype == np.int32
    lib().ulm_oracle_dlaswp(n, _ptr(A), lda, k1, k2, _ptr(piv), inc_piv)
    return A


# ---------------------------------------------------------------------------
# the compiled reference (present only where /root/reference was available at
# build time)
# ---------------------------------------------------------------------------

_ref_libs = {}


def have_ref(name: str = "libulmref.so") -> bool:
    return os.path.exists(os.path.join(REF_DIR, name))


def ref(name: str = "libulmref.so"):
    """A library built from the reference's own sources, or None."""
    if name not in _ref_libs:
        path = os.path.join(REF_DIR, name)
        if not os.path.exists(path):
            return None
        L = C.CDLL(path)
        i32, dbl, flt, vp = C.c_int, C.c_double, C.c_float, C.c_void_p
        if name != "libulmref_iface.so":
            L.ulmref_gemm_d.argtypes = [i32, i32, i32, dbl, vp, i32, i32, vp, i32, i32, dbl, vp, i32, i32]
            L.ulmref_gemm_s.argtypes = [i32, i32, i32, flt, vp, i32, i32, vp, i32, i32, flt, vp, i32, i32]
            L.ulmref_gemm_s_f64.argtypes = [i32, i32, i32, dbl, vp, i32, i32, vp, i32, i32, dbl, vp, i32, i32]
            L.ulmref_trsm_d.argtypes = [i32, i32, i32, dbl, i32, vp, i32, i32, vp, i32, i32]
            L.ulmref_trsm_s.argtypes = [i32, i32, i32, flt, i32, vp, i32, i32, vp, i32, i32]
            L.ulmref_trsm_s_f64.argtypes = [i32, i32, i32, dbl, i32, vp, i32, i32, vp, i32, i32]
            for f in ("ulmref_gemm_d", "ulmref_gemm_s", "ulmref_gemm_s_f64", "ulmref_trsm_d", "ulmref_trsm_s",
                      "ulmref_trsm_s_f64"):
                getattr(L, f).restype = None
            L.ulmref_syrk_d.argtypes = [i32, i32, i32, dbl, vp, i32, i32, dbl, vp, i32, i32]
            L.ulmref_symm_d.argtypes = [i32, i32, i32, dbl, vp, i32, i32, vp, i32, i32, dbl, vp, i32, i32]
            L.ulmref_trmm_d.argtypes = [i32, i32, i32, dbl, i32, vp, i32, i32, vp, i32, i32]
            for suf in ("z", "c"):
                getattr(L, "ulmref_gemm_" + suf).argtypes = [i32, i32, i32, vp, i32, vp, i32, i32, i32, vp, i32, i32, vp,
                                                             vp, i32, i32]
                getattr(L, "ulmref_gemm_" + suf).restype = None
            L.ulmref_syr2k_d.argtypes = [i32, i32, i32, dbl, vp, i32, i32, vp, i32, i32, dbl, vp, i32, i32]
            for f in ("ulmref_syrk_d", "ulmref_symm_d", "ulmref_trmm_d", "ulmref_syr2k_d"):
                getattr(L, f).restype = None
            L.ulmref_getrf_d.argtypes = [i32, i32, vp, i32, i32, vp, i32]
            L.ulmref_getf2_d.argtypes = [i32, i32, vp, i32, i32, vp, i32]
            L.ulmref_laswp_d.argtypes = [i32, vp, i32, i32, i32, i32, vp, i32]
            L.ulmref_getrf_d.restype = i32
            L.ulmref_getf2_d.restype = i32
            L.ulmref_laswp_d.restype = None
        else:
            L.cblas_dgemm.argtypes = [i32, i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32]
            L.cblas_sgemm.argtypes = [i32, i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32]
            L.ulmblas_dgemm.argtypes = [i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32]
            L.ulmblas_sgemm.argtypes = [i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32]
            L.cblas_dtrsm.argtypes = [i32] * 7 + [dbl, vp, i32, vp, i32]
            L.cblas_strsm.argtypes = [i32] * 7 + [flt, vp, i32, vp, i32]
            for f in ("cblas_dgemm", "cblas_sgemm", "ulmblas_dgemm", "ulmblas_sgemm", "dgemm_", "sgemm_",
                      "cblas_dtrsm", "cblas_strsm", "dtrsm_", "strsm_"):
                getattr(L, f).restype = None
            L.ulmblas_dgetrf.argtypes = [i32, i32, i32, vp, i32, vp]
            L.ulmblas_dgetrf.restype = i32
            L.ulmblas_dlaswp.argtypes = [i32, vp, i32, i32, i32, vp, i32]
            L.ulmblas_dlaswp.restype = None
        _ref_libs[name] = L
    return _ref_libs[name]


def ref_gemm(variant, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, libname="libulmref.so"):
    L = ref(libname)
    fn = {"d": L.ulmref_gemm_d, "s": L.ulmref_gemm_s, "s_f64": L.ulmref_gemm_s_f64}[variant]
    sa, sb = _strides(is_trans(transA), lda), _strides(is_trans(transB), ldb)
    fn(m, n, k, alpha, _ptr(A), sa[0], sa[1], _ptr(B), sb[0], sb[1], beta, _ptr(Cm), 1, ldc)
    return Cm


def ref_cgemm(variant, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, libname="libulmref.so"):
    """The reference's ulmBLAS::gemm on complex operands with conjugation flags."""
    dt = np.complex128 if variant == "z" else np.complex64
    sa, sb = _strides(is_trans(transA), lda), _strides(is_trans(transB), ldb)
    al, be = _scalar2(alpha, dt), _scalar2(beta, dt)
    getattr(ref(libname), "ulmref_gemm_" + variant)(m, n, k, _ptr(al), int(is_conj(transA)), _ptr(A), sa[0], sa[1],
                                                    int(is_conj(transB)), _ptr(B), sb[0], sb[1], _ptr(be), _ptr(Cm),
                                                    1, ldc)
    return Cm


def ref_f77_cgemm(prec, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc):
    """zgemm_ / cgemm_ of the reference's own F77 interface (everything by reference)."""
    L = ref("libulmref_iface.so")
    dt = np.complex128 if prec == "z" else np.complex64
    fn = getattr(L, prec + "gemm_")
    fn.restype = None
    ta, tb = C.c_char(_ch(transA)), C.c_char(_ch(transB))
    ints = [C.c_int(v) for v in (m, n, k, lda, ldb, ldc)]
    al, be = _scalar2(alpha, dt), _scalar2(beta, dt)
    fn(C.byref(ta), C.byref(tb), C.byref(ints[0]), C.byref(ints[1]), C.byref(ints[2]), _ptr(al), _ptr(A),
       C.byref(ints[3]), _ptr(B), C.byref(ints[4]), _ptr(be), _ptr(Cm), C.byref(ints[5]))
    return Cm


def ref_cblas_cgemm(prec, order, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc):
    """cblas_zgemm / cblas_cgemm of the reference's own C interface."""
    L = ref("libulmref_iface.so")
    dt = np.complex128 if prec == "z" else np.complex64
    fn = getattr(L, f"cblas_{prec}gemm")
    fn.restype = None
    fn.argtypes = [C.c_int] * 6 + [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int]
    al, be = _scalar2(alpha, dt), _scalar2(beta, dt)
    fn(order, transA, transB, m, n, k, _ptr(al), _ptr(A), lda, _ptr(B), ldb, _ptr(be), _ptr(Cm), ldc)
    return Cm


def ref_blocksize(variant="d", libname="libulmref.so"):
    L = ref(libname)
    out = (C.c_int * 5)()
    (L.ulmref_blocksize_s if variant == "s" else L.ulmref_blocksize_d)(out)
    return tuple(out)


def ref_f77_gemm(prec, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc):
    """dgemm_ / sgemm_ of the reference's own F77 interface (by reference)."""
    L = ref("libulmref_iface.so")
    ct = C.c_double if prec == "d" else C.c_float
    fn = L.dgemm_ if prec == "d" else L.sgemm_
    ta, tb = C.c_char(_ch(transA)), C.c_char(_ch(transB))
    ints = [C.c_int(v) for v in (m, n, k, lda, ldb, ldc)]
    al, be = ct(alpha), ct(beta)
    fn(C.byref(ta), C.byref(tb), C.byref(ints[0]), C.byref(ints[1]), C.byref(ints[2]), C.byref(al), _ptr(A),
       C.byref(ints[3]), _ptr(B), C.byref(ints[4]), C.byref(be), _ptr(Cm), C.byref(ints[5]))
    return Cm


def ref_trsm_strided(variant, lower, m, n, alpha, unit, A, sa, B, sb, libname="libulmref.so"):
    L = ref(libname)
    fn = {"d": L.ulmref_trsm_d, "s": L.ulmref_trsm_s, "s_f64": L.ulmref_trsm_s_f64}[variant]
    fn(int(lower), m, n, alpha, int(unit), _ptr(A), sa[0], sa[1], _ptr(B), sb[0], sb[1])
    return B


def ref_f77_trsm(prec, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb):
    """dtrsm_ / strsm_ of the reference's own F77 interface (by reference)."""
    L = ref("libulmref_iface.so")
    ct = C.c_double if prec == "d" else C.c_float
    fn = L.dtrsm_ if prec == "d" else L.strsm_
    chars = [C.c_char(_ch(c)) for c in (side, uplo, trans, diag)]
    ints = [C.c_int(v) for v in (m, n, lda, ldb)]
    al = ct(alpha)
    fn(*[C.byref(c) for c in chars], C.byref(ints[0]), C.byref(ints[1]), C.byref(al), _ptr(A), C.byref(ints[2]),
       _ptr(B), C.byref(ints[3]))
    return B


def ref_getrf_strided(m, n, A, sa, libname="libulmref.so"):
    piv = np.zeros(max(min(m, n), 1), dtype=np.int32)
    info = ref(libname).ulmref_getrf_d(m, n, _ptr(A), sa[0], sa[1], _ptr(piv), 1)
    return info, piv[:min(m, n)]


def ref_getf2_strided(m, n, A, sa, libname="libulmref.so"):
    piv = np.zeros(max(min(m, n), 1), dtype=np.int32)
    info = ref(libname).ulmref_getf2_d(m, n, _ptr(A), sa[0], sa[1], _ptr(piv), 1)
    return info, piv[:min(m, n)]


def ref_dgetrf(order, m, n, A, lda):
    """ulmblas_dgetrf of the reference's own LAPACK interface object."""
    piv = np.zeros(max(min(m, n), 1), dtype=np.int32)
    info = ref("libulmref_iface.so").ulmblas_dgetrf(order, m, n, _ptr(A), lda, _ptr(piv))
    return info, piv[:min(m, n)]


def ref_dlaswp(n, A, lda, k1, k2, piv, inc_piv=1):
    ref("libulmref_iface.so").ulmblas_dlaswp(n, _ptr(A), lda, k1, k2, _ptr(piv), inc_piv)
    return A


def ref_f77_l3(routine, prec, chars, ints_before, scalars, arrays):
    """A level-3 routine of the reference's own F77 interface, e.g.
    ref_f77_l3("syrk", "d", "LN", (n, k), (alpha, beta), ((A, lda), (C, ldc))):
    arguments go by reference in the BLAS order chars, sizes, then scalars and
    (array, ld) pairs interleaved as alpha, A, lda, [B, ldb,] [beta,] C, ldc."""
    L = ref("libulmref_iface.so")
    fn = getattr(L, f"{prec}{routine}_")
    fn.restype = None
    ct = C.c_double if prec == "d" else C.c_float
    keep = [C.c_char(_ch(c)) for c in chars] + [C.c_int(v) for v in ints_before]
    args = [C.byref(x) for x in keep]
    sc = [ct(v) for v in scalars]
    lds = [C.c_int(ld) for _, ld in arrays]
    args.append(C.byref(sc[0]))
    for idx_, (arr, _) in enumerate(arrays):
        if idx_ == len(arrays) - 1 and len(sc) > 1:
            args.append(C.byref(sc[1]))
        args += [_ptr(arr), C.byref(lds[idx_])]
    fn(*args)


def ref_syrk_d(uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, libname="libulmref.so"):
    """dsyrk's dispatch (interfaces/blas/F77/syrk.cc:139-153) onto the reference's sylrk / syurk."""
    low, tr = uplo.upper() == "L", is_trans(trans)
    sa, sc = ((lda, 1), (ldc, 1)) if tr else ((1, lda), (1, ldc))
    ref(libname).ulmref_syrk_d(int(low != tr), n, k, alpha, _ptr(A), sa[0], sa[1], beta, _ptr(Cm), sc[0], sc[1])
    return Cm


def ref_syr2k_d(uplo, trans, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, libname="libulmref.so"):
    """dsyr2k's dispatch onto the reference's sylr2k / syur2k.  The reference reads B on A's
    strides: only meaningful with lda == ldb."""
    assert lda == ldb, "the reference's rank-2k frame addresses B with A's leading dimension"
    low, tr = uplo.upper() == "L", is_trans(trans)
    sa, sb, sc = ((lda, 1), (ldb, 1), (ldc, 1)) if tr else ((1, lda), (1, ldb), (1, ldc))
    ref(libname).ulmref_syr2k_d(int(low != tr), n, k, alpha, _ptr(A), sa[0], sa[1], _ptr(B), sb[0], sb[1], beta,
                                _ptr(Cm), sc[0], sc[1])
    return Cm


def ref_symm_d(side, uplo, m, n, alpha, A, lda, B, ldb, beta, Cm, ldc, libname="libulmref.so"):
    low = uplo.upper() == "L"
    if side.upper() == "L":
        ref(libname).ulmref_symm_d(int(low), m, n, alpha, _ptr(A), 1, lda, _ptr(B), 1, ldb, beta, _ptr(Cm), 1, ldc)
    else:
        ref(libname).ulmref_symm_d(int(not low), n, m, alpha, _ptr(A), lda, 1, _ptr(B), ldb, 1, beta, _ptr(Cm), ldc,
                                   1)
    return Cm


def ref_trmm_d(side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, libname="libulmref.so"):
    lower, rows, cols, sa, sb = trsm_dispatch(side, uplo, trans, m, n, lda, ldb)
    ref(libname).ulmref_trmm_d(int(lower), rows, cols, alpha, int(diag.upper() == "U"), _ptr(A), sa[0], sa[1],
                               _ptr(B), sb[0], sb[1])
    return B
