"""The BLAS / CBLAS GEMM and TRSM entry points of libulmblas_gpu on numpy and torch data.

The functions keep the names and argument order of the C symbols they call
(`dgemm_`, `sgemm_`, `cblas_dgemm`, `cblas_sgemm`, `ulmblas_dgemm`, ...), which
are the ones ulmBLAS's interface layer exports (interfaces/blas/F77/gemm.cc,
interfaces/blas/C/gemm.cc).  Host matrices are numpy arrays whose memory is the
column-major (or, for CblasRowMajor, row-major) window the BLAS call describes;
C is updated in place.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from .lib import load

CblasRowMajor, CblasColMajor = 101, 102
CblasNoTrans, CblasTrans, CblasConjTrans, AtlasConj = 111, 112, 113, 114
CblasUpper, CblasLower = 121, 122
CblasNonUnit, CblasUnit = 131, 132
CblasLeft, CblasRight = 141, 142


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _check(a, dtype, name):
    if a is not None and a.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}")


def _f77(fn, ctype, dtype, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    for a, nm in ((A, "A"), (B, "B"), (Cm, "C")):
        _check(a, dtype, nm)
    ta = transA.encode() if isinstance(transA, str) else transA
    tb = transB.encode() if isinstance(transB, str) else transB
    ints = [C.c_int(v) for v in (m, n, k, ldA, ldB, ldC)]
    al, be = ctype(alpha), ctype(beta)
    fn(ta, tb, C.byref(ints[0]), C.byref(ints[1]), C.byref(ints[2]), C.byref(al), _p(A), C.byref(ints[3]), _p(B),
       C.byref(ints[4]), C.byref(be), _p(Cm), C.byref(ints[5]))
    return Cm


def dgemm_(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    return _f77(load().dgemm_, C.c_double, np.float64, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC)


def sgemm_(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    return _f77(load().sgemm_, C.c_float, np.float32, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC)


def cblas_dgemm(order, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    for a, nm in ((A, "A"), (B, "B"), (Cm, "C")):
        _check(a, np.float64, nm)
    load().cblas_dgemm(order, transA, transB, m, n, k, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def cblas_sgemm(order, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    for a, nm in ((A, "A"), (B, "B"), (Cm, "C")):
        _check(a, np.float32, nm)
    load().cblas_sgemm(order, transA, transB, m, n, k, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def ulmblas_dgemm(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC, symbol="ulmblas_dgemm"):
    getattr(load(), symbol)(transA, transB, m, n, k, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def ulmblas_sgemm(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC, symbol="ulmblas_sgemm"):
    getattr(load(), symbol)(transA, transB, m, n, k, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def _zdt(prec):
    return np.complex128 if prec == "z" else np.complex64


def _pair(x, prec):
    """A complex scalar as the (re, im) array the complex interfaces take by pointer."""
    return np.array([np.real(x), np.imag(x)], dtype=np.float64 if prec == "z" else np.float32)


TRANS_OF_CHAR = {"N": 111, "T": 112, "C": 113, "R": 114}


def cgemm_(prec, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    """zgemm_ / cgemm_ (interfaces/blas/F77/gemm.cc:382-506, 251-380); prec "z" or "c",
    operands complex Fortran-ordered numpy arrays."""
    dt = _zdt(prec)
    for a, nm in ((A, "A"), (B, "B"), (Cm, "C")):
        _check(a, dt, nm)
    ints = [C.c_int(v) for v in (m, n, k, ldA, ldB, ldC)]
    al, be = _pair(alpha, prec), _pair(beta, prec)
    getattr(load(), f"{prec}gemm_")(_ch(transA), _ch(transB), C.byref(ints[0]), C.byref(ints[1]), C.byref(ints[2]),
                                    _p(al), _p(A), C.byref(ints[3]), _p(B), C.byref(ints[4]), _p(be), _p(Cm),
                                    C.byref(ints[5]))
    return Cm


def cblas_cgemm(prec, order, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    al, be = _pair(alpha, prec), _pair(beta, prec)
    getattr(load(), f"cblas_{prec}gemm")(order, transA, transB, m, n, k, _p(al), _p(A), ldA, _p(B), ldB, _p(be),
                                         _p(Cm), ldC)
    return Cm


def ulmblas_cgemm(prec, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC, prefix="ulmblas_"):
    al, be = _pair(alpha, prec), _pair(beta, prec)
    getattr(load(), f"{prefix}{prec}gemm")(transA, transB, m, n, k, _p(al), _p(A), ldA, _p(B), ldB, _p(be), _p(Cm), ldC)
    return Cm


def _ch(c):
    return c.encode() if isinstance(c, str) else c


def _f77_trsm(fn, ctype, dtype, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    _check(A, dtype, "A")
    _check(B, dtype, "B")
    ints = [C.c_int(v) for v in (m, n, ldA, ldB)]
    al = ctype(alpha)
    fn(_ch(side), _ch(uplo), _ch(transA), _ch(diag), C.byref(ints[0]), C.byref(ints[1]), C.byref(al), _p(A),
       C.byref(ints[2]), _p(B), C.byref(ints[3]))
    return B


def dtrsm_(side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    """interfaces/blas/F77/trsm.cc:120-227: B <- alpha inv(op(A)) B or alpha B inv(op(A)), in place."""
    return _f77_trsm(load().dtrsm_, C.c_double, np.float64, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB)


def strsm_(side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    return _f77_trsm(load().strsm_, C.c_float, np.float32, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB)


def cblas_dtrsm(order, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    _check(A, np.float64, "A")
    _check(B, np.float64, "B")
    load().cblas_dtrsm(order, side, uplo, transA, diag, m, n, alpha, _p(A), ldA, _p(B), ldB)
    return B


def cblas_strsm(order, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    _check(A, np.float32, "A")
    _check(B, np.float32, "B")
    load().cblas_strsm(order, side, uplo, transA, diag, m, n, alpha, _p(A), ldA, _p(B), ldB)
    return B


def ulmblas_dtrsm(side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB, symbol="ulmblas_dtrsm"):
    getattr(load(), symbol)(side, uplo, transA, diag, m, n, alpha, _p(A), ldA, _p(B), ldB)
    return B


def ulmblas_strsm(side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB, symbol="ulmblas_strsm"):
    getattr(load(), symbol)(side, uplo, transA, diag, m, n, alpha, _p(A), ldA, _p(B), ldB)
    return B


def _dt(prec):
    return (C.c_double, np.float64) if prec == "d" else (C.c_float, np.float32)


def trmm_(prec, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    """dtrmm_ / strmm_ (interfaces/blas/F77/trmm.cc): B <- alpha op(A) B or alpha B op(A), in place."""
    ct, dt = _dt(prec)
    return _f77_trsm(getattr(load(), f"{prec}trmm_"), ct, dt, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB)


def cblas_trmm(prec, order, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB):
    getattr(load(), f"cblas_{prec}trmm")(order, side, uplo, transA, diag, m, n, alpha, _p(A), ldA, _p(B), ldB)
    return B


def ulmblas_trmm(prec, side, uplo, transA, diag, m, n, alpha, A, ldA, B, ldB, prefix="ulmblas_"):
    getattr(load(), f"{prefix}{prec}trmm")(side, uplo, transA, diag, m, n, alpha, _p(A), ldA, _p(B), ldB)
    return B


def syrk_(prec, uplo, trans, n, k, alpha, A, ldA, beta, Cm, ldC):
    """dsyrk_ / ssyrk_ (interfaces/blas/F77/syrk.cc): one triangle of C <- alpha op(A) op(A)^T + beta C."""
    ct, dt = _dt(prec)
    _check(A, dt, "A")
    _check(Cm, dt, "C")
    ints = [C.c_int(v) for v in (n, k, ldA, ldC)]
    al, be = ct(alpha), ct(beta)
    getattr(load(), f"{prec}syrk_")(_ch(uplo), _ch(trans), C.byref(ints[0]), C.byref(ints[1]), C.byref(al), _p(A),
                                    C.byref(ints[2]), C.byref(be), _p(Cm), C.byref(ints[3]))
    return Cm


def cblas_syrk(prec, order, uplo, trans, n, k, alpha, A, ldA, beta, Cm, ldC):
    getattr(load(), f"cblas_{prec}syrk")(order, uplo, trans, n, k, alpha, _p(A), ldA, beta, _p(Cm), ldC)
    return Cm


def ulmblas_syrk(prec, uplo, trans, n, k, alpha, A, ldA, beta, Cm, ldC, prefix="ulmblas_"):
    getattr(load(), f"{prefix}{prec}syrk")(uplo, trans, n, k, alpha, _p(A), ldA, beta, _p(Cm), ldC)
    return Cm


def syr2k_(prec, uplo, trans, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    """dsyr2k_ / ssyr2k_ (interfaces/blas/F77/syr2k.cc): one triangle of
    C <- alpha op(A) op(B)^T + alpha op(B) op(A)^T + beta C."""
    ct, dt = _dt(prec)
    for a, nm in ((A, "A"), (B, "B"), (Cm, "C")):
        _check(a, dt, nm)
    ints = [C.c_int(v) for v in (n, k, ldA, ldB, ldC)]
    al, be = ct(alpha), ct(beta)
    getattr(load(), f"{prec}syr2k_")(_ch(uplo), _ch(trans), C.byref(ints[0]), C.byref(ints[1]), C.byref(al), _p(A),
                                     C.byref(ints[2]), _p(B), C.byref(ints[3]), C.byref(be), _p(Cm), C.byref(ints[4]))
    return Cm


def cblas_syr2k(prec, order, uplo, trans, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    getattr(load(), f"cblas_{prec}syr2k")(order, uplo, trans, n, k, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def ulmblas_syr2k(prec, uplo, trans, n, k, alpha, A, ldA, B, ldB, beta, Cm, ldC, prefix="ulmblas_"):
    getattr(load(), f"{prefix}{prec}syr2k")(uplo, trans, n, k, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def symm_(prec, side, uplo, m, n, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    """dsymm_ / ssymm_ (interfaces/blas/F77/symm.cc): C <- alpha A B + beta C or alpha B A + beta C."""
    ct, dt = _dt(prec)
    for a, nm in ((A, "A"), (B, "B"), (Cm, "C")):
        _check(a, dt, nm)
    ints = [C.c_int(v) for v in (m, n, ldA, ldB, ldC)]
    al, be = ct(alpha), ct(beta)
    getattr(load(), f"{prec}symm_")(_ch(side), _ch(uplo), C.byref(ints[0]), C.byref(ints[1]), C.byref(al), _p(A),
                                    C.byref(ints[2]), _p(B), C.byref(ints[3]), C.byref(be), _p(Cm), C.byref(ints[4]))
    return Cm


def cblas_symm(prec, order, side, uplo, m, n, alpha, A, ldA, B, ldB, beta, Cm, ldC):
    getattr(load(), f"cblas_{prec}symm")(order, side, uplo, m, n, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def ulmblas_symm(prec, side, uplo, m, n, alpha, A, ldA, B, ldB, beta, Cm, ldC, prefix="ulmblas_"):
    getattr(load(), f"{prefix}{prec}symm")(side, uplo, m, n, alpha, _p(A), ldA, _p(B), ldB, beta, _p(Cm), ldC)
    return Cm


def ulmblas_dgetrf(order, m, n, A, ldA, symbol="ulmblas_dgetrf"):
    """interfaces/lapack/C/getrf.cc:7-19: LU in place in A.  Returns (info, piv)."""
    _check(A, np.float64, "A")
    piv = np.zeros(max(min(m, n), 1), dtype=np.int32)
    info = getattr(load(), symbol)(order, m, n, _p(A), ldA, _p(piv))
    return info, piv[:max(min(m, n), 0)]


def ulmblas_dlaswp(n, A, ldA, k1, k2, piv, incPiv=1, symbol="ulmblas_dlaswp"):
    """interfaces/lapack/C/laswp.cc:7-18: row exchanges in place in A."""
    _check(A, np.float64, "A")
    _check(piv, np.int32, "piv")
    getattr(load(), symbol)(n, _p(A), ldA, k1, k2, _p(piv), incPiv)
    return A


class GpuError(RuntimeError):
    pass


def _status(rc):
    if rc != 0:
        raise GpuError(f"status {rc}: {load().ulmblas_gpu_last_error().decode()}")


def _dev_ptr(x):
    return C.c_void_p(x.data_ptr()) if x is not None else None


_ELEMENT_BYTES = {"s": 4, "d": 8, "c": 8, "z": 16}


def room(x):
    """Bytes of device memory from the first element of tensor x to the end of its storage."""
    return x.untyped_storage().nbytes() - x.storage_offset() * x.element_size()


def _fits(what, prec, x, rows, cols, ld):
    """The kernels trust the shapes they are given, and a read or write past an
    operand is a memory fault on the GPU: a column-major rows x cols window
    with leading dimension ld must fit the tensor it is said to live in."""
    if x is None or rows <= 0 or cols <= 0:
        return
    if ld < rows:
        return                      # the library refuses this itself and launches nothing
    need = ((cols - 1) * ld + rows) * _ELEMENT_BYTES[prec]
    if room(x) < need:
        raise ValueError(f"{what}: a {rows} x {cols} window with leading dimension {ld} needs {need} bytes, "
                         f"the tensor holds {room(x)}")


def gpu_dgemm(transA, transB, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream=None):
    """Device-resident dgemm: dA, dB, dC are torch CUDA tensors (any shape)
    whose storage holds the column-major windows; `stream` is a raw
    hipStream_t value (default: torch's current stream).  Asynchronous."""
    import torch
    _fits("A", "d", dA, *((k, m) if transA else (m, k)), ldA)
    _fits("B", "d", dB, *((n, k) if transB else (k, n)), ldB)
    _fits("C", "d", dC, m, n, ldC)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    _status(load().ulmblas_gpu_dgemm(int(transA), int(transB), m, n, k, alpha, _dev_ptr(dA), ldA, _dev_ptr(dB), ldB,
                                     beta, _dev_ptr(dC), ldC, C.c_void_p(s)))
    return dC


def gpu_sgemm(transA, transB, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream=None):
    import torch
    _fits("A", "s", dA, *((k, m) if transA else (m, k)), ldA)
    _fits("B", "s", dB, *((n, k) if transB else (k, n)), ldB)
    _fits("C", "s", dC, m, n, ldC)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    _status(load().ulmblas_gpu_sgemm(int(transA), int(transB), m, n, k, alpha, _dev_ptr(dA), ldA, _dev_ptr(dB), ldB,
                                     beta, _dev_ptr(dC), ldC, C.c_void_p(s)))
    return dC


def gpu_dtrsm(right, lower, transA, unit, m, n, alpha, dA, ldA, dB, ldB, stream=None):
    """Device-resident triangular solve on torch CUDA tensors, in place in dB.  Asynchronous."""
    import torch
    _fits("A", "d", dA, n if right else m, n if right else m, ldA)
    _fits("B", "d", dB, m, n, ldB)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    _status(load().ulmblas_gpu_dtrsm(int(right), int(lower), int(transA), int(unit), m, n, alpha, _dev_ptr(dA), ldA,
                                     _dev_ptr(dB), ldB, C.c_void_p(s)))
    return dB


def gpu_strsm(right, lower, transA, unit, m, n, alpha, dA, ldA, dB, ldB, stream=None):
    import torch
    _fits("A", "s", dA, n if right else m, n if right else m, ldA)
    _fits("B", "s", dB, m, n, ldB)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    _status(load().ulmblas_gpu_strsm(int(right), int(lower), int(transA), int(unit), m, n, alpha, _dev_ptr(dA), ldA,
                                     _dev_ptr(dB), ldB, C.c_void_p(s)))
    return dB


def _stream(stream):
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)


def gpu_trmm(prec, right, lower, transA, unit, m, n, alpha, dA, ldA, dB, ldB, stream=None):
    """Device-resident triangular product on torch CUDA tensors, in place in dB.  Asynchronous."""
    _fits("A", prec, dA, n if right else m, n if right else m, ldA)
    _fits("B", prec, dB, m, n, ldB)
    _status(getattr(load(), f"ulmblas_gpu_{prec}trmm")(int(right), int(lower), int(transA), int(unit), m, n, alpha,
                                                       _dev_ptr(dA), ldA, _dev_ptr(dB), ldB, _stream(stream)))
    return dB


def gpu_syrk(prec, lower, trans, n, k, alpha, dA, ldA, beta, dC, ldC, stream=None):
    _fits("A", prec, dA, *((k, n) if trans else (n, k)), ldA)
    _fits("C", prec, dC, n, n, ldC)
    _status(getattr(load(), f"ulmblas_gpu_{prec}syrk")(int(lower), int(trans), n, k, alpha, _dev_ptr(dA), ldA, beta,
                                                       _dev_ptr(dC), ldC, _stream(stream)))
    return dC


def gpu_syr2k(prec, lower, trans, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream=None):
    _fits("A", prec, dA, *((k, n) if trans else (n, k)), ldA)
    _fits("B", prec, dB, *((k, n) if trans else (n, k)), ldB)
    _fits("C", prec, dC, n, n, ldC)
    _status(getattr(load(), f"ulmblas_gpu_{prec}syr2k")(int(lower), int(trans), n, k, alpha, _dev_ptr(dA), ldA,
                                                        _dev_ptr(dB), ldB, beta, _dev_ptr(dC), ldC, _stream(stream)))
    return dC


def gpu_symm(prec, right, lower, m, n, alpha, dA, ldA, dB, ldB, beta, dC, ldC, work, stream=None):
    ka = n if right else m
    _fits("A", prec, dA, ka, ka, ldA)
    _fits("B", prec, dB, m, n, ldB)
    _fits("C", prec, dC, m, n, ldC)
    if alpha != 0:
        _fits("work", prec, work, min(ka, 2048), min(ka, 2048), min(ka, 2048))
    _status(getattr(load(), f"ulmblas_gpu_{prec}symm")(int(right), int(lower), m, n, alpha, _dev_ptr(dA), ldA,
                                                       _dev_ptr(dB), ldB, beta, _dev_ptr(dC), ldC, _dev_ptr(work),
                                                       _stream(stream)))
    return dC


def gpu_cgemm(prec, transA, transB, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream=None, work=None):
    """Device-resident complex GEMM on torch CUDA tensors (complex dtype, column-major
    windows); transA / transB are characters N, T, C, R.  Allocates the workspace unless
    one is passed.  Asynchronous; returns (dC, work)."""
    import torch
    L = load()
    tb = TRANS_OF_CHAR[transB.upper()]
    if work is None:
        size = getattr(L, f"ulmblas_gpu_{prec}gemm_worksize")(tb, m, n, k)
        work = torch.empty(max(size, 16), dtype=torch.uint8, device="cuda")
    al, be = _pair(alpha, prec), _pair(beta, prec)
    _fits("A", prec, dA, *((m, k) if transA.upper() in "NR" else (k, m)), ldA)
    _fits("B", prec, dB, *((k, n) if transB.upper() in "NR" else (n, k)), ldB)
    _fits("C", prec, dC, m, n, ldC)
    _status(getattr(L, f"ulmblas_gpu_{prec}gemm")(TRANS_OF_CHAR[transA.upper()], tb, m, n, k, _p(al), _dev_ptr(dA), ldA,
                                                  _dev_ptr(dB), ldB, _p(be), _dev_ptr(dC), ldC, _dev_ptr(work),
                                                  _stream(stream)))
    return dC, work


def gpu_dgetrf(m, n, dA, ldA, stream=None, work=None):
    """Device-resident LU on a torch CUDA tensor holding the column-major
    window.  Returns (dPiv, dInfo) as int32 device tensors; asynchronous.
    `work`: a caller's workspace of at least ulmblas_gpu_dgetrf_worksize()
    bytes (any contents; one factorisation at a time may use it)."""
    import torch
    _fits("A", "d", dA, m, n, ldA)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    L = load()
    dPiv = torch.zeros(max(min(m, n), 1), dtype=torch.int32, device="cuda")
    dInfo = torch.zeros(1, dtype=torch.int32, device="cuda")
    if work is None:
        work = torch.zeros((L.ulmblas_gpu_dgetrf_worksize() + 7) // 8, dtype=torch.float64, device="cuda")
    elif work.numel() * work.element_size() < L.ulmblas_gpu_dgetrf_worksize():
        raise ValueError("workspace smaller than ulmblas_gpu_dgetrf_worksize()")
    _status(L.ulmblas_gpu_dgetrf(m, n, _dev_ptr(dA), ldA, _dev_ptr(dPiv), _dev_ptr(dInfo), _dev_ptr(work),
                                 C.c_void_p(s)))
    dInfo._ulm_work = work          # keep the workspace alive until the results are read
    return dPiv[:min(m, n)], dInfo


def gpu_dlaswp(n, dA, ldA, k1, k2, dPiv, incPiv=1, stream=None):
    import torch
    _fits("A", "d", dA, max(k2, 1), n, ldA)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    _status(load().ulmblas_gpu_dlaswp(n, _dev_ptr(dA), ldA, k1, k2, _dev_ptr(dPiv), incPiv, C.c_void_p(s)))
    return dA


TEST_NARROW_LOADS, TEST_LU_SPIN_LIMIT, TEST_SHARED_PIECES, TEST_SHARED_MUTE, TEST_SHARED_SPIN_LIMIT, TEST_FAIL_ALLOC, \
    TEST_WHOLE_C, TEST_LU_SIMPLE_PANELS, TEST_TRSM_PARTS, TEST_HOST_HEAD, TEST_TRI_WAY = 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11
SHARED_PIECES_DEFAULT = 32      # the library's own setting of TEST_SHARED_PIECES


def test_control(what: int, value: int):
    """The library's switches for its own tests (ulmblas_gpu_test_control)."""
    _status(load().ulmblas_gpu_test_control(what, value))


test_control.__test__ = False       # not a test, whatever its name says to pytest


def plan(precision, m, n, k, reads_c, ldA, ldB):
    """(variant id, whole_c, sharing workgroups, shared tiles) of the launch the library would make."""
    out = (C.c_int * 4)()
    _status(load().ulmblas_gpu_plan(ord(precision), m, n, k, int(reads_c), ldA, ldB, C.byref(out)))
    return tuple(out)


def device_status():
    """Returns if no workgroup launched through the device entry points gave up a
    bounded wait since the last call; raises GpuError (status 4: recovered, the
    results are complete all the same) otherwise."""
    _status(load().ulmblas_gpu_device_status())


def last_status():
    """Status of the calling thread's most recent host entry point call."""
    return load().ulmblas_gpu_last_status()


def set_variant(precision: str, variant: int):
    _status(load().ulmblas_gpu_set_variant(ord(precision), variant))


def variant_names(precision: str):
    out, i = [], 1
    while True:
        nm = load().ulmblas_gpu_variant_name(ord(precision), i)
        if nm is None:
            return out
        out.append(nm.decode())
        i += 1
