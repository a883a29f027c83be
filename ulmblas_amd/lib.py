"""Locating, building and loading libulmblas_gpu.so."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libulmblas_gpu.so")
_lib = None


def library_path() -> str:
    return _SO


def build() -> str:
    """Compile the HIP sources for gfx950 (hipcc cross-compiles without a GPU)."""
    subprocess.run(["make", "-s", "-B", "-j4", "-C", os.path.join(_HERE, "csrc")], check=True)
    return _SO


def load() -> C.CDLL:
    """The shared library, with argument types declared.  Raises if it has not
    been built: there is no other implementation to fall back to."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        raise RuntimeError(
            f"{_SO} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or ulmblas_amd.build()); ulmblas_amd has no CPU fallback")
    L = C.CDLL(_SO)
    i32, dbl, flt, vp = C.c_int, C.c_double, C.c_float, C.c_void_p
    pi, pd, pf, pc = C.POINTER(C.c_int), C.POINTER(C.c_double), C.POINTER(C.c_float), C.c_char_p
    L.dgemm_.argtypes = [pc, pc, pi, pi, pi, pd, vp, pi, vp, pi, pd, vp, pi]
    L.sgemm_.argtypes = [pc, pc, pi, pi, pi, pf, vp, pi, vp, pi, pf, vp, pi]
    L.cblas_dgemm.argtypes = [i32, i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32]
    L.cblas_sgemm.argtypes = [i32, i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32]
    for name in ("ulmblas_dgemm", "ATL_dgemm"):
        getattr(L, name).argtypes = [i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32]
    for name in ("ulmblas_sgemm", "ATL_sgemm"):
        getattr(L, name).argtypes = [i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32]
    for name in ("dgemm_", "sgemm_", "cblas_dgemm", "cblas_sgemm", "ulmblas_dgemm", "ulmblas_sgemm", "ATL_dgemm",
                 "ATL_sgemm", "ulmblas_gpu_release"):
        getattr(L, name).restype = None
    L.ulmblas_gpu_dgemm.argtypes = [i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, dbl, vp, i32, vp]
    L.ulmblas_gpu_sgemm.argtypes = [i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, flt, vp, i32, vp]
    L.ulmblas_gpu_dgemm.restype = i32
    L.ulmblas_gpu_sgemm.restype = i32
    # triangular solve
    L.dtrsm_.argtypes = [pc, pc, pc, pc, pi, pi, pd, vp, pi, vp, pi]
    L.strsm_.argtypes = [pc, pc, pc, pc, pi, pi, pf, vp, pi, vp, pi]
    L.cblas_dtrsm.argtypes = [i32] * 7 + [dbl, vp, i32, vp, i32]
    L.cblas_strsm.argtypes = [i32] * 7 + [flt, vp, i32, vp, i32]
    for name in ("ulmblas_dtrsm", "ATL_dtrsm"):
        getattr(L, name).argtypes = [i32] * 6 + [dbl, vp, i32, vp, i32]
    for name in ("ulmblas_strsm", "ATL_strsm"):
        getattr(L, name).argtypes = [i32] * 6 + [flt, vp, i32, vp, i32]
    for name in ("dtrsm_", "strsm_", "cblas_dtrsm", "cblas_strsm", "ulmblas_dtrsm", "ulmblas_strsm", "ATL_dtrsm",
                 "ATL_strsm"):
        getattr(L, name).restype = None
    L.ulmblas_gpu_dtrsm.argtypes = [i32, i32, i32, i32, i32, i32, dbl, vp, i32, vp, i32, vp]
    L.ulmblas_gpu_strsm.argtypes = [i32, i32, i32, i32, i32, i32, flt, vp, i32, vp, i32, vp]
    L.ulmblas_gpu_dtrsm.restype = i32
    L.ulmblas_gpu_strsm.restype = i32
    # triangular product, symmetric rank-k and rank-2k updates, symmetric product
    L.dtrmm_.argtypes = [pc, pc, pc, pc, pi, pi, pd, vp, pi, vp, pi]
    L.strmm_.argtypes = [pc, pc, pc, pc, pi, pi, pf, vp, pi, vp, pi]
    L.dsyrk_.argtypes = [pc, pc, pi, pi, pd, vp, pi, pd, vp, pi]
    L.ssyrk_.argtypes = [pc, pc, pi, pi, pf, vp, pi, pf, vp, pi]
    L.dsymm_.argtypes = [pc, pc, pi, pi, pd, vp, pi, vp, pi, pd, vp, pi]
    L.dsyr2k_.argtypes = [pc, pc, pi, pi, pd, vp, pi, vp, pi, pd, vp, pi]
    L.ssyr2k_.argtypes = [pc, pc, pi, pi, pf, vp, pi, vp, pi, pf, vp, pi]
    L.ssymm_.argtypes = [pc, pc, pi, pi, pf, vp, pi, vp, pi, pf, vp, pi]
    for p_, sc in (("d", dbl), ("s", flt)):
        getattr(L, f"cblas_{p_}trmm").argtypes = [i32] * 7 + [sc, vp, i32, vp, i32]
        getattr(L, f"cblas_{p_}syrk").argtypes = [i32] * 5 + [sc, vp, i32, sc, vp, i32]
        getattr(L, f"cblas_{p_}symm").argtypes = [i32] * 5 + [sc, vp, i32, vp, i32, sc, vp, i32]
        getattr(L, f"cblas_{p_}syr2k").argtypes = [i32] * 5 + [sc, vp, i32, vp, i32, sc, vp, i32]
        for pre in ("ulmblas_", "ATL_"):
            getattr(L, f"{pre}{p_}trmm").argtypes = [i32] * 6 + [sc, vp, i32, vp, i32]
            getattr(L, f"{pre}{p_}syrk").argtypes = [i32] * 4 + [sc, vp, i32, sc, vp, i32]
            getattr(L, f"{pre}{p_}symm").argtypes = [i32] * 4 + [sc, vp, i32, vp, i32, sc, vp, i32]
            getattr(L, f"{pre}{p_}syr2k").argtypes = [i32] * 4 + [sc, vp, i32, vp, i32, sc, vp, i32]
        for r in ("trmm", "syrk", "symm", "syr2k"):
            for name in (f"{p_}{r}_", f"cblas_{p_}{r}", f"ulmblas_{p_}{r}", f"ATL_{p_}{r}"):
                getattr(L, name).restype = None
        getattr(L, f"ulmblas_gpu_{p_}trmm").argtypes = [i32, i32, i32, i32, i32, i32, sc, vp, i32, vp, i32, vp]
        getattr(L, f"ulmblas_gpu_{p_}syrk").argtypes = [i32, i32, i32, i32, sc, vp, i32, sc, vp, i32, vp]
        getattr(L, f"ulmblas_gpu_{p_}symm").argtypes = [i32, i32, i32, i32, sc, vp, i32, vp, i32, sc, vp, i32, vp, vp]
        getattr(L, f"ulmblas_gpu_{p_}syr2k").argtypes = [i32, i32, i32, i32, sc, vp, i32, vp, i32, sc, vp, i32, vp]
        for r in ("trmm", "syrk", "symm", "syr2k"):
            getattr(L, f"ulmblas_gpu_{p_}{r}").restype = i32
    # complex GEMM: scalars and matrices by pointer to (re, im) pairs
    for p_ in "zc":
        getattr(L, f"{p_}gemm_").argtypes = [pc, pc, pi, pi, pi, vp, vp, pi, vp, pi, vp, vp, pi]
        getattr(L, f"cblas_{p_}gemm").argtypes = [i32] * 6 + [vp, vp, i32, vp, i32, vp, vp, i32]
        for pre in ("ulmblas_", "ATL_"):
            getattr(L, f"{pre}{p_}gemm").argtypes = [i32] * 5 + [vp, vp, i32, vp, i32, vp, vp, i32]
        for name in (f"{p_}gemm_", f"cblas_{p_}gemm", f"ulmblas_{p_}gemm", f"ATL_{p_}gemm"):
            getattr(L, name).restype = None
        getattr(L, f"ulmblas_gpu_{p_}gemm_worksize").argtypes = [i32, i32, i32, i32]
        getattr(L, f"ulmblas_gpu_{p_}gemm_worksize").restype = C.c_long
        getattr(L, f"ulmblas_gpu_{p_}gemm").argtypes = [i32] * 5 + [vp, vp, i32, vp, i32, vp, vp, i32, vp, vp]
        getattr(L, f"ulmblas_gpu_{p_}gemm").restype = i32
    # LU
    for name in ("ulmblas_dgetrf", "ATL_dgetrf"):
        getattr(L, name).argtypes = [i32, i32, i32, vp, i32, vp]
        getattr(L, name).restype = i32
    for name in ("ulmblas_dlaswp", "ATL_dlaswp"):
        getattr(L, name).argtypes = [i32, vp, i32, i32, i32, vp, i32]
        getattr(L, name).restype = None
    L.ulmblas_gpu_dgetrf_worksize.restype = C.c_long
    L.ulmblas_gpu_dgetrf.argtypes = [i32, i32, vp, i32, vp, vp, vp, vp]
    L.ulmblas_gpu_dgetrf.restype = i32
    L.ulmblas_gpu_dgetrf_static.argtypes = [i32, i32, vp, i32, vp, vp, vp]
    L.ulmblas_gpu_dgetrf_static.restype = i32
    L.ulmblas_gpu_dlaswp.argtypes = [i32, vp, i32, i32, i32, vp, i32, vp]
    L.ulmblas_gpu_dlaswp.restype = i32
    L.ulmblas_gpu_set_variant.argtypes = [i32, i32]
    L.ulmblas_gpu_set_variant.restype = i32
    L.ulmblas_gpu_test_control.argtypes = [i32, C.c_long]
    L.ulmblas_gpu_test_control.restype = i32
    L.ulmblas_gpu_device_status.restype = i32
    L.ulmblas_gpu_plan.argtypes = [i32, i32, i32, i32, i32, C.c_long, C.c_long, C.POINTER(C.c_int * 4)]
    L.ulmblas_gpu_plan.restype = i32
    L.ulmblas_gpu_variant_name.argtypes = [i32, i32]
    L.ulmblas_gpu_variant_name.restype = C.c_char_p
    L.ulmblas_gpu_last_error.restype = C.c_char_p
    L.ulmblas_gpu_last_status.restype = i32
    L.ulmblas_gpu_alloc_count.restype = C.c_long
    _lib = L
    return L
