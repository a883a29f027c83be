"""The C ABI of libulmblas_gpu.so, without a GPU: every symbol the public
header declares is exported, the error exits report the reference's info codes
through an overridable xerbla and leave C alone, and calls that have nothing
to compute return without touching the device."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import netlib
from ulmblas_amd import blas, lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ulmblas_gpu.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?(?:void|int|long|char)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


LEVEL3 = tuple(f"{head}{p}{r}{tail}" for r in ("trmm", "syrk", "syr2k", "symm") for p in "ds"
               for head, tail in (("", "_"), ("cblas_", ""), ("ulmblas_", ""), ("ATL_", ""), ("ulmblas_gpu_", "")))


def test_header_symbols_exported():
    names = declared_symbols()
    for must in ("dgemm_", "sgemm_", "cblas_dgemm", "cblas_sgemm", "ulmblas_dgemm", "ulmblas_sgemm", "ATL_dgemm",
                 "ATL_sgemm", "xerbla_", "cblas_xerbla", "ulmblas_xerbla", "ulmblas_gpu_dgemm", "ulmblas_gpu_sgemm",
                 "ulmblas_gpu_set_variant", "ulmblas_gpu_variant_name", "ulmblas_gpu_last_error",
                 "ulmblas_gpu_alloc_count", "ulmblas_gpu_release", "dtrsm_", "strsm_", "cblas_dtrsm", "cblas_strsm",
                 "ulmblas_dtrsm", "ulmblas_strsm", "ATL_dtrsm", "ATL_strsm", "ulmblas_gpu_dtrsm", "ulmblas_gpu_strsm",
                 "ulmblas_dgetrf", "ulmblas_dlaswp", "ATL_dgetrf", "ATL_dlaswp", "ulmblas_gpu_dgetrf",
                 "ulmblas_gpu_dgetrf_worksize", "ulmblas_gpu_dlaswp", "zgemm_", "cgemm_", "cblas_zgemm", "cblas_cgemm",
                 "ulmblas_zgemm", "ulmblas_cgemm", "ATL_zgemm", "ATL_cgemm", "ulmblas_gpu_zgemm", "ulmblas_gpu_cgemm",
                 "ulmblas_gpu_zgemm_worksize", "ulmblas_gpu_cgemm_worksize") + LEVEL3:
        assert must in names, f"{must} not found in the header"
    L = C.CDLL(lib.library_path())
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/ulmblas_gpu.h but not exported"


def test_missing_library_is_loud(monkeypatch):
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "_SO", "/nonexistent/libulmblas_gpu.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        lib.load()


@pytest.mark.parametrize("prec", ["d", "s"])
def test_f77_error_exits(prec, xerbla):
    """DCHKE, test/F77/dblat3.f:1838-1921 (SCHKE in sblat3.f likewise)."""
    dt = np.float64 if prec == "d" else np.float32
    f = blas.dgemm_ if prec == "d" else blas.sgemm_
    name = b"DGEMM " if prec == "d" else b"SGEMM "
    for (ta, tb, m, n, k, lda, ldb, ldc), info in netlib.F77_ERROR_EXITS:
        xerbla.capture_reset()
        a = np.full((2, 1), 7.0, dtype=dt, order="F")
        b = a.copy(order="F")
        c = a.copy(order="F")
        f(ta, tb, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, ldc)
        assert xerbla.capture_count() == 1, (ta, tb, m, n, k)
        assert xerbla.capture_last_info() == info, (ta, tb, m, n, k, lda, ldb, ldc)
        assert xerbla.capture_last_name() == name
        assert (c == 7.0).all()


@pytest.mark.parametrize("prec", ["d", "s"])
def test_cblas_error_exits(prec, xerbla):
    """test/C/c_d3chke.c:46-273 (c_s3chke.c likewise); the tester's xerbla
    swaps the row-major positions back before comparing."""
    dt = np.float64 if prec == "d" else np.float32
    f = blas.cblas_dgemm if prec == "d" else blas.cblas_sgemm
    name = b"cblas_dgemm" if prec == "d" else b"cblas_sgemm"
    for (order, ta, tb, m, n, k, lda, ldb, ldc), info in netlib.CBLAS_ERROR_EXITS:
        xerbla.capture_reset()
        a = np.full(2, 7.0, dtype=dt)
        c = a.copy()
        f(order, ta, tb, m, n, k, 1.0, a, lda, a, ldb, 0.0, c, ldc)
        assert xerbla.capture_count() == 1, (order, ta, tb, m, n, k)
        assert netlib.cblas_tester_info(order, xerbla.capture_last_info()) == info
        assert xerbla.capture_last_name() == name
        assert (c == 7.0).all()


def test_info_codes_match_oracle_everywhere(oracle, xerbla):
    """Beyond the testers' lists: a grid of argument combinations, first
    failing check wins, same code as the reference's checks restated in the
    oracle (which are pinned against the reference's own objects)."""
    a = np.zeros(1)
    sizes = (-1, 0, 2)
    for ta in "NTXc":
        for tb in "NTXr":
            for m in sizes:
                for n in sizes:
                    for k in sizes:
                        for lda, ldb, ldc in ((1, 1, 1), (2, 1, 2), (1, 2, 2), (2, 2, 1)):
                            want = oracle.f77_info(ta, tb, m, n, k, lda, ldb, ldc)
                            if want == 0 and m > 0 and n > 0:
                                continue        # would compute: needs a GPU
                            xerbla.capture_reset()
                            blas.dgemm_(ta, tb, m, n, k, 0.0, a, lda, a, ldb, 1.0, a, ldc)
                            got = xerbla.capture_last_info() if xerbla.capture_count() else 0
                            assert got == want, (ta, tb, m, n, k, lda, ldb, ldc)
    for order in (101, 102, 7):
        for ta in (111, 112, 113, 114, 0):
            for tb in (111, 112, 5):
                for m in sizes:
                    for n in sizes:
                        for k in sizes:
                            for lda, ldb, ldc in ((1, 1, 1), (2, 1, 2), (1, 2, 2), (2, 2, 1)):
                                want = oracle.cblas_info(order, ta, tb, m, n, k, lda, ldb, ldc)
                                if want == 0 and m > 0 and n > 0:
                                    continue
                                xerbla.capture_reset()
                                blas.cblas_dgemm(order, ta, tb, m, n, k, 0.0, a, lda, a, ldb, 1.0, a, ldc)
                                got = xerbla.capture_last_info() if xerbla.capture_count() else 0
                                assert got == want, (order, ta, tb, m, n, k, lda, ldb, ldc)


def test_nothing_to_do_returns_without_device(xerbla):
    """m == 0 or n == 0 writes nothing (test/F77/dblat3.f:552-553); alpha == 0
    or k == 0 with beta == 1 leaves C as it is (ulmblas/level3/gemm.tcc:52-55,
    ulmblas/level1extensions/gescal.tcc:20-22).  None of these needs the GPU."""
    c0 = np.arange(12.0).reshape((4, 3), order="F")
    a = np.ones((4, 4), order="F")
    for (m, n, k, alpha, beta) in [(0, 3, 2, 1.0, 0.0), (3, 0, 2, 1.0, 0.0), (3, 3, 0, 1.0, 1.0), (3, 3, 2, 0.0, 1.0)]:
        c = c0.copy(order="F")
        blas.dgemm_("N", "N", m, n, k, alpha, a, 4, a, 4, beta, c, 4)
        assert c.tobytes() == c0.tobytes()
        c = c0.copy(order="F")
        blas.cblas_dgemm(blas.CblasColMajor, blas.CblasNoTrans, blas.CblasTrans, m, n, k, alpha, a, 4, a, 4, beta, c, 4)
        assert c.tobytes() == c0.tobytes()
    assert xerbla.capture_count() == 0


def test_device_entry_rejects_bad_arguments():
    L = lib.load()
    for args in [(0, 0, -1, 1, 1, 1, 1, 1), (0, 0, 1, -1, 1, 1, 1, 1), (0, 0, 1, 1, -1, 1, 1, 1),
                 (0, 0, 4, 1, 1, 3, 1, 4), (1, 0, 4, 1, 2, 1, 2, 4), (0, 0, 4, 1, 2, 4, 1, 4), (0, 0, 4, 1, 2, 4, 2, 3)]:
        ta, tb, m, n, k, lda, ldb, ldc = args
        rc = L.ulmblas_gpu_dgemm(ta, tb, m, n, k, 1.0, None, lda, None, ldb, 0.0, None, ldc, None)
        assert rc == 1, args
        assert L.ulmblas_gpu_last_error() != b""
    # nothing to do: fine even with null pointers
    assert L.ulmblas_gpu_dgemm(0, 0, 0, 5, 5, 1.0, None, 1, None, 5, 0.0, None, 1, None) == 0
    assert L.ulmblas_gpu_set_variant(ord("d"), 999) == 1
    assert L.ulmblas_gpu_set_variant(ord("d"), 0) == 0
    assert L.ulmblas_gpu_variant_name(ord("d"), 1) is not None
    assert L.ulmblas_gpu_variant_name(ord("d"), 999) is None


def test_plan_query_and_test_switches():
    """The launch plan can be asked for without a GPU: the headline product takes
    whole tiles of the largest variant with nothing shared (8 full rounds on
    256 CUs); the strided BASELINE case goes out as one launch over all of C;
    437 tiles share the tiles of their second round."""
    from ulmblas_amd import blas
    names = blas.variant_names("d")
    vid, whole_c, groups, tiles = blas.plan("d", 8192, 8192, 8192, 0, 8192, 8192)
    assert names[vid - 1].startswith("whole_256x128") and (whole_c, groups, tiles) == (0, 0, 0)
    vid, whole_c, groups, tiles = blas.plan("d", 5000, 3000, 7000, 1, 7037, 7011)
    assert names[vid - 1].startswith("whole_256x128") and whole_c == 1
    vid, whole_c, groups, tiles = blas.plan("d", 256 * 19, 128 * 23, 7000, 0, 7000, 7000)
    assert names[vid - 1].startswith("whole_256x128") and whole_c == 0 and groups == 256 and tiles == 181
    # leading dimensions beyond the reach of the 32-bit packet offsets: no sharing kernel
    vid, whole_c, groups, tiles = blas.plan("d", 256 * 19, 128 * 23, 7000, 0, 5_000_000, 5_000_000)
    assert groups == 0 and whole_c == 0
    L = lib.load()
    assert L.ulmblas_gpu_test_control(99, 0) == 1
    assert L.ulmblas_gpu_test_control(blas.TEST_SHARED_PIECES, 0) == 0
    try:
        assert blas.plan("d", 256 * 19, 128 * 23, 7000, 0, 7000, 7000)[2] == 0
    finally:
        assert L.ulmblas_gpu_test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT) == 0


def test_failure_on_the_gpu_side_is_reported_and_leaves_c_alone(xerbla):
    """A host entry point returns nothing; when its GPU side cannot run (here:
    no device at all, or -- on a GPU box -- a device allocation that fails on
    request) the status is recorded, the overridable hook is called once with
    the routine's name, and C is left exactly as it was."""
    import torch
    L = lib.load()
    m = 40
    A = np.full((m, m), 2.0, order="F")
    B = np.full((m, m), 3.0, order="F")
    C0 = np.full((m, m), 7.0, order="F")
    have_gpu = torch.cuda.is_available()
    if have_gpu:
        blas.dgemm_("N", "N", m, m, m, 1.0, A, m, B, m, 0.0, C0.copy(order="F"), m)      # contexts and streams exist now
        L.ulmblas_gpu_release()                                                        # ... and hold no buffers
        assert L.ulmblas_gpu_test_control(blas.TEST_FAIL_ALLOC, 1) == 0
    xerbla.hook_reset()
    Cm = C0.copy(order="F")
    try:
        blas.dgemm_("N", "N", m, m, m, 1.0, A, m, B, m, 0.5, Cm, m)
    finally:
        L.ulmblas_gpu_test_control(blas.TEST_FAIL_ALLOC, 0)
    assert xerbla.hook_count() == 1 and xerbla.hook_last_routine() == b"dgemm_"
    assert xerbla.hook_last_status() == L.ulmblas_gpu_last_status() == (2 if have_gpu else 3)
    assert Cm.tobytes() == C0.tobytes()
    if have_gpu:                # the next call works again, and clears the status
        blas.dgemm_("N", "N", m, m, m, 1.0, A, m, B, m, 0.5, Cm, m)
        assert L.ulmblas_gpu_last_status() == 0 and np.allclose(Cm, 2.0 * 3.0 * m + 3.5)
    # a call with nothing to do succeeds without a device
    blas.dgemm_("N", "N", 0, m, m, 1.0, A, m, B, m, 0.5, Cm, m)
    assert L.ulmblas_gpu_last_status() == 0


def test_device_wrappers_refuse_windows_that_do_not_fit():
    """The kernels trust the shapes they are given; the Python wrappers of the
    device entry points and the benchmark's timing loop check every window
    against the memory behind its tensor before anything is launched."""
    import torch
    import bench
    A = torch.empty(64 * 64, dtype=torch.float64)
    B = torch.empty(64 * 32, dtype=torch.float64)
    small = torch.empty(64 * 31, dtype=torch.float64)
    with pytest.raises(ValueError, match="C: a 64 x 32 window"):
        blas.gpu_dgemm(0, 0, 64, 32, 64, 1.0, A, 64, B, 64, 0.0, small, 64)
    with pytest.raises(ValueError, match="B: a 64 x 32 window"):
        blas.gpu_trmm("d", 0, 1, 0, 0, 64, 32, 1.0, A, 64, small, 64)
    with pytest.raises(ValueError, match="A: a 64 x 64 window"):
        blas.gpu_syrk("d", 1, 0, 64, 64, 1.0, B, 64, 0.0, A, 64)
    with pytest.raises(ValueError, match="work"):
        blas.gpu_symm("d", 0, 1, 64, 32, 1.0, A, 64, B, 64, 0.0, B, 64, small)
    with pytest.raises(ValueError, match="A: a 65 x 64 window"):
        blas.gpu_dgetrf(65, 64, A, 65)
    # a view counts from its own first element to the end of the storage
    assert blas.room(A[64:]) == (64 * 64 - 64) * 8
    with pytest.raises(ValueError, match="time_gemm: B is a 64 x 32 window"):
        bench.time_gemm("d", "N", "N", 64, 32, 64, 1.0, 0.0, [bench.operand_set(A, small, B)], 64, 64, 64, 1, 1, 0)
