"""The host entry points beside dgemm_ / sgemm_ on operands large enough for
the streamed paths: dtrsm_ / dtrmm_ send B in panels of right-hand sides
(columns for the left side, rows for the right side), each panel up, solved
and on its way back while its neighbours travel; dsyrk_ / dsymm_ / zgemm_ /
ulmblas_dgetrf move their operands through the pinned rings.  Same checks as
for the small shapes of the conformance sweeps, on leading dimensions with
padding whose sentinels must survive: parity with the oracle where it
finishes in seconds (a panel of right-hand sides), the reference tester's
residual ratios, and numpy in float64 under the bound of gpu_util.TOL_C."""
import numpy as np
import pytest

import netlib
from gpu_util import TOL_C
from test_gpu_trsm import TOL_X, forward_ratio, triangle
from ulmblas_amd import blas, synth

pytestmark = pytest.mark.gpu

SENTINEL = -2560000000.0


def _padded(seed, rows, cols, ld, dtype=np.float64):
    a = synth.matrix(seed, rows, cols, ld, dtype=dtype)
    a[rows:] = SENTINEL
    return a


@pytest.mark.parametrize("side,uplo,trans", [("L", "L", "N"), ("L", "U", "T"), ("R", "U", "N"), ("R", "L", "T")])
def test_dtrsm_streamed(side, uplo, trans, oracle):
    """4200 right-hand sides in two panels (2304 and 1896)."""
    m = n = 4200
    na = m if side == "L" else n
    lda, ldb = na + 3, m + 5
    full, window = triangle(81, uplo, "N", na, lda, np.float64)
    B0 = _padded(82, m, n, ldb)
    W0 = window.copy(order="F")
    got = B0.copy(order="F")
    blas.dtrsm_(side, uplo, trans, "N", m, n, 0.7, window, lda, got, ldb)
    assert window.tobytes(order="F") == W0.tobytes(order="F")
    assert np.array_equal(got[m:], B0[m:]), "padding rows of B were written"
    assert not np.isnan(got[:m]).any()
    err = netlib.trsm_check(side, trans, m, n, 0.7, full, B0, got, np.float64)
    assert err < na / 16, (side, uplo, trans, err)
    # parity with the oracle on right-hand sides from both panels
    if side == "L":
        for c0 in (0, n - 48):
            want = B0[:, c0:c0 + 48].copy(order="F")
            oracle.trsm("d", side, uplo, trans, "N", m, 48, 0.7, window, lda, want, ldb)
            r = forward_ratio(side, trans, full, got[:m, c0:c0 + 48], want[:m], np.float64)
            assert r <= TOL_X, (side, uplo, trans, c0, r)
    else:
        for r0 in (0, m - 48):
            want = np.asfortranarray(B0[r0:r0 + 48, :].copy())
            oracle.trsm("d", side, uplo, trans, "N", 48, n, 0.7, window, lda, want, 48)
            r = forward_ratio(side, trans, full, got[r0:r0 + 48], want, np.float64)
            assert r <= TOL_X, (side, uplo, trans, r0, r)


@pytest.mark.parametrize("side,uplo,trans", [("L", "U", "N"), ("R", "L", "N")])
def test_strsm_streamed(side, uplo, trans):
    """The same paths on four-byte elements (twice the columns per pinned chunk):
    6300 right-hand sides in three panels, the tester's residual."""
    m, n = (3000, 6300) if side == "L" else (6300, 3000)
    na = m if side == "L" else n
    lda, ldb = na + 1, m + 3
    full, window = triangle(92, uplo, "N", na, lda, np.float32)
    B0 = _padded(93, m, n, ldb, dtype=np.float32)
    got = B0.copy(order="F")
    blas.strsm_(side, uplo, trans, "N", m, n, 0.7, window, lda, got, ldb)
    assert np.array_equal(got[m:], B0[m:]), "padding rows of B were written"
    assert not np.isnan(got[:m]).any()
    err = netlib.trsm_check(side, trans, m, n, 0.7, full, B0, got, np.float32)
    assert err < na / 16, (side, uplo, trans, err)


def test_dtrmm_streamed():
    m, n = 2900, 3100
    for side, uplo, trans in (("L", "U", "N"), ("R", "L", "T")):
        na = m if side == "L" else n
        lda, ldb = na + 2, m + 6
        full, window = triangle(83, uplo, "N", na, lda, np.float64)
        B0 = _padded(84, m, n, ldb)
        got = B0.copy(order="F")
        blas.trmm_("d", side, uplo, trans, "N", m, n, -0.5, window, lda, got, ldb)
        assert np.array_equal(got[m:], B0[m:])
        t = full.T if trans == "T" else full
        b = B0[:m].astype(np.float64)
        want = -0.5 * (t @ b if side == "L" else b @ t)
        g = 0.5 * (np.abs(t) @ np.abs(b) if side == "L" else np.abs(b) @ np.abs(t))
        assert (np.abs(got[:m] - want) <= TOL_C * na * np.finfo(np.float64).eps * g).all(), (side, uplo, trans)


@pytest.mark.parametrize("uplo,trans", [("L", "N"), ("U", "T")])
def test_dsyrk_streamed(uplo, trans):
    n, k = 3000, 2600
    ra, ca = (k, n) if trans == "T" else (n, k)
    lda, ldc = ra + 3, n + 4
    A = _padded(85, ra, ca, lda)
    C0 = _padded(86, n, n, ldc)
    mask = netlib.triangle_mask(uplo, n)
    C0[:n][~mask] = np.nan                       # the other triangle is neither read nor written
    got = C0.copy(order="F")
    blas.syrk_("d", uplo, trans, n, k, 0.7, A, lda, 1.3, got, ldc)
    assert np.array_equal(got[n:], C0[n:])
    assert np.isnan(got[:n][~mask]).all() and not np.isnan(got[:n][mask]).any()
    a = (A[:ra].T if trans == "T" else A[:ra]).astype(np.float64)
    c0 = np.nan_to_num(C0[:n])
    want = 0.7 * (a @ a.T) + 1.3 * c0
    g = 0.7 * (np.abs(a) @ np.abs(a).T) + 1.3 * np.abs(c0)
    bad = np.abs(got[:n] - want) > TOL_C * k * np.finfo(np.float64).eps * g
    assert not bad[mask].any()


def test_dsymm_streamed():
    """Two panels of B and C on either side (columns for the left side, rows for the right side)."""
    m, n = 3000, 3100
    for side, uplo in (("L", "U"), ("R", "L")):
        na = m if side == "L" else n
        lda, ldb, ldc = na + 3, m + 1, m + 2
        A = _padded(87, na, na, lda)
        amask = netlib.triangle_mask(uplo, na)
        full = np.where(amask, A[:na], A[:na].T).astype(np.float64)
        A[:na][~amask] = np.nan
        B = _padded(88, m, n, ldb)
        C0 = _padded(89, m, n, ldc)
        got = C0.copy(order="F")
        blas.symm_("d", side, uplo, m, n, 0.7, A, lda, B, ldb, 1.3, got, ldc)
        assert np.array_equal(got[m:], C0[m:]) and not np.isnan(got[:m]).any()
        b = B[:m].astype(np.float64)
        want = 0.7 * (full @ b if side == "L" else b @ full) + 1.3 * C0[:m]
        g = 0.7 * (np.abs(full) @ np.abs(b) if side == "L" else np.abs(b) @ np.abs(full)) + 1.3 * np.abs(C0[:m])
        assert (np.abs(got[:m] - want) <= TOL_C * na * np.finfo(np.float64).eps * g).all(), (side, uplo)


@pytest.mark.parametrize("shape", [(1500, 1700, 1900), (2900, 3000, 700)], ids=["whole_operands", "panels_of_c"])
def test_zgemm_streamed(shape):
    """The smaller shape moves whole operands through the rings; the larger one
    (8.7 M elements of C) is cut into five column panels of C, op(B) brought
    into the product's form panel by panel."""
    m, n, k = shape
    rng = np.random.default_rng(90)
    for ta, tb, beta in (("N", "N", 0.3 + 1.1j), ("C", "T", -0.5 + 0j), ("T", "R", 0j), ("R", "C", 1.0 + 0j)):
        ra, ca = (k, m) if ta in "TC" else (m, k)
        rb, cb = (n, k) if tb in "TC" else (k, n)
        lda, ldb, ldc = ra + 2, rb + 3, m + 1
        def cplx(rows, cols, ld):
            x = np.asfortranarray(rng.uniform(-1, 1, (ld, cols)) + 1j * rng.uniform(-1, 1, (ld, cols)))
            x[rows:] = SENTINEL
            return x
        A, B, C0 = cplx(ra, ca, lda), cplx(rb, cb, ldb), cplx(m, n, ldc)
        Cin = C0.copy(order="F")
        if beta == 0:
            Cin[:m] = np.nan                        # never read
        got = Cin.copy(order="F")
        alpha = 0.7 - 0.2j
        blas.cgemm_("z", ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, got, ldc)
        assert np.array_equal(got[m:], C0[m:])
        op = {"N": lambda x: x, "T": lambda x: x.T, "C": lambda x: x.conj().T, "R": lambda x: x.conj()}
        a, b = op[ta](A[:ra]), op[tb](B[:rb])
        c0 = C0[:m] if beta != 0 else 0.0
        want = alpha * (a @ b) + beta * c0
        g = abs(alpha) * (np.abs(a) @ np.abs(b)) + abs(beta) * np.abs(c0)
        assert not np.isnan(got[:m]).any()
        assert (np.abs(got[:m] - want) <= 2 * TOL_C * 2 * k * np.finfo(np.float64).eps * g).all(), (ta, tb)


def test_cgemm_streamed_panels():
    """Single-precision complex, five column panels of C."""
    m, n, k = 2900, 3000, 700
    rng = np.random.default_rng(94)
    def cplx(rows, cols, ld):
        x = np.asfortranarray((rng.uniform(-1, 1, (ld, cols)) + 1j * rng.uniform(-1, 1, (ld, cols))).astype(np.complex64))
        x[rows:] = SENTINEL
        return x
    for ta, tb in (("N", "T"), ("C", "N")):
        ra, ca = (k, m) if ta in "TC" else (m, k)
        rb, cb = (n, k) if tb in "TC" else (k, n)
        lda, ldb, ldc = ra + 2, rb + 3, m + 1
        A, B, C0 = cplx(ra, ca, lda), cplx(rb, cb, ldb), cplx(m, n, ldc)
        got = C0.copy(order="F")
        alpha, beta = 0.7 - 0.2j, 0.3 + 1.1j
        blas.cgemm_("c", ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, got, ldc)
        assert np.array_equal(got[m:], C0[m:])
        op = {"N": lambda x: x, "T": lambda x: x.T, "C": lambda x: x.conj().T}
        a, b = op[ta](A[:ra]).astype(np.complex128), op[tb](B[:rb]).astype(np.complex128)
        want = alpha * (a @ b) + beta * C0[:m].astype(np.complex128)
        g = abs(alpha) * (np.abs(a) @ np.abs(b)) + abs(beta) * np.abs(C0[:m])
        assert (np.abs(got[:m] - want) <= 2 * TOL_C * 2 * k * np.finfo(np.float32).eps * g).all(), (ta, tb)


def test_dgetrf_streamed():
    """3000 x 2800: P A = L U under the bound of Gaussian elimination, the
    pivots those of partial pivoting (every multiplier at most 1)."""
    m, n = 3000, 2800
    lda = m + 5
    A0 = _padded(91, m, n, lda)
    A = A0.copy(order="F")
    info, piv = blas.ulmblas_dgetrf(blas.CblasColMajor, m, n, A, lda)
    assert info == 0
    assert np.array_equal(A[m:], A0[m:])
    mn = min(m, n)
    L = np.tril(A[:m, :mn], -1) + np.eye(m, mn)
    U = np.triu(A[:mn, :n])
    assert np.abs(np.tril(A[:m, :mn], -1)).max() <= 1.0
    PA = A0[:m].copy()
    for i, p in enumerate(piv):
        if p != i:
            PA[[i, p]] = PA[[p, i]]
    bound = 2 * mn * np.finfo(np.float64).eps * (np.abs(L) @ np.abs(U))
    assert (np.abs(PA - L @ U) <= bound).all()
