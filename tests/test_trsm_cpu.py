"""The triangular solve without a GPU: the oracle's restatement of
ulmBLAS::trlsm / trusm against the committed outputs of the reference, against
the compiled reference where it has been built, against what the mathematics
fixes, and the error exits of the library's dtrsm_ / cblas_dtrsm."""
import hashlib
import itertools
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import netlib
from golden.golden_cases import TRSM_CASES, trsm_operands
from ulmblas_amd import blas, lib

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(
    not os.path.exists(os.path.join(os.path.dirname(GOLDEN), "..", "oracle", "_ref", "libulmref.so")),
    reason="oracle/_ref not built (reference tree absent)")


def test_golden_bit_exact(oracle):
    """tests/golden/trsm.json: sha256 of B after ulmBLAS::trlsm / trusm of the
    compiled reference, production and small block sizes, three type flavours."""
    with open(os.path.join(GOLDEN, "trsm.json")) as f:
        want = json.load(f)
    assert len(want) == len(TRSM_CASES)
    for case in TRSM_CASES:
        A, B = trsm_operands(case)
        oracle.trsm(case["variant"], case["side"], case["uplo"], case["trans"], case["diag"], case["m"], case["n"],
                    case["alpha"], A, case["lda"], B, case["ldb"], blocksize=case["blocksize"])
        assert hashlib.sha256(B.tobytes(order="F")).hexdigest() == want[case["key"]], case["key"]


@needs_ref
@pytest.mark.parametrize("variant", ["d", "s", "s_f64"])
def test_live_reference_bit_exact(oracle, variant):
    """Element strides the interfaces never produce, shapes around the MC
    boundary, and the F77 interface object of the reference itself."""
    dt = np.float64 if variant == "d" else np.float32
    rng = np.random.default_rng(5)
    for (m, n) in [(1, 1), (7, 5), (33, 17), (385, 9), (400, 70), (770, 13)]:
        for lower, unit, ta, tb in itertools.product((0, 1), repeat=4):
            for alpha in (1.0, 0.0, 0.7):
                lda, ldb = m + 2, (n if tb else m) + 3
                A = np.asfortranarray(rng.uniform(-1, 1, (lda, m)).astype(dt) * dt(min(1.0, 8.0 / m)))
                A[np.arange(m), np.arange(m)] += 2
                B0 = np.asfortranarray(rng.uniform(-1, 1, (ldb, m if tb else n)).astype(dt))
                sa = (lda, 1) if ta else (1, lda)
                sb = (ldb, 1) if tb else (1, ldb)
                B1, B2 = B0.copy(order="F"), B0.copy(order="F")
                oracle.trsm_strided(variant, lower, m, n, alpha, unit, A, sa, B1, sb)
                oracle.ref_trsm_strided(variant, lower, m, n, alpha, unit, A, sa, B2, sb)
                assert B1.tobytes() == B2.tobytes(), (variant, m, n, lower, unit, ta, tb, alpha)
    if variant == "s":
        return
    prec = "d" if variant == "d" else "s"
    f = oracle.dtrsm_f77 if prec == "d" else oracle.strsm_f77
    for (m, n) in [(9, 13), (40, 3)]:
        for side, uplo, trans, diag in itertools.product("LR", "UL", "NTC", "UN"):
            na = m if side == "L" else n
            A = np.asfortranarray(rng.uniform(-1, 1, (na + 1, na)).astype(dt))
            A[np.arange(na), np.arange(na)] += 2
            B0 = np.asfortranarray(rng.uniform(-1, 1, (m + 2, n)).astype(dt))
            B1, B2 = B0.copy(order="F"), B0.copy(order="F")
            assert f(side, uplo, trans, diag, m, n, 0.7, A, na + 1, B1, m + 2) == 0
            oracle.ref_f77_trsm(prec, side, uplo, trans, diag, m, n, 0.7, A, na + 1, B2, m + 2)
            assert B1.tobytes() == B2.tobytes(), (prec, side, uplo, trans, diag, m, n)


def test_brute_force_rational(oracle):
    """Small integer triangles with unit diagonal (or diagonal entries that
    are powers of two) have exactly representable solutions: the oracle must
    hit the solution computed in rational arithmetic bit for bit.  A wrong
    index, a transposed operand or a swapped side fails here."""
    rng = np.random.default_rng(11)
    for side, uplo, trans, diag in itertools.product("LR", "UL", "NT", "UN"):
        m, n = 6, 5
        na = m if side == "L" else n
        T = rng.integers(-3, 4, (na, na)).astype(np.float64)
        T = np.triu(T) if uplo == "U" else np.tril(T)
        d = np.array([1.0, -2.0, 0.5, 4.0, -1.0, 2.0])[:na]
        T[np.arange(na), np.arange(na)] = 1.0 if diag == "U" else d
        B0 = rng.integers(-4, 5, (m, n)).astype(np.float64)
        alpha = 2.0
        opT = T.T if trans == "T" else T
        # exact solve in Fractions
        F = [[Fraction(v) for v in row] for row in opT.tolist()]
        R = [[Fraction(alpha) * Fraction(v) for v in row] for row in B0.tolist()]
        X = [[Fraction(0)] * n for _ in range(m)]
        lower = np.allclose(opT, np.tril(opT))
        if side == "L":
            order = range(na) if lower else range(na - 1, -1, -1)
            for j in range(n):
                for i in order:
                    s = R[i][j] - sum(F[i][l] * X[l][j] for l in range(na) if l != i)
                    X[i][j] = s / F[i][i]
        else:
            order = range(na - 1, -1, -1) if lower else range(na)
            for i in range(m):
                for j in order:
                    s = R[i][j] - sum(X[i][l] * F[l][j] for l in range(na) if l != j)
                    X[i][j] = s / F[j][j]
        want = np.array([[float(v) for v in row] for row in X])
        A = np.asfortranarray(T.copy())
        hide = (np.tril(np.ones((na, na)), -1) if uplo == "U" else np.triu(np.ones((na, na)), 1)).astype(bool)
        if diag == "U":
            hide |= np.eye(na, dtype=bool)
        A[hide] = np.nan                      # must not be read
        B = np.asfortranarray(B0.copy())
        oracle.trsm("d", side, uplo, trans, diag, m, n, alpha, A, na, B, m)
        assert np.array_equal(B, want), (side, uplo, trans, diag)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_netlib_sweep_through_oracle(oracle, prec):
    """DCHK3 for the solve (test/F77/dblat3.f:907-1209, sblat3.f likewise):
    every call of the tester's sweep, checked the tester's way (multiply X
    back, ratio < 16), padding rows and the tester's ROGUE-filled unreferenced
    parts of A left out of the result."""
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    dt = np.float64 if prec == "d" else np.float32
    f = oracle.dtrsm_f77 if prec == "d" else oracle.strsm_f77
    worst, calls = 0.0, 0
    for c in netlib.chk3_cases(params, dt):
        bb = c["bb"].copy(order="F")
        aa = c["aa"].copy(order="F")
        assert f(c["side"], c["uplo"], c["transa"], c["diag"], c["m"], c["n"], c["alpha"], aa, c["lda"], bb,
                 c["ldb"]) == 0
        calls += 1
        assert aa.tobytes() == c["aa"].tobytes()
        assert np.array_equal(bb[c["m"]:], c["bb"][c["m"]:])
        if c["m"] > 0 and c["n"] > 0:
            worst = max(worst, netlib.trsm_check(c["side"], c["transa"], c["m"], c["n"], c["alpha"], c["a"], c["bb"],
                                                 bb, dt))
    assert calls == len(params["idim"]) ** 2 * 72
    assert worst < params["thresh"], worst


def test_special_cases(oracle):
    rng = np.random.default_rng(3)
    A = np.asfortranarray(np.triu(rng.uniform(1, 2, (5, 5))))
    B0 = np.asfortranarray(rng.uniform(-1, 1, (5, 4)))
    # alpha == 0: zeros, A and B not read (NaN everywhere)
    B = np.full((5, 4), np.nan, order="F")
    oracle.trsm("d", "L", "U", "N", "N", 5, 4, 0.0, np.full((5, 5), np.nan, order="F"), 5, B, 5)
    assert (B == 0).all()
    # identity triangle: X = alpha * B exactly
    B = B0.copy(order="F")
    oracle.trsm("d", "R", "L", "T", "N", 5, 4, 0.5, np.asfortranarray(np.eye(4)), 4, B, 5)
    assert np.array_equal(B, 0.5 * B0)
    # diagonal triangle: division by the diagonal, through the reciprocal
    D = np.asfortranarray(np.diag([2.0, 4.0, 0.5, 8.0, 1.0]))
    B = B0.copy(order="F")
    oracle.trsm("d", "L", "L", "N", "N", 5, 4, 1.0, D, 5, B, 5)
    assert np.array_equal(B, B0 / np.diag(D)[:, None])
    # right side equals the left side of the transposed problem, bit for bit
    Bl = np.asfortranarray(B0.T.copy())                       # 4 x 5
    Br = B0.copy(order="F")                                   # 5 x 4, X * A^T... uses A 4 x 4
    A4 = np.asfortranarray(np.triu(rng.uniform(1, 2, (4, 4))))
    oracle.trsm("d", "L", "U", "T", "N", 4, 5, 0.7, A4, 4, Bl, 4)      # A4^T X = 0.7 B^T
    oracle.trsm("d", "R", "U", "N", "N", 5, 4, 0.7, A4, 4, Br, 5)      # X A4 = 0.7 B
    assert np.array_equal(Bl.T, Br)


def test_row_major_is_flipped_col_major(oracle):
    """interfaces/blas/C/trsm.cc:452-458."""
    rng = np.random.default_rng(8)
    m, n = 6, 4
    for side, uplo, trans, diag in itertools.product((141, 142), (121, 122), (111, 112), (131, 132)):
        na = m if side == 141 else n
        A = rng.uniform(1, 2, (na, na))
        B0 = rng.uniform(-1, 1, (m, n))
        Brow = B0.copy(order="C")                             # row-major m x n, ld = n
        assert oracle.cblas_dtrsm(101, side, uplo, trans, diag, m, n, 0.7, np.ascontiguousarray(A), na, Brow, n) == 0
        Bcol = np.asfortranarray(B0)
        assert oracle.cblas_dtrsm(102, side, uplo, trans, diag, m, n, 0.7, np.asfortranarray(A), na, Bcol, m) == 0
        # same mathematical problem, different association order: equal within rounding
        np.testing.assert_allclose(Brow, Bcol, rtol=1e-12, atol=1e-13)
        # and exactly the flipped column-major call on the same memory
        Bflip = B0.copy(order="C")
        flip_side = 142 if side == 141 else 141
        flip_uplo = 122 if uplo == 121 else 121
        assert oracle.cblas_dtrsm(102, flip_side, flip_uplo, trans, diag, n, m, 0.7, np.ascontiguousarray(A), na,
                                  Bflip, n) == 0
        assert Brow.tobytes() == Bflip.tobytes()


def test_error_exit_tables(oracle):
    for args, info in netlib.F77_TRSM_ERROR_EXITS:
        assert oracle.f77_trsm_info(*args) == info, args
    for args, info in netlib.CBLAS_TRSM_ERROR_EXITS:
        assert netlib.cblas_tester_info_trsm(args[0], oracle.cblas_trsm_info(*args)) == info, args


# ---------------------------------------------------------------------------
# the library's entry points (no GPU needed: error exits and empty problems)
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("prec", ["d", "s"])
def test_library_f77_error_exits(prec, xerbla):
    """DCHKE's DTRSM block, test/F77/dblat3.f:2098-2205."""
    dt = np.float64 if prec == "d" else np.float32
    f = blas.dtrsm_ if prec == "d" else blas.strsm_
    name = b"DTRSM " if prec == "d" else b"STRSM "
    for (side, uplo, ta, diag, m, n, lda, ldb), info in netlib.F77_TRSM_ERROR_EXITS:
        xerbla.capture_reset()
        a = np.full((2, 2), 7.0, dtype=dt, order="F")
        b = a.copy(order="F")
        f(side, uplo, ta, diag, m, n, 1.0, a, lda, b, ldb)
        assert xerbla.capture_count() == 1
        assert xerbla.capture_last_info() == info, (side, uplo, ta, diag, m, n, lda, ldb)
        assert xerbla.capture_last_name() == name
        assert (b == 7.0).all()


@pytest.mark.parametrize("prec", ["d", "s"])
def test_library_cblas_error_exits(prec, xerbla):
    """test/C/c_d3chke.c:730-1009."""
    dt = np.float64 if prec == "d" else np.float32
    f = blas.cblas_dtrsm if prec == "d" else blas.cblas_strsm
    name = b"cblas_dtrsm" if prec == "d" else b"cblas_strsm"
    for args, info in netlib.CBLAS_TRSM_ERROR_EXITS:
        order, side, uplo, ta, diag, m, n, lda, ldb = args
        xerbla.capture_reset()
        a = np.full(4, 7.0, dtype=dt)
        b = a.copy()
        f(order, side, uplo, ta, diag, m, n, 1.0, a, lda, b, ldb)
        assert xerbla.capture_count() == 1, args
        assert netlib.cblas_tester_info_trsm(order, xerbla.capture_last_info()) == info, args
        assert xerbla.capture_last_name() == name
        assert (b == 7.0).all()


def test_library_info_codes_match_oracle(oracle, xerbla):
    a = np.zeros(4)
    sizes = (-1, 0, 2)
    for side, uplo, ta, diag in itertools.product("LRx", "ULx", "NTcx", "UNx"):
        for m, n in itertools.product(sizes, sizes):
            for lda, ldb in ((1, 1), (2, 1), (1, 2), (2, 2)):
                want = oracle.f77_trsm_info(side, uplo, ta, diag, m, n, lda, ldb)
                if want == 0 and m > 0 and n > 0:
                    continue            # would compute: needs a GPU
                xerbla.capture_reset()
                blas.dtrsm_(side, uplo, ta, diag, m, n, 1.0, a, lda, a, ldb)
                got = xerbla.capture_last_info() if xerbla.capture_count() else 0
                assert got == want, (side, uplo, ta, diag, m, n, lda, ldb)
    for order, side, uplo, ta, diag in itertools.product((101, 102, 7), (141, 142, 0), (121, 122, 0),
                                                         (111, 112, 113, 114, 0), (131, 132, 0)):
        for m, n in itertools.product(sizes, sizes):
            for lda, ldb in ((1, 1), (2, 1), (1, 2), (2, 2)):
                want = oracle.cblas_trsm_info(order, side, uplo, ta, diag, m, n, lda, ldb)
                if want == 0 and m > 0 and n > 0:
                    continue
                xerbla.capture_reset()
                blas.cblas_dtrsm(order, side, uplo, ta, diag, m, n, 1.0, a, lda, a, ldb)
                got = xerbla.capture_last_info() if xerbla.capture_count() else 0
                assert got == want, (order, side, uplo, ta, diag, m, n, lda, ldb)


def test_device_entry_rejects_bad_arguments():
    L = lib.load()
    for (right, m, n, lda, ldb) in [(0, -1, 1, 1, 1), (0, 1, -1, 1, 1), (0, 4, 2, 3, 4), (1, 4, 2, 1, 4),
                                    (0, 4, 2, 4, 3)]:
        assert L.ulmblas_gpu_dtrsm(right, 1, 0, 0, m, n, 1.0, None, lda, None, ldb, None) == 1
        assert L.ulmblas_gpu_last_error() != b""
    assert L.ulmblas_gpu_dtrsm(0, 1, 0, 0, 0, 5, 1.0, None, 1, None, 1, None) == 0
