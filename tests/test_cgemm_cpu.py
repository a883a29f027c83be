"""Complex GEMM without a GPU: the oracle's complex instantiation of the GEMM
frame against the committed outputs of the reference, against the compiled
reference where it has been built, against exact and numpy results, the
netlib complex tester's sweep and criterion, and the error exits of the
library's zgemm_ / cgemm_ / cblas_?gemm symbols."""
import hashlib
import itertools
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import netlib
from golden.golden_cases import CGEMM_CASES, cgemm_operands
from ulmblas_amd import blas, lib

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(
    not os.path.exists(os.path.join(os.path.dirname(GOLDEN), "..", "oracle", "_ref", "libulmref_iface.so")),
    reason="oracle/_ref not built (reference tree absent)")


def test_golden_bit_exact(oracle):
    """tests/golden/cgemm.json: sha256 of the whole C window (padding included)
    after the compiled reference's ulmBLAS::gemm on complex operands; C holds
    NaN where beta == 0 says it must not be read."""
    with open(os.path.join(GOLDEN, "cgemm.json")) as f:
        want = json.load(f)
    assert len(want) == len(CGEMM_CASES)
    for case in CGEMM_CASES:
        A, B, Cm = cgemm_operands(case)
        oracle.cgemm(case["variant"], case["ta"], case["tb"], case["m"], case["n"], case["k"], case["alpha"], A,
                     case["lda"], B, case["ldb"], case["beta"], Cm, case["ldc"], blocksize=case["blocksize"])
        assert hashlib.sha256(Cm.tobytes(order="F")).hexdigest() == want[case["key"]], case["key"]


@needs_ref
def test_live_reference(oracle):
    """The reference's templates and its own zgemm_ / cgemm_ / cblas_?gemm objects."""
    rng = np.random.default_rng(7)

    def mk(dt, ld, cols):
        r = np.float64 if dt == np.complex128 else np.float32
        z = rng.uniform(-1, 1, (ld, max(cols, 1))).astype(r) + 1j * rng.uniform(-1, 1, (ld, max(cols, 1))).astype(r)
        return np.asfortranarray(z.astype(dt))

    for var, dt in (("z", np.complex128), ("c", np.complex64)):
        for (m, n, k) in [(0, 3, 2), (5, 7, 0), (5, 7, 3), (33, 40, 50), (193, 5, 385), (3, 390, 200)]:
            for ta, tb in itertools.product("NTCR", "NTCR"):
                for alpha, beta in ((1.0, 0.0), (0.7 - 0.9j, 1.3 - 1.1j), (0.0, 1.3 - 1.1j), (0.5, 2.0)):
                    ra, ca = (k, m) if ta in "TC" else (m, k)
                    rb, cb = (n, k) if tb in "TC" else (k, n)
                    lda, ldb, ldc = max(ra, 1) + 2, max(rb, 1) + 1, max(m, 1) + 3
                    A, B, C0 = mk(dt, lda, ca), mk(dt, ldb, cb), mk(dt, ldc, n)
                    C1, C2, C3 = C0.copy(order="F"), C0.copy(order="F"), C0.copy(order="F")
                    oracle.cgemm(var, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C1, ldc)
                    oracle.ref_cgemm(var, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C2, ldc)
                    oracle.ref_f77_cgemm(var, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C3, ldc)
                    assert C1.tobytes() == C2.tobytes() == C3.tobytes(), (var, m, n, k, ta, tb, alpha, beta)
    # the C interface in both storage orders: row-major is the swapped column-major call
    m, n, k = 9, 7, 11
    for ta, tb in itertools.product("NTCR", "NTCR"):
        cta, ctb = blas.TRANS_OF_CHAR[ta], blas.TRANS_OF_CHAR[tb]
        ra, ca = (k, m) if ta in "TC" else (m, k)
        rb, cb = (n, k) if tb in "TC" else (k, n)
        A, B, C0 = mk(np.complex128, ra + 1, ca), mk(np.complex128, rb + 2, cb), mk(np.complex128, m + 1, n)
        C1, C2 = C0.copy(order="F"), C0.copy(order="F")
        oracle.cgemm("z", ta, tb, m, n, k, 0.7 - 0.9j, A, ra + 1, B, rb + 2, 1.3 - 1.1j, C1, m + 1)
        oracle.ref_cblas_cgemm("z", blas.CblasColMajor, cta, ctb, m, n, k, 0.7 - 0.9j, A, ra + 1, B, rb + 2, 1.3 - 1.1j,
                               C2, m + 1)
        assert C1.tobytes() == C2.tobytes(), (ta, tb)
        # row-major: the same memory is the transposed problem
        # (C read row-major is the n x m matrix C^T = op(B)^T op(A)^T: operands and flags change places)
        C4 = C0.copy(order="F")
        oracle.ref_cblas_cgemm("z", blas.CblasRowMajor, ctb, cta, n, m, k, 0.7 - 0.9j, B, rb + 2, A, ra + 1,
                               1.3 - 1.1j, C4, m + 1)
        assert C4.tobytes() == C1.tobytes(), ("row-major", ta, tb)


def test_exact_small_integers(oracle):
    """Gaussian integers: every product and sum is exact, so the result is the
    exact one whatever the order of summation -- a wrong conjugation, sign or
    transposition cannot hide in rounding."""
    rng = np.random.default_rng(3)
    m, n, k = 6, 5, 7

    def gi(rows, cols):
        return np.asfortranarray(rng.integers(-9, 10, (rows, cols)) + 1j * rng.integers(-9, 10, (rows, cols)))

    for var, dt in (("z", np.complex128), ("c", np.complex64)):
        for ta, tb in itertools.product("NTCR", "NTCR"):
            A = gi(*((k, m) if ta in "TC" else (m, k))).astype(dt)
            B = gi(*((n, k) if tb in "TC" else (k, n))).astype(dt)
            C0 = gi(m, n).astype(dt)
            alpha, beta = 2 - 3j, -1 + 2j
            opa = A.T if ta in "TC" else A
            opa = opa.conj() if ta in "CR" else opa
            opb = B.T if tb in "TC" else B
            opb = opb.conj() if tb in "CR" else opb
            want = np.zeros((m, n), dtype=object)
            for i in range(m):
                for j in range(n):
                    acc_re, acc_im = Fraction(0), Fraction(0)
                    for l in range(k):
                        ar, ai = int(opa[i, l].real), int(opa[i, l].imag)
                        br, bi = int(opb[l, j].real), int(opb[l, j].imag)
                        acc_re += ar * br - ai * bi
                        acc_im += ar * bi + ai * br
                    cr, ci = int(C0[i, j].real), int(C0[i, j].imag)
                    re = 2 * acc_re + 3 * acc_im + (-1) * cr - 2 * ci
                    im = 2 * acc_im - 3 * acc_re + (-1) * ci + 2 * cr
                    want[i, j] = complex(int(re), int(im))
            Cm = C0.copy(order="F")
            oracle.cgemm(var, ta, tb, m, n, k, alpha, np.asfortranarray(A), A.shape[0], np.asfortranarray(B),
                         B.shape[0], beta, Cm, m)
            assert np.array_equal(Cm, want.astype(dt)), (var, ta, tb)


@pytest.mark.parametrize("prec", ["z", "c"])
def test_netlib_sweep_through_oracle(oracle, prec):
    """ZCHK1 / CCHK1 (test/F77/zblat3.f:411-600): every call of the sweep, the
    tester's ratio < 16, padding untouched, A and B unchanged."""
    dt = np.complex128 if prec == "z" else np.complex64
    params = netlib.ZBLAT3
    worst, calls = 0.0, 0
    for c in netlib.chk1_cases(params, dt):
        cc = c["cc"].copy(order="F")
        oracle.cgemm(prec, c["transa"], c["transb"], c["m"], c["n"], c["k"], c["alpha"], c["aa"], c["lda"], c["bb"],
                     c["ldb"], c["beta"], cc, c["ldc"])
        calls += 1
        m, n, k = c["m"], c["n"], c["k"]
        assert np.array_equal(cc[m:], c["cc"][m:])
        if m > 0 and n > 0:
            err, _ = netlib.zmmch(c["transa"], c["transb"], m, n, k, c["alpha"], c["aa"], c["bb"], c["beta"], c["cc"],
                                  cc, dt)
            worst = max(worst, err)
    assert calls == len(params["idim"]) ** 3 * 81
    assert worst < params["thresh"], worst


def test_generator_known_values():
    """ZBEG by hand (zblat3.f:3309-3335): I = 7*891 mod 1000 = 237, J = 7*457 mod
    1000 = 199 -> (237-500)/1001, (199-500)/1001; the fifth call takes two steps."""
    z = netlib.ZBeg()
    v = z.take(6)
    assert v[0] == complex((237 - 500) / 1001.0, (199 - 500) / 1001.0)
    i, j = 7, 7
    seq = []
    for call in range(1, 7):
        i, j = i * 891 % 1000, j * 457 % 1000
        if call == 5:
            i, j = i * 891 % 1000, j * 457 % 1000
        seq.append(complex((i - 500) / 1001.0, (j - 500) / 1001.0))
    assert np.array_equal(v, np.array(seq))


def test_error_exit_tables(oracle):
    """ZCHKE's ZGEMM block and c_z3chke.c's cblas_zgemm block against the info functions."""
    for args, info in netlib.F77_ZGEMM_ERROR_EXITS:
        assert oracle.f77_info(*args) == info, args
    assert len(netlib.F77_ZGEMM_ERROR_EXITS) == 60


@pytest.mark.parametrize("prec", ["z", "c"])
def test_library_error_exits(prec, xerbla):
    dt = np.complex128 if prec == "z" else np.complex64
    name = f"{prec.upper()}GEMM ".encode()

    def fresh():
        return np.full((2, 2), 7.0 + 3.0j, dtype=dt, order="F")

    for (ta, tb, m, n, k, lda, ldb, ldc), info in netlib.F77_ZGEMM_ERROR_EXITS:
        xerbla.capture_reset()
        a, b, c = fresh(), fresh(), fresh()
        blas.cgemm_(prec, ta, tb, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, ldc)
        assert xerbla.capture_count() == 1 and xerbla.capture_last_info() == info, (ta, tb, m, n, k)
        assert xerbla.capture_last_name() == name
        assert (c == 7.0 + 3.0j).all()
    for args, info in netlib.CBLAS_ERROR_EXITS:
        order, ta, tb, m, n, k, lda, ldb, ldc = args
        xerbla.capture_reset()
        a, b, c = fresh(), fresh(), fresh()
        blas.cblas_cgemm(prec, order, ta, tb, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, ldc)
        assert xerbla.capture_count() == 1, args
        assert netlib.cblas_tester_info(order, xerbla.capture_last_info()) == info, args
        assert xerbla.capture_last_name() == f"cblas_{prec}gemm".encode()
        assert (c == 7.0 + 3.0j).all()


def test_library_nothing_to_do(xerbla):
    """m == 0, n == 0, or alpha == 0 / k == 0 with beta == 1: nothing is written
    and no device is needed (ulmblas/level3/gemm.tcc:52-55)."""
    c0 = np.asfortranarray(np.arange(16.0).reshape((4, 4)) * (1 + 2j))
    a = np.ones((4, 4), dtype=np.complex128, order="F")
    for (m, n, k, alpha, beta) in [(0, 3, 3, 1.0, 0.0), (3, 0, 3, 1.0, 0.0), (3, 3, 0, 1.0, 1.0), (3, 3, 3, 0.0, 1.0)]:
        c = c0.copy(order="F")
        blas.cgemm_("z", "C", "R", m, n, k, alpha, a, 4, a, 4, beta, c, 4)
        blas.cblas_cgemm("z", blas.CblasRowMajor, 113, 111, m, n, k, alpha, a, 4, a, 4, beta, c, 4)
        blas.ulmblas_cgemm("z", 111, 114, m, n, k, alpha, a, 4, a, 4, beta, c, 4, prefix="ATL_")
        assert c.tobytes() == c0.tobytes()
    assert xerbla.capture_count() == 0
    L = lib.load()
    one = np.array([1.0, 0.0])
    p = one.ctypes.data
    assert L.ulmblas_gpu_zgemm(111, 111, -1, 1, 1, p, None, 1, None, 1, p, None, 1, None, None) == 1
    assert L.ulmblas_gpu_zgemm(110, 111, 1, 1, 1, p, None, 1, None, 1, p, None, 1, None, None) == 1
    assert L.ulmblas_gpu_zgemm(112, 111, 4, 2, 3, p, None, 2, None, 3, p, None, 4, None, None) == 1
    assert L.ulmblas_gpu_zgemm(111, 111, 0, 5, 5, p, None, 1, None, 5, p, None, 1, None, None) == 0
    assert L.ulmblas_gpu_zgemm_worksize(111, 8, 4, 2) == 4 * 8 * 2 * 8
    assert L.ulmblas_gpu_zgemm_worksize(113, 8, 4, 2) == 4 * 8 * 2 * 8 + 2 * 2 * 4 * 8
    assert L.ulmblas_gpu_cgemm_worksize(112, 8, 4, 2) == 4 * 8 * 2 * 4 + 2 * 2 * 4 * 4
