"""The CPU oracle against outputs of the reference itself.

1. Committed golden fixtures (tests/golden): results of ulmBLAS::gemm compiled
   from the reference's headers, production block sizes and the three small
   block-size variants of its own test suite.  Bit-exact.
2. Where oracle/_ref has been built (the container that has the reference
   tree), the same comparison live on further shapes, plus the reference's
   dgemm_/sgemm_/cblas_* interface objects against the oracle's restatement of
   the interface layer.
"""
import hashlib
import json
import os

import numpy as np
import pytest

from golden.golden_cases import LARGE_CASES, SMALL_CASES, operands
from ulmblas_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _run_oracle(O, case):
    A, B, C0 = operands(case)
    Cm = C0.copy(order="F")
    bs = case["blocksize"]
    O.gemm(case["variant"], case["ta"], case["tb"], case["m"], case["n"], case["k"], case["alpha"], A, case["lda"], B,
           case["ldb"], case["beta"], Cm, case["ldc"], blocksize=bs)
    return Cm


def test_small_golden_bit_exact(oracle):
    data = np.load(os.path.join(GOLDEN, "gemm_small.npz"))
    assert len(data.files) == len(SMALL_CASES)
    for case in SMALL_CASES:
        got = _run_oracle(oracle, case)
        want = data[case["key"]]
        assert got.tobytes(order="F") == want.tobytes(order="F"), case["key"]


def test_large_golden_bit_exact(oracle):
    with open(os.path.join(GOLDEN, "gemm_large.json")) as f:
        want = json.load(f)
    assert len(want) == len(LARGE_CASES)
    for case in LARGE_CASES:
        got = _run_oracle(oracle, case)
        flat = got.reshape(-1, order="F")
        head = [float(x).hex() for x in flat[:4].astype(np.float64)]
        assert head == want[case["key"]]["head"], case["key"]
        assert hashlib.sha256(got.tobytes(order="F")).hexdigest() == want[case["key"]]["sha256"], case["key"]


def test_golden_outputs_are_sane():
    """The fixtures themselves: no NaN leaked from the NaN-filled C of the
    beta == 0 cases, and the padding rows still hold the sentinel."""
    data = np.load(os.path.join(GOLDEN, "gemm_small.npz"))
    for case in SMALL_CASES:
        want = data[case["key"]]
        m = case["m"]
        assert not np.isnan(want[:m, :]).any(), case["key"]
        assert (want[m:, :] == -2560000000.0).all(), case["key"]


needs_ref = pytest.mark.skipif(not os.path.exists(os.path.join(os.path.dirname(GOLDEN), "..", "oracle", "_ref",
                                                               "libulmref.so")),
                               reason="oracle/_ref not built (reference tree absent)")


@needs_ref
@pytest.mark.parametrize("variant", ["d", "s", "s_f64"])
def test_live_reference_bit_exact(oracle, variant):
    dt = np.float64 if variant == "d" else np.float32
    shapes = [(4, 4, 4), (100, 100, 100), (384, 384, 384), (385, 4097 // 8, 385), (33, 4100, 7), (800, 3, 1153)]
    for (m, n, k) in shapes:
        for ta in "NT":
            for tb in "NT":
                for alpha, beta in [(1.0, 0.0), (1.5, 0.5), (-1.0, 1.0), (0.0, 0.0)]:
                    ra, ca = (k, m) if ta == "T" else (m, k)
                    rb, cb = (n, k) if tb == "T" else (k, n)
                    A = synth.matrix(21, ra, ca, ra + 1, dtype=dt)
                    B = synth.matrix(22, rb, cb, rb + 2, dtype=dt)
                    C0 = synth.matrix(23, m, n, m + 3, dtype=dt)
                    if beta == 0.0:
                        C0[:m, :] = np.nan
                    c1, c2 = C0.copy(order="F"), C0.copy(order="F")
                    oracle.gemm(variant, ta, tb, m, n, k, alpha, A, ra + 1, B, rb + 2, beta, c1, m + 3)
                    oracle.ref_gemm(variant, ta, tb, m, n, k, alpha, A, ra + 1, B, rb + 2, beta, c2, m + 3)
                    assert c1.tobytes(order="F") == c2.tobytes(order="F"), (variant, m, n, k, ta, tb, alpha, beta)


@needs_ref
def test_live_reference_interfaces(oracle, xerbla):
    """dgemm_/sgemm_/cblas_dgemm/cblas_sgemm objects of the reference against
    the oracle's interface layer: trans decoding incl. lower case and 'C',
    AtlasConj, the row-major swap, and sgemm_'s double accumulation."""
    L = oracle.ref("libulmref_iface.so")
    m, n, k = 37, 29, 50
    for prec, dt in (("d", np.float64), ("s", np.float32)):
        for ta in "NnTtCc":
            for tb in "NtC":
                tra, trb = ta.upper() in "TC", tb.upper() in "TC"
                ra, ca = (k, m) if tra else (m, k)
                rb, cb = (n, k) if trb else (k, n)
                A = synth.matrix(31, ra, ca, ra + 2, dtype=dt)
                B = synth.matrix(32, rb, cb, rb + 2, dtype=dt)
                C0 = synth.matrix(33, m, n, m + 2, dtype=dt)
                c1, c2 = C0.copy(order="F"), C0.copy(order="F")
                f = oracle.dgemm_f77 if prec == "d" else oracle.sgemm_f77
                assert f(ta, tb, m, n, k, 0.7, A, ra + 2, B, rb + 2, 1.3, c1, m + 2) == 0
                oracle.ref_f77_gemm(prec, ta, tb, m, n, k, 0.7, A, ra + 2, B, rb + 2, 1.3, c2, m + 2)
                assert c1.tobytes(order="F") == c2.tobytes(order="F"), (prec, ta, tb)
        # CBLAS, both orders; numpy C-ordered arrays are row-major windows
        for order in (oracle.COL_MAJOR, oracle.ROW_MAJOR):
            for ta in (oracle.NO_TRANS, oracle.TRANS, oracle.CONJ_TRANS, oracle.ATLAS_CONJ):
                for tb in (oracle.NO_TRANS, oracle.TRANS):
                    tra = ta in (oracle.TRANS, oracle.CONJ_TRANS)
                    trb = tb in (oracle.TRANS, oracle.CONJ_TRANS)
                    ra, ca = (k, m) if tra else (m, k)      # logical shape of stored A
                    rb, cb = (n, k) if trb else (k, n)
                    if order == oracle.ROW_MAJOR:           # leading dimension runs along a row
                        lda, ldb, ldc = ca + 2, cb + 2, n + 2
                        A = synth.uniform(41, ra * lda, dtype=dt)
                        B = synth.uniform(42, rb * ldb, dtype=dt)
                        C0 = synth.uniform(43, m * ldc, dtype=dt)
                    else:
                        lda, ldb, ldc = ra + 2, rb + 2, m + 2
                        A = synth.uniform(41, ca * lda, dtype=dt)
                        B = synth.uniform(42, cb * ldb, dtype=dt)
                        C0 = synth.uniform(43, n * ldc, dtype=dt)
                    c1, c2 = C0.copy(), C0.copy()
                    f = oracle.cblas_dgemm if prec == "d" else oracle.cblas_sgemm
                    g = L.cblas_dgemm if prec == "d" else L.cblas_sgemm
                    assert f(order, ta, tb, m, n, k, 0.7, A, lda, B, ldb, 1.3, c1, ldc) == 0
                    g(order, ta, tb, m, n, k, 0.7, A.ctypes.data, lda, B.ctypes.data, ldb, 1.3, c2.ctypes.data, ldc)
                    assert c1.tobytes() == c2.tobytes(), (prec, order, ta, tb)
    assert xerbla.capture_count() == 0


@needs_ref
def test_live_reference_error_exits(oracle, xerbla):
    """The reference's own interface objects report the info codes of the
    testers' error-exit lists; the oracle's check functions agree call by call."""
    import ctypes as C
    from netlib import CBLAS_ERROR_EXITS, F77_ERROR_EXITS, cblas_tester_info
    L = oracle.ref("libulmref_iface.so")
    buf = np.zeros(4)
    for (ta, tb, m, n, k, lda, ldb, ldc), info in F77_ERROR_EXITS:
        xerbla.capture_reset()
        oracle.ref_f77_gemm("d", ta, tb, m, n, k, 0.0, buf, lda, buf, ldb, 0.0, buf, ldc)
        assert xerbla.capture_count() == 1 and xerbla.capture_last_info() == info
        assert xerbla.capture_last_name() == b"DGEMM "
        assert oracle.f77_info(ta, tb, m, n, k, lda, ldb, ldc) == info
    for (order, ta, tb, m, n, k, lda, ldb, ldc), info in CBLAS_ERROR_EXITS:
        xerbla.capture_reset()
        L.cblas_dgemm(order, ta, tb, m, n, k, 0.0, buf.ctypes.data, lda, buf.ctypes.data, ldb, 0.0, buf.ctypes.data,
                      ldc)
        assert xerbla.capture_count() == 1
        assert cblas_tester_info(order, xerbla.capture_last_info()) == info
        assert xerbla.capture_last_name() == b"cblas_dgemm"
        assert oracle.cblas_info(order, ta, tb, m, n, k, lda, ldb, ldc) == xerbla.capture_last_info()
