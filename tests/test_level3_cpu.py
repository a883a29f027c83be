"""Symmetric rank-k update, symmetric product and triangular product without
a GPU: the oracle's restatements against the committed outputs of the
reference, against the compiled reference where it has been built, against
plain numpy under the netlib testers' criterion, and the error exits of the
library's entry points."""
import hashlib
import itertools
import json
import os

import numpy as np
import pytest

import netlib
from golden.golden_cases import L3_CASES, l3_operands, l3_run
from ulmblas_amd import blas, lib

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(
    not os.path.exists(os.path.join(os.path.dirname(GOLDEN), "..", "oracle", "_ref", "libulmref_iface.so")),
    reason="oracle/_ref not built (reference tree absent)")


def test_golden_bit_exact(oracle):
    """tests/golden/level3.json: sha256 of the results of the compiled
    reference's sylrk/syurk, sylr2k/syur2k, sylmm/syumm, trlmm/trumm.  The operands hold NaN
    wherever the routines must not read, so the hashes also pin that."""
    with open(os.path.join(GOLDEN, "level3.json")) as f:
        want = json.load(f)
    assert len(want) == len(L3_CASES)
    for case in L3_CASES:
        ops = l3_operands(case)
        out = l3_run(case, ops, lambda *a, **k: oracle.syrk("d", *a, **k), lambda *a, **k: oracle.symm("d", *a, **k),
                     lambda *a, **k: oracle.trmm("d", *a, **k), lambda *a, **k: oracle.syr2k("d", *a, **k),
                     blocksize=case["blocksize"])
        assert hashlib.sha256(out.tobytes(order="F")).hexdigest() == want[case["key"]]["sha256"], case["key"]
        assert int(np.isnan(out).sum()) == want[case["key"]]["nans"], case["key"]


@needs_ref
def test_live_reference_interfaces(oracle):
    """The reference's own dsyrk_/ssyrk_, dsymm_/ssymm_, dtrmm_/strmm_ objects
    (ssyrk_ and ssymm_ compute in double, strmm_ in float)."""
    rng = np.random.default_rng(3)

    def mk(dt, ld, cols):
        return np.asfortranarray(rng.uniform(-1, 1, (ld, max(cols, 1))).astype(dt))

    for prec, var in (("d", "d"), ("s", "s_f64")):
        dt = np.float64 if prec == "d" else np.float32
        for (n, k) in [(0, 3), (5, 0), (5, 7), (100, 400), (390, 390), (400, 800)]:
            for uplo, trans in itertools.product("UL", "NTC"):
                for alpha, beta in ((1.0, 0.0), (0.7, 1.3), (0.0, 1.3)):
                    alpha, beta = float(dt(alpha)), float(dt(beta))
                    ra, ca = (k, n) if trans in "TC" else (n, k)
                    lda, ldc = max(ra, 1) + 2, max(n, 1) + 1
                    A, C0 = mk(dt, lda, ca), mk(dt, ldc, n)
                    C1, C2 = C0.copy(order="F"), C0.copy(order="F")
                    oracle.syrk(var, uplo, trans, n, k, alpha, A, lda, beta, C1, ldc)
                    oracle.ref_f77_l3("syrk", prec, (uplo, trans), (n, k), (alpha, beta), ((A, lda), (C2, ldc)))
                    assert C1.tobytes() == C2.tobytes(), ("syrk", prec, n, k, uplo, trans, alpha, beta)
                    # rank-2k: both operands on one leading dimension (the reference reads B with A's)
                    B = mk(dt, lda, ca)
                    C1, C2 = C0.copy(order="F"), C0.copy(order="F")
                    oracle.syr2k(var, uplo, trans, n, k, alpha, A, lda, B, lda, beta, C1, ldc)
                    oracle.ref_f77_l3("syr2k", prec, (uplo, trans), (n, k), (alpha, beta),
                                      ((A, lda), (B, lda), (C2, ldc)))
                    assert C1.tobytes() == C2.tobytes(), ("syr2k", prec, n, k, uplo, trans, alpha, beta)
        for (m, n) in [(0, 3), (5, 7), (390, 20), (20, 390), (400, 10)]:
            for side, uplo in itertools.product("LR", "UL"):
                for alpha, beta in ((1.0, 0.0), (0.7, 1.3), (0.0, 1.3)):
                    alpha, beta = float(dt(alpha)), float(dt(beta))
                    na = m if side == "L" else n
                    lda, ldb, ldc = max(na, 1) + 2, max(m, 1) + 1, max(m, 1) + 3
                    A, B, C0 = mk(dt, lda, na), mk(dt, ldb, n), mk(dt, ldc, n)
                    C1, C2 = C0.copy(order="F"), C0.copy(order="F")
                    oracle.symm(var, side, uplo, m, n, alpha, A, lda, B, ldb, beta, C1, ldc)
                    oracle.ref_f77_l3("symm", prec, (side, uplo), (m, n), (alpha, beta),
                                      ((A, lda), (B, ldb), (C2, ldc)))
                    assert C1.tobytes() == C2.tobytes(), ("symm", prec, m, n, side, uplo, alpha, beta)
    for prec, var in (("d", "d"), ("s", "s")):
        dt = np.float64 if prec == "d" else np.float32
        for (m, n) in [(0, 3), (5, 7), (390, 20), (20, 390), (800, 5), (1200, 3)]:
            for side, uplo, trans, diag in itertools.product("LR", "UL", "NT", "UN"):
                for alpha in (1.0, 0.7, 0.0):
                    alpha = float(dt(alpha))
                    na = m if side == "L" else n
                    lda, ldb = max(na, 1) + 2, max(m, 1) + 1
                    A, B0 = mk(dt, lda, na), mk(dt, ldb, n)
                    B1, B2 = B0.copy(order="F"), B0.copy(order="F")
                    oracle.trmm(var, side, uplo, trans, diag, m, n, alpha, A, lda, B1, ldb)
                    oracle.ref_f77_l3("trmm", prec, (side, uplo, trans, diag), (m, n), (alpha,), ((A, lda), (B2, ldb)))
                    assert B1.tobytes() == B2.tobytes(), ("trmm", prec, m, n, side, uplo, trans, diag, alpha)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_netlib_sweeps_through_oracle(oracle, prec):
    """DCHK2 (symm), DCHK3 (trmm), DCHK4 (syrk) and DCHK5 (syr2k) of test/F77/dblat3.f /
    sblat3.f: every call of the testers' sweeps, checked the testers' way
    (DMMCH ratio < 16 against a wide product), untouched padding and, for the
    rank-k update, an untouched other triangle (it holds ROGUE)."""
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    dt = np.float64 if prec == "d" else np.float32
    var = "d" if prec == "d" else "s_f64"
    worst = 0.0
    calls = 0
    for c in netlib.chk2_cases(params, dt):
        cc = c["cc"].copy(order="F")
        oracle.symm(var, c["side"], c["uplo"], c["m"], c["n"], c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"],
                    c["beta"], cc, c["ldc"])
        calls += 1
        m, n = c["m"], c["n"]
        assert np.array_equal(cc[m:], c["cc"][m:])
        if m > 0 and n > 0:
            if c["side"] == "L":
                err, _ = netlib.mmch("N", "N", m, n, m, c["alpha"], c["a"], c["bb"], c["beta"], c["cc"], cc, dt)
            else:
                err, _ = netlib.mmch("N", "N", m, n, n, c["alpha"], c["bb"], c["a"], c["beta"], c["cc"], cc, dt)
            worst = max(worst, err)
    assert calls == len(params["idim"]) ** 2 * 36
    for c in netlib.chk3_cases(params, dt):
        bb = c["bb"].copy(order="F")
        oracle.trmm("d" if prec == "d" else "s", c["side"], c["uplo"], c["transa"], c["diag"], c["m"], c["n"],
                    c["alpha"], c["aa"], c["lda"], bb, c["ldb"])
        m, n = c["m"], c["n"]
        assert np.array_equal(bb[m:], c["bb"][m:])
        if m > 0 and n > 0:
            zero = np.zeros_like(c["bb"])
            if c["side"] == "L":
                err, _ = netlib.mmch(c["transa"], "N", m, n, m, c["alpha"], c["a"], c["bb"], 0.0, zero, bb, dt)
            else:
                err, _ = netlib.mmch("N", c["transa"], m, n, n, c["alpha"], c["bb"], c["a"], 0.0, zero, bb, dt)
            worst = max(worst, err)
    for c in netlib.chk4_cases(params, dt):
        cc = c["cc"].copy(order="F")
        oracle.syrk(var, c["uplo"], c["trans"], c["n"], c["k"], c["alpha"], c["aa"], c["lda"], c["beta"], cc, c["ldc"])
        n, k = c["n"], c["k"]
        if n == 0:
            continue
        mask = netlib.triangle_mask(c["uplo"], n)
        assert np.array_equal(cc[:n][~mask], c["cc"][:n][~mask]) and np.array_equal(cc[n:], c["cc"][n:])
        ta, tb = ("T", "N") if c["trans"] in "TC" else ("N", "T")
        full = np.where(mask, cc[:n], c["c"])                  # the checker only looks at the triangle
        err_full = netlib.mmch(ta, tb, n, n, k, c["alpha"], c["aa"], c["aa"], c["beta"], c["c"], full, dt)[1]
        eps = np.finfo(dt).eps
        a = c["aa"].astype(np.float64)
        op = a[:k, :n].T if ta == "T" else a[:n, :k]
        g = abs(c["alpha"]) * (np.abs(op) @ np.abs(op).T) + abs(c["beta"]) * np.abs(c["c"].astype(np.float64))
        erri = np.abs(err_full - full.astype(np.float64)) / eps
        nz = g != 0
        erri[nz] /= g[nz]
        worst = max(worst, float(erri[mask].max()))
    ncalls = 0
    for c in netlib.chk5_cases(params, dt):
        cc = c["cc"].copy(order="F")
        oracle.syr2k(var, c["uplo"], c["trans"], c["n"], c["k"], c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"],
                     c["beta"], cc, c["ldc"])
        ncalls += 1
        n, k = c["n"], c["k"]
        if n == 0:
            assert cc.tobytes() == c["cc"].tobytes()
            continue
        mask = netlib.triangle_mask(c["uplo"], n)
        assert np.array_equal(cc[:n][~mask], c["cc"][:n][~mask]) and np.array_equal(cc[n:], c["cc"][n:])
        erri = netlib.syr2k_check(c["trans"], n, k, c["alpha"], c["aa"], c["bb"], c["beta"], c["c"], cc, dt)
        worst = max(worst, float(erri[mask].max()))
    assert ncalls == len(params["idim"]) ** 2 * 54
    assert worst < params["thresh"], worst


def test_against_numpy(oracle):
    """Independent of the testers' generator: random operands, numpy products."""
    rng = np.random.default_rng(12)
    n, k, m = 37, 29, 23
    A = np.asfortranarray(rng.uniform(-1, 1, (n, k)))
    C0 = np.asfortranarray(rng.uniform(-1, 1, (n, n)))
    for uplo, trans in itertools.product("UL", "NT"):
        Cm = C0.copy(order="F")
        Aop = A if trans == "N" else np.asfortranarray(A.T.copy())
        oracle.syrk("d", uplo, trans, n, k, 0.7, Aop, Aop.shape[0], 1.3, Cm, n)
        want = 0.7 * A @ A.T + 1.3 * C0
        mask = netlib.triangle_mask(uplo, n)
        np.testing.assert_allclose(Cm[mask], want[mask], rtol=0, atol=1e-13)
        assert np.array_equal(Cm[~mask], C0[~mask])
    # rank-2k with different leading dimensions for A and B
    for uplo, trans in itertools.product("UL", "NT"):
        ra = k if trans == "T" else n
        Aop = np.asfortranarray(np.vstack([A if trans == "N" else A.T, np.full((1, A.shape[1 if trans == "N" else 0]), np.nan)]))
        B = rng.uniform(-1, 1, (n, k))
        Bop = np.asfortranarray(np.vstack([B if trans == "N" else B.T, np.full((4, Aop.shape[1]), np.nan)]))
        Cm = C0.copy(order="F")
        oracle.syr2k("d", uplo, trans, n, k, 0.7, Aop, ra + 1, Bop, ra + 4, 1.3, Cm, n)
        want = 0.7 * (A @ B.T + B @ A.T) + 1.3 * C0
        mask = netlib.triangle_mask(uplo, n)
        np.testing.assert_allclose(Cm[mask], want[mask], rtol=0, atol=1e-13)
        assert np.array_equal(Cm[~mask], C0[~mask])
    S = rng.uniform(-1, 1, (m, m))
    S = S + S.T
    B = np.asfortranarray(rng.uniform(-1, 1, (m, n)))
    Cg = np.asfortranarray(rng.uniform(-1, 1, (m, n)))
    for side, uplo in itertools.product("LR", "UL"):
        na = m if side == "L" else n
        Sg = S if side == "L" else (lambda Z: Z + Z.T)(rng.uniform(-1, 1, (n, n)))
        stored = np.asfortranarray(np.where(netlib.triangle_mask(uplo, na), Sg, np.nan))
        Cm = Cg.copy(order="F")
        oracle.symm("d", side, uplo, m, n, 0.7, stored, na, B, m, 1.3, Cm, m)
        want = 0.7 * (Sg @ B if side == "L" else B @ Sg) + 1.3 * Cg
        np.testing.assert_allclose(Cm, want, rtol=0, atol=1e-13)
    for side, uplo, trans, diag in itertools.product("LR", "UL", "NT", "UN"):
        na = m if side == "L" else n
        T = rng.uniform(-1, 1, (na, na))
        mask = netlib.triangle_mask(uplo, na)
        full = np.where(mask, T, 0.0)
        stored = np.where(mask, T, np.nan)
        if diag == "U":
            full[np.arange(na), np.arange(na)] = 1.0
            stored[np.arange(na), np.arange(na)] = np.nan
        Bm = B.copy(order="F")
        oracle.trmm("d", side, uplo, trans, diag, m, n, 0.7, np.asfortranarray(stored), na, Bm, m)
        op = full.T if trans == "T" else full
        want = 0.7 * (op @ B if side == "L" else B @ op)
        np.testing.assert_allclose(Bm, want, rtol=0, atol=1e-13)


def test_error_exit_tables(oracle):
    for args, info in netlib.F77_SYRK_ERROR_EXITS:
        assert oracle.f77_syrk_info(*args) == info, args
    for args, info in netlib.CBLAS_SYRK_ERROR_EXITS:
        assert oracle.cblas_syrk_info(*args) == info, args
    for args, info in netlib.F77_SYR2K_ERROR_EXITS:
        assert oracle.f77_syr2k_info(*args) == info, args
    for args, info in netlib.CBLAS_SYR2K_ERROR_EXITS:
        assert oracle.cblas_syr2k_info(*args) == info, args
    for args, info in netlib.F77_SYMM_ERROR_EXITS:
        assert oracle.f77_symm_info(*args) == info, args
    for args, info in netlib.CBLAS_SYMM_ERROR_EXITS:
        assert netlib.cblas_tester_info_symm(args[0], oracle.cblas_symm_info(*args)) == info, args
    for args, info in netlib.F77_TRMM_ERROR_EXITS:
        assert oracle.f77_trsm_info(*args) == info, args
    for args, info in netlib.CBLAS_TRMM_ERROR_EXITS:
        assert netlib.cblas_tester_info_trsm(args[0], oracle.cblas_trsm_info(*args)) == info, args


@pytest.mark.parametrize("prec", ["d", "s"])
def test_library_error_exits(prec, xerbla):
    """The DSYRK / DSYR2K / DSYMM / DTRMM blocks of DCHKE (test/F77/dblat3.f) and of
    test/C/c_d3chke.c through the library's symbols."""
    dt = np.float64 if prec == "d" else np.float32
    up = prec.upper()

    def fresh():
        return np.full((2, 2), 7.0, dtype=dt, order="F")

    def expect(info, name, out, transform=lambda o, i: i, order=None):
        assert xerbla.capture_count() == 1
        assert transform(order, xerbla.capture_last_info()) == info
        assert xerbla.capture_last_name() == name
        assert (out == 7.0).all()

    for (uplo, trans, n, k, lda, ldc), info in netlib.F77_SYRK_ERROR_EXITS:
        xerbla.capture_reset()
        a, c = fresh(), fresh()
        blas.syrk_(prec, uplo, trans, n, k, 1.0, a, lda, 1.0, c, ldc)
        expect(info, f"{up}SYRK ".encode(), c)
    for args, info in netlib.CBLAS_SYRK_ERROR_EXITS:
        order, uplo, trans, n, k, lda, ldc = args
        xerbla.capture_reset()
        a, c = fresh(), fresh()
        blas.cblas_syrk(prec, order, uplo, trans, n, k, 1.0, a, lda, 1.0, c, ldc)
        expect(info, f"cblas_{prec}syrk".encode(), c)
    for (uplo, trans, n, k, lda, ldb, ldc), info in netlib.F77_SYR2K_ERROR_EXITS:
        xerbla.capture_reset()
        a, b, c = fresh(), fresh(), fresh()
        blas.syr2k_(prec, uplo, trans, n, k, 1.0, a, lda, b, ldb, 1.0, c, ldc)
        expect(info, f"{up}SYR2K".encode(), c)
    for args, info in netlib.CBLAS_SYR2K_ERROR_EXITS:
        order, uplo, trans, n, k, lda, ldb, ldc = args
        xerbla.capture_reset()
        a, b, c = fresh(), fresh(), fresh()
        blas.cblas_syr2k(prec, order, uplo, trans, n, k, 1.0, a, lda, b, ldb, 1.0, c, ldc)
        expect(info, f"cblas_{prec}syr2k".encode(), c)
    for (side, uplo, m, n, lda, ldb, ldc), info in netlib.F77_SYMM_ERROR_EXITS:
        xerbla.capture_reset()
        a, b, c = fresh(), fresh(), fresh()
        blas.symm_(prec, side, uplo, m, n, 1.0, a, lda, b, ldb, 1.0, c, ldc)
        expect(info, f"{up}SYMM ".encode(), c)
    for args, info in netlib.CBLAS_SYMM_ERROR_EXITS:
        order, side, uplo, m, n, lda, ldb, ldc = args
        xerbla.capture_reset()
        a, b, c = fresh(), fresh(), fresh()
        blas.cblas_symm(prec, order, side, uplo, m, n, 1.0, a, lda, b, ldb, 1.0, c, ldc)
        expect(info, f"cblas_{prec}symm".encode(), c, netlib.cblas_tester_info_symm, order)
    for (side, uplo, ta, diag, m, n, lda, ldb), info in netlib.F77_TRMM_ERROR_EXITS:
        xerbla.capture_reset()
        a, b = fresh(), fresh()
        blas.trmm_(prec, side, uplo, ta, diag, m, n, 1.0, a, lda, b, ldb)
        expect(info, f"{up}TRMM ".encode(), b)
    for args, info in netlib.CBLAS_TRMM_ERROR_EXITS:
        order, side, uplo, ta, diag, m, n, lda, ldb = args
        xerbla.capture_reset()
        a, b = fresh(), fresh()
        blas.cblas_trmm(prec, order, side, uplo, ta, diag, m, n, 1.0, a, lda, b, ldb)
        expect(info, f"cblas_{prec}trmm".encode(), b, netlib.cblas_tester_info_trsm, order)


def test_library_nothing_to_do(xerbla):
    """n == 0, or alpha == 0 / k == 0 with beta == 1: nothing is written and
    no device is needed (ulmblas/level3/sylrk.tcc:38-40, sylmm.tcc:47-49)."""
    c0 = np.arange(16.0).reshape((4, 4), order="F")
    a = np.ones((4, 4), order="F")
    for (n, k, alpha, beta) in [(0, 3, 1.0, 0.0), (3, 0, 1.0, 1.0), (3, 3, 0.0, 1.0)]:
        c = c0.copy(order="F")
        blas.syrk_("d", "L", "N", n, k, alpha, a, 4, beta, c, 4)
        blas.cblas_syrk("d", blas.CblasRowMajor, blas.CblasUpper, blas.CblasTrans, n, k, alpha, a, 4, beta, c, 4)
        blas.syr2k_("d", "U", "T", n, k, alpha, a, 4, a, 4, beta, c, 4)
        blas.cblas_syr2k("d", blas.CblasRowMajor, blas.CblasLower, blas.CblasNoTrans, n, k, alpha, a, 4, a, 4, beta, c, 4)
        assert c.tobytes() == c0.tobytes()
    for (m, n, alpha, beta) in [(0, 3, 1.0, 0.0), (3, 0, 1.0, 0.0), (3, 3, 0.0, 1.0)]:
        c = c0.copy(order="F")
        blas.symm_("d", "R", "U", m, n, alpha, a, 4, a, 4, beta, c, 4)
        assert c.tobytes() == c0.tobytes()
    for (m, n) in [(0, 3), (3, 0)]:
        c = c0.copy(order="F")
        blas.trmm_("d", "L", "U", "N", "N", m, n, 1.0, a, 4, c, 4)
        assert c.tobytes() == c0.tobytes()
    assert xerbla.capture_count() == 0
    L = lib.load()
    assert L.ulmblas_gpu_dsyrk(1, 0, -1, 1, 1.0, None, 1, 0.0, None, 1, None) == 1
    assert L.ulmblas_gpu_dsymm(0, 1, 4, 2, 1.0, None, 3, None, 4, 0.0, None, 4, None, None) == 1
    assert L.ulmblas_gpu_dtrmm(0, 1, 0, 0, 4, 2, 1.0, None, 3, None, 4, None) == 1
    assert L.ulmblas_gpu_dsyrk(1, 0, 0, 5, 1.0, None, 1, 0.0, None, 1, None) == 0
    assert L.ulmblas_gpu_dsyr2k(1, 0, 4, 2, 1.0, None, 4, None, 3, 0.0, None, 4, None) == 1
    assert L.ulmblas_gpu_dsyr2k(1, 1, 0, 5, 1.0, None, 5, None, 5, 0.0, None, 1, None) == 0
