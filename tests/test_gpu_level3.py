"""Symmetric rank-k and rank-2k updates, symmetric product and triangular
product on the GPU: the reference's DCHK2 / DCHK3 / DCHK4 / DCHK5 sweeps (test/F77/dblat3.f,
sblat3.f and the CBLAS drivers) through the drop-in symbols of
libulmblas_gpu.so, and the device-resident entry points on larger and ragged
shapes against the CPU oracle.

Parity bound (the one of the GEMM tests, tests/gpu_util.py): elementwise
|R_gpu - R_oracle| <= TOL_C * k * eps * gauge with k the length of the inner
products and gauge = |alpha| |op(A)| |op(B)| + |beta| |C|.
"""
import itertools

import numpy as np
import pytest

import netlib
from gpu_util import TOL_C, parity_ratio, to_device, to_host
from ulmblas_amd import blas, synth

pytestmark = pytest.mark.gpu

UPLO = {"U": blas.CblasUpper, "L": blas.CblasLower}
SIDE = {"L": blas.CblasLeft, "R": blas.CblasRight}
TRANS = {"N": blas.CblasNoTrans, "T": blas.CblasTrans, "C": blas.CblasConjTrans}
DIAG = {"U": blas.CblasUnit, "N": blas.CblasNonUnit}


def gauge_syrk(trans, n, k, alpha, a, beta, c_full):
    op = a[:k, :n].T if trans in "TC" else a[:n, :k]
    op = np.abs(op.astype(np.float64))
    g = abs(alpha) * (op @ op.T) if k > 0 and alpha != 0 else np.zeros((n, n))
    return g + (abs(beta) * np.abs(c_full.astype(np.float64)) if beta != 0 else 0.0)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_chk4_syrk(prec, oracle, xerbla):
    dt = np.float64 if prec == "d" else np.float32
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    variants = ("d",) if prec == "d" else ("s", "s_f64")
    ncalls, worst = 0, 0.0
    for c in netlib.chk4_cases(params, dt):
        n, k = c["n"], c["k"]
        cc, aa = c["cc"].copy(order="F"), c["aa"].copy(order="F")
        blas.syrk_(prec, c["uplo"], c["trans"], n, k, c["alpha"], aa, c["lda"], c["beta"], cc, c["ldc"])
        ncalls += 1
        assert aa.tobytes() == c["aa"].tobytes()
        if n == 0:
            assert cc.tobytes() == c["cc"].tobytes()
            continue
        mask = netlib.triangle_mask(c["uplo"], n)
        tag = (c["uplo"], c["trans"], n, k, c["alpha"], c["beta"])
        assert np.array_equal(cc[:n][~mask], c["cc"][:n][~mask]), tag      # the other triangle holds ROGUE
        assert np.array_equal(cc[n:], c["cc"][n:]), tag
        assert not np.isnan(cc[:n][mask]).any(), tag
        g = gauge_syrk(c["trans"], n, k, c["alpha"], c["aa"], c["beta"], c["c"])
        for v in variants:
            want = c["cc"].copy(order="F")
            oracle.syrk(v, c["uplo"], c["trans"], n, k, c["alpha"], c["aa"], c["lda"], c["beta"], want, c["ldc"])
            diff = np.abs(cc[:n].astype(np.float64) - want[:n].astype(np.float64))
            scale = max(k, 1) * np.finfo(dt).eps * g
            with np.errstate(divide="ignore", invalid="ignore"):
                r = np.where(diff == 0, 0.0, diff / scale)[mask].max()
            assert r <= TOL_C, (tag, v, r)
            worst = max(worst, float(r))
    assert xerbla.capture_count() == 0
    assert ncalls == len(params["idim"]) ** 2 * 54
    print(f"chk4 {prec}: {ncalls} calls, max parity ratio {worst:.3f}")


def gauge_syr2k(trans, n, k, alpha, a, b, beta, c_full):
    opa = np.abs((a[:k, :n].T if trans in "TC" else a[:n, :k]).astype(np.float64))
    opb = np.abs((b[:k, :n].T if trans in "TC" else b[:n, :k]).astype(np.float64))
    g = abs(alpha) * (opa @ opb.T + opb @ opa.T) if k > 0 and alpha != 0 else np.zeros((n, n))
    return g + (abs(beta) * np.abs(c_full.astype(np.float64)) if beta != 0 else 0.0)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_chk5_syr2k(prec, oracle, xerbla):
    """DCHK5 (test/F77/dblat3.f:1487-1790): the inner products have length 2k."""
    dt = np.float64 if prec == "d" else np.float32
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    variants = ("d",) if prec == "d" else ("s", "s_f64")
    ncalls, worst = 0, 0.0
    for c in netlib.chk5_cases(params, dt):
        n, k = c["n"], c["k"]
        cc, aa, bb = c["cc"].copy(order="F"), c["aa"].copy(order="F"), c["bb"].copy(order="F")
        blas.syr2k_(prec, c["uplo"], c["trans"], n, k, c["alpha"], aa, c["lda"], bb, c["ldb"], c["beta"], cc, c["ldc"])
        ncalls += 1
        assert aa.tobytes() == c["aa"].tobytes() and bb.tobytes() == c["bb"].tobytes()
        if n == 0:
            assert cc.tobytes() == c["cc"].tobytes()
            continue
        mask = netlib.triangle_mask(c["uplo"], n)
        tag = (c["uplo"], c["trans"], n, k, c["alpha"], c["beta"])
        assert np.array_equal(cc[:n][~mask], c["cc"][:n][~mask]), tag
        assert np.array_equal(cc[n:], c["cc"][n:]), tag
        erri = netlib.syr2k_check(c["trans"], n, k, c["alpha"], c["aa"], c["bb"], c["beta"], c["c"], cc, dt)
        assert erri[mask].max() < params["thresh"], (tag, erri[mask].max())
        g = gauge_syr2k(c["trans"], n, k, c["alpha"], c["aa"], c["bb"], c["beta"], c["c"])
        for v in variants:
            want = c["cc"].copy(order="F")
            oracle.syr2k(v, c["uplo"], c["trans"], n, k, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"], c["beta"],
                         want, c["ldc"])
            diff = np.abs(cc[:n].astype(np.float64) - want[:n].astype(np.float64))
            scale = max(2 * k, 1) * np.finfo(dt).eps * g
            with np.errstate(divide="ignore", invalid="ignore"):
                r = np.where(diff == 0, 0.0, diff / scale)[mask].max()
            assert r <= TOL_C, (tag, v, r)
            worst = max(worst, float(r))
    assert xerbla.capture_count() == 0
    assert ncalls == len(params["idim"]) ** 2 * 54
    print(f"chk5 {prec}: {ncalls} calls, max parity ratio {worst:.3f}")


@pytest.mark.parametrize("prec", ["d", "s"])
def test_chk2_symm(prec, oracle, xerbla):
    dt = np.float64 if prec == "d" else np.float32
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    variants = ("d",) if prec == "d" else ("s", "s_f64")
    ncalls, worst = 0, 0.0
    for c in netlib.chk2_cases(params, dt):
        m, n = c["m"], c["n"]
        cc = c["cc"].copy(order="F")
        aa, bb = c["aa"].copy(order="F"), c["bb"].copy(order="F")
        blas.symm_(prec, c["side"], c["uplo"], m, n, c["alpha"], aa, c["lda"], bb, c["ldb"], c["beta"], cc, c["ldc"])
        ncalls += 1
        assert aa.tobytes() == c["aa"].tobytes() and bb.tobytes() == c["bb"].tobytes()
        if m == 0 or n == 0:
            assert cc.tobytes() == c["cc"].tobytes()
            continue
        tag = (c["side"], c["uplo"], m, n, c["alpha"], c["beta"])
        assert np.array_equal(cc[m:], c["cc"][m:]), tag
        k = m if c["side"] == "L" else n
        if c["side"] == "L":
            err, _ = netlib.mmch("N", "N", m, n, m, c["alpha"], c["a"], c["bb"], c["beta"], c["cc"], cc, dt)
            g = oracle.gauge("N", "N", m, n, m, c["alpha"], c["a"], c["bb"], c["beta"], c["cc"])
        else:
            err, _ = netlib.mmch("N", "N", m, n, n, c["alpha"], c["bb"], c["a"], c["beta"], c["cc"], cc, dt)
            g = oracle.gauge("N", "N", m, n, n, c["alpha"], c["bb"], c["a"], c["beta"], c["cc"])
        assert err < params["thresh"], (tag, err)
        for v in variants:
            want = c["cc"].copy(order="F")
            oracle.symm(v, c["side"], c["uplo"], m, n, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"], c["beta"],
                        want, c["ldc"])
            r = parity_ratio(cc[:m], want[:m], g, k, dt)
            assert r <= TOL_C, (tag, v, r)
            worst = max(worst, r)
    assert xerbla.capture_count() == 0
    assert ncalls == len(params["idim"]) ** 2 * 36
    print(f"chk2 {prec}: {ncalls} calls, max parity ratio {worst:.3f}")


@pytest.mark.parametrize("prec", ["d", "s"])
def test_chk3_trmm(prec, oracle, xerbla):
    dt = np.float64 if prec == "d" else np.float32
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    ncalls, worst = 0, 0.0
    for c in netlib.chk3_cases(params, dt):
        m, n = c["m"], c["n"]
        aa, bb = c["aa"].copy(order="F"), c["bb"].copy(order="F")
        blas.trmm_(prec, c["side"], c["uplo"], c["transa"], c["diag"], m, n, c["alpha"], aa, c["lda"], bb, c["ldb"])
        ncalls += 1
        assert aa.tobytes() == c["aa"].tobytes()
        if m == 0 or n == 0:
            assert bb.tobytes() == c["bb"].tobytes()
            continue
        tag = (c["side"], c["uplo"], c["transa"], c["diag"], m, n, c["alpha"])
        assert np.array_equal(bb[m:], c["bb"][m:]), tag
        assert not np.isnan(bb[:m]).any(), tag
        zero = np.zeros_like(c["bb"])
        if c["side"] == "L":
            err, _ = netlib.mmch(c["transa"], "N", m, n, m, c["alpha"], c["a"], c["bb"], 0.0, zero, bb, dt)
            g = oracle.gauge(c["transa"], "N", m, n, m, c["alpha"], c["a"], c["bb"], 0.0, zero)
        else:
            err, _ = netlib.mmch("N", c["transa"], m, n, n, c["alpha"], c["bb"], c["a"], 0.0, zero, bb, dt)
            g = oracle.gauge("N", c["transa"], m, n, n, c["alpha"], c["bb"], c["a"], 0.0, zero)
        assert err < params["thresh"], (tag, err)
        want = c["bb"].copy(order="F")
        oracle.trmm(prec, c["side"], c["uplo"], c["transa"], c["diag"], m, n, c["alpha"], c["aa"], c["lda"], want,
                    c["ldb"])
        r = parity_ratio(bb[:m], want[:m], g, m if c["side"] == "L" else n, dt)
        assert r <= TOL_C, (tag, r)
        worst = max(worst, r)
    assert xerbla.capture_count() == 0
    assert ncalls == len(params["idim"]) ** 2 * 72
    print(f"chk3 trmm {prec}: {ncalls} calls, max parity ratio {worst:.3f}")


def test_cblas_orders_and_aliases(oracle, xerbla):
    """The CBLAS drivers' sweeps in both storage orders (test/C/c_dblat3.f with
    test/C/c_dblas3.c), and the ulmblas_ / ATL_ symbols, for double."""
    dt = np.float64
    rogue = netlib.ROGUE
    for c in netlib.chk4_cases(netlib.DIN3, dt):
        n, k = c["n"], c["k"]
        want = c["cc"].copy(order="F")
        oracle.syrk("d", c["uplo"], c["trans"], n, k, c["alpha"], c["aa"], c["lda"], c["beta"], want, c["ldc"])
        outs = []
        for call in (lambda x: blas.cblas_syrk("d", blas.CblasColMajor, UPLO[c["uplo"]], TRANS[c["trans"]], n, k,
                                               c["alpha"], c["aa"], c["lda"], c["beta"], x, c["ldc"]),
                     lambda x: blas.ulmblas_syrk("d", UPLO[c["uplo"]], TRANS[c["trans"]], n, k, c["alpha"], c["aa"],
                                                 c["lda"], c["beta"], x, c["ldc"]),
                     lambda x: blas.ulmblas_syrk("d", UPLO[c["uplo"]], TRANS[c["trans"]], n, k, c["alpha"], c["aa"],
                                                 c["lda"], c["beta"], x, c["ldc"], prefix="ATL_")):
            cc = c["cc"].copy(order="F")
            call(cc)
            outs.append(cc)
        assert outs[0].tobytes() == outs[1].tobytes() == outs[2].tobytes()
        mask = netlib.triangle_mask(c["uplo"], n)
        np.testing.assert_allclose(outs[0][:n][mask], want[:n][mask], rtol=1e-13, atol=1e-14)
        # row-major copies of the operands
        ma, na = (k, n) if c["trans"] in "TC" else (n, k)
        a_row = np.full((ma, na + 1), rogue)
        a_row[:, :na] = c["aa"][:ma, :]
        c_row = np.full((n, n + 1), rogue)
        c_row[:, :n] = c["cc"][:n, :]
        blas.cblas_syrk("d", blas.CblasRowMajor, UPLO[c["uplo"]], TRANS[c["trans"]], n, k, c["alpha"], a_row, na + 1,
                        c["beta"], c_row, n + 1)
        np.testing.assert_allclose(c_row[:, :n][mask], want[:n][mask], rtol=1e-13, atol=1e-14)
        assert np.array_equal(c_row[:, :n][~mask], c["cc"][:n][~mask]) and (c_row[:, n] == rogue).all()
    for c in netlib.chk5_cases(netlib.DIN3, dt):
        n, k = c["n"], c["k"]
        want = c["cc"].copy(order="F")
        oracle.syr2k("d", c["uplo"], c["trans"], n, k, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"], c["beta"],
                     want, c["ldc"])
        outs = []
        for call in (lambda x: blas.cblas_syr2k("d", blas.CblasColMajor, UPLO[c["uplo"]], TRANS[c["trans"]], n, k,
                                                c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"], c["beta"], x,
                                                c["ldc"]),
                     lambda x: blas.ulmblas_syr2k("d", UPLO[c["uplo"]], TRANS[c["trans"]], n, k, c["alpha"], c["aa"],
                                                  c["lda"], c["bb"], c["ldb"], c["beta"], x, c["ldc"]),
                     lambda x: blas.ulmblas_syr2k("d", UPLO[c["uplo"]], TRANS[c["trans"]], n, k, c["alpha"], c["aa"],
                                                  c["lda"], c["bb"], c["ldb"], c["beta"], x, c["ldc"], prefix="ATL_")):
            cc = c["cc"].copy(order="F")
            call(cc)
            outs.append(cc)
        assert outs[0].tobytes() == outs[1].tobytes() == outs[2].tobytes()
        mask = netlib.triangle_mask(c["uplo"], n)
        np.testing.assert_allclose(outs[0][:n][mask], want[:n][mask], rtol=1e-13, atol=1e-14)
        ma, na = (k, n) if c["trans"] in "TC" else (n, k)
        a_row = np.full((ma, na + 1), rogue)
        a_row[:, :na] = c["aa"][:ma, :]
        b_row = np.full((ma, na + 3), rogue)
        b_row[:, :na] = c["bb"][:ma, :]
        c_row = np.full((n, n + 1), rogue)
        c_row[:, :n] = c["cc"][:n, :]
        blas.cblas_syr2k("d", blas.CblasRowMajor, UPLO[c["uplo"]], TRANS[c["trans"]], n, k, c["alpha"], a_row, na + 1,
                         b_row, na + 3, c["beta"], c_row, n + 1)
        np.testing.assert_allclose(c_row[:, :n][mask], want[:n][mask], rtol=1e-13, atol=1e-14)
        assert np.array_equal(c_row[:, :n][~mask], c["cc"][:n][~mask]) and (c_row[:, n] == rogue).all()
    for c in netlib.chk2_cases(netlib.DIN3, dt):
        m, n = c["m"], c["n"]
        na = m if c["side"] == "L" else n
        want = c["cc"].copy(order="F")
        oracle.symm("d", c["side"], c["uplo"], m, n, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"], c["beta"], want,
                    c["ldc"])
        cc = c["cc"].copy(order="F")
        blas.cblas_symm("d", blas.CblasColMajor, SIDE[c["side"]], UPLO[c["uplo"]], m, n, c["alpha"], c["aa"], c["lda"],
                        c["bb"], c["ldb"], c["beta"], cc, c["ldc"])
        c2 = c["cc"].copy(order="F")
        blas.ulmblas_symm("d", SIDE[c["side"]], UPLO[c["uplo"]], m, n, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"],
                          c["beta"], c2, c["ldc"], prefix="ATL_")
        assert cc.tobytes() == c2.tobytes()
        np.testing.assert_allclose(cc[:m], want[:m], rtol=1e-13, atol=1e-14)
        a_row = np.full((na, na + 1), rogue)
        a_row[:, :na] = c["aa"][:na, :]
        b_row = np.full((m, n + 2), rogue)
        b_row[:, :n] = c["bb"][:m, :]
        c_row = np.full((m, n + 1), rogue)
        c_row[:, :n] = c["cc"][:m, :]
        blas.cblas_symm("d", blas.CblasRowMajor, SIDE[c["side"]], UPLO[c["uplo"]], m, n, c["alpha"], a_row, na + 1,
                        b_row, n + 2, c["beta"], c_row, n + 1)
        np.testing.assert_allclose(c_row[:, :n], want[:m], rtol=1e-13, atol=1e-14)
        assert (c_row[:, n] == rogue).all()
    for c in netlib.chk3_cases(netlib.DIN3, dt):
        m, n = c["m"], c["n"]
        na = m if c["side"] == "L" else n
        args = (SIDE[c["side"]], UPLO[c["uplo"]], TRANS[c["transa"]], DIAG[c["diag"]])
        want = c["bb"].copy(order="F")
        oracle.trmm("d", c["side"], c["uplo"], c["transa"], c["diag"], m, n, c["alpha"], c["aa"], c["lda"], want,
                    c["ldb"])
        bb = c["bb"].copy(order="F")
        blas.cblas_trmm("d", blas.CblasColMajor, *args, m, n, c["alpha"], c["aa"], c["lda"], bb, c["ldb"])
        b2 = c["bb"].copy(order="F")
        blas.ulmblas_trmm("d", *args, m, n, c["alpha"], c["aa"], c["lda"], b2, c["ldb"], prefix="ATL_")
        assert bb.tobytes() == b2.tobytes()
        np.testing.assert_allclose(bb[:m], want[:m], rtol=1e-13, atol=1e-14)
        a_row = np.full((na, na + 1), rogue)
        a_row[:, :na] = c["aa"][:na, :]
        b_row = np.full((m, n + 1), rogue)
        b_row[:, :n] = c["bb"][:m, :]
        blas.cblas_trmm("d", blas.CblasRowMajor, *args, m, n, c["alpha"], a_row, na + 1, b_row, n + 1)
        np.testing.assert_allclose(b_row[:, :n], want[:m], rtol=1e-13, atol=1e-14)
        assert (b_row[:, n] == rogue).all()
    assert xerbla.capture_count() == 0


@pytest.mark.parametrize("prec", ["d", "s"])
def test_device_entries_on_larger_shapes(prec, oracle):
    """Orders that exercise the recursion and the masked diagonal launches;
    unreferenced parts hold NaN."""
    import torch
    dt = np.float64 if prec == "d" else np.float32
    tdt = torch.float64 if prec == "d" else torch.float32
    worst = 0.0
    # syrk
    for (n, k) in [(1, 1), (65, 33), (513, 200), (700, 64), (1300, 300)]:
        for uplo, trans in itertools.product("UL", "NT"):
            ra, ca = (k, n) if trans == "T" else (n, k)
            lda, ldc = ra + 3, n + 2
            A = synth.matrix(61, ra, ca, lda, dtype=dt)
            C0 = synth.matrix(62, n, n, ldc, dtype=dt)
            mask = netlib.triangle_mask(uplo, n)
            C0[:n][~mask] = np.nan
            for alpha, beta in ((0.7, 1.3), (1.0, 0.0)):
                Cin = C0.copy(order="F")
                if beta == 0.0:
                    Cin[:n][mask] = np.nan
                dC = to_device(Cin)
                blas.gpu_syrk(prec, uplo == "L", trans == "T", n, k, alpha, to_device(A), lda, beta, dC, ldc)
                torch.cuda.synchronize()
                got = to_host(dC)
                want = Cin.copy(order="F")
                oracle.syrk(prec, uplo, trans, n, k, alpha, A, lda, beta, want, ldc)
                assert np.isnan(got[:n][~mask]).all() and np.array_equal(got[n:], Cin[n:])
                assert not np.isnan(got[:n][mask]).any()
                full = np.where(mask, np.nan_to_num(Cin[:n]), np.nan_to_num(Cin[:n]).T)
                g = gauge_syrk(trans, n, k, alpha, A, beta, full)
                diff = np.abs(got[:n].astype(np.float64) - want[:n].astype(np.float64))
                with np.errstate(divide="ignore", invalid="ignore"):
                    r = np.where(diff == 0, 0.0, diff / (k * np.finfo(dt).eps * g))[mask].max()
                assert r <= TOL_C, ("syrk", uplo, trans, n, k, alpha, beta, r)
                worst = max(worst, float(r))
    # syr2k, A and B on different leading dimensions
    for (n, k) in [(1, 1), (65, 33), (513, 200), (1300, 64)]:
        for uplo, trans in itertools.product("UL", "NT"):
            ra, ca = (k, n) if trans == "T" else (n, k)
            lda, ldb, ldc = ra + 3, ra + 6, n + 2
            A = synth.matrix(68, ra, ca, lda, dtype=dt)
            B = synth.matrix(69, ra, ca, ldb, dtype=dt)
            C0 = synth.matrix(70, n, n, ldc, dtype=dt)
            mask = netlib.triangle_mask(uplo, n)
            C0[:n][~mask] = np.nan
            dC = to_device(C0)
            blas.gpu_syr2k(prec, uplo == "L", trans == "T", n, k, 0.7, to_device(A), lda, to_device(B), ldb, 1.3, dC,
                           ldc)
            torch.cuda.synchronize()
            got = to_host(dC)
            want = C0.copy(order="F")
            oracle.syr2k(prec, uplo, trans, n, k, 0.7, A, lda, B, ldb, 1.3, want, ldc)
            assert np.isnan(got[:n][~mask]).all() and np.array_equal(got[n:], C0[n:])
            assert not np.isnan(got[:n][mask]).any()
            full = np.where(mask, np.nan_to_num(C0[:n]), np.nan_to_num(C0[:n]).T)
            g = gauge_syr2k(trans, n, k, 0.7, A, B, 1.3, full)
            diff = np.abs(got[:n].astype(np.float64) - want[:n].astype(np.float64))
            with np.errstate(divide="ignore", invalid="ignore"):
                r = np.where(diff == 0, 0.0, diff / (2 * k * np.finfo(dt).eps * g))[mask].max()
            assert r <= TOL_C, ("syr2k", uplo, trans, n, k, r)
            worst = max(worst, float(r))
    # symm
    for (m, n) in [(1, 1), (65, 33), (300, 517), (517, 300)]:
        for side, uplo in itertools.product("LR", "UL"):
            na = m if side == "L" else n
            lda, ldb, ldc = na + 3, m + 1, m + 2
            A = synth.matrix(63, na, na, lda, dtype=dt)
            amask = netlib.triangle_mask(uplo, na)
            full = np.where(amask, A[:na], A[:na].T)
            A[:na][~amask] = np.nan
            B = synth.matrix(64, m, n, ldb, dtype=dt)
            C0 = synth.matrix(65, m, n, ldc, dtype=dt)
            dC = to_device(C0)
            work = torch.empty(na * na, dtype=tdt, device="cuda")
            blas.gpu_symm(prec, side == "R", uplo == "L", m, n, 0.7, to_device(A), lda, to_device(B), ldb, 1.3, dC, ldc,
                          work)
            torch.cuda.synchronize()
            got = to_host(dC)
            want = C0.copy(order="F")
            oracle.symm(prec, side, uplo, m, n, 0.7, A, lda, B, ldb, 1.3, want, ldc)
            assert np.array_equal(got[m:], C0[m:]) and not np.isnan(got[:m]).any()
            if side == "L":
                g = oracle.gauge("N", "N", m, n, m, 0.7, full, B, 1.3, C0)
            else:
                g = oracle.gauge("N", "N", m, n, n, 0.7, B, full, 1.3, C0)
            r = parity_ratio(got[:m], want[:m], g, na, dt)
            assert r <= TOL_C, ("symm", side, uplo, m, n, r)
            worst = max(worst, r)
    # trmm
    for (m, n) in [(1, 1), (65, 33), (200, 130), (256, 40), (40, 256), (300, 96), (130, 517)]:
        for side, uplo, trans, diag in itertools.product("LR", "UL", "NT", "UN"):
            na = m if side == "L" else n
            lda, ldb = na + 3, m + 2
            A = synth.matrix(66, na, na, lda, dtype=dt)
            tmask = netlib.triangle_mask(uplo, na)
            full = np.where(tmask, A[:na], 0)
            if diag == "U":
                full[np.arange(na), np.arange(na)] = 1
                A[np.arange(na), np.arange(na)] = np.nan
            A[:na][~tmask] = np.nan
            B0 = synth.matrix(67, m, n, ldb, dtype=dt)
            dB = to_device(B0)
            blas.gpu_trmm(prec, side == "R", uplo == "L", trans == "T", diag == "U", m, n, 0.7, to_device(A), lda, dB,
                          ldb)
            torch.cuda.synchronize()
            got = to_host(dB)
            want = B0.copy(order="F")
            oracle.trmm(prec, side, uplo, trans, diag, m, n, 0.7, A, lda, want, ldb)
            assert np.array_equal(got[m:], B0[m:]) and not np.isnan(got[:m]).any()
            zero = np.zeros_like(B0)
            if side == "L":
                g = oracle.gauge(trans, "N", m, n, m, 0.7, full, B0, 0.0, zero)
            else:
                g = oracle.gauge("N", trans, m, n, n, 0.7, B0, full, 0.0, zero)
            r = parity_ratio(got[:m], want[:m], g, na, dt)
            assert r <= TOL_C, ("trmm", side, uplo, trans, diag, m, n, r)
            worst = max(worst, r)
    print(f"device level-3 {prec}: max parity ratio {worst:.3f}")


@pytest.mark.parametrize("prec", ["d", "s"])
def test_rank_k_update_with_shared_tiles(prec, oracle):
    """The launch over the whole tiles inside the triangle shares the tiles of
    its last round along k like a plain product does (forced here: the orders
    that fit a test have too few tiles for it to pay): 6 and 28 tiles of
    256 x 128 (f64; 3 and 15 of 256 x 256 in f32) cut into up to four pieces, a k that
    ends inside a slab, both triangles, beta == 0 on NaN."""
    import torch
    dt = np.float64 if prec == "d" else np.float32
    blas.test_control(blas.TEST_SHARED_PIECES, -4)
    try:
        for (n, k) in [(1024 + 17, 333), (2048, 515)]:
            for uplo, trans in itertools.product("UL", "NT"):
                ra, ca = (k, n) if trans == "T" else (n, k)
                lda, ldc = ra + 3, n + 2
                A = synth.matrix(71, ra, ca, lda, dtype=dt)
                C0 = synth.matrix(72, n, n, ldc, dtype=dt)
                mask = netlib.triangle_mask(uplo, n)
                C0[:n][~mask] = np.nan
                for alpha, beta in ((0.7, 1.3), (1.0, 0.0)):
                    Cin = C0.copy(order="F")
                    if beta == 0.0:
                        Cin[:n][mask] = np.nan
                    dC = to_device(Cin)
                    blas.gpu_syrk(prec, uplo == "L", trans == "T", n, k, alpha, to_device(A), lda, beta, dC, ldc)
                    torch.cuda.synchronize()
                    got = to_host(dC)
                    want = Cin.copy(order="F")
                    oracle.syrk(prec, uplo, trans, n, k, alpha, A, lda, beta, want, ldc)
                    assert np.isnan(got[:n][~mask]).all() and np.array_equal(got[n:], Cin[n:])
                    assert not np.isnan(got[:n][mask]).any()
                    full = np.where(mask, np.nan_to_num(Cin[:n]), np.nan_to_num(Cin[:n]).T)
                    g = gauge_syrk(trans, n, k, alpha, A, beta, full)
                    diff = np.abs(got[:n].astype(np.float64) - want[:n].astype(np.float64))
                    with np.errstate(divide="ignore", invalid="ignore"):
                        r = np.where(diff == 0, 0.0, diff / (k * np.finfo(dt).eps * g))[mask].max()
                    assert r <= TOL_C, ("syrk", uplo, trans, n, k, alpha, beta, r)
        blas.device_status()
    finally:
        blas.test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_rank_k_update_every_way_it_is_cut_up(prec, oracle):
    """Orders that are no multiple of the block of 256: the square of whole
    blocks with the rows beyond it as a product of their own and the triangle
    at their end on a side stream (ways 1 and 2: all whole blocks, an even
    number of them; 4 and 5: the same with the second largest tile, whose
    blocks are smaller), the any-shape kernel alone (3), and the planner's own
    choice (0).  Every way against the oracle, the other triangle (NaN) and
    the padding rows untouched; syr2k, whose two sweeps meet on the side
    stream, as well."""
    import torch
    dt = np.float64 if prec == "d" else np.float32
    try:
        for way in (1, 2, 3, 4, 5, 0):
            blas.test_control(blas.TEST_TRI_WAY, way)
            for (n, k) in [(1300, 130), (1024 + 17, 333), (3 * 256, 70), (700, 257)]:
                for uplo, trans in itertools.product("UL", "NT"):
                    ra, ca = (k, n) if trans == "T" else (n, k)
                    lda, ldb, ldc = ra + 3, ra + 1, n + 2
                    A = synth.matrix(71, ra, ca, lda, dtype=dt)
                    B = synth.matrix(73, ra, ca, ldb, dtype=dt)
                    C0 = synth.matrix(72, n, n, ldc, dtype=dt)
                    mask = netlib.triangle_mask(uplo, n)
                    C0[:n][~mask] = np.nan
                    for two, (alpha, beta) in itertools.product((False, True), ((0.7, 1.3), (1.0, 0.0))):
                        if two and (way == 0 or trans == "T" and uplo == "U"):
                            continue
                        Cin = C0.copy(order="F")
                        if beta == 0.0:
                            Cin[:n][mask] = np.nan
                        dC = to_device(Cin)
                        want = Cin.copy(order="F")
                        full = np.where(mask, np.nan_to_num(Cin[:n]), np.nan_to_num(Cin[:n]).T)
                        if two:
                            blas.gpu_syr2k(prec, uplo == "L", trans == "T", n, k, alpha, to_device(A), lda, to_device(B), ldb,
                                           beta, dC, ldc)
                            oracle.syr2k(prec, uplo, trans, n, k, alpha, A, lda, B, ldb, beta, want, ldc)
                            g = gauge_syr2k(trans, n, k, alpha, A, B, beta, full)
                        else:
                            blas.gpu_syrk(prec, uplo == "L", trans == "T", n, k, alpha, to_device(A), lda, beta, dC, ldc)
                            oracle.syrk(prec, uplo, trans, n, k, alpha, A, lda, beta, want, ldc)
                            g = gauge_syrk(trans, n, k, alpha, A, beta, full)
                        torch.cuda.synchronize()
                        got = to_host(dC)
                        tag = (way, two, uplo, trans, n, k, alpha, beta)
                        assert np.isnan(got[:n][~mask]).all() and np.array_equal(got[n:], Cin[n:]), tag
                        assert not np.isnan(got[:n][mask]).any(), tag
                        diff = np.abs(got[:n].astype(np.float64) - want[:n].astype(np.float64))
                        with np.errstate(divide="ignore", invalid="ignore"):
                            r = np.where(diff == 0, 0.0, diff / ((2 if two else 1) * k * np.finfo(dt).eps * g))[mask].max()
                        assert r <= TOL_C, tag + (r,)
        blas.device_status()
    finally:
        blas.test_control(blas.TEST_TRI_WAY, 0)


def test_special_cases():
    import torch
    n, k = 100, 40
    A = synth.matrix(71, n, k, n)
    # alpha == 0 scales the triangle only; beta == 0 stores zeros without reading
    dC = torch.full((n, n), float("nan"), dtype=torch.float64, device="cuda")
    blas.gpu_syrk("d", 1, 0, n, k, 0.0, None, n, 0.0, dC, n)
    torch.cuda.synchronize()
    got = to_host(dC)
    mask = netlib.triangle_mask("L", n)
    assert (got[mask] == 0).all() and np.isnan(got[~mask]).all()
    # k == 0 with beta == 1.3
    C0 = synth.matrix(72, n, n, n)
    dC = to_device(C0)
    blas.gpu_syrk("d", 0, 1, n, 0, 1.0, to_device(A), 1, 1.3, dC, n)
    torch.cuda.synchronize()
    got = to_host(dC)
    um = netlib.triangle_mask("U", n)
    assert np.array_equal(got[um], (C0 * 1.3)[um]) and np.array_equal(got[~um], C0[~um])
    # rank-2k: alpha == 0 scales the triangle without reading A or B
    dC = to_device(C0)
    blas.gpu_syr2k("d", 0, 0, n, k, 0.0, None, n, None, n, 1.3, dC, n)
    torch.cuda.synchronize()
    got = to_host(dC)
    assert np.array_equal(got[um], (C0 * 1.3)[um]) and np.array_equal(got[~um], C0[~um])
    # symm with alpha == 0: C <- beta C, A and B not read
    dC = to_device(C0)
    blas.gpu_symm("d", 0, 1, n, n, 0.0, None, n, None, n, 0.5, dC, n, None)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dC), 0.5 * C0)
    # trmm with alpha == 0: zeros without reading
    dB = torch.full((n, n), float("nan"), dtype=torch.float64, device="cuda")
    blas.gpu_trmm("d", 1, 0, 1, 0, n, n, 0.0, None, n, dB, n)
    torch.cuda.synchronize()
    assert (to_host(dB) == 0).all()
    # identity triangle: B <- alpha B exactly
    B0 = synth.matrix(73, n, k, n)
    dB = to_device(B0)
    blas.gpu_trmm("d", 0, 1, 0, 0, n, k, 2.0, to_device(np.asfortranarray(np.eye(n))), n, dB, n)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dB), 2.0 * B0)


def test_large_identities():
    """Order 4096 on the device: whole-matrix identities in float64 that no
    localised error escapes (R x against the same product evaluated as
    matrix-vector products), with the bound 4 (k + n) eps |.||.||x|."""
    import torch
    n, k = 4096, 2048
    eps = np.finfo(np.float64).eps
    A = synth.matrix(201, n, k, n)
    B = synth.matrix(202, n, k, n)
    C0 = synth.matrix(203, n, n, n)
    x = synth.matrix(204, n, 1, n)[:, 0]
    low = netlib.triangle_mask("L", n)
    sym = lambda M: np.where(low, M, M.T)          # the symmetric matrix behind a stored lower triangle
    dA, dB = to_device(A), to_device(B)
    # syrk and syr2k, lower triangle; the upper triangle of C holds NaN and must stay so
    Cin = np.where(low, C0, np.nan)
    Cin = np.asfortranarray(Cin)
    for two in (False, True):
        dC = to_device(Cin)
        if two:
            blas.gpu_syr2k("d", 1, 0, n, k, 0.7, dA, n, dB, n, 1.3, dC, n)
        else:
            blas.gpu_syrk("d", 1, 0, n, k, 0.7, dA, n, 1.3, dC, n)
        torch.cuda.synchronize()
        got = to_host(dC)
        assert np.isnan(got[~low]).all() and not np.isnan(got[low]).any()
        lhs = sym(np.nan_to_num(got)) @ x
        c0x = sym(C0) @ x
        if two:
            rhs = 0.7 * (A @ (B.T @ x) + B @ (A.T @ x)) + 1.3 * c0x
            scale = 0.7 * 2 * (np.abs(A) @ (np.abs(B).T @ np.abs(x))) + 1.3 * (np.abs(sym(C0)) @ np.abs(x))
        else:
            rhs = 0.7 * (A @ (A.T @ x)) + 1.3 * c0x
            scale = 0.7 * (np.abs(A) @ (np.abs(A).T @ np.abs(x))) + 1.3 * (np.abs(sym(C0)) @ np.abs(x))
        assert (np.abs(lhs - rhs) <= 4 * (2 * k + n) * eps * scale).all(), ("syr2k" if two else "syrk")
    # symm, both sides and both triangles, order 4192: diagonal blocks of 2048, 2048 and 96, completed one
    # after the other in a workspace of one block; the blocks off the diagonal are read where they are
    # stored.  The triangle that is not stored holds NaN; beta == 0 on a C full of NaN for two of the four.
    ka, other = 4096 + 96, 640
    S = synth.matrix(205, ka, ka, ka)
    work = torch.empty(2048 * 2048, dtype=torch.float64, device="cuda")
    for right, lower in itertools.product((0, 1), (0, 1)):
        stored = netlib.triangle_mask("L" if lower else "U", ka)
        Sfull = np.where(stored, S, S.T)
        Sin = np.asfortranarray(np.where(stored, S, np.nan))
        m_, n_ = (other, ka) if right else (ka, other)
        Bm = synth.matrix(206, m_, n_, m_)
        Cm = synth.matrix(207, m_, n_, m_)
        beta = 1.3 if right == lower else 0.0
        dC = to_device(Cm if beta != 0.0 else np.full_like(Cm, np.nan))
        blas.gpu_symm("d", right, lower, m_, n_, 0.7, to_device(Sin), ka, to_device(Bm), m_, beta, dC, m_, work)
        torch.cuda.synchronize()
        got = to_host(dC)
        assert not np.isnan(got).any(), ("symm", right, lower)
        y = synth.matrix(208, n_, 1, n_)[:, 0]
        lhs = got @ y
        if right:
            rhs = 0.7 * (Bm @ (Sfull @ y)) + beta * (Cm @ y)
            scale = 0.7 * (np.abs(Bm) @ (np.abs(Sfull) @ np.abs(y))) + abs(beta) * (np.abs(Cm) @ np.abs(y))
        else:
            rhs = 0.7 * (Sfull @ (Bm @ y)) + beta * (Cm @ y)
            scale = 0.7 * (np.abs(Sfull) @ (np.abs(Bm) @ np.abs(y))) + abs(beta) * (np.abs(Cm) @ np.abs(y))
        assert (np.abs(lhs - rhs) <= 4 * (ka + n_) * eps * scale).all(), ("symm", right, lower)
    # trmm, right side, lower triangle, transposed, unit diagonal (diagonal and upper part hold NaN)
    T = synth.matrix(209, k, k, k)
    lowk = netlib.triangle_mask("L", k)
    Tfull = np.where(lowk, T, 0.0)
    Tfull[np.arange(k), np.arange(k)] = 1.0
    Tin = np.where(lowk, T, np.nan)
    Tin[np.arange(k), np.arange(k)] = np.nan
    Bm = synth.matrix(206, n, k, n)
    y = synth.matrix(208, k, 1, k)[:, 0]
    dB2 = to_device(Bm)
    blas.gpu_trmm("d", 1, 1, 1, 1, n, k, 0.7, to_device(np.asfortranarray(Tin)), k, dB2, n)
    torch.cuda.synchronize()
    got = to_host(dB2)
    lhs = got @ y
    rhs = 0.7 * (Bm @ (Tfull.T @ y))
    scale = 0.7 * (np.abs(Bm) @ (np.abs(Tfull).T @ np.abs(y)))
    assert not np.isnan(got).any()
    assert (np.abs(lhs - rhs) <= 4 * (n + k) * eps * scale).all(), "trmm"
