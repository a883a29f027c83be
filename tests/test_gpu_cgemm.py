"""Complex GEMM on the GPU through the C ABI: the complex netlib tester's sweep
(ZCHK1 / CCHK1 of test/F77/zblat3.f, cblat3.f) through zgemm_ / cgemm_, the
CBLAS driver's sweep in both storage orders, and the device-resident entry
points on larger and ragged shapes against the CPU oracle.

Parity bound: each component of C is a sum of 2k real products on the GPU and
a sequence of k complex multiply-adds in the reference, so

    max(|Re d|, |Im d|) <= TOL_C * (2k + 2) * eps * G,
    G = ABS1(alpha) sum ABS1(a) ABS1(b) + ABS1(beta) ABS1(c),  ABS1(z) = |Re z| + |Im z|

(the tester's own gauge, zblat3.f:2935-3000; the + 2 covers alpha folded into
the elements of A and a complex beta applied in a pass of its own).
"""
import itertools

import numpy as np
import pytest

import netlib
from gpu_util import TOL_C
from ulmblas_amd import blas, synth

pytestmark = pytest.mark.gpu


def cparity(got, want, gauge, k, dtype):
    eps = np.finfo(dtype).eps
    d = got.astype(np.complex128) - want.astype(np.complex128)
    diff = np.maximum(np.abs(d.real), np.abs(d.imag))
    scale = (2 * k + 2) * eps * gauge
    with np.errstate(divide="ignore", invalid="ignore"):
        r = np.where(diff == 0, 0.0, diff / scale)
    return float(r.max()) if r.size else 0.0


def cmatrix(seed, rows, cols, ld, dtype):
    z = synth.matrix(seed, rows, cols, ld) + 1j * synth.matrix(seed + 100, rows, cols, ld)
    return np.asfortranarray(z.astype(dtype))


def to_dev(X):
    import torch
    return torch.from_numpy(np.ascontiguousarray(X.T)).cuda()


def to_host(dX):
    return np.asfortranarray(dX.cpu().numpy().T)


@pytest.mark.parametrize("prec", ["z", "c"])
def test_chk1_f77(prec, oracle, xerbla):
    dt = np.complex128 if prec == "z" else np.complex64
    params = netlib.ZBLAT3
    calls, worst, errmax = 0, 0.0, 0.0
    for c in netlib.chk1_cases(params, dt):
        m, n, k = c["m"], c["n"], c["k"]
        aa, bb, cc = c["aa"].copy(order="F"), c["bb"].copy(order="F"), c["cc"].copy(order="F")
        blas.cgemm_(prec, c["transa"], c["transb"], m, n, k, c["alpha"], aa, c["lda"], bb, c["ldb"], c["beta"], cc,
                    c["ldc"])
        calls += 1
        assert aa.tobytes() == c["aa"].tobytes() and bb.tobytes() == c["bb"].tobytes()
        if m == 0 or n == 0:
            assert cc.tobytes() == c["cc"].tobytes()
            continue
        tag = (c["transa"], c["transb"], m, n, k, c["alpha"], c["beta"])
        assert np.array_equal(cc[m:], c["cc"][m:]), tag
        err, _ = netlib.zmmch(c["transa"], c["transb"], m, n, k, c["alpha"], c["aa"], c["bb"], c["beta"], c["cc"], cc,
                              dt)
        assert err < params["thresh"], (tag, err)
        errmax = max(errmax, err)
        want = c["cc"].copy(order="F")
        oracle.cgemm(prec, c["transa"], c["transb"], m, n, k, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"],
                     c["beta"], want, c["ldc"])
        g = oracle.cgauge(c["transa"], c["transb"], m, n, k, c["alpha"], c["aa"], c["bb"], c["beta"], c["cc"])
        r = cparity(cc[:m], want[:m], g, k, dt)
        assert r <= TOL_C, (tag, r)
        worst = max(worst, r)
    assert xerbla.capture_count() == 0
    assert calls == len(params["idim"]) ** 3 * 81
    print(f"chk1 {prec}: {calls} calls, max tester ratio {errmax:.3f}, max parity ratio {worst:.3f}")


def test_chk1_cblas_both_orders(oracle, xerbla):
    """test/C/c_zblat3.f with test/C/c_zblas3.c: the same calls through
    cblas_zgemm, column-major as they are and row-major on transposed copies;
    the unchecked ulmblas_ / ATL_ symbols on the column-major calls."""
    dt = np.complex128
    params = netlib.ZIN3
    rogue = netlib.ZROGUE
    calls = 0
    for c in netlib.chk1_cases(params, dt):
        m, n, k = c["m"], c["n"], c["k"]
        ta, tb = blas.TRANS_OF_CHAR[c["transa"]], blas.TRANS_OF_CHAR[c["transb"]]
        want = c["cc"].copy(order="F")
        oracle.cgemm("z", c["transa"], c["transb"], m, n, k, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"],
                     c["beta"], want, c["ldc"])
        cc = c["cc"].copy(order="F")
        blas.cblas_cgemm("z", blas.CblasColMajor, ta, tb, m, n, k, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"],
                         c["beta"], cc, c["ldc"])
        c2 = c["cc"].copy(order="F")
        blas.ulmblas_cgemm("z", ta, tb, m, n, k, c["alpha"], c["aa"], c["lda"], c["bb"], c["ldb"], c["beta"], c2,
                           c["ldc"], prefix="ATL_" if calls % 2 else "ulmblas_")
        calls += 1
        assert cc.tobytes() == c2.tobytes()
        np.testing.assert_allclose(cc[:m], want[:m], rtol=0, atol=1e-13)
        assert np.array_equal(cc[m:], c["cc"][m:])
        # row-major copies of the three windows, one rogue column of padding each
        ra, ca = (k, m) if c["transa"] in "TC" else (m, k)
        rb, cb = (n, k) if c["transb"] in "TC" else (k, n)
        a_row = np.full((ra, ca + 1), rogue)
        a_row[:, :ca] = c["aa"][:ra, :]
        b_row = np.full((rb, cb + 2), rogue)
        b_row[:, :cb] = c["bb"][:rb, :]
        c_row = np.full((m, n + 1), rogue)
        c_row[:, :n] = c["cc"][:m, :]
        blas.cblas_cgemm("z", blas.CblasRowMajor, ta, tb, m, n, k, c["alpha"], a_row, ca + 1, b_row, cb + 2, c["beta"],
                         c_row, n + 1)
        np.testing.assert_allclose(c_row[:, :n], want[:m], rtol=0, atol=1e-13)
        assert (c_row[:, n] == rogue).all()
    assert xerbla.capture_count() == 0
    assert calls == len(params["idim"]) ** 3 * 81


@pytest.mark.parametrize("prec", ["z", "c"])
def test_device_entry_all_flags(prec, oracle):
    """All sixteen N/T/C/R combinations, real, complex and zero beta, ragged
    shapes with padded leading dimensions; NaN where nothing may be read."""
    import torch
    dt = np.complex128 if prec == "z" else np.complex64
    worst = 0.0
    shapes = [(1, 1, 1), (65, 33, 47), (300, 130, 257), (517, 259, 1100)]
    for (m, n, k) in shapes:
        combos = itertools.product("NTCR", "NTCR") if m <= 300 else [("N", "N"), ("C", "T"), ("T", "R"), ("R", "C")]
        for ta, tb in combos:
            ra, ca = (k, m) if ta in "TC" else (m, k)
            rb, cb = (n, k) if tb in "TC" else (k, n)
            lda, ldb, ldc = ra + 3, rb + 1, m + 2
            A, B, C0 = cmatrix(81, ra, ca, lda, dt), cmatrix(82, rb, cb, ldb, dt), cmatrix(83, m, n, ldc, dt)
            for alpha, beta in ((0.7 - 0.9j, 1.3 - 1.1j), (1.0, 0.0), (-0.5j, 2.0)):
                Cin = C0.copy(order="F")
                if beta == 0:
                    Cin[:m] = complex(np.nan, np.nan)
                dC = to_dev(Cin)
                blas.gpu_cgemm(prec, ta, tb, m, n, k, alpha, to_dev(A), lda, to_dev(B), ldb, beta, dC, ldc)
                torch.cuda.synchronize()
                got = to_host(dC)
                want = Cin.copy(order="F")
                oracle.cgemm(prec, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, want, ldc)
                tag = (prec, ta, tb, m, n, k, alpha, beta)
                assert not np.isnan(got[:m]).any(), tag
                assert np.array_equal(got[m:], Cin[m:]), tag
                g = oracle.cgauge(ta, tb, m, n, k, alpha, A, B, beta, C0)
                r = cparity(got[:m], want[:m], g, k, dt)
                assert r <= TOL_C, (tag, r)
                worst = max(worst, r)
    print(f"device {prec}gemm: max parity ratio {worst:.3f}")


def test_special_cases():
    import torch
    m, n, k = 40, 30, 20
    dt = np.complex128
    A, B, C0 = cmatrix(91, m, k, m, dt), cmatrix(92, k, n, k, dt), cmatrix(93, m, n, m, dt)
    # alpha == 0: C <- beta C without reading A or B, for a complex and a real beta; beta == 0 stores zeros
    for beta in (1.3 - 1.1j, 2.0):
        dC = to_dev(C0)
        blas.gpu_cgemm("z", "N", "N", m, n, k, 0.0, None, m, None, k, beta, dC, m, work=torch.empty(16, dtype=torch.uint8, device="cuda"))
        torch.cuda.synchronize()
        np.testing.assert_allclose(to_host(dC), beta * C0, rtol=0, atol=1e-15)
    dC = to_dev(np.full_like(C0, complex(np.nan, np.nan)))
    blas.gpu_cgemm("z", "T", "C", m, n, 0, 1.0, to_dev(A), 1, to_dev(B), n, 0.0, dC, m)
    torch.cuda.synchronize()
    assert (to_host(dC) == 0).all()
    # identity: C <- alpha B exactly when alpha has one non-zero part
    eye = np.asfortranarray(np.eye(k, dtype=dt))
    dC = to_dev(np.zeros((k, n), dtype=dt, order="F"))
    blas.gpu_cgemm("z", "C", "N", k, n, k, 2.0j, to_dev(eye), k, to_dev(B), k, 0.0, dC, k)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dC), 2.0j * B)
    # conjugation flags against numpy on Gaussian integers (exact)
    rng = np.random.default_rng(5)
    Ai = np.asfortranarray((rng.integers(-9, 10, (k, m)) + 1j * rng.integers(-9, 10, (k, m))).astype(dt))
    Bi = np.asfortranarray((rng.integers(-9, 10, (n, k)) + 1j * rng.integers(-9, 10, (n, k))).astype(dt))
    dC = to_dev(np.zeros((m, n), dtype=dt, order="F"))
    blas.gpu_cgemm("z", "C", "T", m, n, k, 1.0, to_dev(Ai), k, to_dev(Bi), n, 0.0, dC, m)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dC), Ai.conj().T @ Bi.T)


def test_large_identity():
    """2048^3 complex double on the device: the whole-matrix identity
    C x = alpha op(A) (op(B) x) + beta C0 x in complex128, and parity of a
    block of rows with numpy's product."""
    import torch
    n = 2048
    dt = np.complex128
    A, B, C0 = cmatrix(95, n, n, n, dt), cmatrix(96, n, n, n, dt), cmatrix(97, n, n, n, dt)
    alpha, beta = 0.7 - 0.9j, 1.3 - 1.1j
    dC = to_dev(C0)
    blas.gpu_cgemm("z", "N", "C", n, n, n, alpha, to_dev(A), n, to_dev(B), n, beta, dC, n)
    torch.cuda.synchronize()
    got = to_host(dC)
    x = cmatrix(98, n, 1, n, dt)[:, 0]
    lhs = got @ x
    rhs = alpha * (A @ (B.conj().T @ x)) + beta * (C0 @ x)
    abs1 = lambda z: np.abs(z.real) + np.abs(z.imag)
    scale = abs1(np.array(alpha)) * (abs1(A) @ (abs1(B).T @ abs1(x))) + abs1(np.array(beta)) * (abs1(C0) @ abs1(x))
    assert (np.abs(lhs - rhs) <= 4 * n * np.finfo(np.float64).eps * scale).all()
    rows = slice(1000, 1064)
    want = alpha * (A[rows] @ B.conj().T) + beta * C0[rows]
    g = abs1(np.array(alpha)) * (abs1(A[rows]) @ abs1(B).T) + abs1(np.array(beta)) * abs1(C0[rows])
    d = got[rows] - want
    assert (np.maximum(np.abs(d.real), np.abs(d.imag)) <= TOL_C * (2 * n + 2) * np.finfo(np.float64).eps * g).all()
