"""What pins the CPU oracle without the reference: the exact known answers of
the reference's level-3 tester, a higher-precision brute-force product, the
special cases the interface defines, invariants of the call, and the
(call -> info) tables of the reference's error-exit tests."""
import itertools
from fractions import Fraction

import numpy as np
import pytest

import netlib
from ulmblas_amd import synth


def test_exact_known_answers(oracle):
    """test/F77/dblat3.f:195-256: A(i,j) = max(i-j+1, 0), b = 1..n, n = 32 =>
    c_j = j*((j+1)*j)/2 - ((j+1)*j*(j-1))/3 exactly, and the transposed /
    reversed variants.  Integers, so any summation order must reproduce them;
    a dropped term, a transposed operand or an index slip does not."""
    n, nmax = 32, 65
    ab = np.zeros((nmax, 2 * nmax), order="F")
    for j in range(1, n + 1):
        for i in range(1, n + 1):
            ab[i - 1, j - 1] = max(i - j + 1, 0)
        ab[j - 1, nmax] = j            # column vector b for 'N'
        ab[0, nmax + j - 1] = j        # row vector b for 'T'
    cc = np.array([j * ((j + 1) * j) // 2 - ((j + 1) * j * (j - 1)) // 3 for j in range(1, n + 1)], dtype=np.float64)
    A = ab[:, :nmax]
    B = ab[:, nmax:]

    def run(variant, ta, tb, Bmat, want):
        dt = np.float64 if variant == "d" else np.float32
        c = np.full((nmax, 1), np.nan, dtype=dt, order="F")
        oracle.gemm(variant, ta, tb, n, 1, n, 1.0, np.asfortranarray(A.astype(dt)), nmax,
                    np.asfortranarray(Bmat.astype(dt)), nmax, 0.0, c, nmax)
        assert np.array_equal(c[:n, 0], want.astype(dt)), (variant, ta, tb)

    for variant in ("d", "s", "s_f64"):
        run(variant, "N", "N", B, cc)
        run(variant, "N", "T", B, cc)
    for j in range(1, n + 1):
        ab[j - 1, nmax] = n - j + 1
        ab[0, nmax + j - 1] = n - j + 1
    ccr = cc[::-1].copy()
    for variant in ("d", "s", "s_f64"):
        run(variant, "T", "N", B, ccr)
        run(variant, "T", "T", B, ccr)


def test_brute_force_rational(oracle):
    """Tiny shapes against exact rational arithmetic: the oracle's result must
    lie within the DMMCH gauge bound (threshold 16, test/F77/dblat3.dat.in:8)
    of the true value for every trans combination."""
    rng = np.random.default_rng(5)
    for (m, n, k) in [(3, 4, 5), (5, 2, 17), (1, 1, 30)]:
        for ta, tb in itertools.product("NT", repeat=2):
            ra, ca = (k, m) if ta == "T" else (m, k)
            rb, cb = (n, k) if tb == "T" else (k, n)
            A = np.asfortranarray(rng.uniform(-1, 1, (ra, ca)))
            B = np.asfortranarray(rng.uniform(-1, 1, (rb, cb)))
            C0 = np.asfortranarray(rng.uniform(-1, 1, (m, n)))
            alpha, beta = 0.7, 1.3
            Cm = C0.copy(order="F")
            oracle.gemm("d", ta, tb, m, n, k, alpha, A, ra, B, rb, beta, Cm, m)
            for i in range(m):
                for j in range(n):
                    s = Fraction(0)
                    g = Fraction(0)
                    for l in range(k):
                        a = Fraction(A[l, i] if ta == "T" else A[i, l])
                        b = Fraction(B[j, l] if tb == "T" else B[l, j])
                        s += a * b
                        g += abs(a * b)
                    exact = Fraction(alpha) * s + Fraction(beta) * Fraction(C0[i, j])
                    gauge = abs(Fraction(alpha)) * g + abs(Fraction(beta)) * abs(Fraction(C0[i, j]))
                    err = abs(Fraction(Cm[i, j]) - exact)
                    assert err <= 16 * Fraction(np.finfo(np.float64).eps) * gauge, (m, n, k, ta, tb, i, j)


@pytest.mark.parametrize("variant", ["d", "s", "s_f64"])
def test_gauge_bound_vs_wide_product(oracle, variant):
    """k beyond one KC slice, edge tiles in m and n: compare with a float64
    (for float data) or long-double (for double data) product."""
    dt = np.float64 if variant == "d" else np.float32
    wide = np.longdouble if variant == "d" else np.float64
    m, n, k = 70, 45, 900
    for ta, tb in itertools.product("NT", repeat=2):
        ra, ca = (k, m) if ta == "T" else (m, k)
        rb, cb = (n, k) if tb == "T" else (k, n)
        A = synth.matrix(51, ra, ca, ra + 1, dtype=dt)
        B = synth.matrix(52, rb, cb, rb + 1, dtype=dt)
        C0 = synth.matrix(53, m, n, m + 1, dtype=dt)
        Cm = C0.copy(order="F")
        oracle.gemm(variant, ta, tb, m, n, k, -0.75, A, ra + 1, B, rb + 1, 0.25, Cm, m + 1)
        opa = (A[:ra].T if ta == "T" else A[:ra]).astype(wide)
        opb = (B[:rb].T if tb == "T" else B[:rb]).astype(wide)
        want = -0.75 * (opa @ opb) + 0.25 * C0[:m].astype(wide)
        g = 0.75 * (np.abs(opa) @ np.abs(opb)) + 0.25 * np.abs(C0[:m].astype(wide))
        ratio = np.abs(Cm[:m].astype(wide) - want) / (np.finfo(dt).eps * g)
        # sequential fp summation: error grows at most like k, typically sqrt(k)
        assert float(ratio.max()) < (k if variant == "s" else 64), (variant, ta, tb, float(ratio.max()))
        assert np.array_equal(Cm[m:], C0[m:])          # padding untouched


@pytest.mark.parametrize("variant", ["d", "s", "s_f64"])
def test_special_cases(oracle, variant):
    dt = np.float64 if variant == "d" else np.float32
    m, n, k = 19, 23, 40
    A = synth.matrix(61, m, k, m + 2, dtype=dt)
    B = synth.matrix(62, k, n, k + 2, dtype=dt)
    C0 = synth.matrix(63, m, n, m + 2, dtype=dt)

    # alpha == 0: C <- beta*C exactly, A and B are never looked at (NaN there is harmless)
    An = np.full_like(A, np.nan)
    Cm = C0.copy(order="F")
    oracle.gemm(variant, "N", "N", m, n, k, 0.0, An, m + 2, An[:k + 2, :n].copy(order="F"), k + 2, 1.3, Cm, m + 2)
    # sgemm_ scales in double and rounds once (interfaces/blas/F77/gemm.cc:36), cblas_sgemm in float
    want = C0[:m] * dt(1.3) if variant != "s_f64" else (C0[:m].astype(np.float64) * 1.3).astype(dt)
    assert np.array_equal(Cm[:m], want)
    # k == 0 likewise; beta == 1 leaves C bit-identical, beta == 0 gives zeros even from NaN
    Cm = C0.copy(order="F")
    oracle.gemm(variant, "N", "N", m, n, 0, 1.0, A, m + 2, B, k + 2, 1.0, Cm, m + 2)
    assert Cm.tobytes() == C0.tobytes()
    Cn = C0.copy(order="F")
    Cn[:m] = np.nan
    oracle.gemm(variant, "N", "N", m, n, 0, 1.0, A, m + 2, B, k + 2, 0.0, Cn, m + 2)
    assert np.array_equal(Cn[:m], np.zeros((m, n), dtype=dt)) and np.array_equal(Cn[m:], C0[m:])
    # beta == 0 with NaN in C: the product alone, no NaN
    Cn[:m] = np.nan
    oracle.gemm(variant, "N", "N", m, n, k, 1.0, A, m + 2, B, k + 2, 0.0, Cn, m + 2)
    assert not np.isnan(Cn[:m]).any()
    # m == 0 or n == 0: nothing is written
    Cm = C0.copy(order="F")
    oracle.gemm(variant, "N", "N", 0, n, k, 1.0, A, m + 2, B, k + 2, 0.0, Cm, m + 2)
    oracle.gemm(variant, "N", "N", m, 0, k, 1.0, A, m + 2, B, k + 2, 0.0, Cm, m + 2)
    assert Cm.tobytes() == C0.tobytes()
    # B = identity: C = alpha*A exactly (one non-zero product per element)
    I = np.zeros((k + 2, k), dtype=dt, order="F")
    I[:k] = np.eye(k, dtype=dt)
    Cm = np.full((m + 2, k), np.nan, dtype=dt, order="F")
    oracle.gemm(variant, "N", "N", m, k, k, 2.0, A, m + 2, I, k + 2, 0.0, Cm, m + 2)
    assert np.array_equal(Cm[:m], 2 * A[:m])
    # A = identity with B transposed in memory: C = B^T
    Bt = np.asfortranarray(B[:k, :n].T.copy())
    Ik = np.asfortranarray(np.eye(k, dtype=dt))
    Cm = np.full((k, n), np.nan, dtype=dt, order="F")
    oracle.gemm(variant, "T", "T", k, n, k, 1.0, Ik, k, Bt, n, 0.0, Cm, k)
    assert np.array_equal(Cm, B[:k, :n])


def test_result_depends_on_kc_only(oracle):
    """The rounding pattern is fixed by KC alone: MC, NC, MR, NR re-tile the
    same per-element sums (they differ between the reference's test variants,
    test/F77/config/make.testcase0[1-3].inc), KC changes where partial sums
    are folded into C."""
    m, n, k = 37, 29, 100
    A = synth.matrix(71, m, k)
    B = synth.matrix(72, k, n)
    C0 = synth.matrix(73, m, n)
    outs = {}
    for bs in [(8, 12, 12, 4, 4), (8, 12, 12, 2, 4), (8, 12, 12, 4, 2), (16, 12, 8, 8, 4), (6, 12, 10, 3, 5),
               (8, 24, 12, 4, 4), (8, 100, 12, 4, 4)]:
        Cm = C0.copy(order="F")
        oracle.gemm("d", "N", "N", m, n, k, 0.7, A, m, B, k, 1.3, Cm, m, blocksize=bs)
        outs[bs] = Cm
    # MC must be a multiple of MR and NC of NR (the pack buffers are sized MC*KC+MR, KC*NC+NR)
    with pytest.raises(RuntimeError):
        oracle.gemm("d", "N", "N", m, n, k, 0.7, A, m, B, k, 1.3, C0.copy(order="F"), m, blocksize=(5, 12, 7, 3, 5))
    base = outs[(8, 12, 12, 4, 4)]
    for bs, Cm in outs.items():
        if bs[1] == 12:
            assert np.array_equal(Cm, base), bs
    assert not np.array_equal(outs[(8, 24, 12, 4, 4)], base)
    assert np.allclose(outs[(8, 100, 12, 4, 4)], base, rtol=1e-13)


def test_samples_equal_full_product(oracle):
    """The per-element restatement used to check samples of large products
    returns exactly the element the full frame computes."""
    rng = np.random.default_rng(3)
    for variant, dt in (("d", np.float64), ("s", np.float32), ("s_f64", np.float32)):
        m, n, k = 50, 41, 1000
        for ta, tb in itertools.product("NT", repeat=2):
            for alpha, beta in [(1.0, 0.0), (0.7, 1.3), (-1.0, 1.0), (0.0, 0.5)]:
                ra, ca = (k, m) if ta == "T" else (m, k)
                rb, cb = (n, k) if tb == "T" else (k, n)
                A = synth.matrix(81, ra, ca, ra + 1, dtype=dt)
                B = synth.matrix(82, rb, cb, rb + 3, dtype=dt)
                C0 = synth.matrix(83, m, n, m + 2, dtype=dt)
                Cm = C0.copy(order="F")
                oracle.gemm(variant, ta, tb, m, n, k, alpha, A, ra + 1, B, rb + 3, beta, Cm, m + 2)
                rows = rng.integers(0, m, 64)
                cols = rng.integers(0, n, 64)
                vals, g = oracle.samples(variant, ta, tb, m, n, k, alpha, A, ra + 1, B, rb + 3, beta, C0, m + 2, rows,
                                         cols)
                assert np.array_equal(vals, Cm[rows, cols]), (variant, ta, tb, alpha, beta)
                gfull = oracle.gauge(ta, tb, m, n, k, alpha, A, B, beta, C0)
                assert np.allclose(g, gfull[rows, cols], rtol=1e-12)


def test_row_major_is_swapped_col_major(oracle):
    """interfaces/blas/C/gemm.cc:478-484: a row-major call equals the
    column-major call on swapped operands; checked against numpy on C-ordered
    arrays, so the swap itself is pinned, not restated."""
    m, n, k = 11, 7, 13
    rng = np.random.default_rng(9)
    for ta in (oracle.NO_TRANS, oracle.TRANS):
        for tb in (oracle.NO_TRANS, oracle.TRANS):
            A = rng.uniform(-1, 1, (k, m) if ta == oracle.TRANS else (m, k))
            B = rng.uniform(-1, 1, (n, k) if tb == oracle.TRANS else (k, n))
            C0 = rng.uniform(-1, 1, (m, n))
            Cm = C0.copy()
            assert oracle.cblas_dgemm(oracle.ROW_MAJOR, ta, tb, m, n, k, 0.5, A, A.shape[1], B, B.shape[1], 2.0, Cm,
                                      n) == 0
            opa = A.T if ta == oracle.TRANS else A
            opb = B.T if tb == oracle.TRANS else B
            assert np.allclose(Cm, 0.5 * opa @ opb + 2.0 * C0, rtol=1e-13, atol=1e-14)


def test_error_exit_tables(oracle):
    """(call -> info) pairs of DCHKE (test/F77/dblat3.f:1838-1921) and of
    test/C/c_d3chke.c:46-273."""
    for args, info in netlib.F77_ERROR_EXITS:
        assert oracle.f77_info(*args) == info, args
    for args, info in netlib.CBLAS_ERROR_EXITS:
        assert netlib.cblas_tester_info(args[0], oracle.cblas_info(*args)) == info, args
    # valid calls, incl. lower case and 'R' (interfaces/blas/F77/gemm.cc:171-182)
    for ta, tb in itertools.product("NnTtCcRr", repeat=2):
        assert oracle.f77_info(ta, tb, 3, 4, 5, 5, 5, 3) == 0
    # a failed check leaves C alone
    Cm = np.ones((2, 2), order="F")
    assert oracle.dgemm_f77("N", "N", 2, 2, 2, 1.0, Cm, 1, Cm, 2, 0.0, Cm, 2) == 8
    assert (Cm == 1).all()


def test_netlib_generator():
    """DBEG (test/F77/dblat3.f:2673-2718): I = I*891 mod 1000 from 7, every
    fifth call skips one value; first values by hand."""
    b = netlib.Beg()
    want_i = []
    i, ic = 7, 0
    for _ in range(12):
        ic += 1
        i = (i * 891) % 1000
        if ic >= 5:
            ic = 0
            i = (i * 891) % 1000
        want_i.append(i)
    assert want_i[:5] == [237, 167, 797, 127, 887]       # 157 is skipped by the fifth call
    got = [b.next() for _ in range(12)]
    assert got == [(v - 500) / 1001.0 for v in want_i]
    assert all(-0.5 < v < 0.5 for v in got)
    aa = netlib.make_ge(netlib.Beg(), 3, 5, 4)
    assert (aa[3, :] == netlib.ROGUE).all() and aa[0, 1] == 0.0 and aa[1, 1] != 0.0   # column n/2 = 2 zeroed off-diagonal
