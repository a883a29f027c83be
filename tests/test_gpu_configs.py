"""The benchmark configurations, checked for parity with the CPU oracle.

Shapes the oracle recomputes in seconds are compared in full.  Larger ones are
checked on (a) sampled elements, whose reference values come from the oracle's
per-element restatement (equal to what the full frame would write) and (b) a
whole-matrix identity, C x = alpha op(A) (op(B) x) + beta C0 x for a random x,
evaluated in fp64, which no localised error escapes.  The bound is the one
stated in gpu_util.TOL_C: |delta| <= 2 k eps (|alpha||A||B| + |beta||C|).
"""
import numpy as np
import pytest

from gpu_util import TOL_C, parity_ratio, to_device, to_host
from ulmblas_amd import blas, synth

pytestmark = pytest.mark.gpu

SENTINEL = -2560000000.0


def _operands(prec, ta, tb, m, n, k, lda, ldb, ldc, dist, beta, seed=1000):
    dt = np.float64 if prec == "d" else np.float32
    ra, ca = (k, m) if ta == "T" else (m, k)
    rb, cb = (n, k) if tb == "T" else (k, n)
    A = synth.matrix(seed + 1, ra, ca, lda, dist=dist, dtype=dt)
    B = synth.matrix(seed + 2, rb, cb, ldb, dist=dist, dtype=dt)
    C0 = synth.matrix(seed + 3, m, n, ldc, dist=dist, dtype=dt)
    if beta == 0.0:
        C0[:m, :] = np.nan        # beta == 0 must not read C
    return A, B, C0


def _full(oracle, prec, ta, tb, m, n, k, alpha, beta, lda=None, ldb=None, ldc=None, dist="uniform", host=False,
          variants=None):
    dt = np.float64 if prec == "d" else np.float32
    lda = lda or max(1, k if ta == "T" else m)
    ldb = ldb or max(1, n if tb == "T" else k)
    ldc = ldc or max(1, m)
    A, B, C0 = _operands(prec, ta, tb, m, n, k, lda, ldb, ldc, dist, beta)
    if host:
        got = C0.copy(order="F")
        (blas.dgemm_ if prec == "d" else blas.sgemm_)(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, got, ldc)
    else:
        import torch
        dC = to_device(C0)
        (blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm)(ta == "T", tb == "T", m, n, k, alpha, to_device(A), lda,
                                                           to_device(B), ldb, beta, dC, ldc)
        torch.cuda.synchronize()
        got = to_host(dC)
    assert not np.isnan(got[:m]).any()
    assert np.array_equal(got[m:], C0[m:])
    g = oracle.gauge(ta, tb, m, n, k, alpha, A, B, beta, C0)
    worst = 0.0
    for v in variants or (("d",) if prec == "d" else ("s", "s_f64")):
        want = C0.copy(order="F")
        oracle.gemm(v, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, want, ldc)
        r = parity_ratio(got[:m], want[:m], g, k, dt)
        assert r <= TOL_C, (prec, v, ta, tb, m, n, k, r)
        worst = max(worst, r)
    return worst


def _sampled(oracle, prec, ta, tb, m, n, k, alpha, beta, lda=None, ldb=None, ldc=None, dist="uniform", nsamples=4096,
             check_inputs=False):
    import torch
    dt = np.float64 if prec == "d" else np.float32
    tdt = torch.float64
    lda = lda or max(1, k if ta == "T" else m)
    ldb = ldb or max(1, n if tb == "T" else k)
    ldc = ldc or max(1, m)
    A, B, C0 = _operands(prec, ta, tb, m, n, k, lda, ldb, ldc, dist, beta)
    dA, dB, dC = to_device(A), to_device(B), to_device(C0)
    (blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm)(ta == "T", tb == "T", m, n, k, alpha, dA, lda, dB, ldb, beta,
                                                       dC, ldc)
    torch.cuda.synchronize()

    # (b) whole-matrix identity in fp64 on the device (tensor views: (cols, ld), element (i, j) at [j, i])
    x = torch.from_numpy(synth.uniform(77, n)).cuda()
    Cv = dC[:, :m].to(tdt)
    assert not torch.isnan(Cv).any()
    opB = (dB[:, :(n if tb == "T" else k)]).to(tdt)     # stored B: (colsB, rowsB)
    opA = (dA[:, :(k if ta == "T" else m)]).to(tdt)
    # op(B) x : (k)
    bx = opB @ x if tb == "T" else opB.T @ x            # tb: stored (k cols, n rows) -> [l, j]; else stored (n cols, k rows) -> [j, l]
    abx = opA @ bx if ta == "T" else opA.T @ bx         # ta: stored (m cols, k rows) -> [i, l]; else (k cols, m rows) -> [l, i]
    lhs = Cv.T @ x
    rhs = alpha * abx
    gx = abs(alpha) * ((opA.abs() @ ((opB.abs() @ x.abs()) if tb == "T" else (opB.abs().T @ x.abs()))) if ta == "T"
                       else (opA.abs().T @ ((opB.abs() @ x.abs()) if tb == "T" else (opB.abs().T @ x.abs()))))
    if beta != 0.0:
        C0v = to_device(C0)[:, :m].to(tdt)
        rhs = rhs + beta * (C0v.T @ x)
        gx = gx + abs(beta) * (C0v.abs().T @ x.abs())
    eps = np.finfo(dt).eps
    ident = float(((lhs - rhs).abs() / (k * eps * gx)).max())
    assert ident <= TOL_C, ("C x identity", prec, ta, tb, m, n, k, ident)

    # (a) sampled elements: corners, last row / column, random interior
    rng = np.random.default_rng(12345)
    rows = np.concatenate([[0, 0, m - 1, m - 1], np.full(16, m - 1), rng.integers(0, m, 16), rng.integers(0, m, nsamples)])
    cols = np.concatenate([[0, n - 1, 0, n - 1], rng.integers(0, n, 16), np.full(16, n - 1), rng.integers(0, n, nsamples)])
    got_all = to_host(dC)
    assert np.array_equal(got_all[m:], C0[m:]), "padding rows of C were written"
    if check_inputs:
        assert to_host(dA).tobytes(order="F") == A.tobytes(order="F")
        assert to_host(dB).tobytes(order="F") == B.tobytes(order="F")
    got = got_all[rows, cols]
    worst = 0.0
    for v in (("d",) if prec == "d" else ("s", "s_f64")):
        want, g = oracle.samples(v, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C0, ldc, rows, cols)
        r = parity_ratio(got, want, g, k, dt)
        assert r <= TOL_C, ("samples", prec, v, ta, tb, m, n, k, r)
        worst = max(worst, r)
    return worst, ident


def test_config1_plumbing(oracle):
    """dgemm N,N 1024^3, alpha = 1.5, beta = 0.5: device entry and dgemm_."""
    _full(oracle, "d", "N", "N", 1024, 1024, 1024, 1.5, 0.5)
    _full(oracle, "d", "N", "N", 1024, 1024, 1024, 1.5, 0.5, host=True)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_config2_square_sweep(oracle, ta, tb):
    """alpha = 1, beta = 0, C pre-filled with NaN."""
    _full(oracle, "d", ta, tb, 512, 512, 512, 1.0, 0.0)
    _full(oracle, "d", ta, tb, 2048, 2048, 2048, 1.0, 0.0)
    for n in (4096, 8192):
        _sampled(oracle, "d", ta, tb, n, n, n, 1.0, 0.0)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_config2_largest(oracle, ta, tb):
    """n = 16384: 2 GiB per operand, element offsets beyond 2^31 bytes, in every
    one of the four staging patterns."""
    _sampled(oracle, "d", ta, tb, 16384, 16384, 16384, 1.0, 0.0, nsamples=2048)


def test_config3_sgemm(oracle):
    """fp32, N,T, alpha = beta = 1, N(0,1) data; against both arithmetics the
    reference has for single precision (fp32 and fp64 accumulation)."""
    _full(oracle, "s", "N", "T", 1024, 1024, 1024, 1.0, 1.0, dist="normal")
    _full(oracle, "s", "N", "T", 1024, 1024, 1024, 1.0, 1.0, dist="normal", host=True)
    for n in (4096, 8192, 16384):
        _sampled(oracle, "s", "N", "T", n, n, n, 1.0, 1.0, dist="normal")


def test_config4_rectangular(oracle):
    """alpha = -1, beta = 1: rank-k update, tall-skinny, short-wide."""
    _sampled(oracle, "d", "N", "N", 16384, 16384, 256, -1.0, 1.0)
    _full(oracle, "d", "N", "N", 65536, 64, 1024, -1.0, 1.0)
    _full(oracle, "d", "N", "N", 64, 65536, 1024, -1.0, 1.0)


def test_config5_strided(oracle):
    """transA = T, m = 5000, n = 3000, k = 7000 (no multiple of any tile),
    lda = k+37, ldb = k+11, ldc = m+5, alpha = 0.75, beta = -0.25, sentinel in
    every padding row; A and B bit-unchanged, C's padding bit-unchanged."""
    m, n, k = 5000, 3000, 7000
    _sampled(oracle, "d", "T", "N", m, n, k, 0.75, -0.25, lda=k + 37, ldb=k + 11, ldc=m + 5, check_inputs=True)
    # the same layout at a size the oracle recomputes in full, device and host path
    m, n, k = 500, 300, 700
    _full(oracle, "d", "T", "N", m, n, k, 0.75, -0.25, lda=k + 37, ldb=k + 11, ldc=m + 5)
    _full(oracle, "d", "T", "N", m, n, k, 0.75, -0.25, lda=k + 37, ldb=k + 11, ldc=m + 5, host=True)


@pytest.fixture()
def host_head_switch():
    yield
    blas.test_control(blas.TEST_HOST_HEAD, 1)


@pytest.mark.parametrize("head", [0, 2], ids=["a_first", "head_of_b_first"])
@pytest.mark.parametrize("prec", ["d", "s"])
def test_host_entry_points_large(oracle, prec, head, host_head_switch):
    """dgemm_ / sgemm_ on products large enough for the library to cut C into
    column panels and stream them (upload, kernel, download overlapped): all
    four trans combinations, padded leading dimensions whose sentinels must
    survive, beta != 0 (C panels travel both ways) and beta == 0 with NaN in C
    (C must not travel up at all).  Both orders of the uploads: A first, or a
    head of op(B)'s columns first and the panels of A multiplied into it as they
    land (runs of k accumulated into C for op(A) = A, rows of C for op(A) =
    A'; here 1792 columns and two panels of A, the second shorter)."""
    dt = np.float64 if prec == "d" else np.float32
    f = blas.dgemm_ if prec == "d" else blas.sgemm_
    blas.test_control(blas.TEST_HOST_HEAD, head)
    m, n, k = 3100, 4700, 2300
    rng = np.random.default_rng(7)
    rows, cols = rng.integers(0, m, 3000), rng.integers(0, n, 3000)
    rows[:4], cols[:4] = [0, 0, m - 1, m - 1], [0, n - 1, 0, n - 1]
    x = synth.uniform(5, n).astype(np.float64)
    for ta in "NT":
        for tb in "NT":
            for alpha, beta in ((1.0, 0.0), (-0.5, 1.5)):
                ra, ca = (k, m) if ta == "T" else (m, k)
                rb, cb = (n, k) if tb == "T" else (k, n)
                lda, ldb, ldc = ra + 3, rb + 5, m + 7
                A, B, C0 = _operands(prec, ta, tb, m, n, k, lda, ldb, ldc, "uniform", beta, seed=2000)
                A0, B0 = A.copy(order="F"), B.copy(order="F")
                got = C0.copy(order="F")
                f(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, got, ldc)
                assert A.tobytes(order="F") == A0.tobytes(order="F") and B.tobytes(order="F") == B0.tobytes(order="F")
                assert np.array_equal(got[m:], C0[m:]), "padding rows of C were written"
                assert not np.isnan(got[:m]).any()
                for v in (("d",) if prec == "d" else ("s", "s_f64")):
                    want, g = oracle.samples(v, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C0, ldc, rows, cols)
                    r = parity_ratio(got[rows, cols], want, g, k, dt)
                    assert r <= TOL_C, (prec, v, ta, tb, alpha, beta, r)
                # every panel arrived: C x against alpha op(A) (op(B) x) + beta C0 x in float64
                opa = (A[:ra].T if ta == "T" else A[:ra]).astype(np.float64)
                opb = (B[:rb].T if tb == "T" else B[:rb]).astype(np.float64)
                rhs = alpha * (opa @ (opb @ x))
                gx = abs(alpha) * (np.abs(opa) @ (np.abs(opb) @ np.abs(x)))
                if beta != 0.0:
                    rhs += beta * (C0[:m].astype(np.float64) @ x)
                    gx += abs(beta) * (np.abs(C0[:m].astype(np.float64)) @ np.abs(x))
                lhs = got[:m].astype(np.float64) @ x
                assert float((np.abs(lhs - rhs) / (k * np.finfo(dt).eps * gx)).max()) <= TOL_C, (prec, ta, tb)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_host_entry_points_page_locked(prec):
    """The same streamed host path on page-locked caller memory, which the
    library copies where it lies instead of staging it: results bit-identical
    to the call on pageable memory, for packed and padded leading dimensions,
    with some and with all operands page-locked; sentinels in the padding of C
    survive, A and B are unchanged."""
    import torch
    dt = np.float64 if prec == "d" else np.float32
    tdt = torch.float64 if prec == "d" else torch.float32
    f = blas.dgemm_ if prec == "d" else blas.sgemm_

    def page_locked(arr):
        t = torch.empty(arr.shape[::-1], dtype=tdt, pin_memory=True)
        v = t.numpy().T
        v[...] = arr
        return v, t

    m, n, k = 3100, 4700, 2300
    for ta, tb, pad, alpha, beta in (("N", "N", 0, 1.0, 0.0), ("T", "N", 5, -0.5, 1.5), ("N", "T", 3, 0.75, -0.25)):
        ra = k if ta == "T" else m
        rb = n if tb == "T" else k
        lda, ldb, ldc = ra + pad, rb + pad, m + pad
        A, B, C0 = _operands(prec, ta, tb, m, n, k, lda, ldb, ldc, "uniform", beta, seed=2100)
        want = C0.copy(order="F")
        f(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, want, ldc)
        (pA, kA), (pB, kB) = page_locked(A), page_locked(B)
        for which in ("all", "A and C", "B only"):
            pC, kC = page_locked(C0)
            a = pA if which != "B only" else A
            b = pB if which != "A and C" else B
            c = pC if which != "B only" else C0.copy(order="F")
            f(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc)
            assert c.tobytes(order="F") == want.tobytes(order="F"), (prec, ta, tb, pad, which)
            assert pA.tobytes(order="F") == A.tobytes(order="F") and pB.tobytes(order="F") == B.tobytes(order="F")
