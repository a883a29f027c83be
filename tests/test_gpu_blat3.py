"""The reference's own conformance sweeps, driven through the drop-in symbols
of libulmblas_gpu.so on the GPU: DCHK1 / SCHK1 of the netlib level-3 testers
(test/F77/dblat3.f:356-636, sblat3.f) through dgemm_ / sgemm_, and the CBLAS
variant (test/C/c_dblat3.f with test/C/c_dblas3.c:14-75, both storage orders)
through cblas_dgemm / cblas_sgemm.  Every call is checked three ways:
the tester's own DMMCH ratio against a wide product (threshold 16), parity
with the CPU oracle under the stated bound, and "nothing else changed"
(A, B bit-identical, padding rows of C untouched, C untouched when m*n == 0).
"""
import numpy as np
import pytest

import netlib
from gpu_util import TOL_C, parity_ratio
from ulmblas_amd import blas

pytestmark = pytest.mark.gpu

CB = {"N": blas.CblasNoTrans, "T": blas.CblasTrans, "C": blas.CblasConjTrans}


def _check(case, cc_out, oracle, variant, dtype, errmax):
    m, n, k = case["m"], case["n"], case["k"]
    aa, bb, c0 = case["aa"], case["bb"], case["cc"]
    tag = (case["transa"], case["transb"], m, n, k, case["alpha"], case["beta"])
    if m == 0 or n == 0:
        assert cc_out.tobytes(order="F") == c0.tobytes(order="F"), tag          # dblat3.f:552-553
        return errmax
    assert np.array_equal(cc_out[m:, :], c0[m:, :]), tag                        # LDERES, dblat3.f:2636-2642
    assert not np.isnan(cc_out[:m]).any(), tag
    err, _ = netlib.mmch(case["transa"], case["transb"], m, n, k, case["alpha"], aa, bb, case["beta"], c0, cc_out, dtype)
    assert err < netlib.DBLAT3["thresh"], (tag, err)                            # dblat3.f:605
    want = c0.copy(order="F")
    oracle.gemm(variant, case["transa"], case["transb"], m, n, k, case["alpha"], aa, case["lda"], bb, case["ldb"],
                case["beta"], want, case["ldc"])
    g = oracle.gauge(case["transa"], case["transb"], m, n, k, case["alpha"], aa, bb, case["beta"], c0)
    r = parity_ratio(cc_out[:m], want[:m], g, k, dtype)
    assert r <= TOL_C, (tag, r)
    return max(errmax, err)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_chk1_f77(prec, oracle, xerbla):
    dtype = np.float64 if prec == "d" else np.float32
    params = netlib.DBLAT3 if prec == "d" else netlib.SBLAT3
    f = blas.dgemm_ if prec == "d" else blas.sgemm_
    variants = ("d",) if prec == "d" else ("s", "s_f64")      # sgemm_: both reference arithmetics
    errmax, ncalls = 0.0, 0
    for case in netlib.chk1_cases(params, dtype):
        a_save, b_save = case["aa"].copy(order="F"), case["bb"].copy(order="F")
        cc = case["cc"].copy(order="F")
        f(case["transa"], case["transb"], case["m"], case["n"], case["k"], case["alpha"], case["aa"], case["lda"],
          case["bb"], case["ldb"], case["beta"], cc, case["ldc"])
        ncalls += 1
        assert case["aa"].tobytes(order="F") == a_save.tobytes(order="F")       # dblat3.f:547
        assert case["bb"].tobytes(order="F") == b_save.tobytes(order="F")       # dblat3.f:549
        for v in variants:
            errmax = _check(case, cc, oracle, v, dtype, errmax)
    assert xerbla.capture_count() == 0                                          # no error exit taken, dblat3.f:532
    assert ncalls == len(params["idim"]) ** 3 * 81
    print(f"{prec}gemm_: {ncalls} calls, largest DMMCH ratio {errmax:.3f}")


@pytest.mark.parametrize("prec", ["d", "s"])
def test_chk1_cblas_both_orders(prec, oracle, xerbla):
    """The CBLAS driver runs every case column-major and row-major; for
    row-major its shim hands over physically transposed copies with leading
    dimension cols+1 (test/C/c_dblas3.c:25-68)."""
    dtype = np.float64 if prec == "d" else np.float32
    f = blas.cblas_dgemm if prec == "d" else blas.cblas_sgemm
    variant = "d" if prec == "d" else "s"
    errmax, ncalls = 0.0, 0
    for case in netlib.chk1_cases(netlib.DIN3, dtype):
        m, n, k = case["m"], case["n"], case["k"]
        ta, tb = CB[case["transa"]], CB[case["transb"]]
        # column-major
        cc = case["cc"].copy(order="F")
        f(blas.CblasColMajor, ta, tb, m, n, k, case["alpha"], case["aa"], case["lda"], case["bb"], case["ldb"],
          case["beta"], cc, case["ldc"])
        errmax = _check(case, cc, oracle, variant, dtype, errmax)

        # row-major: stored A is (rows x cols) = the logical stored matrix, C-ordered, ld = cols + 1
        def rowmajor(x, rows, cols):
            out = np.full((rows, cols + 1), netlib.ROGUE, dtype=dtype)
            out[:, :cols] = x[:rows, :cols]
            return out

        ra, ca = (k, m) if case["transa"] in "TC" else (m, k)
        rb, cb = (n, k) if case["transb"] in "TC" else (k, n)
        ar, br, cr = rowmajor(case["aa"], ra, ca), rowmajor(case["bb"], rb, cb), rowmajor(case["cc"], m, n)
        f(blas.CblasRowMajor, ta, tb, m, n, k, case["alpha"], ar, ca + 1, br, cb + 1, case["beta"], cr, n + 1)
        assert (cr[:, n] == netlib.ROGUE).all()
        back = case["cc"].copy(order="F")
        back[:m, :] = cr[:, :n]
        errmax = _check(case, back, oracle, variant, dtype, errmax)
        ncalls += 2
    assert xerbla.capture_count() == 0
    print(f"cblas_{prec}gemm: {ncalls} calls, largest DMMCH ratio {errmax:.3f}")


def test_orderless_and_atlas_symbols(oracle):
    """ulmblas_dgemm / ATL_dgemm (interfaces/blas/C/gemm.cc:75-138,
    config/make.atl.inc:4-5): unchecked column-major entry points; AtlasConj
    counts as 'not transposed' (:93-94)."""
    from ulmblas_amd import synth
    m, n, k = 45, 38, 70
    for prec, dt, variant in (("d", np.float64, "d"), ("s", np.float32, "s")):
        for sym in (f"ulmblas_{prec}gemm", f"ATL_{prec}gemm"):
            for ta, tra in ((blas.CblasNoTrans, "N"), (blas.AtlasConj, "N"), (blas.CblasTrans, "T"),
                            (blas.CblasConjTrans, "T")):
                ra, ca = (k, m) if tra == "T" else (m, k)
                A = synth.matrix(1, ra, ca, ra + 1, dtype=dt)
                B = synth.matrix(2, n, k, n + 1, dtype=dt)
                C0 = synth.matrix(3, m, n, m + 1, dtype=dt)
                got = C0.copy(order="F")
                fn = blas.ulmblas_dgemm if prec == "d" else blas.ulmblas_sgemm
                fn(ta, blas.CblasTrans, m, n, k, 0.7, A, ra + 1, B, n + 1, 1.3, got, m + 1, symbol=sym)
                want = C0.copy(order="F")
                oracle.gemm(variant, tra, "T", m, n, k, 0.7, A, ra + 1, B, n + 1, 1.3, want, m + 1)
                g = oracle.gauge(tra, "T", m, n, k, 0.7, A, B, 1.3, C0)
                assert parity_ratio(got[:m], want[:m], g, k, dt) <= TOL_C
                assert np.array_equal(got[m:], C0[m:])
