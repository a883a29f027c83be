"""The LU factorisation on the GPU: ulmblas_dgetrf / ulmblas_dlaswp of
libulmblas_gpu.so and the device-resident entry points against the CPU oracle.

What "same result as the reference" means here.  Pivots are integers: they
must be IDENTICAL to the oracle's (a pivot could only differ where two
candidates agree to within rounding, which the seeded inputs do not produce).
The factors are compared through the bound that holds for LU with partial
pivoting in any operation order,

    |P A - L U| <= TOL_LU * min(m,n) * eps * |L||U|     elementwise,

which the oracle (block 64, separate multiply and add) and the GPU (recursive
blocks, FMA) both satisfy with constant 1, together with |L| <= 1; and
directly, |F_gpu - F_oracle| <= 1e-9 * max|F| for these orders (a loose
figure: the factors' sensitivity depends on the conditioning of the leading
blocks, not on the algorithm).
"""
import ctypes as C

import numpy as np
import pytest

from gpu_util import to_device, to_host
from ulmblas_amd import blas, lib, synth

pytestmark = pytest.mark.gpu

TOL_LU = 2.0
EPS = np.finfo(np.float64).eps


def split_lu(F, m, n):
    mn = min(m, n)
    return np.tril(F[:m, :mn], -1) + np.eye(m, mn), np.triu(F[:mn, :n])


def permute(A, piv):
    PA = A.copy()
    for i, p in enumerate(piv):
        if p != i:
            PA[[i, p]] = PA[[p, i]]
    return PA


def check_factors(A0, F, piv, m, n, tag):
    """Backward error and |L| <= 1 on the m x n windows."""
    mn = min(m, n)
    L, U = split_lu(F, m, n)
    assert np.abs(np.tril(F[:m, :mn], -1)).max(initial=0.0) <= 1.0 + 4 * EPS, tag
    resid = np.abs(permute(A0[:m, :n], piv) - L @ U)
    bound = mn * EPS * (np.abs(L) @ np.abs(U))
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(resid == 0, 0.0, resid / bound)
    r = float(ratio.max()) if ratio.size else 0.0
    assert r <= TOL_LU, (tag, r)
    return r


def test_device_entry_against_oracle(oracle):
    import torch
    worst = 0.0
    for (m, n) in [(1, 1), (5, 5), (64, 64), (65, 65), (100, 60), (60, 100), (255, 257), (300, 300), (513, 257),
                   (257, 513), (1000, 1000), (1030, 700), (2048, 2048)]:
        lda = m + 3
        A0 = synth.matrix(77, m, n, lda)
        dA = to_device(A0)
        dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, lda)
        torch.cuda.synchronize()
        got, piv, info = to_host(dA), dPiv.cpu().numpy(), int(dInfo.cpu()[0])
        want = A0.copy(order="F")
        oinfo, opiv = oracle.getrf_strided(m, n, want, (1, lda))
        assert info == oinfo == 0, (m, n, info)
        assert np.array_equal(piv, opiv), (m, n)
        assert np.array_equal(got[m:], A0[m:]), "padding rows were written"
        worst = max(worst, check_factors(A0, got, piv, m, n, (m, n)))
        check_factors(A0, want, opiv, m, n, ("oracle", m, n))
        assert np.abs(got[:m] - want[:m]).max() <= 1e-9 * np.abs(want[:m]).max(), (m, n)
    print(f"device getrf: max backward-error ratio {worst:.3f}")


def test_workspace_reused_across_factorisations(oracle):
    """One caller workspace, never cleared by the caller and full of arbitrary
    bits to begin with, serves factorisations of different matrices and sizes
    one after the other: nothing a factorisation leaves behind in it (slots,
    turns, tags of its columns) may be taken for the next one's."""
    import torch
    from ulmblas_amd import lib
    nbytes = lib.load().ulmblas_gpu_dgetrf_worksize()
    work = torch.randint(-2**62, 2**62, ((nbytes + 7) // 8,), dtype=torch.int64, device="cuda")
    for seed, (m, n) in [(81, (1000, 1000)), (82, (700, 650)), (83, (1000, 1000)), (81, (1000, 1000)),
                         (84, (300, 900))]:
        A0 = synth.matrix(seed, m, n, m)
        dA = to_device(A0)
        dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, m, work=work)
        torch.cuda.synchronize()
        got, piv, info = to_host(dA), dPiv.cpu().numpy(), int(dInfo.cpu()[0])
        want = A0.copy(order="F")
        oinfo, opiv = oracle.getrf_strided(m, n, want, (1, m))
        assert info == oinfo == 0, (seed, m, n, info)
        assert np.array_equal(piv, opiv), (seed, m, n)
        check_factors(A0, got, piv, m, n, (seed, m, n))


def test_zero_pivots(oracle):
    """getf2.tcc:51-53: an exactly zero pivot sets info to its 1-based column
    (the first one wins, getrf.tcc:44-46) and the factorisation carries on."""
    import torch
    for (m, n, zero_cols) in [(6, 6, (2,)), (70, 70, (2, 40)), (130, 90, (65,)), (300, 300, (100, 299))]:
        A0 = synth.matrix(78, m, n, m)
        for zc in zero_cols:
            A0[:, zc] = 0.0
        dA = to_device(A0)
        dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, m)
        torch.cuda.synchronize()
        got, piv, info = to_host(dA), dPiv.cpu().numpy(), int(dInfo.cpu()[0])
        want = A0.copy(order="F")
        oinfo, opiv = oracle.getrf_strided(m, n, want, (1, m))
        assert info == oinfo == zero_cols[0] + 1, (m, n, info, oinfo)
        assert np.array_equal(piv, opiv), (m, n)
        assert not np.isnan(got).any()
        check_factors(A0, got, piv, m, n, ("zero pivot", m, n))
    # a matrix of zeros: every pivot is zero, nothing changes, info = 1
    dA = torch.zeros((5, 5), dtype=torch.float64, device="cuda")
    dPiv, dInfo = blas.gpu_dgetrf(5, 5, dA, 5)
    torch.cuda.synchronize()
    assert int(dInfo.cpu()[0]) == 1 and (dA == 0).all() and dPiv.cpu().tolist() == [0, 1, 2, 3, 4]


def test_nan_follows_the_reference_rule(oracle):
    """ulmblas/level1/iamax.tcc:17-27: a NaN is never greater than the running
    maximum, so it is chosen only when it is the first element looked at."""
    import torch
    A0 = synth.matrix(79, 8, 8, 8)
    A0[5, 0] = np.nan             # not in the first row: another row is the pivot of column 0
    dA = to_device(A0)
    dPiv, dInfo = blas.gpu_dgetrf(8, 8, dA, 8)
    torch.cuda.synchronize()
    want = A0.copy(order="F")
    oinfo, opiv = oracle.getrf_strided(8, 8, want, (1, 8))
    assert dPiv.cpu().numpy()[0] == opiv[0] != 5


def test_host_entry_points(oracle):
    for order in (blas.CblasColMajor, blas.CblasRowMajor):
        for (m, n) in [(9, 9), (70, 70), (200, 200), (130, 67), (67, 130), (1100, 1100)]:
            if order == blas.CblasRowMajor and m != n:
                # the reference's row-major branch walks i < n rows of pitch ldA and j < m columns:
                # give it the memory that layout needs
                ld, cols = m + 2, n
            else:
                ld, cols = m + 2, n
            A0 = synth.matrix(80, ld - 2, cols, ld)
            A = A0.copy(order="F")
            info, piv = blas.ulmblas_dgetrf(order, m, n, A, ld)
            want = A0.copy(order="F")
            oinfo, opiv = oracle.dgetrf(order, m, n, want, ld)
            assert info == oinfo == 0, (order, m, n)
            assert np.array_equal(piv, opiv), (order, m, n)
            assert np.array_equal(A[ld - 2:], A0[ld - 2:]), "padding written"
            assert np.abs(A - want).max() <= 1e-9 * np.abs(want).max(), (order, m, n)
            if order == blas.CblasColMajor:
                check_factors(A0, A, piv, m, n, (order, m, n))
            else:
                # the factored matrix is the transposed view: n rows, m columns
                check_factors(np.ascontiguousarray(A0[:m, :n].T), np.ascontiguousarray(A[:m, :n].T), piv, n, m,
                              (order, m, n))
    # ATL_ alias
    A0 = synth.matrix(81, 50, 50, 50)
    A1, A2 = A0.copy(order="F"), A0.copy(order="F")
    i1, p1 = blas.ulmblas_dgetrf(blas.CblasColMajor, 50, 50, A1, 50)
    i2, p2 = blas.ulmblas_dgetrf(blas.CblasColMajor, 50, 50, A2, 50, symbol="ATL_dgetrf")
    assert i1 == i2 and np.array_equal(p1, p2) and A1.tobytes() == A2.tobytes()


def test_laswp(oracle):
    import torch
    rng = np.random.default_rng(4)
    m, n, ld = 300, 77, 303
    A0 = synth.matrix(82, m, n, ld)
    piv = rng.integers(0, m, 120).astype(np.int32)
    piv[:120] = np.maximum(piv[:120], np.arange(120))        # LAPACK pivots point downwards
    for (k1, k2, inc) in [(0, 120, 1), (5, 60, 1), (0, 60, 2), (3, 3, 1)]:
        want = A0.copy(order="F")
        oracle.dlaswp(n, want, ld, k1, k2, piv, inc)
        A = A0.copy(order="F")
        blas.ulmblas_dlaswp(n, A, ld, k1, k2, piv, inc)
        assert A.tobytes() == want.tobytes(), (k1, k2, inc)
        A = A0.copy(order="F")
        blas.ulmblas_dlaswp(n, A, ld, k1, k2, piv, inc, symbol="ATL_dlaswp")
        assert A.tobytes() == want.tobytes()
        dA = to_device(A0)
        blas.gpu_dlaswp(n, dA, ld, k1, k2, torch.from_numpy(piv).cuda(), inc)
        torch.cuda.synchronize()
        assert to_host(dA).tobytes() == want.tobytes(), (k1, k2, inc)
    # backwards: the exchanges of a forward pass undone in reverse order.  The reference indexes
    # piv[i*incPiv] also for a negative stride (ulmblas/lapack/laswp.tcc:23-27,39): the pointer
    # handed over is the one from which those offsets are reached.
    dA = to_device(A0)
    dP = torch.from_numpy(np.ascontiguousarray(piv[:60][::-1])).cuda()       # dP[59 - i] = piv[i]
    blas.gpu_dlaswp(n, dA, ld, 0, 60, torch.from_numpy(piv).cuda(), 1)
    import ctypes as C
    from ulmblas_amd.lib import load
    rc = load().ulmblas_gpu_dlaswp(n, C.c_void_p(dA.data_ptr()), ld, 0, 60, C.c_void_p(dP.data_ptr() + 59 * 4), -1,
                                   C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert to_host(dA).tobytes() == A0.tobytes()


def test_factor_then_solve_on_one_stream(oracle):
    """The use the factorisation is for (ulmblas/lapack/getrs.h): A x = b by
    row exchanges and two triangular solves, everything enqueued on one
    stream without a host synchronisation in between."""
    import torch
    n, nrhs = 1500, 9
    A0 = synth.matrix(83, n, n, n)
    X0 = synth.matrix(84, n, nrhs, n)
    B0 = np.asfortranarray(A0 @ X0)
    s = torch.cuda.Stream()
    dA, dB = to_device(A0), to_device(B0)
    s.wait_stream(torch.cuda.current_stream())
    dPiv, dInfo = blas.gpu_dgetrf(n, n, dA, n, stream=s.cuda_stream)
    blas.gpu_dlaswp(nrhs, dB, n, 0, n, dPiv, 1, stream=s.cuda_stream)
    blas.gpu_dtrsm(0, 1, 0, 1, n, nrhs, 1.0, dA, n, dB, n, stream=s.cuda_stream)       # L y = P b
    blas.gpu_dtrsm(0, 0, 0, 0, n, nrhs, 1.0, dA, n, dB, n, stream=s.cuda_stream)       # U x = y
    s.synchronize()
    assert int(dInfo.cpu()[0]) == 0
    X = to_host(dB)
    resid = np.abs(A0 @ X - B0).max() / (np.abs(A0).max() * np.abs(X).max() * n * EPS)
    assert resid < 16.0, resid


def test_large_factorisation(oracle):
    """8192 x 8192: the residual bound evaluated on the GPU (products through
    this library's own dgemm), pivots against the oracle on the leading 64
    columns (the oracle's full factorisation of this order takes minutes)."""
    import torch
    n = 8192
    A0 = synth.matrix(85, n, n, n)
    dA0 = to_device(A0)
    dA = dA0.clone()
    dPiv, dInfo = blas.gpu_dgetrf(n, n, dA, n)
    torch.cuda.synchronize()
    assert int(dInfo.cpu()[0]) == 0
    piv = dPiv.cpu().numpy()
    panel = A0[:, :64].copy(order="F")
    oinfo, opiv = oracle.getf2_strided(n, 64, panel, (1, n))
    assert np.array_equal(piv[:64], opiv)
    # torch tensors hold the transposed image: F^T = U^T L^T
    Ft = dA                                                   # (n, n) tensor = F transposed
    Ut = torch.tril(Ft)                                       # U^T
    Lt = torch.triu(Ft, 1) + torch.eye(n, dtype=torch.float64, device="cuda")
    # P A on the device: apply the exchanges to a copy of A
    dPA = dA0.clone()
    blas.gpu_dlaswp(n, dPA, n, 0, n, dPiv, 1)
    # R = P A - L U (column-major operands L = Lt^T, U = Ut^T live in Lt, Ut's memory)
    blas.gpu_dgemm(0, 0, n, n, n, -1.0, Lt.contiguous(), n, Ut.contiguous(), n, 1.0, dPA, n)
    # bound |L||U|
    dG = torch.zeros((n, n), dtype=torch.float64, device="cuda")
    blas.gpu_dgemm(0, 0, n, n, n, 1.0, Lt.abs().contiguous(), n, Ut.abs().contiguous(), n, 0.0, dG, n)
    torch.cuda.synchronize()
    ratio = (dPA.abs() / (n * EPS * dG)).max().item()
    assert torch.triu(Ft, 1).abs().max().item() <= 1.0 + 4 * EPS
    assert ratio <= TOL_LU, ratio
    print(f"getrf 8192: backward-error ratio {ratio:.4f}")


def test_tall_matrix_many_workgroups(oracle):
    """40 000 rows: 157 workgroups share a panel, more than one wavefront can
    watch in a single pass (64), and the candidates' row numbers exceed 2^15."""
    import torch
    m, n = 40000, 128
    A0 = synth.matrix(86, m, n, m)
    # make late rows win now and then: scale a few rows far down the matrix
    A0[39990, :] *= 50.0
    A0[20011, :] *= 30.0
    dA = to_device(A0)
    dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, m)
    torch.cuda.synchronize()
    got, piv, info = to_host(dA), dPiv.cpu().numpy(), int(dInfo.cpu()[0])
    want = A0.copy(order="F")
    oinfo, opiv = oracle.getrf_strided(m, n, want, (1, m))
    assert info == oinfo == 0
    assert np.array_equal(piv, opiv)
    assert piv.max() >= 39990
    check_factors(A0, got, piv, m, n, (m, n))
    assert np.abs(got - want).max() <= 1e-9 * np.abs(want).max()


def test_bounded_wait_gives_up_cleanly():
    """With no patience at all (zero polls per wait, set from the host) the
    panel workgroups stop waiting for each other at once: every kernel still
    runs to its end, nothing hangs, the pivots stay in range and the
    device entry point's factorisation reports info = -1.  The host entry
    point reads that status before it copies anything back, sends the matrix up
    again and factors it with the launches that wait for nobody: the caller
    gets the factorisation (the same pivots as on a GPU where the workgroups
    do meet).  Afterwards the default is back and the same matrix factors
    normally."""
    import torch
    n = 1024
    A0 = synth.matrix(91, n, n, n)

    def check(F, piv):
        L, U = np.tril(F, -1) + np.eye(n), np.triu(F)
        PA = A0.copy()
        for i, p in enumerate(piv):
            if p != i:
                PA[[i, p]] = PA[[p, i]]
        bound = n * np.finfo(np.float64).eps * (np.abs(L) @ np.abs(U))
        assert (np.abs(PA - L @ U) <= 2.0 * bound).all()

    try:
        blas.test_control(blas.TEST_LU_SPIN_LIMIT, 0)
        dA = to_device(A0)
        dPiv, dInfo = blas.gpu_dgetrf(n, n, dA, n)
        torch.cuda.synchronize()
        info = int(dInfo.cpu().numpy()[0])
        piv = dPiv.cpu().numpy()
        assert info == -1
        assert ((piv >= 0) & (piv < n)).all()
        A = A0.copy(order="F")
        piv_host = np.full(n, -5, dtype=np.int32)
        rc = lib.load().ulmblas_dgetrf(blas.CblasColMajor, n, n, A.ctypes.data_as(C.c_void_p), n,
                                       piv_host.ctypes.data_as(C.c_void_p))
        assert rc == 0
        check(A, piv_host)
    finally:
        blas.test_control(blas.TEST_LU_SPIN_LIMIT, -1)
    dA = to_device(A0)
    dPiv, dInfo = blas.gpu_dgetrf(n, n, dA, n)
    torch.cuda.synchronize()
    assert int(dInfo.cpu().numpy()[0]) == 0
    F = to_host(dA)
    piv = dPiv.cpu().numpy()
    check(F, piv)
    assert np.array_equal(piv, piv_host)
    assert F.tobytes() == A.tobytes()          # the launches that wait for nobody do the same arithmetic


def test_panels_that_wait_for_nobody_give_the_same_bits(oracle):
    """The panel path of three small launches per column (for panels with more
    rows than the cooperative kernel's workgroups can hold at a time) does the
    cooperative kernel's arithmetic operation for operation: forced on, it
    returns the same pivots and the same bits, zero pivots included."""
    import torch
    for seed, (m, n), zero_col in [(95, (1000, 1000), None), (96, (1030, 700), None), (97, (300, 900), None),
                                   (98, (515, 515), 70)]:
        A0 = synth.matrix(seed, m, n, m + 1)
        if zero_col is not None:
            A0[:, zero_col] = 0.0
        out = []
        for simple in (0, 1):
            blas.test_control(blas.TEST_LU_SIMPLE_PANELS, simple)
            try:
                dA = to_device(A0)
                dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, m + 1)
                torch.cuda.synchronize()
            finally:
                blas.test_control(blas.TEST_LU_SIMPLE_PANELS, 0)
            out.append((to_host(dA), dPiv.cpu().numpy(), int(dInfo.cpu()[0])))
        assert out[0][2] == out[1][2] == (0 if zero_col is None else zero_col + 1)
        assert np.array_equal(out[0][1], out[1][1]), (m, n)
        assert out[0][0].tobytes() == out[1][0].tobytes(), (m, n)
        want = A0.copy(order="F")
        oinfo, opiv = oracle.getrf_strided(m, n, want, (1, m + 1))
        assert np.array_equal(out[1][1], opiv)


def test_more_rows_than_the_panel_kernel_holds(oracle):
    """70 000 rows: the first panels cannot be taken by the cooperative kernel
    (274 workgroups of 256 rows; an MI355X holds 256) and go through the small
    launches, the later ones (fewer rows left) through the cooperative kernel
    again.  Pivots as the oracle's, residual bound, padding untouched."""
    import torch
    m, n = 70000, 100
    lda = m + 2
    A0 = synth.matrix(99, m, n, lda)
    A0[65990, 3] = 7.5              # a pivot far down, beyond what one launch of the cooperative kernel reaches
    dA = to_device(A0)
    dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, lda)
    torch.cuda.synchronize()
    got, piv, info = to_host(dA), dPiv.cpu().numpy(), int(dInfo.cpu()[0])
    want = A0.copy(order="F")
    oinfo, opiv = oracle.getrf_strided(m, n, want, (1, lda))
    assert info == oinfo == 0
    assert np.array_equal(piv, opiv) and piv[3] == 65990
    assert np.array_equal(got[m:], A0[m:]), "padding rows were written"
    check_factors(A0, got, piv, m, n, (m, n))
    assert np.abs(got[:m] - want[:m]).max() <= 1e-9 * np.abs(want[:m]).max()
