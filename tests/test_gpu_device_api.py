"""The device-resident entry points ulmblas_gpu_dgemm / ulmblas_gpu_sgemm:
every tile variant on ragged shapes against the oracle, the semantics of the
special cases, streams, and the operand-buffer cache of the host path."""
import itertools

import numpy as np
import pytest

from gpu_util import TOL_C, parity_ratio, to_device, to_host
from ulmblas_amd import blas, lib, synth

pytestmark = pytest.mark.gpu

SENTINEL = -2560000000.0


def run_dev(prec, ta, tb, m, n, k, alpha, beta, pads=(3, 1, 2), nan_c=None, stream=None):
    if pads == "aligned":
        pads = (0, 0, 0)
        aligned = True
    else:
        aligned = False
    import torch
    dt = np.float64 if prec == "d" else np.float32
    ra, ca = (k, m) if ta else (m, k)
    rb, cb = (n, k) if tb else (k, n)
    lda, ldb, ldc = max(1, ra) + pads[0], max(1, rb) + pads[1], max(1, m) + pads[2]
    if aligned:                 # column pitches of A and B that are multiples of 16 bytes
        lda, ldb, ldc = -(-max(1, ra) // 4) * 4 + 4, -(-max(1, rb) // 4) * 4 + 8, max(1, m) + 1
    A = synth.matrix(101, ra, ca, lda, dtype=dt)
    B = synth.matrix(102, rb, cb, ldb, dtype=dt)
    C0 = synth.matrix(103, m, n, ldc, dtype=dt)
    if nan_c if nan_c is not None else beta == 0:
        C0[:m, :] = np.nan
    dA, dB, dC = to_device(A), to_device(B), to_device(C0)
    f = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    f(ta, tb, m, n, k, alpha, dA, lda, dB, ldb, beta, dC, ldc, stream=stream)
    torch.cuda.synchronize()
    assert to_host(dA).tobytes(order="F") == A.tobytes(order="F")
    assert to_host(dB).tobytes(order="F") == B.tobytes(order="F")
    return A, B, C0, to_host(dC), (lda, ldb, ldc)


def check(oracle, prec, ta, tb, m, n, k, alpha, beta, **kw):
    dt = np.float64 if prec == "d" else np.float32
    A, B, C0, got, (lda, ldb, ldc) = run_dev(prec, ta, tb, m, n, k, alpha, beta, **kw)
    tra, trb = "NT"[ta], "NT"[tb]
    want = C0.copy(order="F")
    oracle.gemm("d" if prec == "d" else "s", tra, trb, m, n, k, alpha, A, lda, B, ldb, beta, want, ldc)
    g = oracle.gauge(tra, trb, m, n, k, alpha, A, B, beta, C0)
    assert np.array_equal(got[m:], C0[m:]), "padding rows of C were written"
    assert not np.isnan(got[:m]).any()
    r = parity_ratio(got[:m], want[:m], g, k, dt)
    assert r <= TOL_C, (prec, ta, tb, m, n, k, alpha, beta, r)
    return r


@pytest.mark.parametrize("prec", ["d", "s"])
def test_every_variant_on_ragged_shapes(prec, oracle):
    names = blas.variant_names(prec)
    assert len(names) >= 4
    shapes = [(1, 1, 1), (16, 16, 4), (17, 15, 5), (128, 128, 64), (129, 127, 33), (200, 150, 77), (31, 7, 12),
              (257, 129, 1000), (64, 300, 17), (300, 64, 19), (513, 511, 130)]
    try:
        for vid in range(1, len(names) + 1):
            blas.set_variant(prec, vid)
            for (m, n, k) in shapes:
                for ta, tb in itertools.product((0, 1), repeat=2):
                    for alpha, beta in ((1.0, 0.0), (0.7, 1.3)):
                        check(oracle, prec, ta, tb, m, n, k, alpha, beta)
                    # the 16-byte-load twin of the whole-tile kernels
                    check(oracle, prec, ta, tb, m, n, k, 0.7, 1.3, pads="aligned")
    finally:
        blas.set_variant(prec, 0)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_automatic_choice_covers_all_shapes(prec, oracle):
    for (m, n, k) in [(5, 2000, 64), (2000, 5, 64), (64, 64, 2000), (1500, 1300, 40), (2048, 2304, 96), (33, 33, 33)]:
        for ta, tb in itertools.product((0, 1), repeat=2):
            check(oracle, prec, ta, tb, m, n, k, -1.0, 1.0)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_special_cases(prec, oracle):
    dt = np.float64 if prec == "d" else np.float32
    m, n, k = 150, 90, 60
    # alpha == 0: C <- beta*C exactly as the oracle does it; A, B may hold anything
    for beta in (0.0, 1.0, 1.3):
        A, B, C0, got, (lda, ldb, ldc) = run_dev(prec, 0, 0, m, n, k, 0.0, beta, nan_c=False)
        want = C0.copy(order="F")
        oracle.gemm("d" if prec == "d" else "s", "N", "N", m, n, k, 0.0, A, lda, B, ldb, beta, want, ldc)
        assert got.tobytes(order="F") == want.tobytes(order="F"), beta
    # k == 0 with beta == 0 and NaN in C: zeros in the window, padding kept
    A, B, C0, got, _ = run_dev(prec, 1, 1, m, n, 0, 1.0, 0.0)
    assert (got[:m] == 0).all() and np.array_equal(got[m:], C0[m:])
    # beta == 0 never reads C: NaN and Inf in C do not reach the result
    check(oracle, prec, 0, 1, m, n, k, 1.0, 0.0, nan_c=True)
    # m == 0 / n == 0: nothing is written
    for (mm, nn) in ((0, n), (m, 0)):
        A, B, C0, got, _ = run_dev(prec, 0, 0, mm, nn, k, 1.0, 0.0, nan_c=False)
        assert got.tobytes(order="F") == C0.tobytes(order="F")
    # identity: C = alpha * A exactly
    import torch
    eye = np.asfortranarray(np.eye(k, dtype=dt))
    A = synth.matrix(5, m, k, m, dtype=dt)
    dC = torch.full((k, m), float("nan"), dtype=torch.float64 if prec == "d" else torch.float32, device="cuda")
    f = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    f(0, 0, m, k, k, 2.0, to_device(A), m, to_device(eye), k, 0.0, dC, m)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dC), 2 * A)


@pytest.mark.parametrize("prec", ["d", "s"])
def test_wide_and_narrow_loads_agree_bitwise(prec):
    """Aligned operands take kernels with 16-byte global loads, anything else
    the element-wise ones; the arithmetic is the same, so the results are
    identical: forced narrow, and A / B moved off alignment by one element."""
    import torch
    dt = np.float64 if prec == "d" else np.float32
    f = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    m, n, k = 640, 515, 301
    for ta, tb in itertools.product((0, 1), repeat=2):
        ra, ca = (k, m) if ta else (m, k)
        rb, cb = (n, k) if tb else (k, n)
        lda, ldb, ldc = -(-ra // 4) * 4 + 4, -(-rb // 4) * 4 + 8, m
        A = synth.matrix(11, ra, ca, lda, dtype=dt)
        B = synth.matrix(12, rb, cb, ldb, dtype=dt)
        C0 = synth.matrix(13, m, n, ldc, dtype=dt)
        dA, dB = to_device(A), to_device(B)
        assert dA.data_ptr() % 16 == 0 and dB.data_ptr() % 16 == 0 and (lda * dt().itemsize) % 16 == 0 \
            and (ldb * dt().itemsize) % 16 == 0
        out = []
        blas.test_control(blas.TEST_SHARED_PIECES, 0)     # the loads alone: tiles shared along k round differently
        for mode in ("wide", "narrow", "shifted"):
            dC = to_device(C0)
            if mode == "narrow":
                blas.test_control(blas.TEST_NARROW_LOADS, 1)
            try:
                if mode == "shifted":
                    # same values one element further on: base pointers no longer 16-byte aligned
                    sA = torch.empty(dA.numel() + 1, dtype=dA.dtype, device="cuda")
                    sB = torch.empty(dB.numel() + 1, dtype=dB.dtype, device="cuda")
                    sA[1:].copy_(dA.reshape(-1))
                    sB[1:].copy_(dB.reshape(-1))
                    assert sA[1:].data_ptr() % 16 != 0
                    f(ta, tb, m, n, k, 0.7, sA[1:], lda, sB[1:], ldb, 1.3, dC, ldc)
                else:
                    f(ta, tb, m, n, k, 0.7, dA, lda, dB, ldb, 1.3, dC, ldc)
                torch.cuda.synchronize()
            finally:
                blas.test_control(blas.TEST_NARROW_LOADS, 0)
            out.append(to_host(dC).tobytes(order="F"))
        blas.test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT)
        assert out[0] == out[1] == out[2], (prec, ta, tb)


def test_caller_stream_and_ordering(oracle):
    """Work goes to the stream handed over: a chain C1 = A*B, C2 = C1*B on a
    side stream equals the same chain run step by step."""
    import torch
    n = 256
    A = synth.matrix(7, n, n)
    B = synth.matrix(8, n, n)
    s = torch.cuda.Stream()
    dA, dB = to_device(A), to_device(B)
    d1 = torch.empty((n, n), dtype=torch.float64, device="cuda")
    d2 = torch.empty((n, n), dtype=torch.float64, device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        blas.gpu_dgemm(0, 0, n, n, n, 1.0, dA, n, dB, n, 0.0, d1, n, stream=s.cuda_stream)
        blas.gpu_dgemm(0, 0, n, n, n, 1.0, d1, n, dB, n, 0.0, d2, n, stream=s.cuda_stream)
    s.synchronize()
    c1 = np.zeros((n, n), order="F")
    oracle.gemm("d", "N", "N", n, n, n, 1.0, A, n, B, n, 0.0, c1, n)
    c2 = np.zeros((n, n), order="F")
    oracle.gemm("d", "N", "N", n, n, n, 1.0, c1, n, B, n, 0.0, c2, n)
    g = np.abs(c1) @ np.abs(B)
    assert parity_ratio(to_host(d2), c2, g, 2 * n, np.float64) <= TOL_C


def test_host_path_reuses_device_buffers():
    """The host entry points keep their operand buffers between calls (the
    reference keeps its pack buffers in a static pool,
    ulmblas/level3/gemm.tcc:50,57-58): a repeat of the same shape allocates
    nothing."""
    L = lib.load()
    n = 300
    A = synth.matrix(1, n, n)
    C0 = synth.matrix(2, n, n)
    blas.dgemm_("N", "N", n, n, n, 1.0, A, n, A, n, 0.0, C0.copy(order="F"), n)
    before = L.ulmblas_gpu_alloc_count()
    for _ in range(5):
        blas.dgemm_("N", "T", n, n, n, 1.0, A, n, A, n, 1.0, C0.copy(order="F"), n)
    assert L.ulmblas_gpu_alloc_count() == before
    L.ulmblas_gpu_release()
    blas.dgemm_("N", "N", n, n, n, 1.0, A, n, A, n, 0.0, C0.copy(order="F"), n)
    assert L.ulmblas_gpu_alloc_count() > before


def test_offsets_beyond_4gib(oracle):
    """Leading dimensions so large that element offsets pass 2^32 bytes: the
    kernel's address arithmetic must be 64-bit throughout.  Only the windows
    are initialised; the padding (gigabytes of it) is never touched."""
    import torch
    m, n, k = 200, 150, 96
    ld = 3_000_000                                   # 24 MB per column; column 179 starts 4.3 GB in
    for ta, tb in ((0, 0), (1, 1)):
        ra, ca = (k, m) if ta else (m, k)
        rb, cb = (n, k) if tb else (k, n)
        A = synth.matrix(301, ra, ca)
        B = synth.matrix(302, rb, cb)
        C0 = synth.matrix(303, m, n)
        dA = torch.empty((ca, ld), dtype=torch.float64, device="cuda")
        dB = torch.empty((cb, ld), dtype=torch.float64, device="cuda")
        dC = torch.empty((n, ld), dtype=torch.float64, device="cuda")
        dA[:, :ra] = torch.from_numpy(A.T.copy()).cuda()
        dB[:, :rb] = torch.from_numpy(B.T.copy()).cuda()
        dC[:, :m] = torch.from_numpy(C0.T.copy()).cuda()
        dC[:, m:m + 8] = -1.0e10
        blas.gpu_dgemm(ta, tb, m, n, k, 0.7, dA, ld, dB, ld, 1.3, dC, ld)
        torch.cuda.synchronize()
        got = dC[:, :m].cpu().numpy().T
        assert (dC[:, m:m + 8] == -1.0e10).all()
        want = C0.copy(order="F")
        oracle.gemm("d", "NT"[ta], "NT"[tb], m, n, k, 0.7, A, ra, B, rb, 1.3, want, m)
        g = oracle.gauge("NT"[ta], "NT"[tb], m, n, k, 0.7, A, B, 1.3, C0)
        assert parity_ratio(got, want, g, k, np.float64) <= TOL_C
        del dA, dB, dC


def test_concurrent_callers(oracle):
    """The host entry points may be called from several threads at once (the
    reference is re-entrant: its pool hands out blocks under a mutex,
    ulmblas/auxiliary/memorypool.tcc:43-57); so may the device entry points,
    each thread on its own stream."""
    import threading
    import torch
    shapes = [(300, 200, 150), (257, 129, 300), (64, 500, 90), (500, 64, 70)]
    results, errors = {}, []

    def host_worker(idx):
        try:
            m, n, k = shapes[idx]
            A = synth.matrix(400 + idx, m, k, m + 1)
            B = synth.matrix(500 + idx, k, n, k + 2)
            C0 = synth.matrix(600 + idx, m, n, m + 3)
            for _ in range(10):
                got = C0.copy(order="F")
                blas.dgemm_("N", "N", m, n, k, 0.7, A, m + 1, B, k + 2, 1.3, got, m + 3)
            results[("host", idx)] = (A, B, C0, got)
        except Exception as e:            # noqa: BLE001
            errors.append(e)

    def device_worker(idx):
        try:
            m, n, k = shapes[idx]
            A = synth.matrix(700 + idx, m, k, m + 1)
            B = synth.matrix(800 + idx, k, n, k + 2)
            C0 = synth.matrix(900 + idx, m, n, m + 3)
            s = torch.cuda.Stream()
            dA, dB = to_device(A), to_device(B)
            torch.cuda.synchronize()
            for _ in range(10):
                dC = to_device(C0)
                torch.cuda.synchronize()
                blas.gpu_dgemm(0, 0, m, n, k, 0.7, dA, m + 1, dB, k + 2, 1.3, dC, m + 3, stream=s.cuda_stream)
                s.synchronize()
            results[("device", idx)] = (A, B, C0, to_host(dC))
        except Exception as e:            # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=host_worker, args=(i,)) for i in range(4)]
    threads += [threading.Thread(target=device_worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert len(results) == 8
    for (kind, idx), (A, B, C0, got) in results.items():
        m, n, k = shapes[idx]
        want = C0.copy(order="F")
        oracle.gemm("d", "N", "N", m, n, k, 0.7, A, m + 1, B, k + 2, 1.3, want, m + 3)
        g = oracle.gauge("N", "N", m, n, k, 0.7, A, B, 1.3, C0)
        assert parity_ratio(got[:m], want[:m], g, k, np.float64) <= TOL_C, (kind, idx)
        assert np.array_equal(got[m:], C0[m:]), (kind, idx)


def test_allocation_failure_is_reported_and_leaves_c_alone(xerbla):
    """The host path with a device allocation that fails on request: status,
    hook and an untouched C (the same test the CPU suite runs without a device)."""
    import test_abi
    test_abi.test_failure_on_the_gpu_side_is_reported_and_leaves_c_alone(xerbla)


def test_host_calls_of_two_threads_overlap():
    """Two threads calling dgemm_ at the same time each get a context of their
    own (the reference is re-entrant the same way, ulmblas/auxiliary/
    memorypool.tcc:39-59): a small product started while a large one is under
    way does not wait for it."""
    import threading
    import time
    n, small = 6000, 200
    A, B, Cm = synth.matrix(40, n, n, n), synth.matrix(41, n, n, n), np.zeros((n, n), order="F")
    a, b, c = synth.matrix(42, small, small, small), synth.matrix(43, small, small, small), \
        np.zeros((small, small), order="F")
    done = {}

    def big():
        blas.dgemm_("N", "N", n, n, n, 1.0, A, n, B, n, 0.0, Cm, n)
        done["big"] = time.perf_counter()

    def little():
        blas.dgemm_("N", "N", small, small, small, 1.0, a, small, b, small, 0.0, c, small)
        done["little"] = time.perf_counter()

    for _ in range(2):          # warm both contexts: buffers, rings, streams
        ts = [threading.Thread(target=big), threading.Thread(target=little)]
        [t.start() for t in ts]
        [t.join() for t in ts]
    t0 = time.perf_counter()
    tb = threading.Thread(target=big)
    tb.start()
    time.sleep(0.004)           # the large call is in the middle of its transfers now
    tl = threading.Thread(target=little)
    tl.start()
    tl.join()
    tb.join()
    x = np.ones(n)
    assert np.allclose(Cm @ x, A @ (B @ x), rtol=1e-9, atol=1e-7)
    assert np.allclose(c, a @ b, rtol=1e-10, atol=1e-10)
    print(f"large call {1e3 * (done['big'] - t0):.1f} ms, small call done after {1e3 * (done['little'] - t0):.1f} ms")
    # (no margins in milliseconds: on a loaded host they would decide the test; a small call that had to
    # wait for the large one's context would end after it)
    assert done["little"] < done["big"]
