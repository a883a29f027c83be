"""Workgroup tiles shared between workgroups along k.

When the tiles of a product do not fill the GPU's last round of workgroups,
the tiles of that round are cut along k and dealt to all workgroup slots; the
pieces of one tile are folded into C in the order of k (first piece
alpha*AB + beta*C, later ones += alpha*AB), each after the one before it.
The reference does the same with its KC slices (ulmblas/level3/gemm.tcc:60-83:
beta for the first slice, 1 for the others).  Checked here: parity with the
oracle under the usual bound in every transposition, with beta == 0 on a
NaN-filled C, with k that ends inside a slab; the same bits on every run; and
the bounded wait, walked by keeping the flags from being raised."""
import itertools

import numpy as np
import pytest

from gpu_util import TOL_C, parity_ratio, to_device, to_host
from ulmblas_amd import blas, synth

pytestmark = pytest.mark.gpu


def _operands(prec, ta, tb, m, n, k, pads=(0, 0, 0)):
    dt = np.float64 if prec == "d" else np.float32
    ra, ca = (k, m) if ta else (m, k)
    rb, cb = (n, k) if tb else (k, n)
    lda, ldb, ldc = ra + pads[0], rb + pads[1], m + pads[2]
    return (synth.matrix(501, ra, ca, lda, dtype=dt), synth.matrix(502, rb, cb, ldb, dtype=dt),
            synth.matrix(503, m, n, ldc, dtype=dt), lda, ldb, ldc)


def _run(prec, ta, tb, m, n, k, alpha, beta, A, B, C0, lda, ldb, ldc, dA=None, dB=None):
    import torch
    f = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    dA = to_device(A) if dA is None else dA
    dB = to_device(B) if dB is None else dB
    dC = to_device(C0)
    f(ta, tb, m, n, k, alpha, dA, lda, dB, ldb, beta, dC, ldc)
    torch.cuda.synchronize()
    return to_host(dC)


@pytest.fixture()
def restore_switches():
    yield
    blas.set_variant("d", 0)
    blas.set_variant("s", 0)
    blas.test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT)
    blas.test_control(blas.TEST_WHOLE_C, -1)
    blas.test_control(blas.TEST_SHARED_MUTE, 0)
    blas.test_control(blas.TEST_SHARED_SPIN_LIMIT, -1)


# (precision, variant id, m, n, k): tile counts that leave a partial last round on 256 CUs
CASES = [
    ("d", 1, 2048, 2048, 700),          # 128 tiles of 256 x 128: every tile in two pieces
    ("d", 1, 4352, 2048, 333),          # 272 tiles: one round and 16 tiles cut in four; k ends inside a slab
    ("d", 1, 256 * 19, 128 * 23, 500),  # 437 tiles: pieces that do not line up with the tiles
    ("d", 2, 128 * 23, 128 * 25, 300),  # 575 tiles of 128 x 128 on 512 slots
    ("d", 1, 512, 512, 2048),           # 8 tiles in four pieces each
    ("s", 1, 2048, 2048, 900),          # 64 tiles of 256 x 256
    ("s", 1, 256 * 11, 256 * 27, 250),  # 297 tiles
    ("s", 2, 256 * 9, 128 * 30, 411),   # 270 tiles of 256 x 128 on 512 slots
    # one launch over all of C: tiles that reach past the edges, shared or not
    ("d", 1, 2049, 2047, 300),          # 9 x 16 tiles, the last row of tiles one row high, the last column one short
    ("d", 1, 1001, 777, 515),
    ("d", 2, 1300, 1100, 129),
    ("d", 1, 5, 7, 40),                 # a single tile, mostly past the edge
    ("d", 2, 130, 4, 33),
    ("s", 1, 2051, 2046, 300),          # 4 floats per packet: every offset of the edge inside a packet
    ("s", 1, 1001, 778, 515),
    ("s", 2, 1303, 1101, 129),
    ("s", 1, 6, 5, 40),
    # the small tiles over odd shapes, in place of the any-shape kernel, and cut along k
    ("d", 6, 1001, 777, 515),
    ("d", 6, 67, 5, 40),
    ("d", 6, 448, 512, 2048),
    # the small single-precision tile, which takes odd shapes with 16-byte loads in place of the any-shape kernel
    ("s", 4, 1001, 778, 515),
    ("s", 4, 70, 5, 40),
    ("s", 4, 512, 448, 2048),           # 56 tiles of 64 x 64 in four pieces each
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s%d_%dx%dx%d" % c)
def test_parity_with_shared_tiles(case, oracle, restore_switches):
    prec, vid, m, n, k = case
    dt = np.float64 if prec == "d" else np.float32
    blas.set_variant(prec, vid)
    blas.test_control(blas.TEST_SHARED_PIECES, -4)        # wherever it can be done, not only where it pays
    blas.test_control(blas.TEST_WHOLE_C, 1)
    for ta, tb in itertools.product((0, 1), repeat=2):
        A, B, C0, lda, ldb, ldc = _operands(prec, ta, tb, m, n, k, pads=(3, 1, 2))
        for alpha, beta in ((1.0, 0.0), (0.75, -0.25)):
            Cin = C0.copy(order="F")
            if beta == 0.0:
                Cin[:m] = np.nan
            got = _run(prec, ta, tb, m, n, k, alpha, beta, A, B, Cin, lda, ldb, ldc)
            assert np.array_equal(got[m:], Cin[m:]), "padding rows of C were written"
            assert not np.isnan(got[:m]).any(), (case, ta, tb)
            # every element against the oracle's per-element values would take minutes here:
            # the whole matrix through the identity C x = alpha op(A) (op(B) x) + beta C0 x, and samples
            rng = np.random.default_rng(7)
            rows = np.concatenate([[0, m - 1, 0, m - 1], rng.integers(0, m, 1500)])
            cols = np.concatenate([[0, 0, n - 1, n - 1], rng.integers(0, n, 1500)])
            for v in (("d",) if prec == "d" else ("s", "s_f64")):
                want, g = oracle.samples(v, "NT"[ta], "NT"[tb], m, n, k, alpha, A, lda, B, ldb, beta,
                                         C0 if beta != 0 else np.zeros_like(C0), ldc, rows, cols)
                r = parity_ratio(got[rows, cols], want, g, k, dt)
                assert r <= TOL_C, (case, ta, tb, alpha, beta, v, r)
            x = rng.standard_normal(n)
            opA = (A[:k, :m].T if ta else A[:m, :k]).astype(np.float64)
            opB = (B[:n, :k].T if tb else B[:k, :n]).astype(np.float64)
            rhs = alpha * (opA @ (opB @ x)) + (beta * (C0[:m].astype(np.float64) @ x) if beta != 0 else 0.0)
            gauge = abs(alpha) * (np.abs(opA) @ (np.abs(opB) @ np.abs(x))) + \
                (abs(beta) * (np.abs(C0[:m]).astype(np.float64) @ np.abs(x)) if beta != 0 else 0.0)
            err = np.abs(got[:m].astype(np.float64) @ x - rhs) / ((k + n) * np.finfo(dt).eps * gauge)
            assert err.max() <= TOL_C, (case, ta, tb, alpha, beta, float(err.max()))


# products of a few tiles and a long k: the planner cuts their tiles into more than four pieces
LONG_K = [
    ("d", 0, 0, 256, 256, 40000),
    ("d", 1, 0, 200, 200, 20000),       # tiles that reach past the edges, A transposed
    ("d", 0, 1, 250, 130, 30011),       # k ends inside a slab
    ("d", 1, 1, 512, 512, 8192),
    ("s", 0, 0, 256, 256, 40000),
    ("s", 1, 0, 300, 200, 20000),
    ("s", 0, 1, 100, 100, 50003),
]


@pytest.mark.parametrize("case", LONG_K, ids=lambda c: "%s_%d%d_%dx%dx%d" % c)
def test_long_k_products_cut_into_many_pieces(case, restore_switches):
    """The planner's own launch of products with few tiles and a long k: the
    chain of folds is 4 to 32 pieces long.  Against numpy in float64 under the
    bound of gpu_util.TOL_C, beta == 0 on a NaN-filled C and beta != 0; the same
    bits on a second run."""
    import torch
    prec, ta, tb, m, n, k = case
    dt = np.float64 if prec == "d" else np.float32
    eps = np.finfo(dt).eps
    f = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    A, B, C0, lda, ldb, ldc = _operands(prec, ta, tb, m, n, k, pads=(1, 2, 3))
    vid, whole_c, groups, tiles = blas.plan(prec, m, n, k, 0, lda, ldb)
    assert vid != 0 and groups >= 4 * tiles, ("the planner does not cut this product into chains of pieces", case, groups, tiles)
    dA, dB = to_device(A), to_device(B)
    opA = (A[:k, :m].T if ta else A[:m, :k]).astype(np.float64)
    opB = (B[:n, :k].T if tb else B[:k, :n]).astype(np.float64)
    for alpha, beta in ((1.0, 0.0), (0.75, -0.25)):
        Cin = C0.copy(order="F")
        if beta == 0.0:
            Cin[:m] = np.nan
        runs = []
        for _ in range(2):
            dC = to_device(Cin)
            f(ta, tb, m, n, k, alpha, dA, lda, dB, ldb, beta, dC, ldc)
            torch.cuda.synchronize()
            runs.append(to_host(dC))
        got = runs[0]
        assert got.tobytes() == runs[1].tobytes()
        assert np.array_equal(got[m:], Cin[m:]), "padding rows of C were written"
        c0 = C0[:m].astype(np.float64) if beta != 0 else 0.0
        want = alpha * (opA @ opB) + beta * c0
        gauge = abs(alpha) * (np.abs(opA) @ np.abs(opB)) + abs(beta) * np.abs(c0)
        err = np.abs(got[:m].astype(np.float64) - want)
        assert (err <= TOL_C * k * eps * gauge).all(), (case, alpha, beta)
    blas.device_status()


@pytest.mark.parametrize("prec", ["d", "s"])
def test_random_shapes_as_the_planner_launches_them(prec):
    """240 products of random shape (1 .. 900 in every dimension, every
    transposition, padded leading dimensions, beta == 0 on NaN or beta != 0),
    launched the way the planner chooses -- whole tiles and strips, one launch
    over all of C with tiles past the edge, tiles shared or not, or the
    any-shape kernel alone -- against numpy in float64 under the bound of
    gpu_util.TOL_C; padding rows must come back untouched."""
    import torch
    dt = np.float64 if prec == "d" else np.float32
    eps = np.finfo(dt).eps
    rng = np.random.default_rng(2024 if prec == "d" else 2025)
    f = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    kinds = set()
    for it in range(240):
        big = it % 6 == 0
        m, n, k = (int(rng.integers(1, 2600 if big else 900)) for _ in range(3))
        if it % 17 == 0:
            m = int(rng.choice([1, 3, 4, 5, 63, 64, 65, 255, 256, 257]))
        if it % 19 == 0:
            n = int(rng.choice([1, 3, 4, 5, 63, 64, 65, 127, 128, 129]))
        ta, tb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pads = tuple(int(x) for x in rng.integers(0, 4, 3))
        A, B, C0, lda, ldb, ldc = _operands(prec, ta, tb, m, n, k, pads=pads)
        alpha, beta = ((1.0, 0.0), (0.75, -0.25), (-1.0, 1.0))[it % 3]
        Cin = C0.copy(order="F")
        if beta == 0.0:
            Cin[:m] = np.nan
        kinds.add(tuple(blas.plan(prec, m, n, k, int(beta != 0), lda, ldb))[:2] +
                  (blas.plan(prec, m, n, k, int(beta != 0), lda, ldb)[2] > 0,))
        dC = to_device(Cin)
        f(ta, tb, m, n, k, alpha, to_device(A), lda, to_device(B), ldb, beta, dC, ldc)
        torch.cuda.synchronize()
        got = to_host(dC)
        assert np.array_equal(got[m:], Cin[m:]), ("padding rows of C were written", m, n, k, ta, tb)
        opA = (A[:k, :m].T if ta else A[:m, :k]).astype(np.float64)
        opB = (B[:n, :k].T if tb else B[:k, :n]).astype(np.float64)
        c0 = C0[:m].astype(np.float64) if beta != 0 else 0.0
        want = alpha * (opA @ opB) + beta * c0
        gauge = abs(alpha) * (np.abs(opA) @ np.abs(opB)) + abs(beta) * np.abs(c0)
        err = np.abs(got[:m].astype(np.float64) - want)
        # the float64 reference carries no error of its own worth counting; the bound is the GPU's half of TOL_C
        assert (err <= TOL_C * k * eps * gauge + 0.0).all(), (prec, m, n, k, ta, tb, alpha, beta, pads)
    blas.device_status()
    # the draw covers the ways a product can be launched: any-shape kernel alone (variant 0), whole tiles,
    # one launch over all of C, shared tiles
    assert any(v == 0 for v, _, _ in kinds) and any(w for _, w, _ in kinds) and any(s for _, _, s in kinds), kinds
    # (in single precision the small tile takes odd shapes in one launch: whole tiles with strips beside them
    # only come up for shapes that the draw does not hold)
    assert prec == "s" or any(v != 0 and not w for v, w, _ in kinds), kinds


def test_same_bits_every_run_and_close_to_unshared(restore_switches):
    """The order in which the pieces are folded into C is fixed, so the result
    does not depend on which workgroup happens to be ahead; and it differs from
    the unshared product only by the extra roundings of the folds."""
    import torch
    prec, m, n, k = "d", 256 * 19, 128 * 23, 1100
    blas.set_variant("d", 1)
    A, B, C0, lda, ldb, ldc = _operands(prec, 1, 0, m, n, k)
    dA, dB = to_device(A), to_device(B)
    outs = []
    for pieces in (-4, -4, -4, -2, -8):
        blas.test_control(blas.TEST_SHARED_PIECES, pieces)
        outs.append(_run(prec, 1, 0, m, n, k, 0.75, -0.25, A, B, C0, lda, ldb, ldc, dA, dB))
        # other work in between, so that the workgroups do not meet the same way twice
        _ = (dA[:64] @ dA[:64].T).sum().item()
    assert outs[0].tobytes() == outs[1].tobytes() == outs[2].tobytes()
    blas.test_control(blas.TEST_SHARED_PIECES, 0)
    plain = _run(prec, 1, 0, m, n, k, 0.75, -0.25, A, B, C0, lda, ldb, ldc, dA, dB)
    assert plain.tobytes() != outs[0].tobytes(), "the launch shared no tile: the test does not test what it says"
    scale = k * np.finfo(np.float64).eps * (0.75 * k + 0.25)
    for o in outs:
        assert np.abs(o - plain).max() <= scale
    blas.device_status()


def test_bounded_wait_runs_out_and_the_result_is_still_complete(restore_switches, oracle):
    """Flags that are never raised: every workgroup that waits gives up after
    its limit and leaves C alone, all kernels end, the launch that follows
    every launch with shared tiles recomputes what is missing, and the device
    status says once that this happened.  Every kind of shared launch: whole
    tiles and tiles past the edge, beta == 0 on NaN and beta != 0, two to eight
    pieces per tile, both precisions, a transposed operand."""
    cases = [("d", 1, 0, 0, 2048, 2048, 512, -4), ("d", 1, 1, 0, 4352, 2048, 333, -4), ("d", 2, 0, 1, 1300, 1100, 700, -8),
             ("d", 6, 0, 0, 448, 512, 2048, -8), ("s", 1, 0, 0, 2051, 2046, 300, -2), ("s", 4, 1, 1, 512, 448, 2048, -4)]
    blas.device_status()
    for prec, vid, ta, tb, m, n, k, pieces in cases:
        dt = np.float64 if prec == "d" else np.float32
        blas.set_variant(prec, vid)
        blas.test_control(blas.TEST_WHOLE_C, 1)
        blas.test_control(blas.TEST_SHARED_PIECES, pieces)
        A, B, C0, lda, ldb, ldc = _operands(prec, ta, tb, m, n, k, pads=(3, 1, 2))
        for alpha, beta in ((1.0, 0.0), (0.75, -0.25)):
            Cin = C0.copy(order="F")
            if beta == 0.0:
                Cin[:m] = np.nan
            blas.test_control(blas.TEST_SHARED_MUTE, 0)
            blas.test_control(blas.TEST_SHARED_SPIN_LIMIT, -1)
            heard = _run(prec, ta, tb, m, n, k, alpha, beta, A, B, Cin, lda, ldb, ldc)
            blas.device_status()
            blas.test_control(blas.TEST_SHARED_MUTE, 1)
            blas.test_control(blas.TEST_SHARED_SPIN_LIMIT, 4)
            got = _run(prec, ta, tb, m, n, k, alpha, beta, A, B, Cin, lda, ldb, ldc)
            tag = (prec, vid, ta, tb, m, n, k, alpha, beta)
            with pytest.raises(blas.GpuError, match="status 4.*ran out"):
                blas.device_status()
            blas.device_status()                       # reported once, then clean
            assert np.array_equal(got[m:], Cin[m:]), tag
            assert not np.isnan(got[:m]).any(), tag
            want = Cin.copy(order="F")
            C_for_oracle = C0 if beta != 0 else np.zeros_like(C0)
            want[:] = C_for_oracle
            oracle.gemm(prec, "NT"[ta], "NT"[tb], m, n, k, alpha, A, lda, B, ldb, beta, want, ldc)
            g = oracle.gauge("NT"[ta], "NT"[tb], m, n, k, alpha, A, B, beta, C_for_oracle)
            assert parity_ratio(got[:m], want[:m], g, k, dt) <= TOL_C, tag
            # the same pieces in the same order of k, only later: within rounding of the run whose flags were heard
            assert parity_ratio(got[:m], heard[:m], g, k, dt) <= TOL_C, tag
    # ... and the rows of flags are in order again for the launches that come after
    blas.test_control(blas.TEST_SHARED_MUTE, 0)
    blas.test_control(blas.TEST_SHARED_SPIN_LIMIT, -1)
    prec, vid, ta, tb, m, n, k, pieces = cases[0]
    blas.set_variant(prec, vid)
    blas.test_control(blas.TEST_SHARED_PIECES, pieces)
    A, B, C0, lda, ldb, ldc = _operands(prec, ta, tb, m, n, k)
    for _ in range(3):
        got = _run(prec, ta, tb, m, n, k, 1.0, 0.0, A, B, C0, lda, ldb, ldc)
        want = A[:m, :k] @ B[:k, :n]
        assert np.abs(got[:m] - want).max() <= 4 * k * np.finfo(np.float64).eps * k
    blas.device_status()


def test_host_entry_points_make_up_for_waits_that_run_out(restore_switches, oracle, xerbla):
    """dgemm_, dsyrk_, dtrsm_ and ulmblas_dgetrf on shapes whose products the
    planner cuts along k, with flags that are never raised and a wait limit of
    a few polls: every call returns the complete result (the reference's
    entry points cannot return anything else, interfaces/blas/F77/gemm.cc:
    131-249), its status is OK, and the hook has been told that the call had
    to make up for waits that ran out."""
    import netlib
    RECOVERED = 4

    def muted(on):
        blas.test_control(blas.TEST_SHARED_MUTE, 1 if on else 0)
        blas.test_control(blas.TEST_SHARED_SPIN_LIMIT, 4 if on else -1)

    rng = np.random.default_rng(11)
    # dgemm_: 3072^3 travels in two column panels of 144 tiles each, which share their k
    for (ta, tb, m, n, k, alpha, beta) in [("N", "N", 3072, 3072, 3072, 1.0, 0.0), ("T", "N", 2304, 2304, 4096, 0.75, -0.25)]:
        ra, ca = (k, m) if ta == "T" else (m, k)
        A, B, C0 = synth.matrix(601, ra, ca, ra + 1), synth.matrix(602, k, n, k + 3), synth.matrix(603, m, n, m + 2)
        assert any(blas.plan("d", m, nn, k, beta != 0, ra + 1, k + 3)[2] > 0 for nn in (n, n // 2)), "the planner shares no tile here"
        Cin = C0.copy(order="F")
        if beta == 0.0:
            Cin[:m] = np.nan
        muted(True)
        xerbla.hook_reset()
        got = Cin.copy(order="F")
        blas.dgemm_(ta, tb, m, n, k, alpha, A, ra + 1, B, k + 3, beta, got, m + 2)
        muted(False)
        assert blas.last_status() == 0
        assert xerbla.hook_count() == 1 and xerbla.hook_last_status() == RECOVERED and xerbla.hook_last_routine() == b"dgemm_"
        rows = np.concatenate([[0, m - 1, 0, m - 1], rng.integers(0, m, 3000)])
        cols = np.concatenate([[0, 0, n - 1, n - 1], rng.integers(0, n, 3000)])
        want, g = oracle.samples("d", ta, tb, m, n, k, alpha, A, ra + 1, B, k + 3, beta, C0 if beta != 0 else np.zeros_like(C0),
                                 m + 2, rows, cols)
        assert parity_ratio(got[rows, cols], want, g, k, np.float64) <= TOL_C, (ta, tb, m, n, k)
        x = rng.standard_normal(n)
        opA = A[:k, :m].T if ta == "T" else A[:m, :k]
        rhs = alpha * (opA @ (B[:k, :n] @ x)) + (beta * (C0[:m] @ x) if beta != 0 else 0.0)
        gauge = abs(alpha) * (np.abs(opA) @ (np.abs(B[:k, :n]) @ np.abs(x))) + abs(beta) * (np.abs(C0[:m]) @ np.abs(x))
        assert (np.abs(got[:m] @ x - rhs) / ((k + n) * np.finfo(np.float64).eps * gauge)).max() <= TOL_C
        assert np.array_equal(got[m:], Cin[m:])
        # the same call with flags that are heard says nothing
        xerbla.hook_reset()
        again = Cin.copy(order="F")
        blas.dgemm_(ta, tb, m, n, k, alpha, A, ra + 1, B, k + 3, beta, again, m + 2)
        assert xerbla.hook_count() == 0 and blas.last_status() == 0
        assert parity_ratio(got[:m], again[:m], np.abs(again[:m]) + 1.0, k, np.float64) <= TOL_C

    # dsyrk_: order 3072 (12 blocks of 256: 66 whole tiles inside the triangle, shared), lower, A*A'
    n, k = 3072, 1500
    A, C0 = synth.matrix(611, n, k, n), synth.matrix(612, n, n, n)
    mask = netlib.triangle_mask("L", n)
    C0[~mask] = np.nan
    muted(True)
    xerbla.hook_reset()
    got = C0.copy(order="F")
    blas.syrk_("d", "L", "N", n, k, 0.7, A, n, 1.3, got, n)
    muted(False)
    assert blas.last_status() == 0
    assert xerbla.hook_count() == 1 and xerbla.hook_last_status() == RECOVERED and xerbla.hook_last_routine() == b"dsyrk_"
    assert np.isnan(got[~mask]).all()
    rows = rng.integers(0, n, 4000)
    cols = rng.integers(0, n, 4000)
    rows, cols = np.maximum(rows, cols), np.minimum(rows, cols)
    At = np.asfortranarray(A.T)
    want, g = oracle.samples("d", "N", "N", n, n, k, 0.7, A, n, At, k, 1.3, np.nan_to_num(C0), n, rows, cols)
    assert parity_ratio(got[rows, cols], want, g, k, np.float64) <= TOL_C

    # dtrsm_: order 6144 on 3072 right-hand sides, whose largest update (3072 x 3072 x 3072) shares tiles
    m, n = 6144, 3072
    assert blas.plan("d", m // 2, n, m // 2, True, m, m)[2] > 0, "the planner shares no tile here"
    T = synth.matrix(621, m, m, m)
    T *= 8.0 / m
    T[np.arange(m), np.arange(m)] += 2.0
    B0 = synth.matrix(622, m, n, m)
    muted(True)
    xerbla.hook_reset()
    X = B0.copy(order="F")
    blas.dtrsm_("L", "L", "N", "N", m, n, 1.0, T, m, X, m)
    muted(False)
    assert blas.last_status() == 0
    assert xerbla.hook_count() == 1 and xerbla.hook_last_status() == RECOVERED and xerbla.hook_last_routine() == b"dtrsm_"
    Tl = np.tril(T)
    resid = np.abs(Tl @ X - B0) / (np.finfo(np.float64).eps * (np.abs(Tl) @ np.abs(X) + np.abs(B0)))
    assert resid.max() <= 16.0, resid.max()
    blas.device_status()
