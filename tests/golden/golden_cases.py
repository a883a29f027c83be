"""The case lists shared by make_golden.py (which writes the fixtures from the
compiled reference) and test_oracle_golden.py (which replays them through the
oracle)."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from ulmblas_amd import synth  # noqa: E402

DTYPES = {"d": np.float64, "s": np.float32, "s_f64": np.float32}

# reference builds and the block sizes they were compiled with
# (MC, KC, NC, MR, NR); None = production sizes for the variant
LIBS = {
    "libulmref.so": None,
    "libulmref_tp01.so": (8, 12, 12, 4, 4),
    "libulmref_tp02.so": (8, 12, 12, 2, 4),
    "libulmref_tp03.so": (8, 12, 12, 4, 2),
}

SCALARS = [(1.0, 0.0), (0.7, 1.3), (0.0, 1.3), (-1.0, 1.0)]
TRANS = [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")]


def _case(lib, variant, ta, tb, m, n, k, alpha, beta):
    ra = k if ta == "T" else m
    rb = n if tb == "T" else k
    return dict(lib=lib, variant=variant, ta=ta, tb=tb, m=m, n=n, k=k, alpha=alpha, beta=beta, lda=max(1, ra) + 3,
                ldb=max(1, rb) + 1, ldc=max(1, m) + 2, blocksize=LIBS[lib],
                key=f"{lib[:-3]}|{variant}|{ta}{tb}|{m}x{n}x{k}|{alpha}|{beta}")


SMALL_CASES = [
    _case(lib, variant, ta, tb, m, n, k, alpha, beta)
    for lib in LIBS
    for variant in ("d", "s", "s_f64")
    for (m, n, k) in [(13, 9, 25), (7, 31, 12), (31, 12, 31), (1, 1, 1), (12, 12, 12), (5, 7, 0)]
    for (ta, tb) in TRANS
    for (alpha, beta) in SCALARS
]

LARGE_CASES = [
    _case("libulmref.so", variant, ta, tb, m, n, k, alpha, beta)
    for variant in ("d", "s", "s_f64")
    for (m, n, k) in [(67, 33, 401), (385, 5, 385), (130, 129, 800), (769, 9, 400)]
    for (ta, tb) in TRANS
    for (alpha, beta) in SCALARS
]


def operands(case):
    """Seeded A, B, C for a case; C's window is NaN when beta == 0, so a
    result that read it shows."""
    dt = DTYPES[case["variant"]]
    m, n, k = case["m"], case["n"], case["k"]
    ra, ca = (k, m) if case["ta"] == "T" else (m, k)
    rb, cb = (n, k) if case["tb"] == "T" else (k, n)
    A = synth.matrix(11, ra, ca, case["lda"], dtype=dt)
    B = synth.matrix(12, rb, cb, case["ldb"], dtype=dt)
    C0 = synth.matrix(13, m, n, case["ldc"], dtype=dt)
    if case["beta"] == 0.0:
        C0[:m, :] = np.nan
    return A, B, C0


# ---------------------------------------------------------------------------
# triangular solve (dtrsm / cblas_strsm / strsm_ arithmetic)
# ---------------------------------------------------------------------------

TRSM_COMBOS = [(side, uplo, trans, diag) for side in "LR" for uplo in "UL" for trans in "NT" for diag in "UN"]


def _trsm_case(lib, variant, side, uplo, trans, diag, m, n, alpha):
    na = m if side == "L" else n
    return dict(lib=lib, variant=variant, side=side, uplo=uplo, trans=trans, diag=diag, m=m, n=n, alpha=alpha,
                lda=max(1, na) + 2, ldb=max(1, m) + 3, blocksize=LIBS[lib],
                key=f"trsm|{lib[:-3]}|{variant}|{side}{uplo}{trans}{diag}|{m}x{n}|{alpha}")


TRSM_CASES = [
    _trsm_case(lib, variant, side, uplo, trans, diag, m, n, alpha)
    for lib in LIBS
    for variant in ("d", "s", "s_f64")
    for (m, n) in [(13, 9), (7, 31), (31, 12), (1, 1)]
    for (side, uplo, trans, diag) in TRSM_COMBOS
    for alpha in (1.0, 0.7)
] + [
    _trsm_case("libulmref.so", variant, side, uplo, trans, diag, m, n, alpha)
    for variant in ("d", "s", "s_f64")
    for (m, n) in [(385, 9), (9, 400), (770, 5), (130, 129)]
    for (side, uplo, trans, diag) in TRSM_COMBOS
    for alpha in (-1.0,)
]


def trsm_operands(case):
    """Seeded triangular A and B.  Off-diagonal entries are scaled by
    min(1, 8/order) so that large triangles stay well conditioned, the
    diagonal is pushed away from zero (|a_jj| >= 2); the triangle the routine
    must not read, and the diagonal of a unit triangle, are NaN, so a result
    that read them shows."""
    dt = DTYPES[case["variant"]]
    m, n = case["m"], case["n"]
    na = m if case["side"] == "L" else n
    A = synth.matrix(21, na, na, case["lda"], dtype=dt)
    B = synth.matrix(22, m, n, case["ldb"], dtype=dt)
    idx = np.arange(na)
    A[:na] *= dt(min(1.0, 8.0 / max(na, 1)))
    A[idx, idx] += np.where(A[idx, idx] < 0, -2.0, 2.0).astype(dt)
    i, j = np.meshgrid(idx, idx, indexing="ij")
    hide = (i > j) if case["uplo"] == "U" else (i < j)
    if case["diag"] == "U":
        hide |= (i == j)
    A[:na][hide] = np.nan
    return A, B


# ---------------------------------------------------------------------------
# LU factorisation (ulmblas_dgetrf arithmetic)
# ---------------------------------------------------------------------------

def _lu_case(lib, m, n, row_major, kind):
    return dict(lib=lib, m=m, n=n, row_major=row_major, kind=kind, blocksize=LIBS[lib],
                key=f"getrf|{lib[:-3]}|{m}x{n}|{'row' if row_major else 'col'}|{kind}")


LU_CASES = [
    _lu_case(lib, m, n, rm, kind)
    for lib in ("libulmref.so", "libulmref_tp01.so", "libulmref_tp03.so")
    for (m, n) in [(1, 1), (5, 5), (7, 3), (3, 7), (64, 64), (65, 65), (100, 130), (130, 100), (200, 200), (129, 257)]
    for rm in (False, True)
    for kind in ("random", "singular")
] + [
    _lu_case("libulmref.so", m, n, False, "random") for (m, n) in [(450, 450), (500, 300), (300, 500)]
]


def lu_operands(case):
    """Seeded matrix in the layout the entry point factors: column-major
    m x n with ld = m + 3, or for the row-major branch of the interface the
    n x m matrix with element (i, j) at i*ld + j, ld = m + 3.  'singular'
    zeroes one column and repeats another, so the factorisation meets an
    exactly zero pivot."""
    m, n = case["m"], case["n"]
    ld = m + 3
    cols = n
    A = synth.matrix(31, m, cols, ld)
    if case["kind"] == "singular" and min(m, n) > 2:
        A[:m, 2] = 0.0
        A[:m, n - 1] = A[:m, 0]
    return A, ld


# ---------------------------------------------------------------------------
# symmetric rank-k and rank-2k updates, symmetric product, triangular product
# ---------------------------------------------------------------------------

L3_LIBS = ("libulmref.so", "libulmref_tp01.so", "libulmref_tp02.so")


def _l3_case(routine, lib, combo, dims, scalars):
    return dict(routine=routine, lib=lib, combo=combo, dims=dims, scalars=scalars, blocksize=LIBS[lib],
                key=f"{routine}|{lib[:-3]}|{combo}|{'x'.join(map(str, dims))}|{'|'.join(map(str, scalars))}")


L3_CASES = (
    [_l3_case("syrk", lib, u + t, dims, sc)
     for lib in L3_LIBS for u in "UL" for t in "NT"
     for dims in ([(13, 9), (7, 31), (31, 12), (1, 1)] + ([(385, 40), (40, 800), (390, 390)] if lib == "libulmref.so" else []))
     for sc in ((1.0, 0.0), (0.7, 1.3), (0.0, 1.3))]
    + [_l3_case("syr2k", lib, u + t, dims, sc)
       for lib in L3_LIBS for u in "UL" for t in "NT"
       for dims in ([(13, 9), (7, 31), (31, 12), (1, 1)] + ([(385, 40), (40, 800), (390, 390)] if lib == "libulmref.so" else []))
       for sc in ((1.0, 0.0), (0.7, 1.3), (0.0, 1.3))]
    + [_l3_case("symm", lib, s_ + u, dims, sc)
       for lib in L3_LIBS for s_ in "LR" for u in "UL"
       for dims in ([(13, 9), (7, 31), (31, 12), (1, 1)] + ([(385, 9), (9, 400), (130, 129)] if lib == "libulmref.so" else []))
       for sc in ((1.0, 0.0), (0.7, 1.3), (0.0, 1.3))]
    + [_l3_case("trmm", lib, s_ + u + t + d, dims, sc)
       for lib in L3_LIBS for s_ in "LR" for u in "UL" for t in "NT" for d in "UN"
       for dims in ([(13, 9), (7, 31), (31, 12), (1, 1)] + ([(385, 9), (9, 400), (800, 5)] if lib == "libulmref.so" else []))
       for sc in ((1.0,), (0.7,))]
)


def l3_operands(case):
    """Seeded double operands of a case, in call order, with the parts the
    routine must not read filled with NaN (the other triangle of a symmetric
    or triangular A, the diagonal of a unit triangle, the other triangle of
    the rank-k update's C, and all of C when beta == 0)."""
    r, combo, dims = case["routine"], case["combo"], case["dims"]
    idx = lambda n: np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    if r in ("syrk", "syr2k"):
        n, k = dims
        ra, ca = (k, n) if combo[1] == "T" else (n, k)
        A = synth.matrix(41, ra, ca, ra + 2)
        Cm = synth.matrix(42, n, n, n + 1)
        i, j = idx(n)
        other = (i > j) if combo[0] == "U" else (i < j)
        Cm[:n][other] = np.nan
        if case["scalars"][1] == 0.0:
            Cm[:n][~other] = np.nan
        if r == "syr2k":
            # both operands on one leading dimension: the reference reads B with A's
            # (ulmblas/level3/sylr2k.tcc:66-67)
            return dict(A=A, lda=ra + 2, B=synth.matrix(48, ra, ca, ra + 2), ldb=ra + 2, C=Cm, ldc=n + 1)
        return dict(A=A, lda=ra + 2, C=Cm, ldc=n + 1)
    if r == "symm":
        m, n = dims
        na = m if combo[0] == "L" else n
        A = synth.matrix(43, na, na, na + 2)
        i, j = idx(na)
        A[:na][(i > j) if combo[1] == "U" else (i < j)] = np.nan
        B = synth.matrix(44, m, n, m + 1)
        Cm = synth.matrix(45, m, n, m + 3)
        if case["scalars"][1] == 0.0:
            Cm[:m] = np.nan
        return dict(A=A, lda=na + 2, B=B, ldb=m + 1, C=Cm, ldc=m + 3)
    m, n = dims
    na = m if combo[0] == "L" else n
    A = synth.matrix(46, na, na, na + 2)
    i, j = idx(na)
    hide = (i > j) if combo[1] == "U" else (i < j)
    if combo[3] == "U":
        hide |= (i == j)
    A[:na][hide] = np.nan
    B = synth.matrix(47, m, n, m + 1)
    return dict(A=A, lda=na + 2, B=B, ldb=m + 1)


def l3_run(case, ops, syrk, symm, trmm, syr2k, **kw):
    """Runs the case through the four callables (oracle or compiled reference) and returns the result array."""
    r, combo, dims, sc = case["routine"], case["combo"], case["dims"], case["scalars"]
    if r == "syr2k":
        return syr2k(combo[0], combo[1], dims[0], dims[1], sc[0], ops["A"], ops["lda"], ops["B"], ops["ldb"], sc[1],
                     ops["C"], ops["ldc"], **kw)
    if r == "syrk":
        return syrk(combo[0], combo[1], dims[0], dims[1], sc[0], ops["A"], ops["lda"], sc[1], ops["C"], ops["ldc"], **kw)
    if r == "symm":
        return symm(combo[0], combo[1], dims[0], dims[1], sc[0], ops["A"], ops["lda"], ops["B"], ops["ldb"], sc[1],
                    ops["C"], ops["ldc"], **kw)
    return trmm(combo[0], combo[1], combo[2], combo[3], dims[0], dims[1], sc[0], ops["A"], ops["lda"], ops["B"],
                ops["ldb"], **kw)


# ---------------------------------------------------------------------------
# complex GEMM
# ---------------------------------------------------------------------------

CGEMM_SCALARS = [(1.0, 0.0), (0.7 - 0.9j, 1.3 - 1.1j), (0.0, 1.3 - 1.1j), (-1.0, 1.0), (0.5, 2.0)]


def _cgemm_case(lib, variant, ta, tb, m, n, k, alpha, beta):
    ra = k if ta in "TC" else m
    rb = n if tb in "TC" else k
    return dict(lib=lib, variant=variant, ta=ta, tb=tb, m=m, n=n, k=k, alpha=alpha, beta=beta, lda=max(1, ra) + 3,
                ldb=max(1, rb) + 1, ldc=max(1, m) + 2, blocksize=LIBS[lib],
                key=f"{lib[:-3]}|{variant}|{ta}{tb}|{m}x{n}x{k}|{alpha}|{beta}")


CGEMM_CASES = [
    _cgemm_case(lib, variant, ta, tb, m, n, k, alpha, beta)
    for lib in LIBS
    for variant in ("z", "c")
    for (m, n, k) in ([(13, 9, 25), (7, 31, 12), (1, 1, 1), (5, 7, 0)]
                      + ([(67, 33, 401), (193, 5, 385), (130, 3, 800)] if lib == "libulmref.so" else []))
    for ta in "NTCR" for tb in "NTCR"
    for (alpha, beta) in CGEMM_SCALARS
]


def cgemm_operands(case):
    """Seeded complex A, B, C (real and imaginary parts from independent streams);
    C's window is NaN when beta == 0."""
    dt = np.complex128 if case["variant"] == "z" else np.complex64
    m, n, k = case["m"], case["n"], case["k"]
    ra, ca = (k, m) if case["ta"] in "TC" else (m, k)
    rb, cb = (n, k) if case["tb"] in "TC" else (k, n)

    def cm(seed, rows, cols, ld):
        z = synth.matrix(seed, rows, cols, ld) + 1j * synth.matrix(seed + 100, rows, cols, ld)
        return np.asfortranarray(z.astype(dt))

    A, B, Cm = cm(51, ra, ca, case["lda"]), cm(52, rb, cb, case["ldb"]), cm(53, m, n, case["ldc"])
    if case["beta"] == 0:
        Cm[:m] = complex(np.nan, np.nan)
    return A, B, Cm
