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
