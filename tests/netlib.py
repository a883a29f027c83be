"""Python restatement of the pieces of the netlib level-3 BLAS testers that the
reference's test suite drives GEMM with (test/F77/dblat3.f, sblat3.f and the
CBLAS variants under test/C): the input generator, the sweep parameters read
from the testers' data files, the result check and the error-exit call lists.
"""
from __future__ import annotations

import numpy as np

ROGUE = -1.0e10            # dblat3.f:2365 -- value of padding rows
NMAX = 65                  # dblat3.f:61


def _beg_cycle():
    """One period of DBEG's output.  Its state (I, IC) moves by a bijection
    (891 is invertible mod 1000), so the stream is purely periodic."""
    out, i, ic = [], 7, 0
    while True:
        ic += 1
        i = (i * 891) % 1000
        if ic >= 5:
            ic = 0
            i = (i * 891) % 1000
        out.append((i - 500) / 1001.0)
        if (i, ic) == (7, 0):
            return np.array(out)


class Beg:
    """DBEG / SBEG (dblat3.f:2673-2718): the tester's deterministic generator
    of values in (-0.5, 0.5): I = 7; each call I = I*891 mod 1000, and every
    fifth call takes one extra step (IC).  One instance carries the SAVEd
    state that the Fortran code keeps across calls of DMAKE within a sweep;
    the stream is served from one precomputed period."""

    _cycle = None

    def __init__(self):
        if Beg._cycle is None:
            Beg._cycle = _beg_cycle()
        self.reset()

    def reset(self):
        self.pos = 0

    def take(self, count: int) -> np.ndarray:
        idx = (self.pos + np.arange(count)) % Beg._cycle.shape[0]
        self.pos = (self.pos + count) % Beg._cycle.shape[0]
        return Beg._cycle[idx]

    def next(self) -> float:
        return float(self.take(1)[0])


def make_ge(beg: Beg, m: int, n: int, lda: int, dtype=np.float64) -> np.ndarray:
    """DMAKE('GE', ...) (dblat3.f:2344-2456): an (lda x n) Fortran-ordered
    window, values from `beg` drawn column by column, the off-diagonal elements
    of column n/2 zeroed when n > 3 (:2397-2398), padding rows = ROGUE."""
    aa = np.full((max(lda, 1), n), ROGUE, dtype=dtype, order="F")
    if m > 0 and n > 0:
        body = beg.take(m * n).reshape((m, n), order="F").copy(order="F")
        if n > 3:
            j = n // 2 - 1                      # Fortran column n/2
            keep = body[j, j] if j < m else None
            body[:, j] = 0.0
            if keep is not None:
                body[j, j] = keep
        aa[:m, :] = body
    return aa


def _zbeg_cycle():
    """One period of ZBEG's output (zblat3.f:3287-3340): I and J step together
    (I*891, J*457 mod 1000, one extra step every fifth call)."""
    out, i, j, ic = [], 7, 7, 0
    while True:
        ic += 1
        i, j = (i * 891) % 1000, (j * 457) % 1000
        if ic >= 5:
            ic = 0
            i, j = (i * 891) % 1000, (j * 457) % 1000
        out.append(complex((i - 500) / 1001.0, (j - 500) / 1001.0))
        if (i, j, ic) == (7, 7, 0):
            return np.array(out)


class ZBeg(Beg):
    """ZBEG / CBEG: the complex testers' generator, served like Beg."""

    _zcycle = None

    def __init__(self):
        if ZBeg._zcycle is None:
            ZBeg._zcycle = _zbeg_cycle()
        self.reset()

    def take(self, count: int) -> np.ndarray:
        idx = (self.pos + np.arange(count)) % ZBeg._zcycle.shape[0]
        self.pos = (self.pos + count) % ZBeg._zcycle.shape[0]
        return ZBeg._zcycle[idx]


ZROGUE = complex(-1.0e10, 1.0e10)      # zblat3.f ZMAKE: value of padding rows


def make_zge(beg: ZBeg, m: int, n: int, lda: int, dtype=np.complex128) -> np.ndarray:
    """ZMAKE('GE', ...) (zblat3.f:3070-3184): as make_ge, complex."""
    aa = np.full((max(lda, 1), n), ZROGUE, dtype=dtype, order="F")
    if m > 0 and n > 0:
        body = beg.take(m * n).reshape((m, n), order="F").copy(order="F")
        if n > 3:
            j = n // 2 - 1
            keep = body[j, j] if j < m else None
            body[:, j] = 0.0
            if keep is not None:
                body[j, j] = keep
        aa[:m, :] = body
    return aa


# Sweep parameters from the testers' data files.
DBLAT3 = dict(idim=[0, 1, 2, 3, 7, 12, 31, 3], alf=[0.0, 1.0, 0.7], bet=[0.0, 1.0, 1.3], thresh=16.0)  # dblat3.dat.in:9-14
SBLAT3 = dict(idim=[0, 1, 2, 3, 7, 31, 63], alf=[0.0, 1.0, 0.7], bet=[0.0, 1.0, 1.3], thresh=16.0)      # sblat3.dat.in:9-14
DIN3 = dict(idim=[1, 2, 3, 5, 7, 9], alf=[0.0, 1.0, 0.7], bet=[0.0, 1.0, 1.3], thresh=16.0)              # test/C/din3:8-13
ZBLAT3 = dict(idim=[0, 1, 2, 3, 7, 31, 63], alf=[0.0, 1.0, 0.7 - 0.9j], bet=[0.0, 1.0, 1.3 - 1.1j],
              thresh=16.0)                                                                               # zblat3.dat.in, cblat3.dat.in
ZIN3 = dict(idim=[0, 1, 2, 3, 5, 9], alf=[0.0, 1.0, 0.7 - 0.9j], bet=[0.0, 1.0, 1.3 - 1.1j], thresh=16.0)  # test/C/zin3, cin3
ICH = "NTC"                                                                                              # dblat3.f:408


def chk1_cases(params, dtype=np.float64, nmax=NMAX):
    """The loop nest of DCHK1 (dblat3.f:415-498): yields one dict per GEMM call
    with freshly generated operands, in the tester's order and with the
    tester's generator state (reset once per sweep, :412)."""
    is_complex = np.issubdtype(dtype, np.complexfloating)      # ZCHK1 (zblat3.f:411-498): same nest, ZMAKE
    beg = ZBeg() if is_complex else Beg()
    make_ge = make_zge if is_complex else globals()["make_ge"]
    for m in params["idim"]:
        for n in params["idim"]:
            ldc = m + 1 if m < nmax else m
            if ldc > nmax:
                continue
            for k in params["idim"]:
                for transa in ICH:
                    trana = transa in "TC"
                    ma, na = (k, m) if trana else (m, k)
                    lda = ma + 1 if ma < nmax else ma
                    if lda > nmax:
                        continue
                    aa = make_ge(beg, ma, na, lda, dtype)
                    for transb in ICH:
                        tranb = transb in "TC"
                        mb, nb = (n, k) if tranb else (k, n)
                        ldb = mb + 1 if mb < nmax else mb
                        if ldb > nmax:
                            continue
                        bb = make_ge(beg, mb, nb, ldb, dtype)
                        for alpha in params["alf"]:
                            for beta in params["bet"]:
                                cc = make_ge(beg, m, n, ldc, dtype)
                                yield dict(transa=transa, transb=transb, m=m, n=n, k=k, alpha=alpha, beta=beta, aa=aa,
                                           lda=lda, bb=bb, ldb=ldb, cc=cc, ldc=ldc)


def mmch(transa, transb, m, n, k, alpha, aa, bb, beta, c0, cc, dtype=np.float64):
    """DMMCH (dblat3.f:2457-2578): the expected result in the working
    precision's wider type, the gauge G = |alpha| sum|a||b| + |beta||c| and the
    test ratio max |ct - cc| / (eps * G).  Returns (err, ct)."""
    eps = np.finfo(dtype).eps
    a = aa.astype(np.float64)
    b = bb.astype(np.float64)
    opa = a[:k, :m].T if transa in "TC" else a[:m, :k]
    opb = b[:n, :k].T if transb in "TC" else b[:k, :n]
    c0w = c0[:m, :n].astype(np.float64)
    ct = alpha * (opa @ opb) + beta * c0w
    g = abs(alpha) * (np.abs(opa) @ np.abs(opb)) + abs(beta) * np.abs(c0w)
    erri = np.abs(ct - cc[:m, :n].astype(np.float64)) / eps
    nz = g != 0
    erri[nz] = erri[nz] / g[nz]
    return (float(erri.max()) if erri.size else 0.0), ct


def zmmch(transa, transb, m, n, k, alpha, aa, bb, beta, c0, cc, dtype=np.complex128):
    """ZMMCH (zblat3.f:2935-3066): the expected result in complex128, the gauge
    G = ABS1(alpha) sum ABS1(a) ABS1(b) + ABS1(beta) ABS1(c) with ABS1(z) =
    |re z| + |im z|, and the ratio max ABS1(ct - cc) / (eps G).  'C' conjugates."""
    eps = np.finfo(dtype).eps
    abs1 = lambda z: np.abs(np.real(z)) + np.abs(np.imag(z))
    a, b = aa.astype(np.complex128), bb.astype(np.complex128)
    opa = a[:k, :m].T if transa in "TC" else a[:m, :k]
    opb = b[:n, :k].T if transb in "TC" else b[:k, :n]
    ga, gb = abs1(opa), abs1(opb)
    if transa == "C":
        opa = opa.conj()
    if transb == "C":
        opb = opb.conj()
    c0w = c0[:m, :n].astype(np.complex128)
    ct = alpha * (opa @ opb) + beta * c0w
    g = abs1(alpha) * (ga @ gb) + abs1(beta) * abs1(c0w)
    erri = abs1(ct - cc[:m, :n].astype(np.complex128)) / eps
    nz = g != 0
    erri[nz] = erri[nz] / g[nz]
    return (float(erri.max()) if erri.size else 0.0), ct


# ZCHKE / CCHKE (zblat3.f, cblat3.f), the ZGEMM block: (transa, transb, m, n, k, lda, ldb, ldc) -> INFOT.
# The CBLAS tester's cblas_zgemm block (test/C/c_z3chke.c) makes the calls of its cblas_dgemm block.
F77_ZGEMM_ERROR_EXITS = [
    (("/", "N", 0, 0, 0, 1, 1, 1), 1), (("/", "C", 0, 0, 0, 1, 1, 1), 1), (("/", "T", 0, 0, 0, 1, 1, 1), 1),
    (("N", "/", 0, 0, 0, 1, 1, 1), 2), (("C", "/", 0, 0, 0, 1, 1, 1), 2), (("T", "/", 0, 0, 0, 1, 1, 1), 2),
    (("N", "N", -1, 0, 0, 1, 1, 1), 3), (("N", "C", -1, 0, 0, 1, 1, 1), 3), (("N", "T", -1, 0, 0, 1, 1, 1), 3),
    (("C", "N", -1, 0, 0, 1, 1, 1), 3), (("C", "C", -1, 0, 0, 1, 1, 1), 3), (("C", "T", -1, 0, 0, 1, 1, 1), 3),
    (("T", "N", -1, 0, 0, 1, 1, 1), 3), (("T", "C", -1, 0, 0, 1, 1, 1), 3), (("T", "T", -1, 0, 0, 1, 1, 1), 3),
    (("N", "N", 0, -1, 0, 1, 1, 1), 4), (("N", "C", 0, -1, 0, 1, 1, 1), 4), (("N", "T", 0, -1, 0, 1, 1, 1), 4),
    (("C", "N", 0, -1, 0, 1, 1, 1), 4), (("C", "C", 0, -1, 0, 1, 1, 1), 4), (("C", "T", 0, -1, 0, 1, 1, 1), 4),
    (("T", "N", 0, -1, 0, 1, 1, 1), 4), (("T", "C", 0, -1, 0, 1, 1, 1), 4), (("T", "T", 0, -1, 0, 1, 1, 1), 4),
    (("N", "N", 0, 0, -1, 1, 1, 1), 5), (("N", "C", 0, 0, -1, 1, 1, 1), 5), (("N", "T", 0, 0, -1, 1, 1, 1), 5),
    (("C", "N", 0, 0, -1, 1, 1, 1), 5), (("C", "C", 0, 0, -1, 1, 1, 1), 5), (("C", "T", 0, 0, -1, 1, 1, 1), 5),
    (("T", "N", 0, 0, -1, 1, 1, 1), 5), (("T", "C", 0, 0, -1, 1, 1, 1), 5), (("T", "T", 0, 0, -1, 1, 1, 1), 5),
    (("N", "N", 2, 0, 0, 1, 1, 2), 8), (("N", "C", 2, 0, 0, 1, 1, 2), 8), (("N", "T", 2, 0, 0, 1, 1, 2), 8),
    (("C", "N", 0, 0, 2, 1, 2, 1), 8), (("C", "C", 0, 0, 2, 1, 1, 1), 8), (("C", "T", 0, 0, 2, 1, 1, 1), 8),
    (("T", "N", 0, 0, 2, 1, 2, 1), 8), (("T", "C", 0, 0, 2, 1, 1, 1), 8), (("T", "T", 0, 0, 2, 1, 1, 1), 8),
    (("N", "N", 0, 0, 2, 1, 1, 1), 10), (("C", "N", 0, 0, 2, 2, 1, 1), 10), (("T", "N", 0, 0, 2, 2, 1, 1), 10),
    (("N", "C", 0, 2, 0, 1, 1, 1), 10), (("C", "C", 0, 2, 0, 1, 1, 1), 10), (("T", "C", 0, 2, 0, 1, 1, 1), 10),
    (("N", "T", 0, 2, 0, 1, 1, 1), 10), (("C", "T", 0, 2, 0, 1, 1, 1), 10), (("T", "T", 0, 2, 0, 1, 1, 1), 10),
    (("N", "N", 2, 0, 0, 2, 1, 1), 13), (("N", "C", 2, 0, 0, 2, 1, 1), 13), (("N", "T", 2, 0, 0, 2, 1, 1), 13),
    (("C", "N", 2, 0, 0, 1, 1, 1), 13), (("C", "C", 2, 0, 0, 1, 1, 1), 13), (("C", "T", 2, 0, 0, 1, 1, 1), 13),
    (("T", "N", 2, 0, 0, 1, 1, 1), 13), (("T", "C", 2, 0, 0, 1, 1, 1), 13), (("T", "T", 2, 0, 0, 1, 1, 1), 13),
]

# DCHKE (dblat3.f:1838-1921): (transa, transb, m, n, k, lda, ldb, ldc) -> INFOT
F77_ERROR_EXITS = [
    (("/", "N", 0, 0, 0, 1, 1, 1), 1), (("/", "T", 0, 0, 0, 1, 1, 1), 1),
    (("N", "/", 0, 0, 0, 1, 1, 1), 2), (("T", "/", 0, 0, 0, 1, 1, 1), 2),
    (("N", "N", -1, 0, 0, 1, 1, 1), 3), (("N", "T", -1, 0, 0, 1, 1, 1), 3),
    (("T", "N", -1, 0, 0, 1, 1, 1), 3), (("T", "T", -1, 0, 0, 1, 1, 1), 3),
    (("N", "N", 0, -1, 0, 1, 1, 1), 4), (("N", "T", 0, -1, 0, 1, 1, 1), 4),
    (("T", "N", 0, -1, 0, 1, 1, 1), 4), (("T", "T", 0, -1, 0, 1, 1, 1), 4),
    (("N", "N", 0, 0, -1, 1, 1, 1), 5), (("N", "T", 0, 0, -1, 1, 1, 1), 5),
    (("T", "N", 0, 0, -1, 1, 1, 1), 5), (("T", "T", 0, 0, -1, 1, 1, 1), 5),
    (("N", "N", 2, 0, 0, 1, 1, 2), 8), (("N", "T", 2, 0, 0, 1, 1, 2), 8),
    (("T", "N", 0, 0, 2, 1, 2, 1), 8), (("T", "T", 0, 0, 2, 1, 1, 1), 8),
    (("N", "N", 0, 0, 2, 1, 1, 1), 10), (("T", "N", 0, 0, 2, 2, 1, 1), 10),
    (("N", "T", 0, 2, 0, 1, 1, 1), 10), (("T", "T", 0, 2, 0, 1, 1, 1), 10),
    (("N", "N", 2, 0, 0, 2, 1, 1), 13), (("N", "T", 2, 0, 0, 2, 1, 1), 13),
    (("T", "N", 2, 0, 0, 1, 1, 1), 13), (("T", "T", 2, 0, 0, 1, 1, 1), 13),
]

COL, ROW, BAD = 102, 101, -1
NT, TR = 111, 112


def _four(order, m, n, k, lda, ldb, ldc, info, combos=((NT, NT), (NT, TR), (TR, NT), (TR, TR))):
    return [((order, ta, tb, m, n, k, lda, ldb, ldc), info) for ta, tb in combos]


# test/C/c_d3chke.c:46-273: (order, transa, transb, m, n, k, lda, ldb, ldc) ->
# the info the TESTER expects after its cblas_xerbla has undone the row-major
# swap of positions 4<->5 and 9<->11 (test/C/c_xerbla.c:27-42).
CBLAS_ERROR_EXITS = (
    _four(BAD, 0, 0, 0, 1, 1, 1, 1)
    + [((COL, BAD, NT, 0, 0, 0, 1, 1, 1), 2), ((COL, BAD, TR, 0, 0, 0, 1, 1, 1), 2),
       ((COL, NT, BAD, 0, 0, 0, 1, 1, 1), 3), ((COL, TR, BAD, 0, 0, 0, 1, 1, 1), 3)]
    + _four(COL, BAD, 0, 0, 1, 1, 1, 4) + _four(COL, 0, BAD, 0, 1, 1, 1, 5) + _four(COL, 0, 0, BAD, 1, 1, 1, 6)
    + [((COL, NT, NT, 2, 0, 0, 1, 1, 2), 9), ((COL, NT, TR, 2, 0, 0, 1, 1, 2), 9),
       ((COL, TR, NT, 0, 0, 2, 1, 2, 1), 9), ((COL, TR, TR, 0, 0, 2, 1, 1, 1), 9),
       ((COL, NT, NT, 0, 0, 2, 1, 1, 1), 11), ((COL, TR, NT, 0, 0, 2, 2, 1, 1), 11),
       ((COL, NT, TR, 0, 2, 0, 1, 1, 1), 11), ((COL, TR, TR, 0, 2, 0, 1, 1, 1), 11),
       ((COL, NT, NT, 2, 0, 0, 2, 1, 1), 14), ((COL, NT, TR, 2, 0, 0, 2, 1, 1), 14),
       ((COL, TR, NT, 2, 0, 0, 1, 1, 1), 14), ((COL, TR, TR, 2, 0, 0, 1, 1, 1), 14)]
    + _four(ROW, BAD, 0, 0, 1, 1, 1, 4) + _four(ROW, 0, BAD, 0, 1, 1, 1, 5) + _four(ROW, 0, 0, BAD, 1, 1, 1, 6)
    + [((ROW, NT, NT, 0, 0, 2, 1, 1, 2), 9), ((ROW, NT, TR, 0, 0, 2, 1, 2, 2), 9),
       ((ROW, TR, NT, 2, 0, 0, 1, 2, 1), 9), ((ROW, TR, TR, 2, 0, 0, 1, 1, 1), 9),
       ((ROW, NT, NT, 0, 2, 0, 1, 1, 1), 11), ((ROW, TR, NT, 0, 2, 0, 2, 1, 1), 11),
       ((ROW, NT, TR, 0, 0, 2, 2, 1, 1), 11), ((ROW, TR, TR, 0, 0, 2, 1, 1, 1), 11),
       ((ROW, NT, NT, 0, 2, 0, 1, 2, 1), 14), ((ROW, NT, TR, 0, 2, 0, 1, 1, 1), 14),
       ((ROW, TR, NT, 0, 2, 0, 1, 2, 1), 14), ((ROW, TR, TR, 0, 2, 0, 1, 1, 1), 14)]
)


def cblas_tester_info(order, info):
    """What the CBLAS tester's xerbla makes of a reported info for *gemm:
    under row-major it swaps 4<->5 and 9<->11 back (test/C/c_xerbla.c:27-42)."""
    if order == ROW:
        return {4: 5, 5: 4, 9: 11, 11: 9}.get(info, info)
    return info


# ---------------------------------------------------------------------------
# triangular solve: DCHK3 (dblat3.f:907-1209), its operand generator and check
# ---------------------------------------------------------------------------

def make_tr(beg: Beg, uplo: str, diag: str, n: int, lda: int, dtype=np.float64):
    """DMAKE('TR', ...) (dblat3.f:2344-2456).  Returns (a, aa): `a` the full
    n x n matrix the checker multiplies with (zeros in the other triangle,
    diagonal + 1, or exactly 1 for a unit triangle), `aa` the (lda x n) window
    handed to the routine, where everything the routine must not read -- the
    other triangle, the diagonal of a unit triangle, the padding -- is ROGUE.
    Values are drawn column by column over the stored triangle, diagonal
    included; the off-diagonal elements of column n/2 are zero when n > 3."""
    a = np.zeros((n, n), dtype=np.float64, order="F")
    upper, unit = uplo.upper() == "U", diag.upper() == "U"
    for j in range(n):
        rows = range(0, j + 1) if upper else range(j, n)
        vals = beg.take(len(rows))
        for i, v in zip(rows, vals):
            a[i, j] = v
            if i != j and n > 3 and j == n // 2 - 1:
                a[i, j] = 0.0
        a[j, j] += 1.0
        if unit:
            a[j, j] = 1.0
    a = a.astype(dtype)
    aa = np.full((max(lda, 1), n), ROGUE, dtype=dtype, order="F")
    for j in range(n):
        if upper:
            lo, hi = 0, (j if unit else j + 1)
        else:
            lo, hi = (j + 1 if unit else j), n
        aa[lo:hi, j] = a[lo:hi, j]
    return a, aa


def chk3_cases(params, dtype=np.float64, nmax=NMAX):
    """The loop nest of DCHK3 (dblat3.f:973-1060) for the solve: one dict per
    call with the tester's operands (generator reset once per sweep)."""
    beg = Beg()
    for m in params["idim"]:
        for n in params["idim"]:
            ldb = m + 1 if m < nmax else m
            if ldb > nmax:
                continue
            for side in "LR":
                na = m if side == "L" else n
                lda = na + 1 if na < nmax else na
                if lda > nmax:
                    break                       # GO TO 130: next n
                for uplo in "UL":
                    for transa in ICH:
                        for diag in "UN":
                            for alpha in params["alf"]:
                                a, aa = make_tr(beg, uplo, diag, na, lda, dtype)
                                bb = make_ge(beg, m, n, ldb, dtype)
                                yield dict(side=side, uplo=uplo, transa=transa, diag=diag, m=m, n=n, alpha=alpha,
                                           a=a, aa=aa, lda=lda, bb=bb, ldb=ldb)


def trsm_check(side, transa, m, n, alpha, a, b0, xx, dtype=np.float64):
    """The solve's check in DCHK3 (dblat3.f:1119-1141): multiply the computed
    X back, op(A) X (left) or X op(A) (right), and compare with alpha*B through
    DMMCH's ratio |ct - alpha b| / (eps * sum|a||x|)."""
    eps = np.finfo(dtype).eps
    af = a.astype(np.float64)
    opa = af.T if transa in "TC" else af
    x = xx[:m, :n].astype(np.float64)
    want = (dtype(alpha) * b0[:m, :n]).astype(np.float64)      # BB = ALPHA*B in the working precision
    if side == "L":
        ct, g = opa @ x, np.abs(opa) @ np.abs(x)
    else:
        ct, g = x @ opa, np.abs(x) @ np.abs(opa)
    erri = np.abs(ct - want) / eps
    nz = g != 0
    erri[nz] = erri[nz] / g[nz]
    return float(erri.max()) if erri.size else 0.0


# DCHKE, the DTRSM block (dblat3.f:2098-2205):
# (side, uplo, transa, diag, m, n, lda, ldb) -> INFOT
F77_TRSM_ERROR_EXITS = [
    (("/", "U", "N", "N", 0, 0, 1, 1), 1), (("L", "/", "N", "N", 0, 0, 1, 1), 2),
    (("L", "U", "/", "N", 0, 0, 1, 1), 3), (("L", "U", "N", "/", 0, 0, 1, 1), 4),
    (("L", "U", "N", "N", -1, 0, 1, 1), 5), (("L", "U", "T", "N", -1, 0, 1, 1), 5),
    (("R", "U", "N", "N", -1, 0, 1, 1), 5), (("R", "U", "T", "N", -1, 0, 1, 1), 5),
    (("L", "L", "N", "N", -1, 0, 1, 1), 5), (("L", "L", "T", "N", -1, 0, 1, 1), 5),
    (("R", "L", "N", "N", -1, 0, 1, 1), 5), (("R", "L", "T", "N", -1, 0, 1, 1), 5),
    (("L", "U", "N", "N", 0, -1, 1, 1), 6), (("L", "U", "T", "N", 0, -1, 1, 1), 6),
    (("R", "U", "N", "N", 0, -1, 1, 1), 6), (("R", "U", "T", "N", 0, -1, 1, 1), 6),
    (("L", "L", "N", "N", 0, -1, 1, 1), 6), (("L", "L", "T", "N", 0, -1, 1, 1), 6),
    (("R", "L", "N", "N", 0, -1, 1, 1), 6), (("R", "L", "T", "N", 0, -1, 1, 1), 6),
    (("L", "U", "N", "N", 2, 0, 1, 2), 9), (("L", "U", "T", "N", 2, 0, 1, 2), 9),
    (("R", "U", "N", "N", 0, 2, 1, 1), 9), (("R", "U", "T", "N", 0, 2, 1, 1), 9),
    (("L", "L", "N", "N", 2, 0, 1, 2), 9), (("L", "L", "T", "N", 2, 0, 1, 2), 9),
    (("R", "L", "N", "N", 0, 2, 1, 1), 9), (("R", "L", "T", "N", 0, 2, 1, 1), 9),
    (("L", "U", "N", "N", 2, 0, 2, 1), 11), (("L", "U", "T", "N", 2, 0, 2, 1), 11),
    (("R", "U", "N", "N", 2, 0, 1, 1), 11), (("R", "U", "T", "N", 2, 0, 1, 1), 11),
    (("L", "L", "N", "N", 2, 0, 2, 1), 11), (("L", "L", "T", "N", 2, 0, 2, 1), 11),
    (("R", "L", "N", "N", 2, 0, 1, 1), 11), (("R", "L", "T", "N", 2, 0, 1, 1), 11),
]

LEFT, RIGHT, UPPER, LOWER, NONUNIT, UNIT = 141, 142, 121, 122, 131, 132

# test/C/c_d3chke.c:730-1009: (order, side, uplo, transa, diag, m, n, lda, ldb)
# -> the info the TESTER expects after its cblas_xerbla has undone the
# row-major swap of positions 6<->7 (test/C/c_xerbla.c:41-45).
CBLAS_TRSM_ERROR_EXITS = [
    ((BAD, LEFT, UPPER, NT, NONUNIT, 0, 0, 1, 1), 1), ((COL, BAD, UPPER, NT, NONUNIT, 0, 0, 1, 1), 2),
    ((COL, LEFT, BAD, NT, NONUNIT, 0, 0, 1, 1), 3), ((COL, LEFT, UPPER, BAD, NONUNIT, 0, 0, 1, 1), 4),
    ((COL, LEFT, UPPER, NT, BAD, 0, 0, 1, 1), 5), ((COL, LEFT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, LEFT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, RIGHT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, RIGHT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, LEFT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, LEFT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, RIGHT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, RIGHT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, LEFT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, LEFT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, RIGHT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, RIGHT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, LEFT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, LEFT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, RIGHT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, RIGHT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, LEFT, UPPER, NT, NONUNIT, 2, 0, 1, 2), 10),
    ((COL, LEFT, UPPER, TR, NONUNIT, 2, 0, 1, 2), 10), ((COL, RIGHT, UPPER, NT, NONUNIT, 0, 2, 1, 1), 10),
    ((COL, RIGHT, UPPER, TR, NONUNIT, 0, 2, 1, 1), 10), ((COL, LEFT, LOWER, NT, NONUNIT, 2, 0, 1, 2), 10),
    ((COL, LEFT, LOWER, TR, NONUNIT, 2, 0, 1, 2), 10), ((COL, RIGHT, LOWER, NT, NONUNIT, 0, 2, 1, 1), 10),
    ((COL, RIGHT, LOWER, TR, NONUNIT, 0, 2, 1, 1), 10), ((COL, LEFT, UPPER, NT, NONUNIT, 2, 0, 2, 1), 12),
    ((COL, LEFT, UPPER, TR, NONUNIT, 2, 0, 2, 1), 12), ((COL, RIGHT, UPPER, NT, NONUNIT, 2, 0, 1, 1), 12),
    ((COL, RIGHT, UPPER, TR, NONUNIT, 2, 0, 1, 1), 12), ((COL, LEFT, LOWER, NT, NONUNIT, 2, 0, 2, 1), 12),
    ((COL, LEFT, LOWER, TR, NONUNIT, 2, 0, 2, 1), 12), ((COL, RIGHT, LOWER, NT, NONUNIT, 2, 0, 1, 1), 12),
    ((COL, RIGHT, LOWER, TR, NONUNIT, 2, 0, 1, 1), 12), ((ROW, LEFT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, LEFT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, RIGHT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, LEFT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, LEFT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, RIGHT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, LEFT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, LEFT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, RIGHT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, LEFT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, LEFT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, RIGHT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, LEFT, UPPER, NT, NONUNIT, 2, 0, 1, 1), 10),
    ((ROW, LEFT, UPPER, TR, NONUNIT, 2, 0, 1, 1), 10), ((ROW, RIGHT, UPPER, NT, NONUNIT, 0, 2, 1, 2), 10),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, 0, 2, 1, 2), 10), ((ROW, LEFT, LOWER, NT, NONUNIT, 2, 0, 1, 1), 10),
    ((ROW, LEFT, LOWER, TR, NONUNIT, 2, 0, 1, 1), 10), ((ROW, RIGHT, LOWER, NT, NONUNIT, 0, 2, 1, 2), 10),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, 0, 2, 1, 2), 10), ((ROW, LEFT, UPPER, NT, NONUNIT, 0, 2, 1, 1), 12),
    ((ROW, LEFT, UPPER, TR, NONUNIT, 0, 2, 1, 1), 12), ((ROW, RIGHT, UPPER, NT, NONUNIT, 0, 2, 2, 1), 12),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, 0, 2, 2, 1), 12), ((ROW, LEFT, LOWER, NT, NONUNIT, 0, 2, 1, 1), 12),
    ((ROW, LEFT, LOWER, TR, NONUNIT, 0, 2, 1, 1), 12), ((ROW, RIGHT, LOWER, NT, NONUNIT, 0, 2, 2, 1), 12),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, 0, 2, 2, 1), 12),
]


def cblas_tester_info_trsm(order, info):
    if order == ROW:
        return {6: 7, 7: 6}.get(info, info)
    return info


# ---------------------------------------------------------------------------
# symmetric product (DCHK2), triangular product (DCHK3), rank-k update (DCHK4)
# ---------------------------------------------------------------------------

def make_sy(beg: Beg, uplo: str, n: int, lda: int, dtype=np.float64):
    """DMAKE('SY', ...) (dblat3.f:2344-2456).  Returns (a, aa): `a` the full
    symmetric n x n matrix, `aa` the (lda x n) window holding only the uplo
    triangle, everything else ROGUE.  Values are drawn column by column over
    the stored triangle; off-diagonal elements of column n/2 are zero when
    n > 3 (and so are their mirror images)."""
    a = np.zeros((n, n), dtype=np.float64, order="F")
    upper = uplo.upper() == "U"
    for j in range(n):
        rows = range(0, j + 1) if upper else range(j, n)
        vals = beg.take(len(rows))
        for i, v in zip(rows, vals):
            if i != j and n > 3 and j == n // 2 - 1:
                v = 0.0
            a[i, j] = v
            a[j, i] = v
    a = a.astype(dtype)
    aa = np.full((max(lda, 1), n), ROGUE, dtype=dtype, order="F")
    for j in range(n):
        lo, hi = (0, j + 1) if upper else (j, n)
        aa[lo:hi, j] = a[lo:hi, j]
    return a, aa


def chk2_cases(params, dtype=np.float64, nmax=NMAX):
    """The loop nest of DCHK2 (dblat3.f:672-760): one dict per DSYMM call."""
    beg = Beg()
    for m in params["idim"]:
        for n in params["idim"]:
            ldc = m + 1 if m < nmax else m
            if ldc > nmax:
                continue
            ldb = ldc
            bb = make_ge(beg, m, n, ldb, dtype)
            for side in "LR":
                na = m if side == "L" else n
                lda = na + 1 if na < nmax else na
                if lda > nmax:
                    continue
                for uplo in "UL":
                    a, aa = make_sy(beg, uplo, na, lda, dtype)
                    for alpha in params["alf"]:
                        for beta in params["bet"]:
                            cc = make_ge(beg, m, n, ldc, dtype)
                            yield dict(side=side, uplo=uplo, m=m, n=n, alpha=alpha, beta=beta, a=a, aa=aa, lda=lda,
                                       bb=bb, ldb=ldb, cc=cc, ldc=ldc)


def chk4_cases(params, dtype=np.float64, nmax=NMAX):
    """The loop nest of DCHK4 (dblat3.f:1249-1300): one dict per DSYRK call.
    `c` is the full symmetric matrix behind the stored triangle `cc`."""
    beg = Beg()
    for n in params["idim"]:
        ldc = n + 1 if n < nmax else n
        if ldc > nmax:
            continue
        for k in params["idim"]:
            for trans in ICH:
                tran = trans in "TC"
                ma, na = (k, n) if tran else (n, k)
                lda = ma + 1 if ma < nmax else ma
                if lda > nmax:
                    continue
                aa = make_ge(beg, ma, na, lda, dtype)
                for uplo in "UL":
                    for alpha in params["alf"]:
                        for beta in params["bet"]:
                            c, cc = make_sy(beg, uplo, n, ldc, dtype)
                            yield dict(uplo=uplo, trans=trans, n=n, k=k, alpha=alpha, beta=beta, aa=aa, lda=lda, c=c,
                                       cc=cc, ldc=ldc)


def chk5_cases(params, dtype=np.float64, nmax=NMAX):
    """The loop nest of DCHK5 (dblat3.f:1541-1600) for DSYR2K: one dict per
    call.  B is drawn right after A with the same shape and leading dimension;
    `c` is the full symmetric matrix behind the stored triangle `cc`."""
    beg = Beg()
    for n in params["idim"]:
        ldc = n + 1 if n < nmax else n
        if ldc > nmax:
            continue
        for k in params["idim"]:
            for trans in ICH:
                tran = trans in "TC"
                ma, na = (k, n) if tran else (n, k)
                lda = ma + 1 if ma < nmax else ma
                if lda > nmax:
                    continue
                aa = make_ge(beg, ma, na, lda, dtype)
                bb = make_ge(beg, ma, na, lda, dtype)
                for uplo in "UL":
                    for alpha in params["alf"]:
                        for beta in params["bet"]:
                            c, cc = make_sy(beg, uplo, n, ldc, dtype)
                            yield dict(uplo=uplo, trans=trans, n=n, k=k, alpha=alpha, beta=beta, aa=aa, lda=lda,
                                       bb=bb, ldb=lda, c=c, cc=cc, ldc=ldc)


def syr2k_check(trans, n, k, alpha, aa, bb, beta, c, got, dtype=np.float64):
    """The check of DCHK5 (dblat3.f:1688-1735): column j of the result against
    alpha * [A B] [B A]^T + beta * C formed in double, as the DMMCH ratio with
    an inner dimension of 2k.  Returns the n x n array of ratios."""
    eps = np.finfo(dtype).eps
    a, b = aa.astype(np.float64), bb.astype(np.float64)
    opa = a[:k, :n].T if trans in "TC" else a[:n, :k]
    opb = b[:k, :n].T if trans in "TC" else b[:n, :k]
    c0 = c.astype(np.float64)
    ct = alpha * (opa @ opb.T + opb @ opa.T) + beta * c0
    g = abs(alpha) * (np.abs(opa) @ np.abs(opb).T + np.abs(opb) @ np.abs(opa).T) + abs(beta) * np.abs(c0)
    erri = np.abs(ct - got[:n, :n].astype(np.float64)) / eps
    nz = g != 0
    erri[nz] = erri[nz] / g[nz]
    return erri


def triangle_mask(uplo, n):
    i, j = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    return (i <= j) if uplo.upper() == "U" else (i >= j)


# DCHKE (dblat3.f:1801-2340), the DSYMM, DTRMM and DSYRK blocks:
# (character arguments..., sizes and leading dimensions in call order) -> INFOT
F77_SYMM_ERROR_EXITS = [
    (("/", "U", 0, 0, 1, 1, 1), 1), (("L", "/", 0, 0, 1, 1, 1), 2), (("L", "U", -1, 0, 1, 1, 1), 3),
    (("R", "U", -1, 0, 1, 1, 1), 3), (("L", "L", -1, 0, 1, 1, 1), 3), (("R", "L", -1, 0, 1, 1, 1), 3),
    (("L", "U", 0, -1, 1, 1, 1), 4), (("R", "U", 0, -1, 1, 1, 1), 4), (("L", "L", 0, -1, 1, 1, 1), 4),
    (("R", "L", 0, -1, 1, 1, 1), 4), (("L", "U", 2, 0, 1, 2, 2), 7), (("R", "U", 0, 2, 1, 1, 1), 7),
    (("L", "L", 2, 0, 1, 2, 2), 7), (("R", "L", 0, 2, 1, 1, 1), 7), (("L", "U", 2, 0, 2, 1, 1), 9),
    (("R", "U", 2, 0, 1, 1, 1), 9), (("L", "L", 2, 0, 2, 1, 1), 9), (("R", "L", 2, 0, 1, 1, 1), 9),
    (("L", "U", 2, 0, 2, 2, 1), 12), (("R", "U", 2, 0, 1, 2, 1), 12), (("L", "L", 2, 0, 2, 2, 1), 12),
    (("R", "L", 2, 0, 1, 2, 1), 12),
]
F77_TRMM_ERROR_EXITS = [
    (("/", "U", "N", "N", 0, 0, 1, 1), 1), (("L", "/", "N", "N", 0, 0, 1, 1), 2),
    (("L", "U", "/", "N", 0, 0, 1, 1), 3), (("L", "U", "N", "/", 0, 0, 1, 1), 4),
    (("L", "U", "N", "N", -1, 0, 1, 1), 5), (("L", "U", "T", "N", -1, 0, 1, 1), 5),
    (("R", "U", "N", "N", -1, 0, 1, 1), 5), (("R", "U", "T", "N", -1, 0, 1, 1), 5),
    (("L", "L", "N", "N", -1, 0, 1, 1), 5), (("L", "L", "T", "N", -1, 0, 1, 1), 5),
    (("R", "L", "N", "N", -1, 0, 1, 1), 5), (("R", "L", "T", "N", -1, 0, 1, 1), 5),
    (("L", "U", "N", "N", 0, -1, 1, 1), 6), (("L", "U", "T", "N", 0, -1, 1, 1), 6),
    (("R", "U", "N", "N", 0, -1, 1, 1), 6), (("R", "U", "T", "N", 0, -1, 1, 1), 6),
    (("L", "L", "N", "N", 0, -1, 1, 1), 6), (("L", "L", "T", "N", 0, -1, 1, 1), 6),
    (("R", "L", "N", "N", 0, -1, 1, 1), 6), (("R", "L", "T", "N", 0, -1, 1, 1), 6),
    (("L", "U", "N", "N", 2, 0, 1, 2), 9), (("L", "U", "T", "N", 2, 0, 1, 2), 9),
    (("R", "U", "N", "N", 0, 2, 1, 1), 9), (("R", "U", "T", "N", 0, 2, 1, 1), 9),
    (("L", "L", "N", "N", 2, 0, 1, 2), 9), (("L", "L", "T", "N", 2, 0, 1, 2), 9),
    (("R", "L", "N", "N", 0, 2, 1, 1), 9), (("R", "L", "T", "N", 0, 2, 1, 1), 9),
    (("L", "U", "N", "N", 2, 0, 2, 1), 11), (("L", "U", "T", "N", 2, 0, 2, 1), 11),
    (("R", "U", "N", "N", 2, 0, 1, 1), 11), (("R", "U", "T", "N", 2, 0, 1, 1), 11),
    (("L", "L", "N", "N", 2, 0, 2, 1), 11), (("L", "L", "T", "N", 2, 0, 2, 1), 11),
    (("R", "L", "N", "N", 2, 0, 1, 1), 11), (("R", "L", "T", "N", 2, 0, 1, 1), 11),
]
F77_SYRK_ERROR_EXITS = [
    (("/", "N", 0, 0, 1, 1), 1), (("U", "/", 0, 0, 1, 1), 2), (("U", "N", -1, 0, 1, 1), 3),
    (("U", "T", -1, 0, 1, 1), 3), (("L", "N", -1, 0, 1, 1), 3), (("L", "T", -1, 0, 1, 1), 3),
    (("U", "N", 0, -1, 1, 1), 4), (("U", "T", 0, -1, 1, 1), 4), (("L", "N", 0, -1, 1, 1), 4),
    (("L", "T", 0, -1, 1, 1), 4), (("U", "N", 2, 0, 1, 2), 7), (("U", "T", 0, 2, 1, 1), 7),
    (("L", "N", 2, 0, 1, 2), 7), (("L", "T", 0, 2, 1, 1), 7), (("U", "N", 2, 0, 2, 1), 10),
    (("U", "T", 2, 0, 1, 1), 10), (("L", "N", 2, 0, 2, 1), 10), (("L", "T", 2, 0, 1, 1), 10),
]

# the DSYR2K block (dblat3.f:2263-2328): (uplo, trans, n, k, lda, ldb, ldc) -> INFOT
F77_SYR2K_ERROR_EXITS = [
    (("/", "N", 0, 0, 1, 1, 1), 1), (("U", "/", 0, 0, 1, 1, 1), 2), (("U", "N", -1, 0, 1, 1, 1), 3),
    (("U", "T", -1, 0, 1, 1, 1), 3), (("L", "N", -1, 0, 1, 1, 1), 3), (("L", "T", -1, 0, 1, 1, 1), 3),
    (("U", "N", 0, -1, 1, 1, 1), 4), (("U", "T", 0, -1, 1, 1, 1), 4), (("L", "N", 0, -1, 1, 1, 1), 4),
    (("L", "T", 0, -1, 1, 1, 1), 4), (("U", "N", 2, 0, 1, 1, 2), 7), (("U", "T", 0, 2, 1, 1, 1), 7),
    (("L", "N", 2, 0, 1, 1, 2), 7), (("L", "T", 0, 2, 1, 1, 1), 7), (("U", "N", 2, 0, 2, 1, 2), 9),
    (("U", "T", 0, 2, 2, 1, 1), 9), (("L", "N", 2, 0, 2, 1, 2), 9), (("L", "T", 0, 2, 2, 1, 1), 9),
    (("U", "N", 2, 0, 2, 2, 1), 12), (("U", "T", 2, 0, 1, 1, 1), 12), (("L", "N", 2, 0, 2, 2, 1), 12),
    (("L", "T", 2, 0, 1, 1, 1), 12),
]

# test/C/c_d3chke.c, the cblas_dsymm, cblas_dtrmm and cblas_dsyrk blocks: what
# the TESTER expects after its cblas_xerbla has undone the row-major swaps
# (test/C/c_xerbla.c:27-60: symm 4<->5, trmm 6<->7, syrk none).
CBLAS_SYMM_ERROR_EXITS = [
    ((BAD, RIGHT, LOWER, 0, 0, 1, 1, 1), 1), ((COL, BAD, UPPER, 0, 0, 1, 1, 1), 2),
    ((COL, LEFT, BAD, 0, 0, 1, 1, 1), 3), ((COL, LEFT, UPPER, BAD, 0, 1, 1, 1), 4),
    ((COL, RIGHT, UPPER, BAD, 0, 1, 1, 1), 4), ((COL, LEFT, LOWER, BAD, 0, 1, 1, 1), 4),
    ((COL, RIGHT, LOWER, BAD, 0, 1, 1, 1), 4), ((COL, LEFT, UPPER, 0, BAD, 1, 1, 1), 5),
    ((COL, RIGHT, UPPER, 0, BAD, 1, 1, 1), 5), ((COL, LEFT, LOWER, 0, BAD, 1, 1, 1), 5),
    ((COL, RIGHT, LOWER, 0, BAD, 1, 1, 1), 5), ((COL, LEFT, UPPER, 2, 0, 1, 2, 2), 8),
    ((COL, RIGHT, UPPER, 0, 2, 1, 1, 1), 8), ((COL, LEFT, LOWER, 2, 0, 1, 2, 2), 8),
    ((COL, RIGHT, LOWER, 0, 2, 1, 1, 1), 8), ((COL, LEFT, UPPER, 2, 0, 2, 1, 1), 10),
    ((COL, RIGHT, UPPER, 2, 0, 1, 1, 1), 10), ((COL, LEFT, LOWER, 2, 0, 2, 1, 1), 10),
    ((COL, RIGHT, LOWER, 2, 0, 1, 1, 1), 10), ((COL, LEFT, UPPER, 2, 0, 2, 2, 1), 13),
    ((COL, RIGHT, UPPER, 2, 0, 1, 2, 1), 13), ((COL, LEFT, LOWER, 2, 0, 2, 2, 1), 13),
    ((COL, RIGHT, LOWER, 2, 0, 1, 2, 1), 13), ((ROW, LEFT, UPPER, BAD, 0, 1, 1, 1), 4),
    ((ROW, RIGHT, UPPER, BAD, 0, 1, 1, 1), 4), ((ROW, LEFT, LOWER, BAD, 0, 1, 1, 1), 4),
    ((ROW, RIGHT, LOWER, BAD, 0, 1, 1, 1), 4), ((ROW, LEFT, UPPER, 0, BAD, 1, 1, 1), 5),
    ((ROW, RIGHT, UPPER, 0, BAD, 1, 1, 1), 5), ((ROW, LEFT, LOWER, 0, BAD, 1, 1, 1), 5),
    ((ROW, RIGHT, LOWER, 0, BAD, 1, 1, 1), 5), ((ROW, LEFT, UPPER, 2, 0, 1, 2, 2), 8),
    ((ROW, RIGHT, UPPER, 0, 2, 1, 1, 1), 8), ((ROW, LEFT, LOWER, 2, 0, 1, 2, 2), 8),
    ((ROW, RIGHT, LOWER, 0, 2, 1, 1, 1), 8), ((ROW, LEFT, UPPER, 0, 2, 2, 1, 1), 10),
    ((ROW, RIGHT, UPPER, 0, 2, 2, 1, 1), 10), ((ROW, LEFT, LOWER, 0, 2, 2, 1, 1), 10),
    ((ROW, RIGHT, LOWER, 0, 2, 2, 1, 1), 10), ((ROW, LEFT, UPPER, 0, 2, 1, 2, 1), 13),
    ((ROW, RIGHT, UPPER, 0, 2, 2, 2, 1), 13), ((ROW, LEFT, LOWER, 0, 2, 1, 2, 1), 13),
    ((ROW, RIGHT, LOWER, 0, 2, 2, 2, 1), 13),
]
CBLAS_TRMM_ERROR_EXITS = [
    ((BAD, LEFT, UPPER, NT, NONUNIT, 0, 0, 1, 1), 1), ((COL, BAD, UPPER, NT, NONUNIT, 0, 0, 1, 1), 2),
    ((COL, LEFT, BAD, NT, NONUNIT, 0, 0, 1, 1), 3), ((COL, LEFT, UPPER, BAD, NONUNIT, 0, 0, 1, 1), 4),
    ((COL, LEFT, UPPER, NT, BAD, 0, 0, 1, 1), 5), ((COL, LEFT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, LEFT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, RIGHT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, RIGHT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, LEFT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, LEFT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, RIGHT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((COL, RIGHT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((COL, LEFT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, LEFT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, RIGHT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, RIGHT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, LEFT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, LEFT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, RIGHT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((COL, RIGHT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((COL, LEFT, UPPER, NT, NONUNIT, 2, 0, 1, 2), 10),
    ((COL, LEFT, UPPER, TR, NONUNIT, 2, 0, 1, 2), 10), ((COL, RIGHT, UPPER, NT, NONUNIT, 0, 2, 1, 1), 10),
    ((COL, RIGHT, UPPER, TR, NONUNIT, 0, 2, 1, 1), 10), ((COL, LEFT, LOWER, NT, NONUNIT, 2, 0, 1, 2), 10),
    ((COL, LEFT, LOWER, TR, NONUNIT, 2, 0, 1, 2), 10), ((COL, RIGHT, LOWER, NT, NONUNIT, 0, 2, 1, 1), 10),
    ((COL, RIGHT, LOWER, TR, NONUNIT, 0, 2, 1, 1), 10), ((COL, LEFT, UPPER, NT, NONUNIT, 2, 0, 2, 1), 12),
    ((COL, LEFT, UPPER, TR, NONUNIT, 2, 0, 2, 1), 12), ((COL, RIGHT, UPPER, NT, NONUNIT, 2, 0, 1, 1), 12),
    ((COL, RIGHT, UPPER, TR, NONUNIT, 2, 0, 1, 1), 12), ((COL, LEFT, LOWER, NT, NONUNIT, 2, 0, 2, 1), 12),
    ((COL, LEFT, LOWER, TR, NONUNIT, 2, 0, 2, 1), 12), ((COL, RIGHT, LOWER, NT, NONUNIT, 2, 0, 1, 1), 12),
    ((COL, RIGHT, LOWER, TR, NONUNIT, 2, 0, 1, 1), 12), ((ROW, LEFT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, LEFT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, RIGHT, UPPER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, LEFT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, LEFT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, RIGHT, LOWER, NT, NONUNIT, BAD, 0, 1, 1), 6),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, BAD, 0, 1, 1), 6), ((ROW, LEFT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, LEFT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, RIGHT, UPPER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, LEFT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, LEFT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, RIGHT, LOWER, NT, NONUNIT, 0, BAD, 1, 1), 7),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, 0, BAD, 1, 1), 7), ((ROW, LEFT, UPPER, NT, NONUNIT, 2, 0, 1, 1), 10),
    ((ROW, LEFT, UPPER, TR, NONUNIT, 2, 0, 1, 1), 10), ((ROW, RIGHT, UPPER, NT, NONUNIT, 0, 2, 1, 2), 10),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, 0, 2, 1, 2), 10), ((ROW, LEFT, LOWER, NT, NONUNIT, 2, 0, 1, 1), 10),
    ((ROW, LEFT, LOWER, TR, NONUNIT, 2, 0, 1, 1), 10), ((ROW, RIGHT, LOWER, NT, NONUNIT, 0, 2, 1, 2), 10),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, 0, 2, 1, 2), 10), ((ROW, LEFT, UPPER, NT, NONUNIT, 0, 2, 1, 1), 12),
    ((ROW, LEFT, UPPER, TR, NONUNIT, 0, 2, 1, 1), 12), ((ROW, RIGHT, UPPER, NT, NONUNIT, 0, 2, 2, 1), 12),
    ((ROW, RIGHT, UPPER, TR, NONUNIT, 0, 2, 2, 1), 12), ((ROW, LEFT, LOWER, NT, NONUNIT, 0, 2, 1, 1), 12),
    ((ROW, LEFT, LOWER, TR, NONUNIT, 0, 2, 1, 1), 12), ((ROW, RIGHT, LOWER, NT, NONUNIT, 0, 2, 2, 1), 12),
    ((ROW, RIGHT, LOWER, TR, NONUNIT, 0, 2, 2, 1), 12),
]
CBLAS_SYRK_ERROR_EXITS = [
    ((BAD, UPPER, NT, 0, 0, 1, 1), 1), ((COL, BAD, NT, 0, 0, 1, 1), 2), ((COL, UPPER, BAD, 0, 0, 1, 1), 3),
    ((COL, UPPER, NT, BAD, 0, 1, 1), 4), ((COL, UPPER, TR, BAD, 0, 1, 1), 4), ((COL, LOWER, NT, BAD, 0, 1, 1), 4),
    ((COL, LOWER, TR, BAD, 0, 1, 1), 4), ((COL, UPPER, NT, 0, BAD, 1, 1), 5), ((COL, UPPER, TR, 0, BAD, 1, 1), 5),
    ((COL, LOWER, NT, 0, BAD, 1, 1), 5), ((COL, LOWER, TR, 0, BAD, 1, 1), 5), ((ROW, UPPER, NT, 0, 2, 1, 2), 8),
    ((ROW, UPPER, TR, 2, 0, 1, 1), 8), ((ROW, LOWER, NT, 0, 2, 1, 2), 8), ((ROW, LOWER, TR, 2, 0, 1, 1), 8),
    ((COL, UPPER, NT, 2, 0, 1, 2), 8), ((COL, UPPER, TR, 0, 2, 1, 1), 8), ((COL, LOWER, NT, 2, 0, 1, 2), 8),
    ((COL, LOWER, TR, 0, 2, 1, 1), 8), ((ROW, UPPER, NT, 2, 0, 1, 1), 11), ((ROW, UPPER, TR, 2, 0, 2, 1), 11),
    ((ROW, LOWER, NT, 2, 0, 1, 1), 11), ((ROW, LOWER, TR, 2, 0, 2, 1), 11), ((COL, UPPER, NT, 2, 0, 2, 1), 11),
    ((COL, UPPER, TR, 2, 0, 1, 1), 11), ((COL, LOWER, NT, 2, 0, 2, 1), 11), ((COL, LOWER, TR, 2, 0, 1, 1), 11),
]


# test/C/c_d3chke.c:1123-1265, the cblas_dsyr2k block (the tester applies no row-major swap to it)
CBLAS_SYR2K_ERROR_EXITS = [
    ((BAD, UPPER, NT, 0, 0, 1, 1, 1), 1), ((COL, BAD, NT, 0, 0, 1, 1, 1), 2),
    ((COL, UPPER, BAD, 0, 0, 1, 1, 1), 3), ((COL, UPPER, NT, BAD, 0, 1, 1, 1), 4),
    ((COL, UPPER, TR, BAD, 0, 1, 1, 1), 4), ((COL, LOWER, NT, BAD, 0, 1, 1, 1), 4),
    ((COL, LOWER, TR, BAD, 0, 1, 1, 1), 4), ((COL, UPPER, NT, 0, BAD, 1, 1, 1), 5),
    ((COL, UPPER, TR, 0, BAD, 1, 1, 1), 5), ((COL, LOWER, NT, 0, BAD, 1, 1, 1), 5),
    ((COL, LOWER, TR, 0, BAD, 1, 1, 1), 5), ((ROW, UPPER, NT, 0, 2, 1, 2, 2), 8),
    ((ROW, UPPER, TR, 2, 0, 1, 2, 1), 8), ((ROW, LOWER, NT, 0, 2, 1, 2, 2), 8),
    ((ROW, LOWER, TR, 2, 0, 1, 2, 1), 8), ((COL, UPPER, NT, 2, 0, 1, 1, 2), 8),
    ((COL, UPPER, TR, 0, 2, 1, 1, 1), 8), ((COL, LOWER, NT, 2, 0, 1, 1, 2), 8),
    ((COL, LOWER, TR, 0, 2, 1, 1, 1), 8), ((ROW, UPPER, NT, 0, 2, 2, 1, 2), 10),
    ((ROW, UPPER, TR, 2, 0, 2, 1, 1), 10), ((ROW, LOWER, NT, 0, 2, 2, 1, 2), 10),
    ((ROW, LOWER, TR, 2, 0, 2, 1, 1), 10), ((COL, UPPER, NT, 2, 0, 2, 1, 2), 10),
    ((COL, UPPER, TR, 0, 2, 2, 1, 1), 10), ((COL, LOWER, NT, 2, 0, 2, 1, 2), 10),
    ((COL, LOWER, TR, 0, 2, 2, 1, 1), 10), ((ROW, UPPER, NT, 2, 0, 1, 1, 1), 13),
    ((ROW, UPPER, TR, 2, 0, 2, 2, 1), 13), ((ROW, LOWER, NT, 2, 0, 1, 1, 1), 13),
    ((ROW, LOWER, TR, 2, 0, 2, 2, 1), 13), ((COL, UPPER, NT, 2, 0, 2, 2, 1), 13),
    ((COL, UPPER, TR, 2, 0, 1, 1, 1), 13), ((COL, LOWER, NT, 2, 0, 2, 2, 1), 13),
    ((COL, LOWER, TR, 2, 0, 1, 1, 1), 13),
]


def cblas_tester_info_symm(order, info):
    if order == ROW:
        return {4: 5, 5: 4}.get(info, info)
    return info
