"""Where the launch planner's figures come from (the Variant tables of
csrc/gemm_host.hip): timings of forced launches on an MI355X, and least-squares
fits of the planner's own cost formulas to them.

    python -m ulmblas_amd.calibrate collect OUTDIR     (needs the GPU; ~1 minute)
    python -m ulmblas_amd.calibrate fit OUTDIR         (prints the table rows)

collect times, through the C timing loop the benchmark uses,
  rates   every whole-tile variant on exact multiples of its tile: a quarter of
          a round of tiles to eight rounds, k = 256, 1024, 4096, beta = 0 and
          != 0, tiles never shared;
  shares  the variants that share tiles and take tiles past the edge of C, one
          launch over all of C, unshared and with 2, 4, 8 pieces a tile;
  strips  every whole-tile variant on shapes that are no multiple of its tile,
          whole tiles with the strips beside them and the whole tiles alone.
fit reproduces estimate_cycles() of gemm_host.hip and fits, per variant,
  eff, latency, ovh0, ovh1, company            to `rates`,
  edge, share_slab, share_base, share_link, share_hidden   to `shares`,
and prints what the strips cost in units of one walk over k (`strips`).
"""
import collections
import json
import math
import os
import re
import sys

CU = 256


def _setup():
    import torch
    ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if ROOT not in sys.path:
        sys.path.insert(0, ROOT)
    import bench
    from ulmblas_amd import blas
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    count = 8192 * 8192
    bufs = {p: [torch.empty(count, dtype=torch.float64 if p == "d" else torch.float32, device="cuda").uniform_(-1, 1)
                for _ in range(3)] for p in "ds"}
    for p in "ds":      # the shader clock needs some tens of milliseconds of load
        bench.time_gemm(p, "N", "N", 4096, 4096, 4096, 1.0, 0.0, [bench.operand_set(*bufs[p])], 4096, 4096, 4096,
                        5, 20, stream)

    def timed(prec, m, n, k, rc, lda, ldb, ldc):
        assert max(lda * k, ldb * n, ldc * n) <= count, "operands larger than the buffers"
        reps = int(min(60, max(3, 2.5e11 // (2.0 * m * n * k))))
        ptrs = [bench.operand_set(*bufs[prec])]
        return min(bench.time_gemm(prec, "N", "N", m, n, k, 1.0, 0.5 if rc else 0.0, ptrs, lda, ldb, ldc,
                                   max(2, reps // 2), reps, stream) for _ in range(2))

    def force(prec, vid, whole_c, pieces):
        blas.set_variant(prec, vid)
        blas.test_control(blas.TEST_WHOLE_C, whole_c)
        blas.test_control(blas.TEST_SHARED_PIECES, pieces)

    def restore():
        for p in "ds":
            blas.set_variant(p, 0)
        blas.test_control(blas.TEST_WHOLE_C, -1)
        blas.test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT)

    return blas, timed, force, restore


def _whole_variants(blas):
    for prec in "ds":
        for vid, name in enumerate(blas.variant_names(prec), 1):
            mo = re.match(r"whole_(\d+)x(\d+)x(\d+)_w(\d+)x(\d+)", name)
            if mo:
                yield prec, vid, name, int(mo.group(1)), int(mo.group(2)), int(mo.group(3))


def collect(outdir):
    blas, timed, force, restore = _setup()
    os.makedirs(outdir, exist_ok=True)
    try:
        with open(os.path.join(outdir, "rates.jsonl"), "w") as f:
            for prec, vid, name, bm, bn, bk in _whole_variants(blas):
                for frac in (0.25, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 8.0):
                    tiles = max(1, int(round(CU * frac)))
                    tm = max(1, int(round(math.sqrt(tiles * bn / bm))))
                    tn = max(1, int(round(tiles / tm)))
                    m, n = tm * bm, tn * bn
                    for k in (256, 1024, 4096):
                        if max(m * k, k * n, m * n) > 8192 * 8192 or max(m, n) > 65536:
                            continue
                        for rc in (0, 1):
                            force(prec, vid, 0, 0)
                            plan = blas.plan(prec, m, n, k, rc, m, k)
                            if plan[0] != vid or plan[2] != 0:
                                continue
                            f.write(json.dumps({"prec": prec, "vid": vid, "name": name, "bm": bm, "bn": bn, "bk": bk, "tm": tm,
                                                "tn": tn, "k": k, "rc": rc, "ms": timed(prec, m, n, k, rc, m, k, m)}) + "\n")
        sharing = {("d", 6): range(400, 1900, 100), ("d", 2): (900, 1100, 1500, 1900, 2100, 2400, 2900, 3100, 3300, 3600),
                   ("d", 1): (1500, 1900, 2300, 2500, 2900, 3300, 3600, 3800, 4400, 5000),
                   ("s", 4): (500, 700, 900, 1100, 1400, 1800), ("s", 2): (1500, 1900, 2500, 2900, 3300, 3800),
                   ("s", 1): (2000, 2500, 3000, 3500, 4100, 5100)}
        with open(os.path.join(outdir, "shares.jsonl"), "w") as f:
            for prec, vid, name, bm, bn, bk in _whole_variants(blas):
                for n in sharing.get((prec, vid), ()):
                    for k in (n, (4 if bm * bn <= 4096 else 2) * n):
                        for rc in (0, 1):
                            row = {"prec": prec, "vid": vid, "bm": bm, "bn": bn, "m": n, "n": n, "k": k, "rc": rc, "t": {}}
                            for pieces in (0, -2, -4, -8):
                                force(prec, vid, 1, pieces)
                                plan = blas.plan(prec, n, n, k, rc, n, k)
                                key = "%d,%d,%d" % plan[1:]
                                if plan[0] == vid and key not in row["t"]:
                                    row["t"][key] = timed(prec, n, n, k, rc, n, k, n)
                            f.write(json.dumps(row) + "\n")
        shapes = [(n, n, n) for n in range(300, 4001, 100)] + [(6658, 2315, 512), (5237, 1161, 3390), (3101, 3715, 3287),
                                                               (5000, 3000, 7000), (1464, 3000, 1536), (4000, 2000, 4000),
                                                               (6000, 1000, 300), (700, 6000, 2000)]
        with open(os.path.join(outdir, "strips.jsonl"), "w") as f:
            for prec, vid, name, bm, bn, bk in _whole_variants(blas):
                for m, n, k in shapes:
                    mw, nw = m // bm * bm, n // bn * bn
                    if mw == 0 or nw == 0 or (mw == m and nw == n):
                        continue
                    force(prec, vid, 0, 0)
                    f.write(json.dumps({"prec": prec, "vid": vid, "bm": bm, "bn": bn, "m": m, "n": n, "k": k,
                                        "both": timed(prec, m, n, k, 1, m, k, m),
                                        "main": timed(prec, mw, nw, k, 1, m, k, m)}) + "\n")
        blas.device_status()
    finally:
        restore()


def _round(prec, bm, bn, bk, cs, slabs, rc, c, eff, lat, o0, o1, comp, loop=1.0):
    size = 8 if prec == "d" else 4
    slab_mfma = 2.0 * bm * bn * bk / (128.0 if size == 8 else 256.0)
    ovh = o0 + o1 * bm * bn * size * (2 if rc else 1)
    return loop * slabs * max(c * slab_mfma / eff, lat) + (ovh if c == 1 else comp * ovh)


def _unshared(prec, bm, bn, bk, cs, wgs, slabs, rc, base, loop=1.0):
    per_cu = (wgs + CU - 1) // CU
    full, rem = per_cu // cs, per_cu % cs
    return full * _round(prec, bm, bn, bk, cs, slabs, rc, cs, *base, loop) + \
        (_round(prec, bm, bn, bk, cs, slabs, rc, rem, *base, loop) if rem else 0.0)


def fit(outdir, clock_ghz=2.4):
    import numpy as np
    from scipy.optimize import least_squares
    ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = open(os.path.join(ROOT, "ulmblas_amd", "csrc", "gemm_host.hip")).read()
    # workgroups per CU of every variant, from the tables themselves
    cs_of = {}
    for mo in re.finditer(r"_VARIANT\((double|float), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+),", src):
        cs_of[("d" if mo.group(1) == "double" else "s", int(mo.group(2)), int(mo.group(3)), int(mo.group(4)),
               int(mo.group(5)) * int(mo.group(6)))] = int(mo.group(7))
    rows = [json.loads(l) for l in open(os.path.join(outdir, "rates.jsonl"))]
    by = collections.defaultdict(list)
    for r in rows:
        by[(r["prec"], r["vid"])].append(r)
    base = {}
    for key, rs in sorted(by.items()):
        r0 = rs[0]
        waves = [int(x) for x in re.search(r"_w(\d+)x(\d+)", r0["name"]).groups()]
        cs = cs_of[(key[0], r0["bm"], r0["bn"], r0["bk"], waves[0] * waves[1])]

        def resid(p, rs=rs, cs=cs):
            return [math.log(max(_unshared(r["prec"], r["bm"], r["bn"], r["bk"], cs, r["tm"] * r["tn"],
                                           -(-r["k"] // r["bk"]), r["rc"], p), 1.0) / (clock_ghz * 1e6) / r["ms"]) for r in rs]
        best = None
        for e0 in (0.7, 0.85, 0.95):
            for l0 in (1000.0, 3000.0, 6000.0):
                sol = least_squares(resid, [e0, l0, 6000.0, 0.02, 0.5], bounds=([0.3, 200.0, 0.0, 0.0, 0.0], [1.0, 20000.0, 60000.0, 1.0, 1.0]))
                if best is None or sol.cost < best.cost:
                    best = sol
        e = np.array(resid(best.x))
        base[key] = (list(best.x), cs, r0)
        print("%s%d %-24s eff %.3f latency %5.0f ovh0 %5.0f ovh1 %.4f company %.2f   | %d launches, rms %.3f, max %.3f"
              % (key[0], key[1], r0["name"], *best.x, len(e), math.sqrt((e * e).mean()), np.abs(e).max()))
    rows = [json.loads(l) for l in open(os.path.join(outdir, "shares.jsonl"))]
    by = collections.defaultdict(list)
    for r in rows:
        by[(r["prec"], r["vid"])].append(r)
    for key, rs in sorted(by.items()):
        b, cs, r0 = base[key]
        bm, bn, bk = r0["bm"], r0["bn"], r0["bk"]
        size = 8 if key[0] == "d" else 4
        slab_mfma = 2.0 * bm * bn * bk / (128.0 if size == 8 else 256.0)

        def est(r, groups, stiles, p):
            edge, sf, sb, link, hidden = p
            wgs, slabs = -(-r["m"] // bm) * -(-r["n"] // bn), -(-r["k"] // bk)
            if groups == 0:
                return _unshared(key[0], bm, bn, bk, cs, wgs, slabs, r["rc"], b, edge)
            slots = CU * cs
            on_cu, run, pieces = (groups + CU - 1) // CU, stiles * slabs / groups, (groups + stiles - 1) // stiles
            fold = 11000.0 + sb + (pieces - 1) * link * (1.0 if wgs < slots else hidden)
            return (wgs // slots) * _round(key[0], bm, bn, bk, cs, slabs, r["rc"], cs, *b, edge) + \
                edge * sf * run * max(on_cu * slab_mfma / b[0], b[1]) + fold

        def resid(p):
            return [math.log(est(r, *[int(x) for x in k.split(",")[1:]], p) / (clock_ghz * 1e6) / t)
                    for r in rs for k, t in r["t"].items()]
        tile_bytes = bm * bn * size
        sol = least_squares(resid, [1.05, 1.06, 5000, 0.25 * tile_bytes, 0.7],
                            bounds=([0.95, 0.95, 0, 0, 0.3], [1.3, 1.4, 60000, 2.0 * tile_bytes, 1.0]))
        e = np.array(resid(sol.x))
        print("%s%d edge %.3f share_slab %.3f share_base %5.0f share_link %6.0f share_hidden %.2f   | %d launches, rms %.3f, "
              "max %.3f" % (key[0], key[1], *sol.x, len(e), math.sqrt((e * e).mean()), np.abs(e).max()))
    rows = [json.loads(l) for l in open(os.path.join(outdir, "strips.jsonl"))]
    by = collections.defaultdict(list)
    for r in rows:
        _, cs, _ = base[(r["prec"], r["vid"])]
        tiles, slots = (r["m"] // r["bm"]) * (r["n"] // r["bn"]), CU * cs
        fill = (tiles % slots) / slots if tiles % slots else 1.0
        walk = 3000.0 * -(-r["k"] // 16) / (clock_ghz * 1e6)
        by[(r["prec"], "alone on its CU" if cs == 1 else "with company", "fill > 0.85" if fill > 0.85 else
            "fill > 0.5" if fill > 0.5 else "fill <= 0.5")].append((r["both"] - r["main"]) / walk)
    for key, v in sorted(by.items()):
        print("strips beside %s tiles %s, %s: median %.2f walks (%d launches)" % (*key, float(np.median(v)), len(v)))


if __name__ == "__main__":
    if len(sys.argv) != 3 or sys.argv[1] not in ("collect", "fit"):
        sys.exit(__doc__)
    (collect if sys.argv[1] == "collect" else fit)(sys.argv[2])
