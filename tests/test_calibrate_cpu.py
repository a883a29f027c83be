"""The tool that fits the launch planner's figures (ulmblas_amd/calibrate.py),
on the CPU: timings made up from known figures through the planner's own cost
formula, with one per cent of noise, must give those figures back."""
import json
import math
import os
import re

from ulmblas_amd import calibrate


def test_fit_recovers_the_figures_behind_synthetic_timings(tmp_path, capsys):
    truth = [0.93, 2300.0, 9000.0, 0.05, 0.8]          # eff, latency, ovh0, ovh1, company
    prec, vid, name, bm, bn, bk, cs = "d", 3, "whole_128x64x16_w2x2", 128, 64, 16, 2
    rows = []
    i = 0
    for frac in (0.25, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 8.0):
        tiles = max(1, int(round(calibrate.CU * frac)))
        tm = max(1, int(round(math.sqrt(tiles * bn / bm))))
        tn = max(1, int(round(tiles / tm)))
        for k in (256, 1024, 4096):
            for rc in (0, 1):
                cycles = calibrate._unshared(prec, bm, bn, bk, cs, tm * tn, -(-k // bk), rc, truth)
                noise = 1.0 + 0.01 * math.sin(1.7 * i)
                i += 1
                rows.append({"prec": prec, "vid": vid, "name": name, "bm": bm, "bn": bn, "bk": bk, "tm": tm, "tn": tn, "k": k,
                             "rc": rc, "ms": cycles / 2.4e6 * noise})
    with open(tmp_path / "rates.jsonl", "w") as f:
        f.writelines(json.dumps(r) + "\n" for r in rows)
    for empty in ("shares.jsonl", "strips.jsonl"):
        open(tmp_path / empty, "w").close()
    calibrate.fit(str(tmp_path))
    out = capsys.readouterr().out
    mo = re.search(r"d3 \S+\s+eff ([\d.]+) latency\s+(\d+) ovh0\s+(\d+) ovh1 ([\d.]+) company ([\d.]+)\s+\| (\d+) launches, rms ([\d.]+)", out)
    assert mo, out
    eff, lat, o0, o1, comp = (float(mo.group(j)) for j in range(1, 6))
    assert int(mo.group(6)) == len(rows) and float(mo.group(7)) < 0.02, out
    assert abs(eff - truth[0]) < 0.02 and abs(lat - truth[1]) < 0.1 * truth[1], out
    # the overhead of a tile as a whole is what the timings pin (its two terms trade against each other)
    tile = lambda a, b, rc: a + b * bm * bn * 8 * (2 if rc else 1)
    for rc in (0, 1):
        assert abs(tile(o0, o1, rc) - tile(truth[2], truth[3], rc)) < 0.15 * tile(truth[2], truth[3], rc), out
    assert abs(comp - truth[4]) < 0.15, out
