#!/usr/bin/env python3
"""Fits the constants of the dispatcher's time estimate to a tuner log.

    python tune.py --search exhaustive --shapes ... --log sweep.log --output /tmp/x.json
    python fit_model.py sweep.log [--model model_gfx950.json] [--write]

The dispatcher (csrc/config_select.cpp: model_plan) prices a plan for a shape without a
tuned entry as  launch + passes over the compute units x (K tiles x step_us + item_us)  plus
what a split costs.  step_us (per pipeline and tile) and item_us (per pipeline) are what
this script measures: over every whole-tile, unsplit timing of the log it solves, per
pipeline, the least-squares problem
    t_us - launch_us = passes * k_tiles * step_us[tile] + passes * item_us
and prints (or writes into the model file, which config/generate_config.py turns into
constants of csrc/config_generated.hpp) the fitted values beside the old ones.  The other
constants of the file (launch, reduce, bytes per microsecond of partial sums and copies)
are kept.  compact() turns a log into the small per-problem table that the regret test of
tests/test_host.py holds as a fixture.

No counterpart in the reference, whose dispatcher has no model: it takes the nearest tuned
shape (reference rocm_wmma_gemm/config/generate_config.py:174-234).
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LINE = re.compile(r"^(\d+),(\d+),(\d+) ([rc]{3}) (\S+) p(\d+) (\d+)x(\d+)x(\d+) w(\d+)x(\d+) sw(-?\d+) sk(-?\d+) "
                  r"touch(\d+) (compiled|jit) ([\d.]+) ms")


def parse(lines):
    """[(M, N, K, layout 'abc', type, pipeline, bm, bn, bk, wm, wn, swizzle, split, touch, ms)]"""
    out = []
    for line in lines:
        m = LINE.match(line)
        if m:
            g = m.groups()
            out.append((int(g[0]), int(g[1]), int(g[2]), g[3], g[4]) + tuple(int(x) for x in g[5:14])
                       + (float(g[15]),))
    return out


def candidate_key(pipe, bm, bn, bk, wm, wn, sw, sk, touch) -> str:
    return f"p{pipe} {bm}x{bn}x{bk} w{wm}x{wn} sw{sw} sk{sk} t{touch}"


def compact(records) -> dict:
    """{"M,N,K abc type": {candidate: ms}}: the log as a table per problem."""
    table: dict = {}
    for (M, N, K, lay, typ, pipe, bm, bn, bk, wm, wn, sw, sk, touch, ms) in records:
        table.setdefault(f"{M},{N},{K} {lay} {typ}", {})[candidate_key(pipe, bm, bn, bk, wm, wn, sw, sk, touch)] = ms
    return table


def expand(table: dict):
    """The records of a compacted log (inverse of compact)."""
    key = re.compile(r"^p(\d+) (\d+)x(\d+)x(\d+) w(\d+)x(\d+) sw(-?\d+) sk(-?\d+) t(\d+)$")
    out = []
    for problem, cands in table.items():
        shape, lay, typ = problem.split(" ")
        M, N, K = (int(x) for x in shape.split(","))
        for cand, ms in cands.items():
            out.append((M, N, K, lay, typ) + tuple(int(x) for x in key.match(cand).groups()) + (float(ms),))
    return out


def fit(records, model: dict) -> dict:
    """New step_us / item_us from the whole-tile, unsplit timings of pipelines in the model."""
    import numpy as np

    cus, launch = model["compute_units"], model["launch_us"]
    best: dict = {}  # (problem, pipeline, tile) -> best ms over band heights
    for (M, N, K, lay, typ, pipe, bm, bn, bk, wm, wn, sw, sk, touch, ms) in records:
        rows, cols = (M, N) if lay[2] == "r" else (N, M)
        if str(pipe) not in model["step_us"] or sk != 1 or touch != 0 or bk != 64:
            continue
        if rows % bm or cols % bn or K % 64:
            continue
        key = ((M, N, K, lay, typ), pipe, f"{bm}x{bn}")
        best[key] = min(best.get(key, ms), ms)
    out = {"step_us": {}, "item_us": {}, "samples": {}}
    for pipe in sorted(model["step_us"]):
        tiles = sorted({t for (_, p, t) in best if str(p) == pipe})
        if not tiles:
            continue
        rows_a, rhs = [], []
        for ((M, N, K, lay, _), p, tile), ms in best.items():
            if str(p) != pipe:
                continue
            bm, bn = (int(x) for x in tile.split("x"))
            rws, cls = (M, N) if lay[2] == "r" else (N, M)
            passes = -(-(rws // bm) * (cls // bn) // cus)
            row = [0.0] * (len(tiles) + 1)
            row[tiles.index(tile)] = passes * (K // 64)
            row[-1] = passes
            rows_a.append(row)
            rhs.append(ms * 1e3 - launch)
        sol, *_ = np.linalg.lstsq(np.array(rows_a), np.array(rhs), rcond=None)
        out["step_us"][pipe] = {t: round(float(s), 3) for t, s in zip(tiles, sol[:-1])}
        out["item_us"][pipe] = round(float(max(sol[-1], 0.0)), 2)
        out["samples"][pipe] = len(rhs)
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("log")
    ap.add_argument("--model", default=os.path.join(HERE, "model_gfx950.json"))
    ap.add_argument("--write", action="store_true", help="write the fitted values into --model")
    ap.add_argument("--compact", default=None, help="also write the log as a per-problem table (JSON)")
    a = ap.parse_args(argv)
    records = parse(open(a.log))
    model = json.load(open(a.model))
    new = fit(records, model)
    for pipe, tiles in new["step_us"].items():
        for tile, us in tiles.items():
            print(f"pipeline {pipe} tile {tile}: step_us {model['step_us'].get(pipe, {}).get(tile)} -> {us} "
                  f"({new['samples'][pipe]} timings)")
        print(f"pipeline {pipe}: item_us {model['item_us'].get(pipe)} -> {new['item_us'][pipe]}")
    if a.write:
        for pipe, tiles in new["step_us"].items():
            model["step_us"].setdefault(pipe, {}).update(tiles)
            model["item_us"][pipe] = new["item_us"][pipe]
        model["fitted_from"] = f"{os.path.basename(a.log)}: {len(records)} timings"
        with open(a.model, "w") as f:
            json.dump(model, f, indent=4)
            f.write("\n")
    if a.compact:
        with open(a.compact, "w") as f:
            json.dump(compact(records), f, separators=(",", ":"), sort_keys=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
