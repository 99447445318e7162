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

With --stream the log is the file written by config/sweep_stream.py, and what is fitted are
the constants of the estimate for the plans of the whole-K streaming kernel
(stream_estimate below, the same arithmetic as csrc/config_select.cpp: stream_plan).

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


STREAM_TILES = ("32x32", "64x32", "32x64", "64x64", "16x32", "16x64", "32x16", "64x16")


def stream_estimate(c: dict, rows: int, cols: int, K: int, a_kmajor: bool, b_kmajor: bool, bm: int, bn: int,
                    slices: int, batch: int = 1, cus: int = 256) -> float:
    """Microseconds of one plan of the whole-K streaming kernel: launch, then per pass over
    the compute units (two workgroups to a unit, one for the 64 x 64 tile) the fill of the
    ring and the workgroup's stages, each at the slower of what a workgroup pulls with its
    ring of loads in flight and its share of the stream of the large operand from memory; plus the exchange of partial tiles when several
    workgroups share a tile.  c = the "stream" object of the model file."""
    tiles = -(-rows // bm) * -(-cols // bn)
    groups = tiles * slices * batch
    resident = cus * (1 if (bm, bn) == (64, 64) else 2)  # workgroups that the LDS lets run at once
    passes = -(-groups // resident)
    active = min(groups, resident)
    stages = -(-K // 128) // slices
    wide = cols >= rows  # the large operand is B
    large_kmajor = b_kmajor if wide else a_kmajor
    large_bytes = (bn if wide else bm) * 256
    sharing = -(-rows // bm) if wide else -(-cols // bn)  # workgroups that read the same panel of it
    # (transposing reads: by the width of the side they fill, in units of 64)
    other = (0 if a_kmajor else bm / 64) + (0 if b_kmajor else bn / 64)
    per_cu = c["stage_us"][f"{bm}x{bn}"] * (1.0 + c["transposed_operand"] * other)
    small_bytes = (bm if wide else bn) * 256  # every workgroup reads its rows of the small operand, from L2
    # (the workgroups that read the same panel find only part of it in L2)
    sharing = 1.0 + (sharing - 1.0) * c["panel_sharing"]
    rate = c["bytes_per_us_kmajor" if large_kmajor else "bytes_per_us_other"]
    if not large_kmajor and (bn if wide else bm) <= 32:
        rate *= c["half_line"]  # k rows of 64 bytes: half a cache line per request
    if max(rows, cols) * K * 2 > 256 << 20:
        # the large operand does not fit the memory-side cache, which serves part of a
        # repeated call on a smaller one (not fitted: left free it soaks up other effects)
        rate *= c["beyond_cache" if large_kmajor else "beyond_cache_other"]
    l2_rate = c["bytes_per_us_l2"]
    if not (a_kmajor if wide else b_kmajor) and (bm if wide else bn) <= 32:
        l2_rate *= c["half_line"]
    from_memory = (large_bytes * (active / sharing) / rate
                   + small_bytes * active / l2_rate)
    # (workgroups that share a compute unit take turns at part of a stage)
    per_cu *= 1.0 + (-(-active // cus) - 1) * c["taking_turns"]
    return (c["launch_us"] + passes * (c["fill_us"] + stages * max(per_cu, from_memory))
            + (c["exchange_us"] + c["exchange_us_per_kb"] * slices * bm * bn * 4 / 1024 if slices > 1 else 0.0))


def stream_plans(rec: dict):
    """(tile, slices, measured us) of a sweep record."""
    for name, us in rec["t"].items():
        tile, slices = name.split("s")
        yield tile, int(slices), us


def fit_stream(records: list, start: dict) -> dict:
    """Least squares on log(estimate / measured) over every timing of the sweep."""
    import math

    from scipy.optimize import least_squares

    keys = ["launch_us", "fill_us", "exchange_us", "bytes_per_us_kmajor", "bytes_per_us_other", "bytes_per_us_l2",
            "transposed_operand", "panel_sharing", "half_line", "exchange_us_per_kb"]

    def unpack(p):
        c = {k: float(v) for k, v in zip(keys, p)}
        # (set by hand: the skinny problems of the sweep are bound by memory and say nothing
        # about turns on a compute unit; left free, beyond_cache soaks up other effects)
        c["beyond_cache"] = start["beyond_cache"]
        c["beyond_cache_other"] = start["beyond_cache_other"]
        c["taking_turns"] = start["taking_turns"]
        c["stage_us"] = {t: float(v) for t, v in zip(STREAM_TILES, p[len(keys):])}
        return c

    rows = []
    for r in records:
        for tile, slices, us in stream_plans(r):
            bm, bn = (int(x) for x in tile.split("x"))
            rows.append((r["M"], r["N"], r["K"], r["lay"][0] == "r", r["lay"][1] == "c", bm, bn, slices, us))

    def residuals(p):
        c = unpack(p)
        return [math.log(stream_estimate(c, *row[:8]) / row[8]) for row in rows]

    p0 = [start[k] for k in keys] + [start["stage_us"][t] for t in STREAM_TILES]
    res = least_squares(residuals, p0, bounds=([0.0] * len(p0), [20, 10, 30, 2e7, 2e7, 2e8, 3, 1, 1, 1] + [2.0] * len(STREAM_TILES)))
    c = unpack(res.x)
    for k in ("launch_us", "fill_us", "exchange_us"):
        c[k] = round(c[k], 2)
    for k in ("bytes_per_us_kmajor", "bytes_per_us_other", "bytes_per_us_l2"):
        c[k] = round(c[k], -4)
    c["transposed_operand"] = round(c["transposed_operand"], 3)
    c["panel_sharing"] = round(c["panel_sharing"], 3)
    c["half_line"] = round(c["half_line"], 3)
    c["exchange_us_per_kb"] = round(c["exchange_us_per_kb"], 4)
    c["stage_us"] = {t: round(v, 4) for t, v in c["stage_us"].items()}
    return c


STREAM_TIE = 1.03  # estimates this close do not tell plans apart (csrc/config_select.cpp: stream_plan)


def stream_pick(c: dict, M: int, N: int, K: int, a_kmajor: bool, b_kmajor: bool, plans: list):
    """The plan (tile, slices, ...) of `plans` that the dispatcher takes (csrc/config_select.cpp:
    stream_plan): of those whose estimate is within STREAM_TIE of the lowest, the fewest
    workgroups per tile, then the lowest estimate; an operand contiguous along M or N sits on a
    16- or 32-wide side of the tile only while it has at most 128 rows."""
    def allowed(p):
        bm, bn = (int(x) for x in p[0].split("x"))
        return not ((not a_kmajor and bm <= 32 and M > 128) or (not b_kmajor and bn <= 32 and N > 128))

    def estimate(p):
        bm, bn = (int(x) for x in p[0].split("x"))
        return stream_estimate(c, M, N, K, a_kmajor, b_kmajor, bm, bn, p[1])

    known = [(estimate(p), p) for p in plans if allowed(p)]
    lowest = min(us for us, _ in known)
    return min((x for x in known if x[0] <= lowest * STREAM_TIE), key=lambda x: (x[1][1], x[0]))[1]


def stream_regret(records: list, c: dict):
    """(geometric mean, worst) of measured time of the plan the estimate picks over the
    best measured plan, per problem of the sweep."""
    import math

    logs, worst = [], 1.0
    for r in records:
        plans = list(stream_plans(r))
        if not plans:
            continue
        a_k, b_k = r["lay"][0] == "r", r["lay"][1] == "c"
        pick = stream_pick(c, r["M"], r["N"], r["K"], a_k, b_k, plans)
        ratio = pick[2] / min(p[2] for p in plans)
        logs.append(math.log(ratio))
        worst = max(worst, ratio)
    return math.exp(sum(logs) / len(logs)), worst


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("log")
    ap.add_argument("--model", default=os.path.join(HERE, "model_gfx950.json"))
    ap.add_argument("--write", action="store_true", help="write the fitted values into --model")
    ap.add_argument("--compact", default=None, help="also write the log as a per-problem table (JSON)")
    ap.add_argument("--stream", action="store_true",
                    help="the log is a sweep_stream.py file: fit the streaming kernel's constants")
    a = ap.parse_args(argv)
    if a.stream:
        model = json.load(open(a.model))
        records = json.load(open(a.log))
        new = fit_stream(records, model["stream"])
        mean, worst = stream_regret(records, new)
        print(json.dumps(new, indent=1))
        print(f"regret of the estimate's pick over {len(records)} problems: mean {mean:.3f}, worst {worst:.2f}")
        if a.write:
            new["fitted_from"] = f"{os.path.basename(a.log)}: {sum(len(r['t']) for r in records)} timings (beyond_cache, beyond_cache_other and taking_turns set by hand)"
            model["stream"] = new
            with open(a.model, "w") as f:
                json.dump(model, f, indent=4)
                f.write("\n")
        return 0
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
