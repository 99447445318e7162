#!/usr/bin/env python3
"""Races tuned-config files of the gfx950 GEMM library against each other.

Role of the reference's config/race.py (reference rocm_wmma_gemm/config/race.py:65-100
head-to-head rounds, :160-226 file-against-file, :227-268 cross-layout check): a tuning
run times each candidate once, minutes apart from its rivals, on a part whose clock
moves with load and temperature; a race times two configurations for the same problem
alternately, round by round, and the one that wins more rounds stays.

Two modes, with the reference's option names:
  --config1 A.json --config2 B.json   entries present in both files with different
        configurations are raced; the winner goes to --output; entries present in one
        file only are kept.
  --config1 A.json --cross-check      a problem with column-major C is, for the kernels,
        the transposed problem with row-major C: (M, N, K, A=a, B=b, C=col) runs exactly
        as (N, M, K, A=not b, B=not a, C=row).  Where a file holds both entries and
        their configurations differ, both are raced on both problems.

Run on a machine with an MI355X:
    python rocm_wmma_gemm_amd/config/race.py --config1 old.json --config2 new.json --output best.json
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.normpath(os.path.join(HERE, "..", "..")))
sys.path.insert(0, HERE)

from tune import LAYOUT_NAME, key_of  # noqa: E402

LAYOUT_CODE = {name: code for code, name in LAYOUT_NAME.items()}
FLIP = {"row_major": "col_major", "col_major": "row_major"}


def hook_split(cfg: dict) -> int:
    """The split argument of the library's tuner hook for a JSON configuration (inverse of
    tune.config_json): s > 1 every tile split, -s only the tail wave, -1 walk by K tile."""
    if cfg.get("stream_k"):
        return -1
    if cfg.get("tail_split", 0) > 1:
        return -int(cfg["tail_split"])
    return int(cfg.get("split_k", 1))


def variant_of(cfg: dict, variants):
    """The compiled variant a JSON configuration names, or None."""
    for v in variants:
        # (block extents rather than tiles per wave: a 16-wide side has warp_tile 0.5 in the file)
        if (v.warps_m, v.warps_n, v.block_m, v.block_n, v.block_k, v.pipeline) == (
                cfg["warps_m"], cfg["warps_n"], int(cfg["warps_m"] * cfg["warp_tile_m"] * 32),
                int(cfg["warps_n"] * cfg["warp_tile_n"] * 32), cfg.get("block_k", 64), cfg.get("pipeline", 0)):
            return v
    return None


def _ms(x):
    return "failed" if x is None else f"{x:.4f} ms"


def head_to_head(timer, key, cfg1: dict, cfg2: dict, rounds: int):
    """Times cfg1 and cfg2 on problem `key` alternately for `rounds` rounds (the order
    within a round alternates too).  timer(key, cfg) -> ms or None.  Returns (winner,
    wins1, wins2, median1, median2) with winner 1, 2, or 0 when neither ran."""
    t1, t2 = [], []
    wins1 = wins2 = 0
    for r in range(rounds):
        order = ((1, cfg1), (2, cfg2)) if r % 2 == 0 else ((2, cfg2), (1, cfg1))
        got = {}
        for which, cfg in order:
            got[which] = timer(key, cfg)
        a, b = got[1], got[2]
        if a is not None:
            t1.append(a)
        if b is not None:
            t2.append(b)
        if a is not None and (b is None or a < b):
            wins1 += 1
        elif b is not None and (a is None or b < a):
            wins2 += 1
    m1 = statistics.median(t1) if t1 else None
    m2 = statistics.median(t2) if t2 else None
    if m1 is None and m2 is None:
        return 0, wins1, wins2, m1, m2
    if wins1 != wins2:
        return (1 if wins1 > wins2 else 2), wins1, wins2, m1, m2
    if m2 is None or (m1 is not None and m1 <= m2):
        return 1, wins1, wins2, m1, m2
    return 2, wins1, wins2, m1, m2


def race_files(table1: dict, table2: dict, timer, rounds: int, log=print) -> dict:
    """Entry by entry: the configuration that wins the race; entries of one file only are
    kept as they are."""
    out = dict(table1)
    for key, e2 in table2.items():
        if key not in table1:
            out[key] = e2
            continue
        e1 = table1[key]
        if e1["config"] == e2["config"]:
            continue
        winner, w1, w2, m1, m2 = head_to_head(timer, key, e1["config"], e2["config"], rounds)
        log(f"{key}: config{winner or '?'} wins {max(w1, w2)}-{min(w1, w2)} "
            f"(medians {_ms(m1)} against {_ms(m2)})")
        if winner == 2:
            out[key] = e2
    return out


def twin_of(key):
    """The row-major-C problem that runs exactly as this column-major-C problem."""
    M, N, K, la, lb, lc = key
    if lc != "col_major":
        return None
    return (N, M, K, FLIP[lb], FLIP[la], "row_major")


def cross_check(table: dict, timer, rounds: int, log=print) -> dict:
    out = dict(table)
    for key in sorted(table):
        twin = twin_of(key)
        if twin is None or twin not in table or table[key]["config"] == table[twin]["config"]:
            continue
        for problem in (key, twin):
            own, other = out[problem]["config"], out[twin if problem == key else key]["config"]
            if own == other:
                continue
            winner, w1, w2, m1, m2 = head_to_head(timer, problem, own, other, rounds)
            log(f"{problem}: {'own' if winner != 2 else 'twin'} configuration wins "
                f"{max(w1, w2)}-{min(w1, w2)} (medians {_ms(m1)} against {_ms(m2)})")
            if winner == 2:
                out[problem] = dict(out[problem], config=dict(other))
    return out


def load_table(path: str) -> dict:
    with open(path) as f:
        return {key_of(e): e for e in json.load(f)["configurations"]}


def gpu_timer(type_name: str, reps: int, warmup: int):
    """timer(key, cfg) on the GPU, through the library's tuner hook; operands are cached
    per problem size."""
    import torch

    import rocm_wmma_gemm_amd as R
    from tune import time_candidate

    L = R.Loader()
    variants = L.variants()
    c_dtype = torch.float32 if type_name.startswith("f32") else (
        torch.bfloat16 if type_name.startswith("bf16") else torch.float16)
    in_dtype = torch.bfloat16 if type_name.endswith("bf16") else torch.float16
    cache = {}

    def timer(key, cfg):
        M, N, K, la, lb, lc = key
        v = variant_of(cfg, variants)
        if v is None:
            return None
        if cache.get("shape") != (M, N, K):
            cache.clear()
            cache["shape"] = (M, N, K)
            cache["A"] = (torch.rand(M * K, device="cuda") * 2 - 1).to(in_dtype)
            cache["B"] = (torch.rand(K * N, device="cuda") * 2 - 1).to(in_dtype)
            cache["C"] = torch.empty(M * N, dtype=c_dtype, device="cuda")
        return time_candidate(L, torch, v.index, int(cfg.get("swizzle", 1)), hook_split(cfg),
                              (int(cfg.get("touch_ahead", 0)) & 15) | (int(cfg.get("k_runs", 0)).bit_length() << 4) | ((int(cfg.get("k_group", 0)).bit_length() - 1 if cfg.get("k_group", 0) else 0) << 8), cache["C"], cache["A"], cache["B"], M, N, K,
                              LAYOUT_CODE[lc], LAYOUT_CODE[la], LAYOUT_CODE[lb], reps, warmup)

    return timer


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--config1", required=True)
    ap.add_argument("--config2", default=None)
    ap.add_argument("--cross-check", action="store_true")
    ap.add_argument("--repeats", type=int, default=5, help="rounds per race")
    ap.add_argument("--reps", type=int, default=10, help="timed launches per round and configuration")
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--output", default="gemm_config_raced.json")
    ap.add_argument("--type", default="f16_f16",
                    choices=["f16_f16", "f32_f16", "bf16_bf16", "f32_bf16"])
    a = ap.parse_args(argv)
    if not a.config2 and not a.cross_check:
        ap.error("give --config2, --cross-check, or both")
    table = load_table(a.config1)
    timer = gpu_timer(a.type, a.reps, a.warmup)
    if a.config2:
        table = race_files(table, load_table(a.config2), timer, a.repeats)
    if a.cross_check:
        table = cross_check(table, timer, a.repeats)
    with open(a.output, "w") as f:
        json.dump({"configurations": [table[k] for k in sorted(table)]}, f, indent=4)
    print(f"wrote {a.output}: {len(table)} entries")
    return 0


if __name__ == "__main__":
    sys.exit(main())
