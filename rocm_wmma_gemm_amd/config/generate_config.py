#!/usr/bin/env python3
"""Build-time step: tuned-config JSON -> csrc/config_generated.hpp.

Reads gemm_config_<arch>_f16.json (type group 0: 16-bit C) and, if present,
gemm_config_<arch>_f32.json (type group 1: fp32 C), checks every entry against the
compiled tile variants listed in csrc/variants.def, and writes the table that
config_select.cpp searches at run time.

File naming, the two type groups and the JSON schema ("configurations": [{"range":
{M,N,K}, "layout": {A,B,C}, "config": {...}}]) follow the reference
(rocm_wmma_gemm/CMakeLists.txt:16-33, config/generate_config.py:9-36,
config/gemm_config_gfx1100_f16.json:1-22).  The "config" object keeps the reference's
keys (warps_m, warps_n, warp_tile_m, warp_tile_n, swizzle, bits) with MFMA meaning
(tiles are 32x32, waves are 64 wide) and adds block_k, pipeline, split_k, tail_split, stream_k
and touch_ahead.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.normpath(os.path.join(HERE, "..", "csrc"))
MFMA_TILE = 32
LAYOUT_CODE = {"row_major": 0, "col_major": 1}

VARIANT_RE = re.compile(
    r"^\s*RWG_VARIANT\(\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*\)")


def read_variants(path: str) -> list[dict]:
    out = []
    with open(path) as f:
        for line in f:
            m = VARIANT_RE.match(line)
            if m:
                idx, bm, bn, bk, wm, wn, pipe = map(int, m.groups())
                if idx != len(out):
                    raise ValueError(f"{path}: variant indices must be dense, got {idx}")
                out.append(dict(index=idx, block_m=bm, block_n=bn, block_k=bk, warps_m=wm,
                                warps_n=wn, pipeline=pipe))
    if not out:
        raise ValueError(f"{path}: no variants found")
    return out


def variant_of(cfg: dict, variants: list[dict]) -> int:
    """Index of the compiled variant a JSON "config" object names."""
    # (warp_tile 0.5: a 16-wide side of the whole-K streaming kernel's tile)
    bm = int(cfg["warps_m"] * cfg["warp_tile_m"] * MFMA_TILE)
    bn = int(cfg["warps_n"] * cfg["warp_tile_n"] * MFMA_TILE)
    bk = cfg.get("block_k", 64)
    pipe = cfg.get("pipeline", 0)
    for v in variants:
        if (v["block_m"], v["block_n"], v["block_k"], v["warps_m"], v["warps_n"], v["pipeline"]) == (
                bm, bn, bk, cfg["warps_m"], cfg["warps_n"], pipe):
            return v["index"]
    raise ValueError(f"no compiled variant for config {cfg} (block {bm}x{bn}x{bk}, pipeline {pipe})")


def load_entries(path: str, type_group: int, variants: list[dict]) -> list[tuple]:
    with open(path) as f:
        doc = json.load(f)
    rows = []
    for conf in doc["configurations"]:
        r, lay, cfg = conf["range"], conf["layout"], conf["config"]
        rows.append((int(r["M"]), int(r["N"]), int(r["K"]), type_group,
                     LAYOUT_CODE[lay["A"]], LAYOUT_CODE[lay["B"]], LAYOUT_CODE[lay["C"]],
                     variant_of(cfg, variants), int(cfg.get("swizzle", 4)),
                     split_field(cfg), touch_field(cfg)))
    return rows


def touch_field(cfg: dict) -> int:
    """The plan's fourth field: bits 0-3 the distance of the line touches ("touch_ahead"),
    bits 4-7 the code of the K run length ("k_runs": 0 = K tiles in order, else a power of two
    up to 16, coded as log2 + 1), bits 8-9 the code of the K group ("k_group": 0, 2, 4 or 8,
    coded as log2)."""
    run = int(cfg.get("k_runs", 0))
    if run < 0 or run > 16 or (run & (run - 1)):
        raise ValueError(f"k_runs must be 0 or a power of two up to 16, not {run}")
    group = int(cfg.get("k_group", 0))
    if group not in (0, 2, 4, 8):
        raise ValueError(f"k_group must be 0, 2, 4 or 8, not {group}")
    return (int(cfg.get("touch_ahead", 0)) & 15) | (run.bit_length() << 4) | ((group.bit_length() - 1 if group else 0) << 8)


def split_field(cfg: dict) -> int:
    """The plan's split field: K slices for every tile ("split_k"), or minus the number of
    slices for the tiles of the last, partial wave only ("tail_split"), or -1 for the
    persistent kernel's walk by K tile ("stream_k": 1); 1 = no split."""
    if int(cfg.get("stream_k", 0)):
        return -1
    tail = int(cfg.get("tail_split", 0))
    return -tail if tail > 1 else int(cfg.get("split_k", 1))


def build_table(f16_json: str, f32_json: str | None, variants: list[dict]) -> list[tuple]:
    rows = load_entries(f16_json, 0, variants)
    if f32_json and os.path.exists(f32_json):
        rows += load_entries(f32_json, 1, variants)
    seen = {}
    for row in rows:  # a later duplicate key replaces an earlier one
        seen[row[:7]] = row
    return sorted(seen.values())


def load_model(path: str) -> dict:
    with open(path) as f:
        m = json.load(f)
    for key in ("compute_units", "launch_us", "reduce_us", "plane_bytes_per_us", "tile_bytes_per_us",
                "copy_bytes_per_us", "operand_bytes_per_us", "step_us", "item_us", "stream"):
        if key not in m:
            raise ValueError(f"{path}: missing {key}")
    return m


def render_model(m: dict) -> list[str]:
    steps = []
    for pipe, tiles in sorted(m["step_us"].items()):
        for tile, us in sorted(tiles.items()):
            bm, bn = (int(x) for x in tile.split("x"))
            steps.append(f"    {{{int(pipe)}, {bm}, {bn}, {float(us)!r}, {float(m['item_us'][pipe])!r}}},")
    st = m["stream"]
    stream = ["constexpr model_stream model_stream_constants = {"
              + ", ".join(repr(float(st[k])) for k in ("launch_us", "fill_us", "exchange_us", "exchange_us_per_kb",
                                                        "bytes_per_us_kmajor", "bytes_per_us_other", "bytes_per_us_l2",
                                                        "transposed_operand", "panel_sharing", "half_line",
                                                        "beyond_cache", "beyond_cache_other", "taking_turns"))
              + ", {" + ", ".join(repr(float(st["stage_us"][t])) for t in ("32x32", "64x32", "32x64", "64x64", "16x32", "16x64", "32x16", "64x16")) + "}};"]
    return ([f"constexpr int model_compute_units = {int(m['compute_units'])};"]
            + [f"constexpr double model_{k} = {float(m[k])!r};" for k in
               ("launch_us", "reduce_us", "plane_bytes_per_us", "tile_bytes_per_us", "copy_bytes_per_us",
                "operand_bytes_per_us")]
            + [f"constexpr int model_step_count = {len(steps)};",
               f"constexpr model_step model_steps[{max(len(steps), 1)}] = {{"]
            + (steps or ["    {0, 0, 0, 0.0, 0.0},"]) + ["};"] + stream)


def render(rows: list[tuple], sources: list[str], model: dict | None = None) -> str:
    lines = [
        "// Generated by config/generate_config.py -- do not edit.",
        "// Sources: " + ", ".join(os.path.basename(s) for s in sources),
        "#ifndef ROCM_WMMA_GEMM_CONFIG_GENERATED_HPP",
        "#define ROCM_WMMA_GEMM_CONFIG_GENERATED_HPP",
        '#include "config_select.hpp"',
        "namespace rocm_wmma_gemm { namespace host { namespace generated {",
        f"constexpr size_t entry_count = {len(rows)};",
        f"constexpr tuned_entry entries[{max(len(rows), 1)}] = {{",
    ]
    if not rows:
        lines.append("    {0, 0, 0, 0, 0, 0, 0, {0, 1, 1, 0}},")
    for m, n, k, tg, la, lb, lc, var, swz, sk, touch in rows:
        lines.append(f"    {{{m}, {n}, {k}, {tg}, {la}, {lb}, {lc}, {{{var}, {swz}, {sk}, {touch}}}}},")
    lines += ["};"]
    lines += render_model(model if model is not None else load_model(os.path.join(HERE, "model_gfx950.json")))
    lines += ["}}} // namespace rocm_wmma_gemm::host::generated", "#endif", ""]
    return "\n".join(lines)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--arch", default="gfx950")
    ap.add_argument("--f16-config", default=None)
    ap.add_argument("--f32-config", default=None)
    ap.add_argument("--variants", default=os.path.join(CSRC, "variants.def"))
    ap.add_argument("--model", default=None, help="constants of the dispatcher's time estimate (model_<arch>.json)")
    ap.add_argument("output", nargs="?", default=os.path.join(CSRC, "config_generated.hpp"))
    a = ap.parse_args(argv)
    f16 = a.f16_config or os.path.join(HERE, f"gemm_config_{a.arch}_f16.json")
    if not os.path.exists(f16):  # legacy un-suffixed name (reference CMakeLists.txt:20-22)
        legacy = os.path.join(HERE, f"gemm_config_{a.arch}.json")
        f16 = legacy if os.path.exists(legacy) else f16
    f32 = a.f32_config or os.path.join(HERE, f"gemm_config_{a.arch}_f32.json")
    variants = read_variants(a.variants)
    rows = build_table(f16, f32, variants)
    model_path = a.model or os.path.join(HERE, f"model_{a.arch}.json")
    text = render(rows, [f16] + ([f32] if os.path.exists(f32) else []) + [model_path], load_model(model_path))
    old = open(a.output).read() if os.path.exists(a.output) else None
    if old != text:
        with open(a.output, "w") as f:
            f.write(text)
    print(f"{a.output}: {len(rows)} tuned entries over {len(variants)} variants")
    return 0


if __name__ == "__main__":
    sys.exit(main())
