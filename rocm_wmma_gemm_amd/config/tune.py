#!/usr/bin/env python3
"""Offline tuner for the gfx950 GEMM library: times every compiled tile variant
(x tile-map band height x split-K factor) on each requested shape, layout triple and
type group through the library's tuner hook, and writes the winners as
gemm_config_gfx950_f16.json / _f32.json in the schema the config generator reads.

Role of the reference's config/tune.py + config/tuner.cpp (reference
rocm_wmma_gemm/config/tune.py:692-765,848-933; config/tuner.cpp:398-521): produce the
tuned-config JSON for one architecture.  The reference searches a large space of
just-in-time compiled kernels with a GOMEA evolutionary search; this library ships a
short list of ahead-of-time compiled variants, so the search here is exhaustive.
What is kept from the reference's tool: the JSON schema (tune.py:905-913), one entry
per (M, N, K, layout triple), `--input` to resume from / extend an existing file
with untouched entries preserved (tune.py:772-822), `--overwrite` to re-tune entries
that already exist (tune.py:874), and timing by GPU events around the enqueue.

Run on a machine with an MI355X:
    python rocm_wmma_gemm_amd/config/tune.py --type-group f16 --shapes 4096,4096,4096:8192,8192,8192
"""
from __future__ import annotations

import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.normpath(os.path.join(HERE, "..", "..")))

LAYOUT_NAME = {0: "row_major", 1: "col_major"}
CUS = 256  # compute units of an MI355X
DEFAULT_SHAPES = [
    # the reference's tuned sizes (gemm_config_gfx1100_f16.json)
    (1024, 1024, 1024), (2048, 2048, 2048), (2048, 5120, 5120), (4096, 2048, 64),
    (4096, 4096, 1024), (4096, 4096, 4096), (4096, 4096, 16384), (4096, 5120, 5120),
    (4096, 16384, 4096), (8192, 4096, 128), (8192, 8192, 1024), (8192, 8192, 8192),
    (32768, 4096, 4096), (65536, 2048, 2048),
    # projection, decode-like, ragged and long-K shapes
    (8192, 4096, 2048), (4096, 14336, 4096), (16, 8192, 8192), (64, 8192, 8192),
    (128, 8192, 8192), (4095, 5121, 3001), (1000, 1000, 1000), (1024, 1024, 65536),
    # small shapes of the parity suite
    (128, 128, 128), (256, 256, 256), (512, 512, 512),
    # square sizes whose tile count does not divide by the CU count
    (1536, 1536, 1536), (3072, 3072, 3072), (6144, 6144, 6144),
    # transformer projection shapes (hidden 4096 / 8192, feed-forward 11008 / 14336 / 28672)
    (4096, 11008, 4096), (4096, 4096, 11008), (8192, 8192, 4096), (4096, 12288, 4096),
    (8192, 1024, 8192), (4096, 4096, 14336), (2048, 8192, 2048), (12288, 4096, 4096),
    (5120, 5120, 5120), (8192, 3584, 7168), (7168, 7168, 7168), (8192, 28672, 8192),
    (8192, 8192, 28672),
]


def parse_shapes(text: str):
    out = []
    for tok in text.split(":"):
        m, n, k = (int(x) for x in tok.split(","))
        out.append((m, n, k))
    return out


def key_of(entry: dict):
    r, lay = entry["range"], entry["layout"]
    return (r["M"], r["N"], r["K"], lay["A"], lay["B"], lay["C"])


def config_json(v, swizzle: int, split_k: int) -> dict:
    """split_k as the library's hook takes it: s > 1 every tile split, -s (s > 1) only the
    tail wave, -1 the persistent kernel's walk by K tile."""
    cfg = {"warps_m": v.warps_m, "warps_n": v.warps_n, "warp_tile_m": v.warp_tile_m,
           "warp_tile_n": v.warp_tile_n, "swizzle": swizzle, "bits": 128,
           "block_k": v.block_k, "pipeline": v.pipeline, "split_k": max(split_k, 1)}
    if split_k < -1:
        cfg["tail_split"] = -split_k
    if split_k == -1:
        cfg["stream_k"] = 1
    return cfg


def candidates(variants, M, N, K, lc):
    """(variant, swizzle, split_k) triples worth timing for this problem."""
    rows, cols = (M, N) if lc == 0 else (N, M)
    out = []
    for v in variants:
        tiles = -(-rows // v.block_m) * -(-cols // v.block_n)
        k_steps = -(-K // v.block_k)
        # a tile much larger than the problem only wastes work
        if (v.block_m >= 192 and rows < 192) or (v.block_n >= 192 and cols < 192):
            continue
        # band height of the tile walk; negative: bands of tile columns instead of rows
        swizzles = [1] if tiles <= 8 else [4, 8, 16, -4, -8]
        splits = [1]
        if tiles < 256 and k_steps >= 16:
            for s in (2, 4, 8, 16, 32):
                if tiles * s <= 2048 and k_steps // s >= 4:
                    splits.append(s)
        # more tiles than CUs and a thin last wave: split only that wave (negative = tail)
        tail = tiles % CUS
        if tiles > CUS and 0 < tail <= CUS * 3 // 4 and k_steps >= 16:
            for s in (2, 3, 4, 6, 8):
                if tail * s <= CUS * 5 // 4 and k_steps // s >= 4:
                    splits.append(-s)
        # the persistent kernel can also give every workgroup the same number of K tiles
        if v.pipeline == 5 and tiles % CUS != 0 and tiles * k_steps >= 4 * CUS:
            splits.append(-1)
        for sw in swizzles:
            for sk in splits:
                out.append((v, sw, sk))
    return out


def time_candidate(L, torch, v, sw, sk, C, A, B, M, N, K, lc, la, lb, reps, warmup):
    for _ in range(warmup):
        rc = L.run_variant(v.index, sw, sk, C, A, B, M, N, K, lc, la, lb)
        if rc != 0:
            return None
    torch.cuda.synchronize()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        start[i].record()
        L.run_variant(v.index, sw, sk, C, A, B, M, N, K, lc, la, lb)
        stop[i].record()
    torch.cuda.synchronize()
    ms = sorted(s.elapsed_time(e) for s, e in zip(start, stop))
    return ms[len(ms) // 2]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--type-group", choices=["f16", "f32"], default="f16",
                    help="f16: 16-bit C (f16_f16 kernels are timed); f32: fp32 C (f32_f16 kernels)")
    ap.add_argument("--shapes", default=None, help="M,N,K:M,N,K:... (default: built-in list)")
    ap.add_argument("--layouts", default="all", help="comma list of A,B,C triples like rcr, or 'all'")
    ap.add_argument("--input", default=None, help="existing JSON to extend")
    ap.add_argument("--output", default=None)
    ap.add_argument("--overwrite", action="store_true", help="re-tune entries present in --input")
    ap.add_argument("--reps", type=int, default=15)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--log", default=None, help="write every timing to this file")
    a = ap.parse_args(argv)

    import torch

    import rocm_wmma_gemm_amd as R

    L = R.Loader()
    variants = L.variants()
    out_path = a.output or os.path.join(HERE, f"gemm_config_{L.arch}_{a.type_group}.json")
    in_path = a.input or (out_path if os.path.exists(out_path) else None)
    table = {}
    if in_path and os.path.exists(in_path):
        for e in json.load(open(in_path))["configurations"]:
            table[key_of(e)] = e
    shapes = parse_shapes(a.shapes) if a.shapes else DEFAULT_SHAPES
    if a.layouts == "all":
        layouts = [(la, lb, lc) for la in (0, 1) for lb in (0, 1) for lc in (0, 1)]
    else:
        layouts = [tuple("rc".index(ch) for ch in tok) for tok in a.layouts.split(",")]
    c_dtype = torch.float16 if a.type_group == "f16" else torch.float32
    log = open(a.log, "w") if a.log else None

    for (M, N, K) in shapes:
        A = (torch.rand(M * K, device="cuda") * 2 - 1).to(torch.float16)
        B = (torch.rand(K * N, device="cuda") * 2 - 1).to(torch.float16)
        C = torch.empty(M * N, dtype=c_dtype, device="cuda")
        for (la, lb, lc) in layouts:
            key = (M, N, K, LAYOUT_NAME[la], LAYOUT_NAME[lb], LAYOUT_NAME[lc])
            if key in table and not a.overwrite:
                continue
            best = None
            for (v, sw, sk) in candidates(variants, M, N, K, lc):
                ms = time_candidate(L, torch, v, sw, sk, C, A, B, M, N, K, lc, la, lb,
                                    a.reps, a.warmup)
                if ms is None:
                    continue
                if log:
                    log.write(f"{M},{N},{K} {'rc'[la]}{'rc'[lb]}{'rc'[lc]} v{v.index} sw{sw} sk{sk} "
                              f"{ms:.4f} ms {2.0 * M * N * K / ms / 1e9:.1f} TFLOP/s\n")
                    log.flush()
                if best is None or ms < best[0]:
                    best = (ms, v, sw, sk)
            if best is None:
                continue
            ms, v, sw, sk = best
            table[key] = {"range": {"M": M, "N": N, "K": K},
                          "layout": {"A": key[3], "B": key[4], "C": key[5]},
                          "config": config_json(v, sw, sk)}
            print(f"{M}x{N}x{K} A={key[3][:3]} B={key[4][:3]} C={key[5][:3]}: variant {v.index} "
                  f"({v.block_m}x{v.block_n}x{v.block_k}, {v.warps_m}x{v.warps_n} waves, pipeline "
                  f"{v.pipeline}) swizzle {sw} split_k {sk}: {ms:.4f} ms, "
                  f"{2.0 * M * N * K / ms / 1e9:.1f} TFLOP/s", flush=True)
        del A, B, C
        # write after every shape: an interrupted run resumes from here with --input
        doc = {"configurations": [table[k] for k in sorted(table)]}
        with open(out_path, "w") as f:
            json.dump(doc, f, indent=4)
    print(f"wrote {out_path}: {len(table)} entries")
    return 0


if __name__ == "__main__":
    sys.exit(main())
