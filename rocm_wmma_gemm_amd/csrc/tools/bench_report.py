#!/usr/bin/env python3
"""Markdown comparison tables (and a bar chart when matplotlib is there) from gemm_bench.

Runs rocm_wmma_gemm_amd/lib/gemm_bench with --rocblas --hipblaslt over a list of shapes and
all eight layouts for one type pair, and writes one table per report in the layout of the
reference's published tables (reference docs/gfx1100_square.md: one row per shape and
input layout pair; this library with C column-major, rocBLAS with C column-major, their
ratio, this library with C row-major, its ratio to the same rocBLAS figure), with more
columns: rocBLAS for C row-major, run as the transposed problem, which the reference's
rocBLAS wrapper does not cover, and hipBLASLt (hipblasLtMatmul with the first algorithm
its heuristic returns) for both C layouts.  The ratio is against the faster of the two
vendor libraries.

    python bench_report.py --type f16_f16 --set square --out docs/gfx950_square_f16.md
    python bench_report.py --type f32_bf16 --shapes 4096,5120,5120:8192,4096,2048 --out x.md

Needs an MI355X: it times the GPU.
"""
from __future__ import annotations

import argparse
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
BENCH = os.path.normpath(os.path.join(HERE, "..", "..", "lib", "gemm_bench"))
SETS = {
    # the reference's published tables (docs/gfx1100_square.md, gfx1100_rectangle.md)
    "square": "1024,1024,1024:2048,2048,2048:4096,4096,4096:8192,8192,8192",
    "rectangle": "4096,2048,64:8192,4096,128:4096,16384,4096:4096,4096,16384:2048,5120,5120:"
                 "4096,5120,5120:32768,4096,4096:65536,2048,2048",
    # projection, decode-like, ragged and long-K shapes
    "other": "8192,4096,2048:4096,14336,4096:16,8192,8192:64,8192,8192:128,8192,8192:"
             "4095,5121,3001:1000,1000,1000:1024,1024,65536:3072,3072,3072:6144,6144,6144",
    # transformer projection shapes (hidden 4096 / 8192 against 11008 / 12288 / 14336 / 28672)
    "projection": "4096,11008,4096:4096,4096,11008:8192,8192,4096:4096,12288,4096:8192,1024,8192:"
                  "4096,4096,14336:2048,8192,2048:12288,4096,4096:5120,5120,5120:8192,3584,7168:"
                  "7168,7168,7168:8192,28672,8192:8192,8192,28672",
    # 256 to 1024 rows of activations against transformer weight matrices
    "prefill": ":".join(f"{m},{n},{k}" for m in (256, 512, 1024)
                        for n, k in ((4096, 4096), (8192, 8192), (4096, 14336), (14336, 4096),
                                     (28672, 8192), (8192, 28672))),
    # many small problems in one strided-batch call (run with --batch_count, default 64)
    "batched": "128,128,128:256,256,256:512,512,512:1024,1024,1024:256,256,4096:"
               "384,640,512:1000,1000,1000:2048,2048,2048",
}
TITLES = {"f16_f16": "FP16 in, FP16 out", "f32_f16": "FP16 in, FP32 out",
          "bf16_bf16": "BF16 in, BF16 out", "f32_bf16": "BF16 in, FP32 out"}
ROW = re.compile(r"^(\S+)\s+(\d+),(\d+),(\d+)\s+([rc]{3})\s+\S+\s+\S+\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)")


def run_bench(type_pair: str, shapes: str, reps: int, batch: int = 1) -> dict:
    """{(m, n, k): {'ours'|'rocblas'|'hipblaslt': {layout 'abc': TFLOP/s}}}"""
    cmd = [BENCH, "--type", type_pair, "--shapes", shapes, "--layouts", "all", "--rocblas", "--hipblaslt",
           "--reps", str(reps), "--batch_count", str(batch)]
    print("running:", " ".join(cmd), file=sys.stderr)
    out = subprocess.run(cmd, capture_output=True, text=True, check=True, timeout=1800).stdout
    res: dict = {}
    for line in out.splitlines():
        m = ROW.match(line)
        if not m:
            continue
        who = m.group(1) if m.group(1) in ("rocblas", "hipblaslt") else "ours"
        key = tuple(int(x) for x in m.group(2, 3, 4))
        res.setdefault(key, {"ours": {}, "rocblas": {}, "hipblaslt": {}})[who][m.group(5)] = float(m.group(8))
    return res


def device_line() -> str:
    try:
        out = subprocess.run([BENCH, "--type", "f16_f16", "--shapes", "128,128,128", "--layouts", "rcr",
                              "--reps", "1", "--warmup", "1"], capture_output=True, text=True,
                             timeout=120).stdout
        return next(l[2:] for l in out.splitlines() if l.startswith("# device"))
    except Exception:  # noqa: BLE001 - the header line is decoration
        return "MI355X"


def table(res: dict, type_pair: str) -> list[str]:
    name = {"r": "row", "c": "col"}
    lines = [
        f"## {TITLES[type_pair]}\n",
        "| Matrix Size | Input Layout (A,B) | this library<br>(C=col) | rocBLAS<br>(C=col) | hipBLASLt<br>(C=col) "
        "| Ratio<br>(C=col) | this library<br>(C=row) | rocBLAS<br>(C=row) | hipBLASLt<br>(C=row) | Ratio<br>(C=row) |",
        "|:---|:---|---:|---:|---:|---:|---:|---:|---:|---:|",
    ]
    for (m, n, k), r in res.items():
        for ab in ("cc", "rc", "cr", "rr"):
            cells = []
            for c in ("c", "r"):
                ours, blas, lt = r["ours"].get(ab + c), r["rocblas"].get(ab + c), r["hipblaslt"].get(ab + c)
                vendor = max([x for x in (blas, lt) if x], default=None)
                ratio = f"{ours / vendor:.2f}" if ours and vendor else "-"
                cells += [f"{ours:.1f}" if ours else "-", f"{blas:.1f}" if blas else "-",
                          f"{lt:.1f}" if lt else "-", ratio]
            lines.append(f"| {m}x{n}x{k} | {name[ab[0]]}, {name[ab[1]]} | " + " | ".join(cells) + " |")
    return lines


def chart(res: dict, type_pair: str, path: str) -> bool:
    try:
        import matplotlib
        matplotlib.use("Agg")
        import matplotlib.pyplot as plt
    except ImportError:
        return False
    labels, ours, blas, lt = [], [], [], []
    for (m, n, k), r in res.items():
        for lay in ("rcr", "rrr", "crr", "ccr"):
            if lay in r["ours"] and lay in r["rocblas"]:
                labels.append(f"{m}x{n}x{k}\n{lay}")
                ours.append(r["ours"][lay])
                blas.append(r["rocblas"][lay])
                lt.append(r["hipblaslt"].get(lay, 0.0))
    if not labels:
        return False
    fig, ax = plt.subplots(figsize=(max(8, 0.45 * len(labels)), 5))
    x = range(len(labels))
    ax.bar([i - 0.27 for i in x], ours, 0.27, label="this library")
    ax.bar([i for i in x], blas, 0.27, label="rocBLAS")
    ax.bar([i + 0.27 for i in x], lt, 0.27, label="hipBLASLt")
    ax.set_xticks(list(x))
    ax.set_xticklabels(labels, fontsize=6, rotation=90)
    ax.set_ylabel("TFLOP/s")
    ax.set_title(f"{TITLES[type_pair]}: C row-major layouts")
    ax.legend()
    fig.tight_layout()
    fig.savefig(path, dpi=120)
    return True


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--type", default="f16_f16", choices=sorted(TITLES))
    ap.add_argument("--set", choices=sorted(SETS), default=None)
    ap.add_argument("--shapes", default=None, help="M,N,K:M,N,K:... instead of --set")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--batch_count", type=int, default=None,
                    help="problems per strided-batch call (default 1; 64 for --set batched); "
                         "rocBLAS then runs rocblas_gemm_strided_batched_ex")
    ap.add_argument("--out", required=True, help="markdown file to write")
    ap.add_argument("--png", default=None, help="bar chart to write (needs matplotlib)")
    a = ap.parse_args(argv)
    shapes = a.shapes or SETS[a.set or "square"]
    batch = a.batch_count or (64 if a.set == "batched" else 1)
    res = run_bench(a.type, shapes, a.reps, batch)
    title = {"square": "Square matrices", "rectangle": "Rectangular matrices",
             "other": "Projection, skinny, ragged and long-K shapes",
             "projection": "Transformer projection shapes",
             "prefill": "256 to 1024 rows against transformer weight matrices",
             "batched": f"Strided batches of {batch} small problems"}.get(a.set, "Selected shapes")
    flops = "2·M·N·K" if batch == 1 else f"{batch}·2·M·N·K"
    lines = [f"# {title}: this library, rocBLAS and hipBLASLt on one MI355X\n",
             f"TFLOP/s = {flops} / median of {a.reps} event-timed launches, seeded random operands; "
             f"{device_line()}.",
             "Produced by `rocm_wmma_gemm_amd/csrc/tools/bench_report.py` "
             f"(`--type {a.type} --shapes {shapes}" + (f" --batch_count {batch}" if batch > 1 else "")
             + "`).\n"]
    lines += table(res, a.type)
    if a.png and chart(res, a.type, a.png):
        lines.append(f"\n![chart]({os.path.basename(a.png)})")
    os.makedirs(os.path.dirname(os.path.abspath(a.out)), exist_ok=True)
    with open(a.out, "w") as f:
        f.write("\n".join(lines) + "\n")
    print("wrote", a.out, file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
