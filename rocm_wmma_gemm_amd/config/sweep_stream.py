#!/usr/bin/env python3
"""Times every plan of the whole-K streaming kernel (pipeline 7) on skinny shapes.

    python sweep_stream.py --out stream_sweep.json [--type f16_f16] [--reps 15]

For each shape M x N x K of a grid of decode-like problems (M = 8..128 against N x K from
1024 to 28672) and each of four layout triples (both operands K-contiguous, either, neither)
it runs every compiled pipeline-7 variant that takes the layout with 1, 2, 4 and 8
workgroups per tile through the tuner hook (rocm_wmma_gemm_run_variant) and writes, per
problem, the time of every plan, of the default dispatch and of hipBLASLt.  fit_model.py
--stream fits the constants of the dispatcher's estimate for these plans to the file.

Needs an MI355X.  No counterpart in the reference, which has no kernel for these shapes.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.normpath(os.path.join(HERE, "..", "..")))

SHAPES = [(M, N, K) for M in (8, 16, 32, 64, 128)
          for (N, K) in ((1024, 8192), (2048, 2048), (4096, 4096), (4096, 14336), (8192, 8192), (14336, 4096),
                         (28672, 8192), (8192, 1024), (2048, 8192))]
# small problems, where a 256 x 256 tiling leaves most compute units idle and a workgroup per
# 32- or 64-wide tile over the whole K is a contender too (--small)
SMALL_SHAPES = [(256, 256, 1024), (512, 512, 512), (512, 512, 4096), (768, 768, 768), (1024, 1024, 1024),
                (1024, 1024, 4096), (1536, 1536, 1536), (2048, 2048, 2048), (2048, 1024, 1024), (512, 2048, 2048),
                (1024, 4096, 1024), (2048, 2048, 512), (256, 4096, 2048), (384, 1536, 1536), (3072, 1024, 1024)]
LAYOUTS = ("rcr", "rrr", "ccr", "crr")  # A, B, C: r row-major, c column-major


def takes(v, a_kmajor: bool, b_kmajor: bool, M: int, N: int, K: int) -> bool:
    """What csrc/gemm.hip: streaming_ok asks of a problem, for C row-major."""
    return (K >= 128 and (K % 8 == 0 or not (a_kmajor or b_kmajor)) and (a_kmajor or M % 8 == 0)
            and (b_kmajor or N % 8 == 0))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--out", required=True)
    ap.add_argument("--type", default="f16_f16", choices=["f16_f16", "bf16_bf16"])
    ap.add_argument("--reps", type=int, default=15)
    ap.add_argument("--small", action="store_true", help="the small square and rectangular shapes instead")
    a = ap.parse_args(argv)

    import torch

    import rocm_wmma_gemm_amd as R
    from rocm_wmma_gemm_amd import vendor

    L = R.Loader()
    try:
        V = vendor.VendorGemm()
    except vendor.VendorGemmError:
        V = None
    dtype = torch.float16 if a.type == "f16_f16" else torch.bfloat16
    variants = [v for v in L.variants() if v.pipeline == 7]

    def timed(fn) -> float:
        """Microseconds per call, back to back; the median of three measurements of at
        least 2 ms each (calls of 10 us timed over 0.15 ms are at the mercy of the clock governor)."""
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(4):
            fn()
        reps, runs = a.reps, []
        while len(runs) < 3:  # (the median of three: a slow spell of the GPU lasts several measurements)
            start.record()
            for _ in range(reps):
                fn()
            stop.record()
            torch.cuda.synchronize()
            ms = start.elapsed_time(stop)
            if ms < 2.0 and reps < 1024:
                reps *= 4
                continue
            runs.append(ms / reps * 1e3)
        return sorted(runs)[1]

    # (clocks up before the first measurement)
    warm = torch.randn(4096 * 4096, device="cuda").to(dtype)
    for _ in range(50):
        L.gemm(warm, warm, warm, 4096, 4096, 4096, 0, 0, 1)
    torch.cuda.synchronize()
    del warm
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    out = []
    for (M, N, K) in (SMALL_SHAPES if a.small else SHAPES):
        A = torch.randn(M * K, device="cuda", generator=gen).to(dtype)
        B = torch.randn(K * N, device="cuda", generator=gen).to(dtype)
        C = torch.empty(M * N, dtype=dtype, device="cuda")
        for lay in LAYOUTS:
            la, lb, lc = ("rc".index(ch) for ch in lay)
            rec = {"M": M, "N": N, "K": K, "lay": lay, "t": {},
                   "default": timed(lambda: L.gemm(C, A, B, M, N, K, lc, la, lb))}
            if V is not None:
                rec["hipblaslt"] = timed(lambda: V.gemm("hipblaslt", C, A, B, M, N, K, lc, la, lb))
            for v in variants:
                if not takes(v, la == 0, lb == 1, M, N, K):
                    continue
                for slices in (1, 2, 4, 8):
                    if -(-K // 128) % slices or -(-K // 128) // slices < 2:
                        continue
                    rec["t"][f"{v.block_m}x{v.block_n}s{slices}"] = round(timed(
                        lambda: L.run_variant(v.index, 1, slices, C, A, B, M, N, K, lc, la, lb)), 2)
            rec["default"] = round(rec["default"], 2)
            if "hipblaslt" in rec:
                rec["hipblaslt"] = round(rec["hipblaslt"], 2)
            best = min(rec["t"].items(), key=lambda kv: kv[1]) if rec["t"] else ("-", 0.0)
            print(f"{M}x{N}x{K} {lay}: default {rec['default']:.1f} us, best {best[0]} {best[1]:.1f} us", flush=True)
            out.append(rec)
    with open(a.out, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    return 0


if __name__ == "__main__":
    sys.exit(main())
