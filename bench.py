#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass over the workload: the fp16 -> fp16 GEMM at M=N=K=4096 in all
eight row/column-major layout combinations of A, B and C (eight launches through the
library's C ABI), on seeded uniform[-1,1] inputs already resident in HBM.  Prints one
JSON line: whole-job TFLOP/s, the roofline of the kernel (against the dense fp16 MFMA
peak), the CPU oracle timed on the host cores as a reported baseline, and context
numbers (per layout, the bf16 -> fp32 8192^3 case, torch.matmul on the same GPU).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2516.6  # 256 CUs x 4 SIMDs x 1024 FLOP/clk x 2.4 GHz: published dense fp16/bf16
METRIC = "TFLOP/s and % of MI355X dense fp16/bf16 MFMA peak at M=N=K=4096/8192"
LAYOUTS = [(la, lb, lc) for la in (0, 1) for lb in (0, 1) for lc in (0, 1)]


def layout_name(la, lb, lc):
    return "rc"[la] + "rc"[lb] + "rc"[lc]


def timed_region(torch, fn, steps):
    """HIP events on the stream the kernels are launched on (torch's current stream)."""
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return e0.elapsed_time(e1) * 1e-3, wall


def load_traffic():
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f)
    except (OSError, ValueError):
        return None


def mfma_ceiling():
    """Sustained MFMA rate of this GPU on pseudo-random operands with nothing else
    running (registers only, ~35 ms per shape): what the power and clock management
    leaves of the published peak for data like the benchmark's.  v_mfma_f32_16x16x32_f16
    is the instruction the large-shape kernels use; 32x32x16 is reported beside it.
    Context only."""
    import subprocess

    exe = os.path.join(ROOT, "rocm_wmma_gemm_amd", "lib", "mfma_probe")
    out = None
    try:
        r = subprocess.run([exe, "--ceiling"], capture_output=True, text=True, timeout=90)
        for line in r.stdout.splitlines():
            if line.startswith("ceiling "):
                _, tf, mhz = line.split()
                out = {"tflops": float(tf), "core_clock_mhz": float(mhz),
                       "what": "v_mfma_f32_16x16x32_f16 only, random fp16 operands, 4 waves/CU, all CUs"}
            elif line.startswith("ceiling_32x32x16 ") and out is not None:
                _, tf, mhz = line.split()
                out["tflops_32x32x16"] = float(tf)
                out["core_clock_mhz_32x32x16"] = float(mhz)
    except (OSError, subprocess.SubprocessError, ValueError):
        pass
    return out


def cpu_baseline(torch, A, B, M, N, K, gpu_c, la, lb, lc):
    """The oracle (a port of the reference's hgemm_cpu) on the host cores, whole
    4096^3 problem in one layout, one run; also used to spot-check the GPU result."""
    import numpy as np

    import oracle as O

    threads = O.default_threads()
    a = A.view(torch.int16).cpu().numpy().view(np.uint16)
    b = B.view(torch.int16).cpu().numpy().view(np.uint16)
    t0 = time.perf_counter()
    cpu, S = O.gemm(a, b, M, N, K, lc, la, lb, O.F16, O.F16, threads=threads, want_scale=True)
    dt = time.perf_counter() - t0
    g = O.bits_to_f32(gpu_c.view(torch.int16).cpu().numpy().view(np.uint16), O.F16).astype(np.float64)
    c = O.bits_to_f32(cpu, O.F16).astype(np.float64)
    tol = O.tolerance(S, K, c, O.F16)
    worst = float((np.abs(g - c) / tol).max())
    # the reference's own CPU-runnable case, 256^3, A row / B column / C row, one thread
    # (reference test/test.hpp:59-129 is single-threaded), in the oracle's two forms: the
    # literal i, j, k loop with a scalar float accumulator, which is what the reference
    # runs, and the strip form the multi-threaded number above uses (the same sums in the
    # same order per element, vectorised across columns: bit-identical results)
    a1 = O.init_matrix(256, 256, O.ROW, O.F16, seed=1)
    b1 = O.init_matrix(256, 256, O.COL, O.F16, seed=1)

    def best_of(fn, runs):
        best = None
        for _ in range(runs):
            t1 = time.perf_counter()
            fn()
            d1 = time.perf_counter() - t1
            best = d1 if best is None else min(best, d1)
        return {"ms": round(best * 1e3, 3), "gflops": round(2.0 * 256 ** 3 / best / 1e9, 2)}

    strip = best_of(lambda: O.gemm(a1, b1, 256, 256, 256, O.ROW, O.ROW, O.COL, O.F16, O.F16, threads=1), 3)
    literal = best_of(lambda: O.gemm(a1, b1, 256, 256, 256, O.ROW, O.ROW, O.COL, O.F16, O.F16, naive=True), 2)
    return {"value": round(2.0 * M * N * K / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads,
            "kind": "port",
            "form": "strip form of the oracle (oracle_gemm_rows): per element the reference's sums in "
                    "the reference's order, vectorised across columns, rows spread over the threads",
            "harness_case_256_cubed_1_thread": dict(strip, form="strip form, 1 thread"),
            "harness_case_256_cubed_literal_loop": dict(literal, form="literal i,j,k loop of the reference "
                                                                      "(oracle_gemm_naive), 1 thread"),
            "sample": f"whole {M}x{N}x{K} fp16->fp16 GEMM, layout {layout_name(la, lb, lc)}, "
                      f"1 run, {dt:.2f} s wall",
            "gpu_vs_cpu_max_err_over_tol": round(worst, 4)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=4096, help="M=N=K of the fp16 workload")
    ap.add_argument("--settle", type=float, default=0.3,
                    help="seconds of untimed steps before the warm-up, for the clock governor")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-context", action="store_true", help="skip the context measurements")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); nothing here shards across "
              "GPUs, so no figure at several GPUs exists", file=sys.stderr)
        return 2

    import torch

    import rocm_wmma_gemm_amd as R

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    loader = R.Loader()  # no fallback: raises if the HIP library is missing
    M = N = K = a.size
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    A = (torch.rand(M * K, device="cuda", generator=gen) * 2 - 1).to(torch.float16)
    B = (torch.rand(K * N, device="cuda", generator=gen) * 2 - 1).to(torch.float16)
    # one output buffer: every GEMM overwrites C, as every call of the library does
    C = torch.empty(M * N, dtype=torch.float16, device="cuda")
    Cs = [C for _ in LAYOUTS]

    def step():
        for (la, lb, lc) in LAYOUTS:
            loader.gemm(C, A, B, M, N, K, lc, la, lb)

    # The GPU comes out of a low-power state: the first few milliseconds of work run at
    # ramping clocks (measured: 128 us per launch in the first 5 ms, 115 us from then on).
    # Let the clock governor settle before the W warm-up steps and the K timed steps.
    settle_until = time.perf_counter() + a.settle
    while time.perf_counter() < settle_until:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(a.warmup):
        step()
    gpu_s, wall_s = timed_region(torch, step, a.steps)
    flop_step = 2.0 * M * N * K * len(LAYOUTS)
    tflops = flop_step * a.steps / gpu_s / 1e12
    launches = a.steps * len(LAYOUTS)
    avg_launch_s = gpu_s / launches

    out = {
        "metric": METRIC, "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(gpu_s / a.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"half_half square GEMM, fp16 in / fp32 accumulate / fp16 out, "
                               f"M=N=K={M}, all 8 row/col-major layouts of A,B,C per step, "
                               f"uniform[-1,1] seed 1",
                   "launches_per_step": len(LAYOUTS)},
        "pct_of_peak": round(100.0 * tflops / PEAK_TFLOPS, 2),
        "wall_s_timed_region": round(wall_s, 4),
    }
    traffic = load_traffic()
    stamp_now = R.source_stamp()
    out["roofline"] = {
        "bound": "mfma", "achieved": round(2.0 * M * N * K / avg_launch_s / 1e12, 2),
        "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(2.0 * M * N * K / avg_launch_s / 1e12 / PEAK_TFLOPS, 4),
        "traffic": traffic.get("hbm_bytes_per_launch") if traffic else None,
        "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, recorded in "
                          "profiles/hbm_traffic.json (a counter run cannot share the timed run)",
        # whether that record was measured on the sources this library is built from
        "traffic_stamp": {"recorded_on": traffic.get("source_stamp") if traffic else None,
                          "this_tree": stamp_now,
                          "matches": bool(traffic) and traffic.get("source_stamp") == stamp_now},
        "kernel": "256x256x64 direct-to-LDS MFMA GEMM kernel solo_gemm (one wave per SIMD, 16x16x32 "
                  "MFMA), the tuned choice for this shape in all 8 layouts; one launch = one GEMM = "
                  "2*M*N*K FLOP",
        "avg_launch_us": round(avg_launch_s * 1e6, 2),
        "algorithmic_bytes_per_launch": (M * K + K * N + M * N) * 2,
    }

    if not a.no_context:
        per_layout = {}
        for C, (la, lb, lc) in zip(Cs, LAYOUTS):
            s, _ = timed_region(torch, lambda: loader.gemm(C, A, B, M, N, K, lc, la, lb), a.steps)
            per_layout[layout_name(la, lb, lc)] = round(2.0 * M * N * K * a.steps / s / 1e12, 1)
        out["per_layout_tflops_ABC"] = per_layout
        # the other half of the headline metric: bf16 -> fp32, 8192^3, A row / B col / C row
        n2 = 8192
        gen.manual_seed(1)
        A2 = torch.randn(n2 * n2, device="cuda", generator=gen).to(torch.bfloat16)
        B2 = torch.randn(n2 * n2, device="cuda", generator=gen).to(torch.bfloat16)
        C2 = torch.empty(n2 * n2, dtype=torch.float32, device="cuda")
        run2 = lambda: loader.gemm(C2, A2, B2, n2, n2, n2, 0, 0, 1)  # noqa: E731
        for _ in range(a.warmup):
            run2()
        s, _ = timed_region(torch, run2, a.steps)
        tf2 = 2.0 * n2 ** 3 * a.steps / s / 1e12
        out["float_bf16_8192_rcr"] = {"tflops": round(tf2, 1),
                                      "pct_of_peak": round(100 * tf2 / PEAK_TFLOPS, 2),
                                      "data": "normal(0,1) seed 1"}
        # the HBM-bound corner of the workload set: M = 16 against N = K = 8192, A row-major,
        # B column-major (weights stored N x K); algorithmic bytes over the time per call
        m3, n3 = 16, 8192
        A3 = (torch.rand(m3 * n3, device="cuda", generator=gen) * 2 - 1).to(torch.float16)
        B3 = (torch.rand(n3 * n3, device="cuda", generator=gen) * 2 - 1).to(torch.float16)
        C3 = torch.empty(m3 * n3, dtype=torch.float16, device="cuda")
        run3 = lambda: loader.gemm(C3, A3, B3, m3, n3, n3, 0, 0, 1)  # noqa: E731
        for _ in range(a.warmup):
            run3()
        s, _ = timed_region(torch, run3, a.steps)
        bytes3 = (m3 * n3 + n3 * n3 + m3 * n3) * 2
        out["skinny_16x8192x8192_rcr"] = {
            "us_per_call_back_to_back": round(s / a.steps * 1e6, 2),
            "tb_per_s": round(bytes3 * a.steps / s / 1e12, 3),
            "frac_of_8_tb_per_s_hbm_roof": round(bytes3 * a.steps / s / 8e12, 3),
            "algorithmic_bytes": bytes3}
        del A3, B3, C3
        # vendor libraries on the same GPU and the same data (context only): rocBLAS and
        # hipBLASLt called directly through libvendor_gemm.so, and torch.matmul
        vendor_ctx = {}
        try:
            from rocm_wmma_gemm_amd.vendor import VendorGemm

            vg = VendorGemm()
            for name in ("rocblas", "hipblaslt"):
                for _ in range(a.warmup):
                    vg.gemm(name, C, A, B, M, N, K, 0, 0, 1)
                s, _ = timed_region(torch, lambda: vg.gemm(name, C, A, B, M, N, K, 0, 0, 1), a.steps)
                vendor_ctx[f"{name}_fp16_{M}_rcr_tflops"] = round(2.0 * M * N * K * a.steps / s / 1e12, 1)
                for _ in range(a.warmup):
                    vg.gemm(name, C2, A2, B2, n2, n2, n2, 0, 0, 1)
                s, _ = timed_region(torch, lambda: vg.gemm(name, C2, A2, B2, n2, n2, n2, 0, 0, 1), a.steps)
                vendor_ctx[f"{name}_bf16_f32_{n2}_rcr_tflops"] = round(2.0 * n2 ** 3 * a.steps / s / 1e12, 1)
            vg.close()
        except Exception as e:  # context only: the line is still valid without it
            vendor_ctx["error"] = repr(e)
        Am, Bm = A.view(M, K), B.view(K, N)
        for _ in range(a.warmup):
            torch.matmul(Am, Bm)
        s, _ = timed_region(torch, lambda: torch.matmul(Am, Bm), a.steps)
        vendor_ctx[f"torch_matmul_fp16_{M}_rrr_tflops"] = round(2.0 * M * N * K * a.steps / s / 1e12, 1)
        out["vendor_context"] = vendor_ctx
        del A2, B2, C2
        ceil = mfma_ceiling()
        if ceil:
            out["mfma_ceiling_random_operands"] = ceil
            out["pct_of_measured_mfma_ceiling"] = round(100.0 * tflops / ceil["tflops"], 2)

    if not a.no_cpu:
        la, lb, lc = 0, 1, 0
        loader.gemm(Cs[0], A, B, M, N, K, lc, la, lb)
        torch.cuda.synchronize()
        out["cpu_baseline"] = cpu_baseline(torch, A, B, M, N, K, Cs[0], la, lb, lc)

    props = torch.cuda.get_device_properties(0)
    out["device"] = {"name": props.name, "arch": props.gcnArchName,
                     "compute_units": props.multi_processor_count}
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
