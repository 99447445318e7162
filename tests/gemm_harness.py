"""Shared helpers for the GPU parity tests: oracle inputs -> device -> C ABI -> compare.

Everything under test goes through the library's C ABI (via the Python loader
mirror); the oracle is only the checker.
"""
from __future__ import annotations

import numpy as np

import oracle as O

TYPE_PAIRS = {  # name: (input dtype code, output dtype code)
    "f16_f16": (O.F16, O.F16),
    "f32_f16": (O.F16, O.F32),
    "bf16_bf16": (O.BF16, O.BF16),
    "f32_bf16": (O.BF16, O.F32),
}
LAYOUTS8 = [(lc, la, lb) for la in (0, 1) for lb in (0, 1) for lc in (0, 1)]  # (C, A, B) codes


def layout_id(lc, la, lb):
    return "A%sB%sC%s" % ("rc"[la], "rc"[lb], "rc"[lc])


def torch_dtype(code):
    import torch

    return {O.F16: torch.float16, O.BF16: torch.bfloat16, O.F32: torch.float32}[code]


def to_device(flat: np.ndarray, code: int):
    import torch

    if code == O.F32:
        return torch.from_numpy(flat).cuda()
    return torch.from_numpy(flat.view(np.int16)).cuda().view(torch_dtype(code))


def to_host(t, code: int) -> np.ndarray:
    import torch

    if code == O.F32:
        return t.cpu().numpy()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def make_inputs(M, N, K, la, lb, din, seed_a=1, seed_b=1, dist="uniform", lo=-1.0, hi=1.0):
    """Reference-style inputs (test/test.hpp:33-54: both matrices from seed 1 by default)."""
    A = O.init_matrix(M, K, la, din, seed=seed_a, dist=dist, lo=lo, hi=hi)
    B = O.init_matrix(K, N, lb, din, seed=seed_b, dist=dist, lo=lo, hi=hi)
    return A, B


def built_for(v, lc, la, lb, K=None, M=None, N=None):
    """Whether tile variant v runs this layout triple (and shape): in the direct-to-LDS
    pipelines a tile extent that is no multiple of 128 needs its operand K-contiguous in
    kernel space (C row-major: A row-major, B column-major; a column-major C swaps the
    operands); the whole-K streaming kernel (pipeline 7) needs at least one stage of 128 of
    K, 16-byte aligned rows (K a multiple of 8 where an operand is K-contiguous; M or N a multiple
    of 8 where an operand is contiguous along it)."""
    if v.pipeline == 0:
        return True
    a_k, b_k = la == 0, lb == 1
    if lc == 1:
        a_k, b_k = b_k, a_k
    if v.pipeline == 7:
        rows, cols = (M, N) if lc == 0 else (N, M)
        return ((K is None or (K >= 128 and (K % 8 == 0 or not (a_k or b_k))))
                and (a_k or rows is None or rows % 8 == 0)
                and (b_k or cols is None or cols % 8 == 0))
    return (v.block_m % 128 == 0 or a_k) and (v.block_n % 128 == 0 or b_k)


def run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, batch=1, poison=True, variant=None):
    import torch

    dA, dB = to_device(A, din), to_device(B, din)
    dC = torch.empty(M * N * batch, dtype=torch_dtype(dout), device="cuda")
    if poison:
        dC.fill_(float("nan"))
    if variant is None:
        loader.gemm(dC, dA, dB, M, N, K, lc, la, lb, batch_count=batch)
    else:
        v, swz, sk = variant
        rc = loader.run_variant(v, swz, sk, dC, dA, dB, M, N, K, lc, la, lb, batch_count=batch)
        assert rc == 0, f"run_variant returned {rc}"
    torch.cuda.synchronize()
    return to_host(dC, dout)


def check_against_oracle(gpu_flat, A, B, M, N, K, lc, la, lb, din, dout, rows=None):
    """Element-wise |gpu - cpu| <= 2*K*2^-24*sum|a*b| + 1 ulp(C type); returns max ratio."""
    cpu, S = O.gemm(A, B, M, N, K, lc, la, lb, din, dout, want_scale=True, rows=rows)
    r0, r1 = rows if rows is not None else (0, M)
    # (cut the band out before converting: a band check must not cost a pass over all of C)
    g = O.bits_to_f32(np.ascontiguousarray(O.logical(gpu_flat, M, N, lc)[r0:r1]), dout).astype(np.float64)
    c = O.bits_to_f32(np.ascontiguousarray(O.logical(cpu, M, N, lc)[r0:r1]), dout).astype(np.float64)
    S = S.reshape(M, N)[r0:r1]
    assert np.isfinite(g).all(), "GPU result holds NaN/Inf (unwritten or corrupted elements)"
    tol = O.tolerance(S, K, c, dout)
    err = np.abs(g - c)
    worst = float((err / np.maximum(tol, 1e-300)).max()) if err.size else 0.0
    bad = np.argwhere(err > tol)
    assert bad.size == 0, (
        f"{bad.shape[0]} elements outside tolerance; first at {tuple(bad[0])} of rows {r0}..{r1}: "
        f"gpu={g[tuple(bad[0])]!r} cpu={c[tuple(bad[0])]!r} tol={tol[tuple(bad[0])]!r}")
    return worst, g, c


def checksum_check(gpu_flat, A, B, M, N, K, lc, la, lb, din, dout):
    """Size-independent property: C*1 == A*(B*1) and 1^T*C == (1^T*A)*B, in float64.

    Covers every element of C at O(MK + KN + MN) host cost.  The bound is statistical, not
    worst-case, so that one wrong tile cannot hide in it: a row (column) sum adds N (M)
    element errors that are independent, so they add in quadrature.  Per element,
      - rounding to the C type: at most half an output ulp, uniformly distributed,
        variance ulp^2 / 12;
      - fp32 accumulation over K products in any order: each of the K additions rounds a
        partial sum whose variance is at most sum_k (a_ik b_kj)^2, so the variance of the
        accumulated error is at most u^2 * K * sum_k (a_ik b_kj)^2 with u = 2^-24 (twice
        what a left-to-right sum gives, to leave room for the matrix cores' own order).
    Tolerance: 16 standard deviations of the sum (the element-wise comparison against the
    oracle is the exact check; this one has to be free of false alarms over ~10^5 sums
    and still far below what a wrong or missing K tile does to a sum: at 4096^3 fp16 it
    is about 5 against 40 for one K tile of 64 missing from one 256-column tile)."""
    Al = O.bits_to_f32(O.logical(A, M, K, la), din).astype(np.float64)
    Bl = O.bits_to_f32(O.logical(B, K, N, lb), din).astype(np.float64)
    g32 = O.bits_to_f32(O.logical(gpu_flat, M, N, lc), dout)
    g = g32.astype(np.float64)
    assert np.isfinite(g).all()
    u = 2.0 ** -24
    ulp2 = O.ulp_out(g32, dout) ** 2 / 12.0
    A2, B2 = Al * Al, Bl * Bl
    # row sums
    want_r = Al @ Bl.sum(axis=1)
    var_r = u * u * K * (A2 @ B2.sum(axis=1)) + ulp2.sum(axis=1)
    tol_r = 16.0 * np.sqrt(var_r) + 1e-30
    err_r = np.abs(g.sum(axis=1) - want_r)
    assert np.all(err_r <= tol_r), (
        f"row checksum outside tolerance: worst {float((err_r / tol_r).max()):.2f} x tol "
        f"at row {int((err_r / tol_r).argmax())}")
    # column sums
    want_c = Al.sum(axis=0) @ Bl
    var_c = u * u * K * (A2.sum(axis=0) @ B2) + ulp2.sum(axis=0)
    tol_c = 16.0 * np.sqrt(var_c) + 1e-30
    err_c = np.abs(g.sum(axis=0) - want_c)
    assert np.all(err_c <= tol_c), (
        f"column checksum outside tolerance: worst {float((err_c / tol_c).max()):.2f} x tol "
        f"at column {int((err_c / tol_c).argmax())}")
    return float(max((err_r / tol_r).max(), (err_c / tol_c).max()))
