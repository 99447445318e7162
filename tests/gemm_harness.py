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


def built_for(v, lc, la, lb):
    """Whether tile variant v is compiled for this layout triple: in the direct-to-LDS
    pipelines a tile extent that is no multiple of 128 needs its operand K-contiguous in
    kernel space (C row-major: A row-major, B column-major; a column-major C swaps the
    operands)."""
    if v.pipeline == 0:
        return True
    a_k, b_k = la == 0, lb == 1
    if lc == 1:
        a_k, b_k = b_k, a_k
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
    g = O.bits_to_f32(O.logical(gpu_flat, M, N, lc), dout).astype(np.float64)
    c = O.bits_to_f32(O.logical(cpu, M, N, lc), dout).astype(np.float64)
    S = S.reshape(M, N)
    if rows is not None:
        g, c, S = g[rows[0]:rows[1]], c[rows[0]:rows[1]], S[rows[0]:rows[1]]
    assert np.isfinite(g).all(), "GPU result holds NaN/Inf (unwritten or corrupted elements)"
    tol = O.tolerance(S, K, c, dout)
    err = np.abs(g - c)
    worst = float((err / np.maximum(tol, 1e-300)).max()) if err.size else 0.0
    bad = np.argwhere(err > tol)
    assert bad.size == 0, (
        f"{bad.shape[0]} elements outside tolerance; first at {tuple(bad[0])}: "
        f"gpu={g[tuple(bad[0])]!r} cpu={c[tuple(bad[0])]!r} tol={tol[tuple(bad[0])]!r}")
    return worst, g, c


def checksum_check(gpu_flat, A, B, M, N, K, lc, la, lb, din, dout):
    """Size-independent property: C*1 == A*(B*1) and 1^T*C == (1^T*A)*B, in float64.

    Covers every element of C at O(MK + KN + MN) host cost."""
    Al = O.bits_to_f32(O.logical(A, M, K, la), din).astype(np.float64)
    Bl = O.bits_to_f32(O.logical(B, K, N, lb), din).astype(np.float64)
    g = O.bits_to_f32(O.logical(gpu_flat, M, N, lc), dout).astype(np.float64)
    assert np.isfinite(g).all()
    u = 2.0 ** -24
    out_eps = {O.F32: 0.0, O.F16: 2.0 ** -11, O.BF16: 2.0 ** -8}[dout]
    absA, absB = np.abs(Al), np.abs(Bl)
    # row sums
    want_r = Al @ Bl.sum(axis=1)
    scale_r = absA @ absB.sum(axis=1)
    tol_r = (2 * K * u + out_eps) * scale_r + 1e-30
    assert np.all(np.abs(g.sum(axis=1) - want_r) <= tol_r), "row checksum outside tolerance"
    # column sums
    want_c = Al.sum(axis=0) @ Bl
    scale_c = absA.sum(axis=0) @ absB
    tol_c = (2 * K * u + out_eps) * scale_c + 1e-30
    assert np.all(np.abs(g.sum(axis=0) - want_c) <= tol_c), "column checksum outside tolerance"
