"""GPU parity: the HIP library, called through its C ABI, against the CPU oracle.

Tolerance (stated once, used everywhere): |gpu - cpu| <= 2*K*2^-24 * sum_k|a_ik*b_kj|
+ 1 ulp of the C element type -- the bound on the difference between two fp32
summation orders of K products, plus output rounding.  Where the reference states
its own criterion it is asserted as well: absolute 1e-4 for fp32 C on its 13 test
shapes (test/gemm/test_float_accum.cpp:128-136), cosine similarity > 0.995 / 0.97
for same-precision C (test/test.hpp:199-215).
"""
import numpy as np
import pytest

import oracle as O
from gemm_harness import (LAYOUTS8, TYPE_PAIRS, built_for, check_against_oracle, checksum_check,
                          layout_id, make_inputs, run_gpu, to_device, to_host, torch_dtype)

pytestmark = pytest.mark.gpu

# reference test/gemm/test_float_accum.cpp:161-224 and test_same_prec.cpp:145-213
REFERENCE_SIZES = [(128, 128, 128), (128, 256, 128), (128, 128, 256), (256, 128, 128),
                   (256, 256, 256), (320, 320, 320), (320, 512, 512), (512, 320, 320),
                   (512, 512, 320), (512, 320, 512), (512, 512, 512), (1024, 256, 256),
                   (256, 1024, 256)]


@pytest.fixture(scope="module")
def loader():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import rocm_wmma_gemm_amd as R

    L = R.Loader()  # probes device 0, opens librocm_wmma_gemm_gfx950.so; raises if missing
    assert L.arch == "gfx950" and L.library_arch() == "gfx950"
    return L


@pytest.mark.parametrize("type_name", list(TYPE_PAIRS))
@pytest.mark.parametrize("lc,la,lb", LAYOUTS8, ids=[layout_id(*l) for l in LAYOUTS8])
def test_reference_test_matrix(loader, type_name, lc, la, lb):
    """The reference's own 13 shapes x 8 layouts x 4 type pairs, seeded as it seeds them."""
    din, dout = TYPE_PAIRS[type_name]
    for (M, N, K) in REFERENCE_SIZES:
        A, B = make_inputs(M, N, K, la, lb, din)
        gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout)
        _, g, c = check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
        if dout == O.F32:
            assert np.abs(g - c).max() <= 1e-4, (M, N, K)
        else:
            cpu = O.gemm(A, B, M, N, K, lc, la, lb, din, dout)
            cos = O.cosine_similarity(gpu, cpu, M, N, lc, dout)
            assert cos > O.cosine_threshold(dout), (M, N, K, cos)


@pytest.mark.parametrize("lc,la,lb", LAYOUTS8, ids=[layout_id(*l) for l in LAYOUTS8])
def test_bit_exact_on_integer_inputs(loader, lc, la, lb):
    """Small-integer operands make every partial sum exact, so any summation order
    must give the oracle's bits exactly -- pins index maps and transpositions."""
    rng = np.random.default_rng(42)
    for din, dout in ((O.F16, O.F32), (O.BF16, O.BF16), (O.F16, O.F16)):
        for (M, N, K) in ((96, 160, 64), (200, 72, 136), (257, 129, 65)):
            Al = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
            Bl = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
            conv = O.f32_to_f16_bits if din == O.F16 else O.f32_to_bf16_bits
            A = np.ascontiguousarray(conv(Al) if la == 0 else conv(Al).T).ravel()
            B = np.ascontiguousarray(conv(Bl) if lb == 0 else conv(Bl).T).ravel()
            gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout)
            cpu = O.gemm(A, B, M, N, K, lc, la, lb, din, dout)
            assert np.array_equal(gpu, cpu), (din, dout, M, N, K)
            if dout == O.F32:
                assert np.array_equal(O.logical(gpu, M, N, lc), Al @ Bl)


@pytest.mark.parametrize("type_name", list(TYPE_PAIRS))
def test_identity_and_ones_closed_forms(loader, type_name):
    din, dout = TYPE_PAIRS[type_name]
    one = 0x3C00 if din == O.F16 else 0x3F80
    # A = I  =>  C = B (exactly, after rounding B's values to the C type: they are already there)
    M = N = K = 192
    for (lc, la, lb) in LAYOUTS8:
        A = np.zeros(M * K, dtype=np.uint16)
        A[np.arange(M) * K + np.arange(M)] = one  # identity is symmetric: same in both layouts
        B = O.init_matrix(K, N, lb, din, seed=5)
        gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout)
        want = O.bits_to_f32(O.logical(B, K, N, lb), din)
        assert np.array_equal(O.bits_to_f32(O.logical(gpu, M, N, lc), dout), want), (lc, la, lb)
    # all ones => C = K (exactly representable: K <= 2048 in f16, <= 256 in bf16)
    Kones = 2048 if dout != O.BF16 else 256
    M, N = 64, 96
    A = np.full(M * Kones, one, dtype=np.uint16)
    B = np.full(Kones * N, one, dtype=np.uint16)
    gpu = run_gpu(loader, A, B, M, N, Kones, 0, 0, 1, din, dout)
    assert np.array_equal(O.bits_to_f32(gpu, dout), np.full(M * N, float(Kones), dtype=np.float32))


EDGE_SHAPES = [(1, 1, 1), (1, 7, 3), (5, 1, 9), (17, 33, 5), (31, 63, 127), (129, 65, 31),
               (64, 64, 8), (100, 36, 1), (255, 257, 259), (1000, 1000, 1000), (33, 4096, 40),
               (3000, 17, 520)]


@pytest.mark.parametrize("type_name", list(TYPE_PAIRS))
@pytest.mark.parametrize("lc,la,lb", LAYOUTS8, ids=[layout_id(*l) for l in LAYOUTS8])
def test_ragged_and_tiny_shapes(loader, type_name, lc, la, lb):
    """Shapes the reference cannot run: M, N not tile multiples, K not a multiple of
    16, odd leading dimensions (2-byte load path), single elements."""
    din, dout = TYPE_PAIRS[type_name]
    for (M, N, K) in EDGE_SHAPES:
        A, B = make_inputs(M, N, K, la, lb, din, seed_a=3, seed_b=4, lo=-0.5, hi=0.5)
        gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout)
        check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)


def _random_problems(seed, count):
    """Seeded shapes across the dispatcher's classes: extents that are multiples of 64, of
    8, even, odd; tiny to a few tiles; every layout and type pair; some strided batches."""
    rng = np.random.RandomState(seed)

    def extent(hi):
        kind = rng.randint(4)
        if kind == 0:
            return 64 * rng.randint(1, hi // 64 + 1)
        if kind == 1:
            return 8 * rng.randint(1, hi // 8 + 1)
        if kind == 2:
            return 2 * rng.randint(1, hi // 2 + 1)
        return rng.randint(1, hi + 1)

    names = list(TYPE_PAIRS)
    out = []
    for _ in range(count):
        M, N, K = extent(1400), extent(1400), extent(2600)
        lc, la, lb = LAYOUTS8[rng.randint(8)]
        batch = 1 if M * N > 300000 else int(rng.choice([1, 1, 2, 3]))
        out.append((M, N, K, lc, la, lb, names[rng.randint(4)], batch))
    return out


@pytest.mark.parametrize("chunk", range(4))
def test_seeded_random_shapes_through_the_default_dispatch(loader, chunk):
    """48 seeded problems that have no tuned entry, so the time-estimate model or the
    nearest entry picks kernel, tile, split and copies for them; each checked element by
    element against the oracle (strided batches: every entry against its own slice)."""
    for (M, N, K, lc, la, lb, tname, batch) in _random_problems(20240 + chunk, 12):
        din, dout = TYPE_PAIRS[tname]
        As, Bs = [], []
        for b in range(batch):
            A, B = make_inputs(M, N, K, la, lb, din, seed_a=11 + 2 * b, seed_b=12 + 2 * b)
            As.append(A)
            Bs.append(B)
        print(f"random problem {M}x{N}x{K} layouts(C,A,B)=({lc},{la},{lb}) {tname} batch {batch}", flush=True)
        gpu = run_gpu(loader, np.concatenate(As), np.concatenate(Bs), M, N, K, lc, la, lb, din, dout, batch=batch)
        for b in range(batch):
            check_against_oracle(gpu[b * M * N:(b + 1) * M * N], As[b], Bs[b], M, N, K, lc, la, lb, din, dout)


def test_seeded_random_skinny_and_small_shapes_through_the_default_dispatch(loader):
    """60 seeded problems of the kinds that the dispatcher's estimate sends to the whole-K
    streaming kernel or prices against it: a few rows or columns (1 to 128, any value) against
    a larger operand, and small problems, K in whole stages of 128; all layouts and type
    pairs, some as strided batches.  Most run on the streaming kernel (several with shared
    tiles), the rest on what beat it; each element against the oracle."""
    rng = np.random.RandomState(4711)
    names = list(TYPE_PAIRS)
    pipelines = {}
    for n in range(60):
        kind = n % 3
        if kind == 0:
            M = [1, 2, 3, 5, 8, 13, 16, 24, 31, 32, 33, 48, 64, 65, 100, 128][rng.randint(16)]
            N = [256, 520, 1000, 1024, 2048, 3000, 4096][rng.randint(7)]
        elif kind == 1:
            N = [1, 4, 8, 16, 30, 64, 96, 128][rng.randint(8)]
            M = [256, 777, 1024, 2048, 4096][rng.randint(5)]
        else:
            M = [130, 256, 300, 512, 768, 1000, 1024][rng.randint(7)]
            N = [130, 256, 384, 512, 1024, 2000][rng.randint(6)]
        K = 128 * rng.randint(2, 33)
        lc, la, lb = LAYOUTS8[rng.randint(8)]
        tname = names[rng.randint(4)]
        batch = [1, 1, 1, 2, 3][rng.randint(5)]
        din, dout = TYPE_PAIRS[tname]
        variant = loader.select(M, N, K, names.index(tname), lc, la, lb, batch)[0]
        pipelines[loader.variants()[variant].pipeline] = pipelines.get(loader.variants()[variant].pipeline, 0) + 1
        print(f"random problem {M}x{N}x{K} layouts(C,A,B)=({lc},{la},{lb}) {tname} batch {batch}", flush=True)
        As = [O.init_matrix(M, K, la, din, seed=300 + n + b) for b in range(batch)]
        Bs = [O.init_matrix(K, N, lb, din, seed=900 + n + b) for b in range(batch)]
        gpu = run_gpu(loader, np.concatenate(As), np.concatenate(Bs), M, N, K, lc, la, lb, din, dout, batch=batch)
        for b in range(batch):
            check_against_oracle(gpu[b * M * N:(b + 1) * M * N], As[b], Bs[b], M, N, K, lc, la, lb, din, dout)
    assert pipelines.get(7, 0) >= 25, pipelines  # the streaming kernel is what most of these run on


def test_fewer_than_sixteen_rows_take_the_plan_tuned_for_sixteen(loader):
    """1 to 15 rows (or columns) against an N x K that has a tuned entry for 16 rows on the
    streaming kernel are served by that entry's plan (same tiles, rows past M read as zeros);
    a small operand stored K x M with rows that are not 16-byte aligned is not.  Each element
    against the oracle."""
    N, K = 4096, 14336
    want = loader.select(16, N, K, 0, 0, 0, 1)
    assert loader.variants()[want[0]].pipeline == 7
    for M in (1, 3, 8, 15):
        assert loader.select(M, N, K, 0, 0, 0, 1) == want, M
        A, B = make_inputs(M, N, K, 0, 1, O.F16, seed_a=60 + M, seed_b=61)
        gpu = run_gpu(loader, A, B, M, N, K, 0, 0, 1, O.F16, O.F16)
        check_against_oracle(gpu, A, B, M, N, K, 0, 0, 1, O.F16, O.F16)
    # (A column-major: 8 rows are 16 bytes per k row and stream, 3 rows do not)
    assert loader.variants()[loader.select(8, N, K, 0, 0, 1, 1)[0]].pipeline == 7
    assert loader.variants()[loader.select(3, N, K, 0, 0, 1, 1)[0]].pipeline != 7
    for M in (8, 3):
        A, B = make_inputs(M, N, K, 1, 1, O.BF16, seed_a=70 + M, seed_b=71)
        gpu = run_gpu(loader, A, B, M, N, K, 0, 1, 1, O.BF16, O.F32)
        check_against_oracle(gpu, A, B, M, N, K, 0, 1, 1, O.BF16, O.F32)


def test_seeded_random_large_shapes_through_the_default_dispatch(loader):
    """The same for 10 problems of many tiles (extents 1500..5200, K 500..4200, all
    alignment classes): every element through the row/column checksums, a 32-row band in
    every block of 128 rows element by element."""
    rng = np.random.RandomState(777)
    names = list(TYPE_PAIRS)
    for n in range(10):
        step = [64, 8, 2, 1][n % 4]
        M = step * rng.randint(1500 // step, 5200 // step + 1)
        N = [64, 8, 1, 2][rng.randint(4)] * 1
        N = N * rng.randint(1500 // N, 5200 // N + 1)
        kstep = [64, 8, 1][rng.randint(3)]
        K = kstep * rng.randint(500 // kstep, 4200 // kstep + 1)
        lc, la, lb = LAYOUTS8[rng.randint(8)]
        tname = names[rng.randint(4)]
        print(f"random problem {M}x{N}x{K} layouts(C,A,B)=({lc},{la},{lb}) {tname}", flush=True)
        _full_size_case(loader, M, N, K, lc, la, lb, tname, seed_a=21 + n, seed_b=40 + n)


def test_subnormal_inputs_are_not_flushed(loader):
    """A holds only subnormal values (fp16 below 6.1e-5, bf16 below 1.2e-38): the products
    and sums must come out as the fp32 arithmetic of the reference's CPU loop gives them,
    subnormal fp32 sums included, on whole tiles and on a ragged shape."""
    for tname, lim in (("f32_f16", 6.0e-5), ("f16_f16", 6.0e-5), ("f32_bf16", 1.0e-38)):
        din, dout = TYPE_PAIRS[tname]
        for (M, N, K) in ((256, 256, 256), (1024, 1024, 512), (130, 70, 51)):
            A = O.init_matrix(M, K, O.ROW, din, seed=5, lo=-lim, hi=lim)
            B = O.init_matrix(K, N, O.COL, din, seed=6, lo=-1.0, hi=1.0)
            a = O.bits_to_f32(A, din)
            assert 0.0 < np.abs(a).max() <= lim * 1.01
            gpu = run_gpu(loader, A, B, M, N, K, 0, 0, 1, din, dout)
            _, g, c = check_against_oracle(gpu, A, B, M, N, K, 0, 0, 1, din, dout)
            assert np.abs(c).max() > 0.0 and np.count_nonzero(g) >= 0.9 * np.count_nonzero(c)


def test_infinities_and_nans_propagate_as_in_the_reference_loop(loader):
    """inf * finite = inf, inf * 0 = NaN, inf - inf = NaN, NaN stays: element (i, k0) of A
    set to +inf (and one to NaN) must mark row i of C exactly as the oracle's fp32 loop does,
    and leave every other row within tolerance."""
    M, N, K = 256, 384, 192
    for tname in ("f32_f16", "bf16_bf16"):
        din, dout = TYPE_PAIRS[tname]
        for (lc, la, lb) in [(0, 0, 1), (1, 1, 0)]:
            A, B = make_inputs(M, N, K, la, lb, din, seed_a=9, seed_b=10)
            inf_bits = 0x7c00 if din == O.F16 else 0x7f80
            nan_bits = 0x7e00 if din == O.F16 else 0x7fc0
            Al = O.logical(A, M, K, la).copy()
            Bl = O.logical(B, K, N, lb).copy()
            Al[3, 17] = inf_bits                   # row 3: +-inf by the sign of B(17, j), NaN where it is 0
            Bl[17, 5] = 0
            Al[100, 40] = inf_bits                 # row 100: +inf and -inf meet in one sum
            Al[100, 41] = inf_bits | 0x8000
            Al[200, 0] = nan_bits                  # row 200: NaN everywhere
            A2 = (Al if la == 0 else Al.T).reshape(-1).copy()
            B2 = (Bl if lb == 0 else Bl.T).reshape(-1).copy()
            gpu = run_gpu(loader, A2, B2, M, N, K, lc, la, lb, din, dout)
            cpu = O.gemm(A2, B2, M, N, K, lc, la, lb, din, dout)
            g = O.bits_to_f32(O.logical(gpu, M, N, lc), dout)
            c = O.bits_to_f32(O.logical(cpu, M, N, lc), dout)
            assert np.array_equal(np.isnan(g), np.isnan(c)), (tname, lc, la, lb)
            assert np.array_equal(np.isposinf(g), np.isposinf(c)) and np.array_equal(np.isneginf(g), np.isneginf(c))
            assert np.isnan(c[3, 5]) and np.isinf(c[3, 6]) and np.isnan(c[200]).all()
            fin = np.isfinite(c)
            assert fin[[0, 1, 2, 4, 99, 101, 199, 201, 255]].all()
            assert np.allclose(g[fin], c[fin], rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("type_name", ["f16_f16", "f32_bf16"])
def test_unaligned_base_pointers(loader, type_name):
    """A, B and C starting one element past a 16-byte boundary: vector loads are not
    legal, so small problems take the 2-byte-load path and large ones the padded copies; a
    skinny shape, which the dispatcher would give to the streaming kernel, goes to the
    general kernel instead."""
    import torch

    din, dout = TYPE_PAIRS[type_name]
    assert loader.variants()[loader.select(16, 1024, 2048, 0, 0, 0, 1)[0]].pipeline == 7
    for (M, N, K) in ((100, 72, 56), (520, 776, 328), (16, 1024, 2048)):
        for (lc, la, lb) in [(0, 0, 1), (1, 1, 0), (0, 1, 1), (0, 0, 0)]:
            A, B = make_inputs(M, N, K, la, lb, din, seed_a=5, seed_b=6)
            bufA = torch.zeros(M * K + 9, dtype=torch_dtype(din), device="cuda")
            bufB = torch.zeros(K * N + 9, dtype=torch_dtype(din), device="cuda")
            bufC = torch.full((M * N + 9,), float("nan"), dtype=torch_dtype(dout), device="cuda")
            dA, dB, dC = bufA[1:1 + M * K], bufB[1:1 + K * N], bufC[1:1 + M * N]
            dA.copy_(to_device(A, din))
            dB.copy_(to_device(B, din))
            assert dA.data_ptr() % 16 != 0 and dB.data_ptr() % 16 != 0
            loader.gemm(dC, dA, dB, M, N, K, lc, la, lb)
            torch.cuda.synchronize()
            assert torch.isnan(bufC[0]) and torch.isnan(bufC[1 + M * N:]).all()
            check_against_oracle(to_host(dC.contiguous(), dout), A, B, M, N, K, lc, la, lb, din, dout)


def test_does_not_write_outside_c(loader):
    """Guard rows/columns around C stay untouched for ragged shapes."""
    import torch

    M, N, K = 130, 70, 50
    for (lc, la, lb) in LAYOUTS8:
        A, B = make_inputs(M, N, K, la, lb, O.F16)
        dA, dB = to_device(A, O.F16), to_device(B, O.F16)
        pad = 4096
        buf = torch.full((M * N + 2 * pad,), 7.0, dtype=torch.float32, device="cuda")
        loader.gemm(buf[pad:pad + M * N], dA, dB, M, N, K, lc, la, lb)
        torch.cuda.synchronize()
        assert torch.all(buf[:pad] == 7.0) and torch.all(buf[pad + M * N:] == 7.0), (lc, la, lb)


@pytest.mark.parametrize("type_name", ["f16_f16", "f32_bf16"])
def test_batched_equals_per_slice_calls(loader, type_name):
    """Batch b equals the unbatched call on slices at b*M*K, b*K*N, b*M*N
    (reference kernel.hpp:165-167); bit-identical because the same kernel runs."""
    import torch

    din, dout = TYPE_PAIRS[type_name]
    M, N, K, batch = 200, 136, 96, 5
    for (lc, la, lb) in [(0, 0, 1), (1, 1, 0), (0, 1, 1), (1, 0, 0)]:
        A = np.concatenate([O.init_matrix(M, K, la, din, seed=10 + b) for b in range(batch)])
        B = np.concatenate([O.init_matrix(K, N, lb, din, seed=20 + b) for b in range(batch)])
        got = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, batch=batch)
        for b in range(batch):
            Ab, Bb = A[b * M * K:(b + 1) * M * K], B[b * K * N:(b + 1) * K * N]
            one = run_gpu(loader, Ab, Bb, M, N, K, lc, la, lb, din, dout)
            assert np.array_equal(got[b * M * N:(b + 1) * M * N], one), (lc, la, lb, b)
            check_against_oracle(one, Ab, Bb, M, N, K, lc, la, lb, din, dout)


def test_every_variant_and_split_k_agree_with_oracle(loader):
    """Each compiled tile variant, forced through the tuner hook, with and without
    split-K, on aligned and ragged shapes."""
    for v in loader.variants():
        for split_k in (1, 3):
            for (M, N, K) in ((512, 512, 512), (300, 520, 264), (77, 91, 1003)):
                for (lc, la, lb) in [(0, 0, 1), (0, 1, 0), (1, 0, 0), (1, 1, 1), (1, 0, 1)]:
                    for tname in ("f16_f16", "f32_bf16"):
                        din, dout = TYPE_PAIRS[tname]
                        A, B = make_inputs(M, N, K, la, lb, din, seed_a=7, seed_b=8)
                        if not built_for(v, lc, la, lb, K, M, N):
                            dA, dB = to_device(A, din), to_device(B, din)
                            dC = to_device(np.zeros(M * N, dtype=A.dtype if dout != O.F32 else np.float32), dout)
                            assert loader.run_variant(v.index, 4, split_k, dC, dA, dB, M, N, K,
                                                      lc, la, lb) == -1, (v.index, lc, la, lb)
                            continue
                        gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout,
                                      variant=(v.index, 4, split_k))
                        try:
                            check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
                        except AssertionError as e:
                            raise AssertionError(
                                f"variant {v.index} split_k {split_k} {M}x{N}x{K} layouts "
                                f"C{lc} A{la} B{lb} {tname}: {e}") from None


def test_whole_k_streaming_kernel_agrees_with_oracle(loader):
    """The kernel for skinny shapes (pipeline 7: tiles of 16, 32 or 64, one workgroup per tile
    over the whole K, ring of up to 8 stages): every tile, skinny M and skinny N (a
    column-major C runs as the transposed problem), either operand K-contiguous or
    contiguous along M or N on a 32- or a 64-wide side, ragged M and N (rows past the edge are read as zeros and not
    stored), one stage and many, a last stage that K cuts short, a strided batch, all type
    pairs, and -1 for what it does not take (rows of either kind that are not 16-byte aligned,
    less than a stage of K)."""
    import torch

    stream = [v for v in loader.variants() if v.pipeline == 7]
    assert {(v.block_m, v.block_n) for v in stream} == {(32, 32), (64, 32), (32, 64), (64, 64),
                                                       (16, 32), (16, 64), (32, 16), (64, 16),
                                                       (128, 64), (64, 128), (128, 32), (32, 128)}
    # (K = 200, 1000 and 1352: a last stage that K cuts short; 1001 where no operand is K-contiguous)
    shapes = [(16, 2048, 1024), (100, 1000, 384), (128, 512, 128), (33, 65, 2048), (2048, 24, 512),
              (40, 520, 200), (1000, 1000, 1000), (64, 128, 1352)]
    ran = set()
    for v in stream:
        for (M, N, K) in shapes:
            # both operands K-contiguous, then the large operand contiguous along N (weights
            # stored K x N), each with C row- and column-major
            for (lc, la, lb) in [(0, 0, 1), (1, 0, 1), (0, 0, 0), (1, 0, 0), (0, 1, 1), (0, 1, 0), (1, 1, 0)]:
                for tname in TYPE_PAIRS:
                    din, dout = TYPE_PAIRS[tname]
                    A, B = make_inputs(M, N, K, la, lb, din, seed_a=3, seed_b=4)
                    if not built_for(v, lc, la, lb, K, M, N):
                        dA, dB = to_device(A, din), to_device(B, din)
                        dC = torch.zeros(M * N, dtype=torch_dtype(dout), device="cuda")
                        assert loader.run_variant(v.index, 1, 1, dC, dA, dB, M, N, K, lc, la, lb) == -1, (
                            v.index, M, N, K, lc, la, lb)
                        continue
                    ran.add((v.block_m, v.block_n, lc, la, lb))
                    gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, variant=(v.index, 1, 1))
                    try:
                        check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
                    except AssertionError as e:
                        raise AssertionError(f"variant {v.index} {M}x{N}x{K} C{lc} A{la} B{lb} {tname}: {e}") from None
    # every tile ran with every pair of operand layouts
    every = {(32, 32), (64, 32), (32, 64), (64, 64), (16, 32), (16, 64), (32, 16), (64, 16),
             (128, 64), (64, 128), (128, 32), (32, 128)}
    for pair in ((0, 1), (0, 0), (1, 1), (1, 0)):
        assert {(bm, bn) for (bm, bn, lc, la, lb) in ran if (la, lb) == pair} == every, pair
    # a strided batch, and bit-identical repeats
    v = stream[0]
    M, N, K, batch = 48, 320, 640, 3
    As = [O.init_matrix(M, K, 0, O.F16, seed=1 + b) for b in range(batch)]
    Bs = [O.init_matrix(K, N, 1, O.F16, seed=9 + b) for b in range(batch)]
    gpu = run_gpu(loader, np.concatenate(As), np.concatenate(Bs), M, N, K, 0, 0, 1, O.F16, O.F32, batch=batch,
                  variant=(v.index, 1, 1))
    again = run_gpu(loader, np.concatenate(As), np.concatenate(Bs), M, N, K, 0, 0, 1, O.F16, O.F32, batch=batch,
                    variant=(v.index, 1, 1))
    assert np.array_equal(gpu, again)
    for b in range(batch):
        check_against_oracle(gpu[b * M * N:(b + 1) * M * N], As[b], Bs[b], M, N, K, 0, 0, 1, O.F16, O.F32)
    # what it does not take
    dA = torch.zeros(64 * 256, dtype=torch.float16, device="cuda")
    dC = torch.zeros(64 * 64, dtype=torch.float16, device="cuda")
    assert loader.run_variant(v.index, 1, 1, dC, dA, dA, 60, 64, 256, 0, 1, 0) == -1   # A contiguous along M, k rows of 120 bytes
    assert loader.run_variant(v.index, 1, 1, dC, dA, dA, 64, 64, 204, 0, 0, 1) == -1   # K-contiguous rows of 408 bytes
    assert loader.run_variant(v.index, 1, 1, dC, dA, dA, 64, 64, 120, 0, 0, 1) == -1   # less than a stage of K


def test_workgroups_that_share_a_tile_of_the_streaming_kernel(loader):
    """Split field s > 1 on pipeline 7: s workgroups per tile, each with K / s, exchange
    their fp32 tiles through the scratch memory inside the one launch; whichever finishes
    last adds them up in slice order.  Against the oracle, and bit-identical from run to
    run (the order of the sum does not depend on who is last); every tile, 2, 4 and 8 workgroups
    per tile, ragged M and N, a strided batch, launches back to back (the counters are back
    at zero after each), the entry point that allocates nothing, and a split that does not
    divide the stages (the tile then stays whole)."""
    import torch

    stream = [v for v in loader.variants() if v.pipeline == 7]
    shapes = [(16, 1024, 2048), (40, 200, 1024), (128, 256, 4096), (1000, 24, 2048), (24, 512, 1000)]
    for v in stream:
        for split in (2, 4, 8):
            for (M, N, K) in shapes:
                for (lc, la, lb) in [(0, 0, 1), (0, 0, 0), (1, 0, 0), (0, 1, 0)]:
                    if not built_for(v, lc, la, lb, K, M, N):
                        continue
                    tname = "f16_f16" if (M + split) % 3 else "f32_bf16"
                    din, dout = TYPE_PAIRS[tname]
                    A, B = make_inputs(M, N, K, la, lb, din, seed_a=5, seed_b=6)
                    runs = [run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, variant=(v.index, 1, split))
                            for _ in range(3)]
                    try:
                        check_against_oracle(runs[0], A, B, M, N, K, lc, la, lb, din, dout)
                    except AssertionError as e:
                        raise AssertionError(
                            f"variant {v.index} split {split} {M}x{N}x{K} C{lc} A{la} B{lb} {tname}: {e}") from None
                    assert all(np.array_equal(r.view(np.uint8), runs[0].view(np.uint8)) for r in runs[1:]), (
                        v.index, split, M, N, K, lc, la, lb)
    # a strided batch (a counter per tile and batch entry)
    v = next(x for x in stream if (x.block_m, x.block_n) == (32, 64))
    M, N, K, batch = 48, 320, 1024, 3
    As = [O.init_matrix(M, K, 0, O.F16, seed=1 + b) for b in range(batch)]
    Bs = [O.init_matrix(K, N, 1, O.F16, seed=9 + b) for b in range(batch)]
    gpu = run_gpu(loader, np.concatenate(As), np.concatenate(Bs), M, N, K, 0, 0, 1, O.F16, O.F32, batch=batch,
                  variant=(v.index, 1, 4))
    for b in range(batch):
        check_against_oracle(gpu[b * M * N:(b + 1) * M * N], As[b], Bs[b], M, N, K, 0, 0, 1, O.F16, O.F32)
    # a split that does not divide the 10 stages: runs, as whole tiles
    A, B = make_inputs(32, 256, 1280, 0, 1, O.F16, seed_a=2, seed_b=3)
    check_against_oracle(run_gpu(loader, A, B, 32, 256, 1280, 0, 0, 1, O.F16, O.F16, variant=(v.index, 1, 4)),
                         A, B, 32, 256, 1280, 0, 0, 1, O.F16, O.F16)
    # the default dispatch shares tiles where they are few and K is long, and the entry
    # point that allocates nothing gives the same bits
    M, N, K = 16, 1024, 8192
    variant, _, split = loader.select(M, N, K, 0, 0, 0, 1)
    assert loader.variants()[variant].pipeline == 7 and split > 1, (variant, split)
    A, B = make_inputs(M, N, K, 0, 1, O.F16, seed_a=7, seed_b=8)
    ordinary = run_gpu(loader, A, B, M, N, K, 0, 0, 1, O.F16, O.F16)
    check_against_oracle(ordinary, A, B, M, N, K, 0, 0, 1, O.F16, O.F16)
    dA, dB = to_device(A, O.F16), to_device(B, O.F16)
    dC = torch.full((M * N,), float("nan"), dtype=torch.float16, device="cuda")
    assert loader.gemm_noalloc(dC, dA, dB, M, N, K, 0, 0, 1) == 0
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dC, O.F16).view(np.uint8), ordinary.view(np.uint8))


def test_split_tail_wave_agrees_with_oracle(loader):
    """Negative split field: only the tiles of the last, partial wave over the 256 CUs are
    cut along K (compact partial tiles + their own reduce kernel).  Shapes with more
    tiles than CUs for both tile sizes, whole and ragged, every pipeline."""
    by_tile = {}
    for v in loader.variants():
        by_tile.setdefault((v.block_m, v.block_n, v.pipeline), v)
    cases = []
    for (bm, bn, pipe), v in sorted(by_tile.items()):
        if (bm, bn) == (256, 256):
            cases += [(v, 4352, 4352, 256), (v, 4300, 4400, 264)]   # 17 x 17 and 17 x 18 tiles
        elif (bm, bn) == (128, 128):
            cases += [(v, 2304, 2304, 256), (v, 2200, 2310, 200)]   # 18 x 18 and 18 x 19 tiles
    assert cases
    for v, M, N, K in cases:
        for split in (-2, -3):
            for (lc, la, lb) in [(0, 0, 1), (1, 1, 0)]:
                din, dout = TYPE_PAIRS["f16_f16" if split == -2 else "f32_bf16"]
                A, B = make_inputs(M, N, K, la, lb, din, seed_a=3, seed_b=4)
                gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout,
                              variant=(v.index, 4, split))
                try:
                    check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
                except AssertionError as e:
                    raise AssertionError(f"variant {v.index} split {split} {M}x{N}x{K} layouts "
                                         f"C{lc} A{la} B{lb}: {e}") from None


def test_mirrored_tile_walk_agrees_with_oracle(loader):
    """Negative swizzle: the tile walk runs in bands of tile columns instead of tile rows.
    Every pipeline, whole K, every tile split, split tail wave and (persistent kernel) the
    walk by K tile, whose reduce kernels must find the tiles by the same mirrored walk; a
    batched call on top (the persistent kernel then deals entries by XCD)."""
    by_pipe = {}
    for v in loader.variants():
        if (v.block_m, v.block_n) in ((256, 256), (128, 128)):
            by_pipe.setdefault(v.pipeline, v)
    assert len(by_pipe) >= 6
    for pipe, v in sorted(by_pipe.items()):
        # 9 x 29 tiles of 256 (261 > 256 CUs: a tail wave of 5) or 18 x 29 of 128
        M, N, K = (2304, 7424, 512) if v.block_m == 256 else (2304, 3700, 512)
        splits = [1, 2, -2] + ([-1] if pipe == 5 else [])
        for split in splits:
            for swz in (-4, -8):
                lc, la, lb = (0, 0, 1) if swz == -4 else (1, 0, 1)
                din, dout = TYPE_PAIRS["f16_f16" if split > 0 else "f32_bf16"]
                A, B = make_inputs(M, N, K, la, lb, din, seed_a=7, seed_b=8)
                print(f"mirrored walk: variant {v.index} pipeline {pipe} split {split} swizzle {swz}", flush=True)
                gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, variant=(v.index, swz, split))
                checksum_check(gpu, A, B, M, N, K, lc, la, lb, din, dout)
                check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout, rows=(M - 40, M))
    v = by_pipe[5]
    M, N, K, batch = 512, 1280, 256, 3
    A = np.concatenate([O.init_matrix(M, K, 0, O.F16, seed=30 + b) for b in range(batch)])
    B = np.concatenate([O.init_matrix(K, N, 1, O.F16, seed=40 + b) for b in range(batch)])
    gpu = run_gpu(loader, A, B, M, N, K, 0, 0, 1, O.F16, O.F16, batch=batch, variant=(v.index, -2, 1))
    for b in range(batch):
        check_against_oracle(gpu[b * M * N:(b + 1) * M * N], A[b * M * K:(b + 1) * M * K],
                             B[b * K * N:(b + 1) * K * N], M, N, K, 0, 0, 1, O.F16, O.F16)


def test_workgroups_that_take_several_tiles_agree_with_oracle(loader):
    """The one-wave-per-SIMD kernel launches one workgroup per CU, and each walks over
    work items CU count apart with ONE load stream running through them.  Cases: more
    tiles than the 256 CUs with 1, 2 and 3 K tiles per item (with one K tile the load
    stream is two items ahead of the MFMAs; with three the ring parity flips from item
    to item), items that straddle batch entries, a K split on top, a ragged edge, fp32
    and 16-bit C; and the walk by K tile, where a workgroup's range of K tiles starts
    and ends anywhere inside a tile and the parts are added up by a second kernel."""
    solo = [v for v in loader.variants() if v.pipeline == 5]
    assert solo, "no one-wave-per-SIMD variant compiled"
    cases = [  # M, N, K, batch, split field
        (4352, 4352, 64, 1, 1),     # 289 items of one K tile
        (4352, 4608, 192, 1, 1),    # 306 items of three K tiles
        (1024, 768, 128, 30, 1),    # 12 tiles x 30 batch entries = 360 items
        (2048, 2304, 320, 2, 2),    # 72 tiles x 2 slices x 2 batch entries = 288 items
        (4344, 4360, 128, 1, 1),    # ragged edges (guarded stores)
        (392, 648, 256, 3, 1),      # ragged, several batch entries: operands are read as they
                                    # are, rows past an edge come from the next batch entry
        # split field -1: the workgroups walk by K tile, each over ceil(all K tiles / 256)
        (3072, 3072, 512, 1, -1),   # 1152 K tiles, 5 per workgroup: tiles cut at odd places
        (1536, 1280, 1024, 1, -1),  # 480 K tiles, 2 per workgroup: every tile in 8 parts
        (768, 512, 640, 7, -1),     # ranges that run from one batch entry into the next
        (1000, 1300, 320, 1, -1),   # ragged edges
        (4096, 4096, 128, 1, -1),   # ranges of whole tiles: nothing to add up
        (512, 512, 64, 1, -1),      # one K tile per workgroup
        (2560, 2304, 4096, 1, -1),  # 90 tiles of 64 K tiles on 256 CUs: 23 per workgroup
    ]
    # every case on the 256 x 256 tile; the other tiles (for them the same shapes are
    # ragged, or hold other tile counts) take every third case, staggered
    runs = [(v, n) for i, v in enumerate(solo) for n in range(len(cases))
            if (v.block_m, v.block_n) == (256, 256) or n % 3 == i % 3]
    for v, n in runs:
        M, N, K, batch, split = cases[n]
        tname = "f16_f16" if n % 2 == 0 else "f32_bf16"
        din, dout = TYPE_PAIRS[tname]
        for (lc, la, lb) in [l for l in [(0, 0, 1), (1, 1, 0), (1, 0, 1)] if built_for(v, *l)][:2]:
            A = np.concatenate([O.init_matrix(M, K, la, din, seed=30 + b) for b in range(batch)])
            B = np.concatenate([O.init_matrix(K, N, lb, din, seed=60 + b) for b in range(batch)])
            gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, batch=batch,
                          variant=(v.index, 4, split))
            for b in range(batch):
                try:
                    check_against_oracle(gpu[b * M * N:(b + 1) * M * N], A[b * M * K:(b + 1) * M * K],
                                         B[b * K * N:(b + 1) * K * N], M, N, K, lc, la, lb, din, dout)
                except AssertionError as e:
                    raise AssertionError(f"variant {v.index} {M}x{N}x{K} batch {b}/{batch} split {split} "
                                         f"layouts C{lc} A{la} B{lb} {tname}: {e}") from None


def test_batch_entries_dealt_by_xcd_agree_with_oracle(loader):
    """Strided batches of whole tiles on the kernels that deal (batch entry, tile) pairs
    to the XCDs in contiguous runs: every entry's every tile must still be computed once.
    Item counts that are and are not multiples of the 8 XCDs, fewer and more items than
    the 256 CUs, one tile per entry, every layout class, 16-bit and fp32 C, and a ragged
    shape on the kernels that take one."""
    kernels = [v for v in loader.variants() if v.pipeline in (5, 6)]
    assert kernels, "no persistent or direct-to-LDS variant compiled"
    cases = [  # M, N, K, batch
        (512, 768, 128, 11),    # 6 tiles of 256 x 256 x 11 entries = 66 items
        (256, 256, 192, 37),    # one 256 x 256 tile per entry
        (768, 1024, 64, 29),    # 12 x 29 = 348 items: more than the CUs, not a multiple of 8
        (328, 456, 128, 9),     # ragged
    ]
    for i, v in enumerate(kernels):
        for n, (M, N, K, batch) in enumerate(cases):
            tname = "f16_f16" if (n + i) % 2 == 0 else "f32_bf16"
            din, dout = TYPE_PAIRS[tname]
            layouts = [l for l in [(0, 0, 1), (1, 1, 0), (0, 0, 0), (1, 1, 1)] if built_for(v, *l)]
            lc, la, lb = layouts[(n + i) % len(layouts)]
            A = np.concatenate([O.init_matrix(M, K, la, din, seed=130 + b) for b in range(batch)])
            B = np.concatenate([O.init_matrix(K, N, lb, din, seed=170 + b) for b in range(batch)])
            gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, batch=batch,
                          variant=(v.index, 2, 1))
            for b in range(batch):
                try:
                    check_against_oracle(gpu[b * M * N:(b + 1) * M * N], A[b * M * K:(b + 1) * M * K],
                                         B[b * K * N:(b + 1) * K * N], M, N, K, lc, la, lb, din, dout)
                except AssertionError as e:
                    raise AssertionError(f"variant {v.index} {M}x{N}x{K} batch {b}/{batch} "
                                         f"layouts C{lc} A{la} B{lb} {tname}: {e}") from None


def test_k_tiles_walked_in_runs_out_of_step_between_xcds(loader):
    """The plan's K-order fields on the persistent kernel: the K tiles of a tile are walked in runs
    of 1 to 16, and within every 8 runs the workgroups of XCD x start at run x; within groups of
    2, 4 or 8 K tiles the workgroup of tile (i, j) starts at tile (i + j) of the group.  Against the
    oracle on K that is whole groups of runs, K with runs left over (walked in order), a
    partial last K tile, ragged M and N, several items per workgroup, batch entries, every
    tile split along K, the split tail wave, the walk by K tile, and line touches on top;
    three runs compared bit for bit (an element's sum has one order, whoever computes it)."""
    solo = [v for v in loader.variants() if v.pipeline == 5 and v.block_k == 64]
    assert solo
    v256 = next(v for v in solo if (v.block_m, v.block_n) == (256, 256))
    field = lambda run, touch=0: (touch & 15) | (run.bit_length() << 4) | (touch & 0x300)  # noqa: E731
    cases = [  # M, N, K, batch, split field, run length, touch distance (+ K group code << 8), variant
        (512, 768, 4096 + 64, 1, 1, 0, 0x200, v256),   # groups of 4 K tiles, one tile left over
        (768, 512, 2048, 1, 1, 0, 0x300, v256),        # groups of 8
        (300, 520, 1024 + 40, 1, 1, 0, 0x100, v256),   # groups of 2, ragged M, N and a partial last K tile
        (2304, 2304, 1024, 1, 1, 0, 0x200, v256),      # workgroups with two items
        (256, 256, 1088, 3, 2, 0, 0x200, v256),        # batch entries, two K slices of 9 and 8 tiles
        (768, 512, 4096, 1, -1, 0, 0x200, v256),       # walk by K tile
        (512, 512, 8192, 1, 1, 8, 0x200, v256),        # groups inside runs
        (512, 512, 2048, 1, 1, 1, 0, v256),      # 32 K tiles: 4 groups of 8 runs of 1
        (512, 768, 4096, 1, 1, 4, 0, v256),      # 64 K tiles: 2 groups of runs of 4
        (256, 512, 8192 + 192, 1, 1, 8, 0, v256),  # 131 K tiles: 2 groups of runs of 8 and 3 tiles in order
        (300, 520, 4096 + 40, 1, 1, 2, 0, v256),  # ragged M, N and a partial last K tile
        (2304, 2304, 1024, 1, 1, 2, 0, v256),    # 81 tiles: workgroups with two items
        (256, 256, 1088, 5, 1, 1, 0, v256),      # batch entries, 17 K tiles
        (512, 512, 8192, 1, 2, 4, 0, v256),      # every tile in two K slices of 64 tiles
        (4352, 256, 2048, 1, -2, 2, 0, v256),    # the tail wave split in two
        (768, 512, 4096, 1, -1, 4, 0, v256),     # walk by K tile: ranges cut anywhere
        (512, 512, 16384, 1, 1, 8, 1, v256),     # with line touches inside the runs
        (512, 512, 4096, 1, 1, 16, 0, v256),     # 64 K tiles are less than a group of runs of 16: in order
    ] + [(384, 576, 2048 + 64, 1, 1, 2, 0, v) for v in solo if v is not v256]
    for n, (M, N, K, batch, split, run, touch, v) in enumerate(cases):
        tname = "f16_f16" if n % 2 == 0 else "f32_bf16"
        din, dout = TYPE_PAIRS[tname]
        for (lc, la, lb) in [l for l in [(0, 0, 1), (1, 1, 0), (0, 0, 0), (1, 1, 1)] if built_for(v, *l)]:
            import torch

            A = np.concatenate([O.init_matrix(M, K, la, din, seed=330 + b) for b in range(batch)])
            B = np.concatenate([O.init_matrix(K, N, lb, din, seed=360 + b) for b in range(batch)])
            dA, dB = to_device(A, din), to_device(B, din)
            outs = []
            for _ in range(3):
                dC = torch.full((M * N * batch,), float("nan"), dtype=torch_dtype(dout), device="cuda")
                rc = loader.run_variant(v.index, 4, split, dC, dA, dB, M, N, K, lc, la, lb, batch_count=batch,
                                        touch_ahead=field(run, touch))
                assert rc == 0, (rc, M, N, K, split, run)
                outs.append(dC)
            torch.cuda.synchronize()
            gpu = to_host(outs[0], dout)
            for b in range(batch):
                try:
                    check_against_oracle(gpu[b * M * N:(b + 1) * M * N], A[b * M * K:(b + 1) * M * K],
                                         B[b * K * N:(b + 1) * K * N], M, N, K, lc, la, lb, din, dout)
                except AssertionError as e:
                    raise AssertionError(f"variant {v.index} {M}x{N}x{K} batch {b}/{batch} split {split} runs of "
                                         f"{run} touch {touch} layouts C{lc} A{la} B{lb} {tname}: {e}") from None
            assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), (M, N, K, split, run)
    # the dispatcher's estimate asks for groups of 8 where the operands outgrow the memory-side cache
    variant, _, _, touch = loader.select_ex(8192, 8192, 20480, 2, 0, 0, 1)
    assert loader.variants()[variant].pipeline == 5 and (touch >> 8) == 3, (variant, touch)
    assert loader.select_ex(6144, 6144, 10240, 2, 0, 0, 1)[3] >> 4 == 0  # 252 MB: fits
    assert loader.select_ex(4096, 4096, 3072, 2, 0, 0, 1)[3] >> 4 == 0
    assert loader.select_ex(8192, 8192, 16384, 2, 0, 0, 0)[3] >> 4 == 0  # B row-major: not before K = 20480


def test_partial_last_k_tile_on_the_persistent_kernel(loader):
    """K that is not a multiple of the 64-wide K tile, rows 16-byte aligned: the
    one-wave-per-SIMD kernel reads the operands where they lie and takes the rest of the
    last K tile as zeros (a K-contiguous operand: the lanes that would fetch columns
    past K load out of range; an M/N-contiguous one: the rows past K lie past the end of
    the batch entry's range).  Cases: the partial tile as tile 0, as tile 1 (both go out
    in the prologue) and later; ragged M and N on top; batch entries; a K split and the
    walk by K tile on top; K not a multiple of 8 where no operand is K-contiguous."""
    solo = [v for v in loader.variants() if v.pipeline == 5]
    assert solo, "no one-wave-per-SIMD variant compiled"
    cases = [  # M, N, K, batch, split field
        (512, 512, 1000, 1, 1),
        (304, 520, 200, 1, 1),     # ragged M and N too
        (256, 256, 8, 1, 1),       # the only K tile is partial
        (256, 512, 72, 1, 1),      # the second
        (256, 256, 136, 5, 1),     # batch entries: each one's range ends at its own K
        (512, 768, 1096, 2, 2),    # every tile in two K slices, the second ends in the partial tile
        (768, 512, 648, 3, -1),    # walk by K tile
        (4352, 256, 40, 1, 1),     # several items per workgroup, each one partial tile
    ]
    for i, v in enumerate(solo):
        for n, (M, N, K, batch, split) in enumerate(cases):
            tname = "f16_f16" if (n + i) % 2 == 0 else "f32_bf16"
            din, dout = TYPE_PAIRS[tname]
            for (lc, la, lb) in [l for l in [(0, 0, 1), (1, 1, 0), (0, 0, 0), (1, 1, 1)] if built_for(v, *l)]:
                k = K + 1 if (la, lb) == (1, 0) and n % 2 == 0 else K  # odd K: no K-contiguous operand
                A = np.concatenate([O.init_matrix(M, k, la, din, seed=230 + b) for b in range(batch)])
                B = np.concatenate([O.init_matrix(k, N, lb, din, seed=260 + b) for b in range(batch)])
                gpu = run_gpu(loader, A, B, M, N, k, lc, la, lb, din, dout, batch=batch,
                              variant=(v.index, 4, split))
                for b in range(batch):
                    try:
                        check_against_oracle(gpu[b * M * N:(b + 1) * M * N], A[b * M * k:(b + 1) * M * k],
                                             B[b * k * N:(b + 1) * k * N], M, N, k, lc, la, lb, din, dout)
                    except AssertionError as e:
                        raise AssertionError(f"variant {v.index} {M}x{N}x{k} batch {b}/{batch} split {split} "
                                             f"layouts C{lc} A{la} B{lb} {tname}: {e}") from None


def test_what_lies_past_k_does_not_reach_c(loader):
    """The columns of the last K tile past K must be zeros, not whatever follows in memory
    times zero: with infinities right behind a row's K columns (the next row's first
    elements, the next batch entry) every other row of C stays finite and correct."""
    solo = next(v for v in loader.variants() if v.pipeline == 5 and (v.block_m, v.block_n) == (256, 256))
    din, dout = TYPE_PAIRS["f16_f16"]
    inf = np.uint16(0x7C00)
    # A row-major (K-contiguous): row 5 starts with infinities, which the loads of row 4's
    # partial tile would reach
    M, N, K = 256, 256, 200
    for lb in (0, 1):
        A = O.init_matrix(M, K, 0, din, seed=301)
        B = O.init_matrix(K, N, lb, din, seed=302)
        A[5 * K:5 * K + 64] = inf
        gpu = run_gpu(loader, A, B, M, N, K, 0, 0, lb, din, dout, variant=(solo.index, 4, 1))
        check_against_oracle(gpu, A, B, M, N, K, 0, 0, lb, din, dout, rows=(0, 5))
        check_against_oracle(gpu, A, B, M, N, K, 0, 0, lb, din, dout, rows=(6, M))
    # A column-major, B row-major (K rows each): the second batch entry is all
    # infinities and starts where the first entry's rows past K would be
    K = 203
    A = np.concatenate([O.init_matrix(M, K, 1, din, seed=303), np.full(M * K, inf, np.uint16)])
    B = np.concatenate([O.init_matrix(K, N, 0, din, seed=304), np.full(K * N, inf, np.uint16)])
    gpu = run_gpu(loader, A, B, M, N, K, 0, 1, 0, din, dout, batch=2, variant=(solo.index, 4, 1))
    check_against_oracle(gpu[:M * N], A[:M * K], B[:K * N], M, N, K, 0, 1, 0, din, dout)


def test_what_lies_past_k_does_not_reach_c_on_the_streaming_kernel(loader):
    """The same for the whole-K streaming kernel (pipeline 7), which relies on the ends of its
    buffer descriptors alone: a last stage of 128 that K cuts short must read zeros, whole
    tiles and tiles shared by two workgroups alike.  K-contiguous operand: the row behind a
    row starts with infinities (inside the allocation, right where the lanes past K would
    fetch).  Operand contiguous along M or N: a second batch entry of infinities starts where
    the k rows past K would be (K = 200, and K = 1001 where no operand is K-contiguous).
    Ragged M and N on top, so that the rows past the edge of a tile are in play too."""
    din, dout = TYPE_PAIRS["f16_f16"]
    inf = np.uint16(0x7C00)
    stream = [v for v in loader.variants() if v.pipeline == 7]
    ran = set()
    for v in stream:
        for split in (1, 2):
            # A row-major: row 5 begins with infinities; B column-major or row-major
            M, N, K = 40, 136, 200
            for lb in (1, 0):
                if not built_for(v, 0, 0, lb, K, M, N):
                    continue
                A = O.init_matrix(M, K, 0, din, seed=311)
                B = O.init_matrix(K, N, lb, din, seed=312)
                A[5 * K:5 * K + 64] = inf
                gpu = run_gpu(loader, A, B, M, N, K, 0, 0, lb, din, dout, variant=(v.index, 1, split))
                check_against_oracle(gpu, A, B, M, N, K, 0, 0, lb, din, dout, rows=(0, 5))
                check_against_oracle(gpu, A, B, M, N, K, 0, 0, lb, din, dout, rows=(6, M))
                ran.add((v.index, split, 0, lb))
            # B column-major: column 7 begins with infinities; A column-major
            if built_for(v, 0, 1, 1, K, M, N):
                A = O.init_matrix(M, K, 1, din, seed=313)
                B = O.init_matrix(K, N, 1, din, seed=314)
                B[7 * K:7 * K + 64] = inf
                gpu = run_gpu(loader, A, B, M, N, K, 0, 1, 1, din, dout, variant=(v.index, 1, split))
                g = O.bits_to_f32(gpu, dout).reshape(M, N)
                cpu = O.bits_to_f32(O.gemm(A, B, M, N, K, 0, 1, 1, din, dout), dout).reshape(M, N)
                keep = [j for j in range(N) if j != 7]
                assert np.isfinite(g[:, keep]).all(), (v.index, split)
                assert np.allclose(g[:, keep], cpu[:, keep], rtol=2e-3, atol=1e-2), (v.index, split)
                ran.add((v.index, split, 1, 1))
            # neither operand K-contiguous: the second batch entry, all infinities, lies where
            # the first entry's k rows past K would be
            for K2 in (200, 1001):
                if not built_for(v, 0, 1, 0, K2, M, N):
                    continue
                A = np.concatenate([O.init_matrix(M, K2, 1, din, seed=315), np.full(M * K2, inf, np.uint16)])
                B = np.concatenate([O.init_matrix(K2, N, 0, din, seed=316), np.full(K2 * N, inf, np.uint16)])
                gpu = run_gpu(loader, A, B, M, N, K2, 0, 1, 0, din, dout, batch=2, variant=(v.index, 1, split))
                check_against_oracle(gpu[:M * N], A[:M * K2], B[:K2 * N], M, N, K2, 0, 1, 0, din, dout)
                ran.add((v.index, split, 1, 0, K2))
    assert len({r[0] for r in ran}) == len(stream), "every streaming tile ran"


def test_degenerate_arguments(loader):
    import torch

    a = torch.ones(64, dtype=torch.float16, device="cuda")
    c = torch.full((64,), 3.0, dtype=torch.float16, device="cuda")
    loader.gemm(c, a, a, 0, 8, 8)          # M == 0: nothing happens
    loader.gemm(c, a, a, 8, 8, 8, batch_count=0)
    torch.cuda.synchronize()
    assert torch.all(c == 3.0)
    loader.gemm(c, a, a, 8, 8, 0)          # K == 0: empty sum, C = 0
    torch.cuda.synchronize()
    assert torch.all(c == 0.0)
    c.fill_(3.0)
    # layout codes outside {0,1}: silent no-op (reference src/gemm.cpp:243)
    loader.gemm_raw(0, c.data_ptr(), a.data_ptr(), a.data_ptr(), 8, 8, 8, 1, 2, 0, 0,
                    torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.all(c == 3.0)
    with pytest.raises(TypeError):
        loader.gemm(c, a.float(), a.float(), 8, 8, 8)


def test_runs_on_the_callers_stream(loader):
    import torch

    M = N = K = 256
    A, B = make_inputs(M, N, K, 0, 1, O.F16)
    dA, dB = to_device(A, O.F16), to_device(B, O.F16)
    dC = torch.zeros(M * N, dtype=torch.float16, device="cuda")
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        loader.gemm(dC, dA, dB, M, N, K, 0, 0, 1)  # picks up torch's current stream
        ev = torch.cuda.Event()
        ev.record(s)
    ev.synchronize()
    check_against_oracle(to_host(dC, O.F16), A, B, M, N, K, 0, 0, 1, O.F16, O.F16)


def test_repeated_calls_give_identical_bits(loader):
    """Every reduction runs in a fixed order (K slices ascending, parts of a tile by
    workgroup number), so a call repeated with other work in between returns the same
    bits: whole tiles, every tile split, split tail wave, walk by K tile, padded copies."""
    import torch

    shapes = [(4096, 4096, 4096), (64, 8192, 8192), (4096, 5120, 5120), (1024, 1024, 65536),
              (4095, 5121, 3001), (1000, 1000, 1000)]
    other = torch.ones(512 * 512, dtype=torch.float16, device="cuda")
    other_c = torch.empty(512 * 512, dtype=torch.float32, device="cuda")
    for (M, N, K) in shapes:
        for (lc, la, lb) in [(0, 0, 1), (1, 1, 0)]:
            dA = (torch.rand(M * K, device="cuda") * 2 - 1).to(torch.float16)
            dB = (torch.rand(K * N, device="cuda") * 2 - 1).to(torch.float16)
            outs = []
            for _ in range(3):
                c = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda")
                loader.gemm(c, dA, dB, M, N, K, lc, la, lb)
                loader.gemm(other_c, other, other, 512, 512, 512, 0, 0, 1)
                loader.gemm(other_c, other, other, 16, 128, 2048, 0, 0, 1)  # a split-K call in between
                outs.append(c)
            torch.cuda.synchronize()
            assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), (M, N, K, lc, la, lb)
            assert not torch.isnan(outs[0]).any()


def test_two_streams_share_the_scratch_memory(loader):
    """Split-K and padded-copy GEMMs issued from two streams at the same time (reference
    contract: concurrent calls are safe when each has its own stream).  Both kinds keep
    fp32 partial sums or operand copies in the library's one per-device buffer; every
    result must equal, bit for bit, what the same call gives when nothing else runs."""
    import torch

    cases = [  # (M, N, K, lc, la, lb): split-K (skinny, long K), padded copies (odd K), and the
        # streaming kernel's shared tiles (partial tiles in the buffer, one set of counters)
        (64, 8192, 8192, 0, 1, 0),
        (1024, 1024, 16384, 0, 0, 1),
        (128, 8192, 8192, 1, 0, 0),
        (1025, 1031, 2049, 0, 0, 1),
        (16, 1024, 8192, 0, 0, 1),
        (32, 2048, 8192, 0, 0, 0),
    ]
    assert loader.select(16, 1024, 8192, 0, 0, 0, 1)[2] > 1 and loader.select(32, 2048, 8192, 0, 0, 0, 0)[2] > 1
    dev = []
    for (M, N, K, lc, la, lb) in cases:
        A, B = make_inputs(M, N, K, la, lb, O.F16)
        dA, dB = to_device(A, O.F16), to_device(B, O.F16)
        want = torch.zeros(M * N, dtype=torch.float32, device="cuda")
        loader.gemm(want, dA, dB, M, N, K, lc, la, lb)
        torch.cuda.synchronize()
        dev.append((dA, dB, want))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    rounds = 6
    got = [[torch.zeros_like(dev[i][2]) for _ in range(rounds)] for i in range(len(cases))]
    for r in range(rounds):
        for i, (M, N, K, lc, la, lb) in enumerate(cases):
            s = streams[(i + r) % 2]
            loader.gemm(got[i][r], dev[i][0], dev[i][1], M, N, K, lc, la, lb, stream=s)
    torch.cuda.synchronize()
    for i in range(len(cases)):
        for r in range(rounds):
            assert torch.equal(got[i][r], dev[i][2]), (cases[i], r)


def test_two_host_threads_each_on_its_own_stream(loader):
    """The reference's threading contract (no mutable state behind the loader: concurrent
    gemm calls from several host threads are safe when each uses its own stream), on
    shapes that share the library's scratch buffer and on one that does not."""
    import threading

    import torch

    cases = [(64, 8192, 8192, 0, 1, 0), (1025, 1031, 2049, 0, 0, 1), (512, 768, 1024, 0, 0, 1)]
    dev = []
    for (M, N, K, lc, la, lb) in cases:
        A, B = make_inputs(M, N, K, la, lb, O.F16)
        dA, dB = to_device(A, O.F16), to_device(B, O.F16)
        want = torch.zeros(M * N, dtype=torch.float16, device="cuda")
        loader.gemm(want, dA, dB, M, N, K, lc, la, lb)
        dev.append((dA, dB, want))
    torch.cuda.synchronize()
    rounds, errors = 8, []
    outs = [[[torch.zeros_like(dev[i][2]) for _ in range(rounds)] for i in range(len(cases))] for _ in range(2)]

    def worker(t):
        try:
            torch.cuda.set_device(0)
            s = torch.cuda.Stream()
            for r in range(rounds):
                for i in range(len(cases)):
                    j = (i + t) % len(cases)
                    M, N, K, lc, la, lb = cases[j]
                    loader.gemm(outs[t][j][r], dev[j][0], dev[j][1], M, N, K, lc, la, lb, stream=s)
            s.synchronize()
        except Exception as e:  # surfaced in the main thread below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
    assert not errors and not any(th.is_alive() for th in threads), errors
    torch.cuda.synchronize()
    for t in range(2):
        for i in range(len(cases)):
            for r in range(rounds):
                assert torch.equal(outs[t][i][r], dev[i][2]), (t, cases[i], r)


def test_scratch_buffer_outlives_a_graph_that_holds_its_address(loader):
    """A split-K call recorded into a HIP graph bakes the library's scratch buffer into the
    graph.  A later eager call that needs a larger buffer must not free the old one (the
    replays would write partial sums into freed memory), and a call recorded while the buffer
    is too small must neither allocate nor synchronise inside the capture: it runs without
    scratch memory instead.  Every replay gives the eager result."""
    import torch

    assert loader.workspace_release() == 0, "run before any other test that captures a graph"
    M, N, K, lc, la, lb = 256, 8192, 8192, 0, 1, 0  # (a split-K plan: partial planes in the buffer)
    assert loader.select(M, N, K, 1, lc, la, lb)[2] > 1
    A, B = make_inputs(M, N, K, la, lb, O.F16)
    dA, dB = to_device(A, O.F16), to_device(B, O.F16)
    want = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    loader.gemm(want, dA, dB, M, N, K, lc, la, lb)  # eager: allocates the first buffer
    torch.cuda.synchronize()
    check_against_oracle(to_host(want, O.F32), A, B, M, N, K, lc, la, lb, O.F16, O.F32)
    out = torch.zeros_like(want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loader.gemm(out, dA, dB, M, N, K, lc, la, lb)
    assert loader.workspace_release() == 1, "a buffer lent to a capture must be kept"

    # an eager call that needs 512 MiB of partial planes: the buffer is replaced
    small = next(v.index for v in loader.variants() if v.pipeline == 1 and v.block_m == 128 and v.block_n == 128)
    M2, N2, K2 = 2048, 2048, 8192
    A2, B2 = make_inputs(M2, N2, K2, 0, 1, O.F16, seed_b=2)
    dA2, dB2 = to_device(A2, O.F16), to_device(B2, O.F16)
    big = torch.full((M2 * N2,), float("nan"), dtype=torch.float32, device="cuda")
    assert loader.run_variant(small, 8, 32, big, dA2, dB2, M2, N2, K2, 0, 0, 1) == 0
    torch.cuda.synchronize()
    check_against_oracle(to_host(big, O.F32), A2, B2, M2, N2, K2, 0, 0, 1, O.F16, O.F32)
    # memory allocated now lands where a freed buffer would have been
    filler = [torch.full((64 << 20,), 7, dtype=torch.uint8, device="cuda") for _ in range(6)]
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        assert all(bool((f == 7).all()) for f in filler), "a replay wrote into memory the library had freed"
        loader.gemm(big, dA2, dB2, M2, N2, K2, 0, 0, 1)  # eager work in between
        torch.cuda.synchronize()

    # recorded while the buffer is too small for it: no growth inside the capture
    M3, N3, K3 = 4096, 2048, 8192
    A3, B3 = make_inputs(M3, N3, K3, 0, 1, O.F16, seed_b=3)
    dA3, dB3 = to_device(A3, O.F16), to_device(B3, O.F16)
    out3 = torch.full((M3 * N3,), float("nan"), dtype=torch.float32, device="cuda")
    graph3 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph3):
        assert loader.run_variant(small, 8, 28, out3, dA3, dB3, M3, N3, K3, 0, 0, 1) == 0
    for replay in range(2):
        out3.fill_(float("nan"))
        torch.cuda.synchronize()
        graph3.replay()
        torch.cuda.synchronize()
        check_against_oracle(to_host(out3, O.F32), A3, B3, M3, N3, K3, 0, 0, 1, O.F16, O.F32)


def test_replays_from_a_hip_graph(loader):
    """GEMM calls recorded into a HIP graph (whole tiles on the persistent kernel, a ragged
    shape, a split-K call whose scratch memory was sized by an eager call before, and a skinny
    call whose workgroups share tiles through that memory and the arrival counters) give the
    eager results on every replay, with eager work and synchronisations in between."""
    import torch

    cases = [(512, 768, 1024, 0, 0, 1), (1000, 1000, 1000, 0, 1, 0), (64, 8192, 8192, 0, 1, 0),
             (16, 1024, 8192, 0, 0, 1)]
    assert loader.select(16, 1024, 8192, 0, 0, 0, 1)[2] > 1
    ops = []
    for (M, N, K, lc, la, lb) in cases:
        A, B = make_inputs(M, N, K, la, lb, O.F16)
        dA, dB = to_device(A, O.F16), to_device(B, O.F16)
        want = torch.zeros(M * N, dtype=torch.float16, device="cuda")
        loader.gemm(want, dA, dB, M, N, K, lc, la, lb)  # eager; also sizes the scratch memory
        ops.append((dA, dB, want, torch.zeros_like(want)))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for (M, N, K, lc, la, lb), (dA, dB, _, out) in zip(cases, ops):
            loader.gemm(out, dA, dB, M, N, K, lc, la, lb)  # torch's current stream is capturing
    for replay in range(3):
        for (_, _, _, out) in ops:
            out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for case, (dA, dB, want, out) in zip(cases, ops):
            assert torch.equal(out, want), (case, replay)
        # eager work between replays, through the same scratch memory
        M, N, K, lc, la, lb = cases[2]
        loader.gemm(ops[2][3], ops[2][0], ops[2][1], M, N, K, lc, la, lb)
        torch.cuda.synchronize()
        assert torch.equal(ops[2][3], ops[2][2])


def test_cpp_client_through_this_repositorys_loader_header():
    """A C++ client of rocm_wmma_gemm::loader (all type pairs, all layouts, batched),
    bit-exact against a host loop on inputs whose sums are exact."""
    import os
    import subprocess

    exe = os.path.join(os.path.dirname(__file__), "..", "rocm_wmma_gemm_amd", "lib", "dropin_check")
    assert os.path.exists(exe), "build the tools first (make -C rocm_wmma_gemm_amd/csrc)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "DROP-IN CHECK PASSED" in r.stdout, r.stdout + r.stderr


def test_cpp_client_through_the_references_own_loader_header():
    """The same client compiled against the REFERENCE's kernel_loader.hpp (built where the
    reference tree is present, see oracle/Makefile target `ref`): the reference's loader
    finds librocm_wmma_gemm_gfx950.so by architecture name and drives it unchanged."""
    import os
    import subprocess

    exe = os.path.join(os.path.dirname(__file__), "..", "oracle", "_ref",
                       "dropin_check_reference_loader")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/dropin_check_reference_loader was not built (no reference tree)")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "DROP-IN CHECK PASSED" in r.stdout, r.stdout + r.stderr


# ---------------------------------------------------------------- full-size configurations
def _full_size_case(loader, M, N, K, lc, la, lb, tname, band_every=128, whole=False, **gen):
    """One full-size configuration: every element of C through the row/column checksums,
    and element by element against the oracle either over the whole of C (`whole`, as
    the reference's tests do, test/gemm/test_float_accum.cpp:118-136) or over one 32-row
    band in every block of `band_every` rows, so that every tile of C, whatever the
    kernel's tile size (128, 192 or 256 rows: each holds a whole aligned block of 128) and
    whichever way round it walks C, has 32 of its rows compared."""
    din, dout = TYPE_PAIRS[tname]
    A, B = make_inputs(M, N, K, la, lb, din, **gen)
    gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout)
    sums = checksum_check(gpu, A, B, M, N, K, lc, la, lb, din, dout)
    if whole:
        worst, _, _ = check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
        compared = M * N
    else:
        worst, compared = 0.0, 0
        for block in range(0, M, band_every):
            # a different place in every block, the last rows of C always among them
            r0 = min(block + (block // band_every * 96) % max(band_every - 32, 1), max(M - 32, 0))
            if block + band_every >= M:
                r0 = max(M - 32, 0)
            r1 = min(M, r0 + 32)
            w, _, _ = check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout, rows=(r0, r1))
            worst, compared = max(worst, w), compared + (r1 - r0) * N
    print(f"full-size {tname} {M}x{N}x{K} {layout_id(lc, la, lb)}: {compared} of {M * N} elements "
          f"compared with the oracle, max |err|/tol = {worst:.3f}; checksums at {sums:.3f} of "
          f"their tolerance", flush=True)


@pytest.mark.parametrize("lc,la,lb", LAYOUTS8, ids=[layout_id(*l) for l in LAYOUTS8])
def test_half_half_4096_cubed_all_layouts(loader, lc, la, lb):
    """fp16 -> fp16, M=N=K=4096, uniform[-1,1] seeded: every element of C against the
    oracle, and the row/column checksums."""
    _full_size_case(loader, 4096, 4096, 4096, lc, la, lb, "f16_f16", whole=True)


def test_float_bf16_8192_cubed(loader):
    """bf16 -> fp32, M=N=K=8192, A row / B col / C row, normal(0,1) seeded: every element
    of C against the oracle."""
    _full_size_case(loader, 8192, 8192, 8192, 0, 0, 1, "f32_bf16", whole=True,
                    dist="normal", lo=0.0, hi=1.0)


@pytest.mark.parametrize("M,N,K", [(4096, 5120, 5120), (8192, 4096, 2048), (4096, 14336, 4096),
                                   (16, 8192, 8192), (64, 8192, 8192), (128, 8192, 8192)])
def test_llm_projection_shapes(loader, M, N, K):
    """fp16 in, fp32 out, through the default dispatch (the tuned entries of these shapes) in
    A row / B column / C row, A column / B row / C row, all row-major, all column-major and
    A row / B row / C column: the skinny shapes compare the whole of C, the others in bands.
    With A column-major the 16-, 64- and 128-row shapes run the streaming kernel's
    transposing reads at N = K = 8192."""
    for (lc, la, lb) in [(0, 0, 1), (0, 1, 0), (0, 0, 0), (1, 1, 1), (1, 0, 0)]:
        _full_size_case(loader, M, N, K, lc, la, lb, "f32_f16", whole=M <= 128)


@pytest.mark.parametrize("M,N,K", [(16, 28672, 8192), (24, 8192, 28672)])
def test_a_few_rows_against_weights_beyond_the_memory_side_cache(loader, M, N, K):
    """470 MB of weights against 16 or 24 rows: the streaming kernel reads an operand of 256 MB
    and more, which one row (or column) of tiles walks exactly once, with the non-temporal
    hint.  Every element of C against the oracle, through the default dispatch and with
    streaming tiles forced (whole tiles and two workgroups per tile), B as the large operand
    (C row-major) and A (C column-major: the transposed problem)."""
    stream = {(v.block_m, v.block_n): v.index for v in loader.variants() if v.pipeline == 7}
    ran = 0
    for (lc, la, lb) in [(0, 0, 1), (0, 0, 0), (1, 1, 1), (1, 0, 1)]:
        din, dout = TYPE_PAIRS["f32_f16"]
        A, B = make_inputs(M, N, K, la, lb, din)
        check_against_oracle(run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout), A, B, M, N, K, lc, la, lb, din, dout)
        small_first = lc == 0  # kernel space: rows = M (C row-major) or N (C column-major)
        for (small, large), split in [((32, 64), 1), ((16, 64), 2), ((32, 32), 1)]:
            tile = (small, large) if small_first else (large, small)
            v = loader.variants()[stream[tile]]
            if not built_for(v, lc, la, lb, K, M, N):
                continue
            gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, variant=(v.index, 1, split))
            check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
            ran += 1
    assert ran >= 6, ran


@pytest.mark.parametrize("M,N,K", [(256, 4096, 4096), (256, 28672, 8192), (512, 14336, 4096),
                                   (512, 8192, 28672), (1024, 4096, 14336)])
def test_a_few_hundred_rows_against_projection_weights(loader, M, N, K):
    """256 to 1024 rows against transformer weight matrices, through the tuned entries of
    these shapes (the streaming kernel, the 128x128 ring of 4, the persistent kernel with
    and without a split, the ping-pong kernel with split-K, depending on shape and layout)."""
    for (lc, la, lb), tname in [((0, 0, 1), "f16_f16"), ((0, 0, 0), "bf16_bf16"), ((1, 1, 1), "f32_bf16")]:
        _full_size_case(loader, M, N, K, lc, la, lb, tname)


@pytest.mark.parametrize("M,N,K", [(4095, 5121, 3001), (1000, 1000, 1000), (1024, 1024, 65536),
                                   (8191, 8191, 8191)])
def test_edge_tile_and_long_k(loader, M, N, K):
    """Non-tile-multiple and long-K shapes; 8191^3 needs padded copies larger than the
    workspace's first allocation, so it also covers the workspace growing."""
    layouts = [(0, 0, 1), (1, 0, 0), (0, 1, 0), (1, 1, 1)] if M < 8000 else [(0, 0, 1), (1, 1, 0)]
    for (lc, la, lb) in layouts:
        _full_size_case(loader, M, N, K, lc, la, lb, "bf16_bf16", whole=M <= 1024 and K <= 1024,
                        lo=-0.5, hi=0.5)
