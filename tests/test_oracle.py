"""Pins the CPU oracle: reference known answers, closed forms, brute force.

None of these checks retypes the oracle's formula: the fixtures come from the
reference's own C++ oracle, and the rest are facts the mathematics fixes
(identity, one-hot, all-ones, float64 brute force, a library matmul).
"""
import json
import os

import numpy as np
import pytest

import oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "oracle_kat.json")))
LAY = {"row": O.ROW, "col": O.COL}
DT = {"f16": O.F16, "bf16": O.BF16, "f32": O.F32}


def test_mt19937_known_answers():
    # The 10000th consecutive draw of a default-seeded (5489) mt19937 is fixed by
    # the C++ standard [rand.predef]; seed 1's first draw is the textbook value.
    assert int(O.raw_draws(5489, 10000)[-1]) == 4123659995
    assert int(O.raw_draws(1, 1)[0]) == 1791095845


def test_uniform_first_six_match_reference_generator():
    got = O.uniform_draws(1, -1.0, 1.0, 6)
    want = np.array(GOLD["uniform_seed1_first6"], dtype=np.float32)
    assert np.array_equal(got, want), (got, want)


def test_uniform_draws_match_the_standard_librarys_generator(tmp_path):
    """The reference draws its inputs with libstdc++'s mt19937 and
    uniform_real_distribution<float> (test/test.hpp:36-38).  tests/golden/
    record_uniform_draws.cpp is that pair and nothing else; the oracle's generator must give
    the same floats, bit for bit, for the reference's range, the harness's other range and
    an asymmetric one, and the fixture's six values are the head of the first."""
    import subprocess

    src = os.path.join(os.path.dirname(__file__), "golden", "record_uniform_draws.cpp")
    exe = str(tmp_path / "record_uniform_draws")
    subprocess.run(["g++", "-O1", "-std=c++17", src, "-o", exe], check=True)
    for seed, lo, hi, count in [(1, -1.0, 1.0, 100000), (1, -0.5, 0.5, 100000), (7, 0.25, 3.0, 20000)]:
        r = subprocess.run([exe, str(seed), repr(lo), repr(hi), str(count)], capture_output=True,
                           text=True, check=True)
        want = np.array([float.fromhex(t) for t in r.stdout.split()], dtype=np.float32)
        got = O.uniform_draws(seed, lo, hi, count)
        assert want.size == count and np.array_equal(got, want), (seed, lo, hi)
        if (seed, lo, hi) == (1, -1.0, 1.0):
            assert np.array_equal(want[:6], np.array(GOLD["uniform_seed1_first6"], dtype=np.float32))


def test_uniform_range_and_moments():
    u = O.uniform_draws(1, -1.0, 1.0, 100000)
    assert u.min() >= -1.0 and u.max() < 1.0
    assert abs(float(u.mean())) < 0.01 and abs(float(u.var()) - 1.0 / 3.0) < 0.01


def test_normal_draws_are_standard_normal():
    """dist='normal' (Box-Muller; harness-only, the 8192^3 configuration's inputs) is what
    it says: moments and a Kolmogorov-Smirnov test against the normal distribution on a
    million values, mean and deviation applied as given, both members of every pair used
    (an odd count keeps the order), and the storage layout does not change the values."""
    from scipy import stats

    n = 1 << 20
    x = O.init_matrix(1024, 1024, O.ROW, O.F32, seed=1, dist="normal", lo=0.0, hi=1.0).astype(np.float64)
    assert abs(x.mean()) < 5.0 / np.sqrt(n)
    assert abs(x.var() - 1.0) < 5.0 * np.sqrt(2.0 / n)
    assert abs(stats.skew(x)) < 5.0 * np.sqrt(6.0 / n)
    assert abs(stats.kurtosis(x)) < 5.0 * np.sqrt(24.0 / n)
    assert stats.kstest(x, "norm").pvalue > 1e-3
    # even and odd members of the pairs are each normal and uncorrelated with each other
    assert stats.kstest(x[0::2], "norm").pvalue > 1e-3 and stats.kstest(x[1::2], "norm").pvalue > 1e-3
    assert abs(np.corrcoef(x[0::2], x[1::2])[0, 1]) < 5.0 / np.sqrt(n / 2)
    assert abs(np.corrcoef(x[:-1], x[1:])[0, 1]) < 5.0 / np.sqrt(n)
    assert 4.5 < np.abs(x).max() < 6.5  # tails are there, and nothing is infinite
    # mean and deviation
    y = O.init_matrix(1024, 1024, O.ROW, O.F32, seed=1, dist="normal", lo=3.0, hi=0.5).astype(np.float64)
    assert np.allclose(y, 3.0 + 0.5 * x, rtol=0, atol=1e-6)
    # a different seed gives different values; the same seed the same ones
    assert not np.array_equal(O.init_matrix(8, 8, O.ROW, O.F32, seed=2, dist="normal", lo=0.0, hi=1.0),
                              x[:64].astype(np.float32))
    # draw order is logical (row by row) whatever the storage, as for the uniform inputs
    r = O.init_matrix(5, 7, O.ROW, O.F32, seed=1, dist="normal", lo=0.0, hi=1.0)
    c = O.init_matrix(5, 7, O.COL, O.F32, seed=1, dist="normal", lo=0.0, hi=1.0)
    assert np.array_equal(r.reshape(5, 7), c.reshape(7, 5).T)
    assert np.array_equal(r, x[:35].astype(np.float32))
    # narrowing is the oracle's own round-to-nearest-even conversion
    b = O.init_matrix(5, 7, O.ROW, O.BF16, seed=1, dist="normal", lo=0.0, hi=1.0)
    import torch

    want = torch.from_numpy(r).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(b, want)


def test_f16_conversion_exhaustive_against_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    L = O.lib()
    wide = np.array([L.oracle_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    ref = bits.view(np.float16).astype(np.float32)
    ok = (wide == ref) | (np.isnan(wide) & np.isnan(ref))
    assert ok.all()
    # round trip is the identity on every non-NaN pattern
    finite = ~np.isnan(ref)
    back = O.f32_to_f16_bits(ref[finite])
    assert np.array_equal(back, bits[finite])


def test_f32_to_f16_rounding_against_numpy():
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-5).astype(np.float32),   # subnormal halves
        (rng.standard_normal(5000) * 1e-8).astype(np.float32),   # underflow
        (rng.standard_normal(2000) * 7e4).astype(np.float32),    # overflow edge
        np.array([65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 0.0, -0.0,
                  np.inf, -np.inf], dtype=np.float32),
        # exact ties between neighbouring halves
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) / 1024.0,
    ])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16_bits(x), want)


def test_bf16_conversion_rne():
    import torch

    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32),
                        np.array([1.00390625, 1.01171875, 3.3895314e38, 0.0, -0.0],
                                 dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(x), want)
    # 1 + 2^-8 ties to even (1.0); 1 + 3*2^-8 ties to even (1 + 2^-6)
    assert O.f32_to_bf16_bits(np.float32(1.00390625)) == 0x3F80
    assert O.f32_to_bf16_bits(np.float32(1.01171875)) == 0x3F82
    assert np.array_equal(O.bits_to_f32(want, O.BF16).view(np.uint32) & 0xFFFF,
                          np.zeros_like(want, dtype=np.uint32))


def test_init_matrix_draw_order_and_shared_stream():
    # A(i,k) = r[i*K+k], B(k,j) = r[k*N+j] for the same stream r, whatever the storage.
    M, K = 5, 7
    r = O.uniform_draws(1, -1.0, 1.0, M * K)
    for lay in (O.ROW, O.COL):
        flat = O.init_matrix(M, K, lay, O.F32)
        assert np.array_equal(O.logical(flat, M, K, lay), r.reshape(M, K))
    f16 = O.init_matrix(M, K, O.COL, O.F16)
    assert np.array_equal(O.logical(f16, M, K, O.COL), r.reshape(M, K).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("case", GOLD["gemm"], ids=lambda c: "%s_%s_%dx%dx%d_%s%s%s" % (
    c["in"], c["out"], c["M"], c["N"], c["K"], c["A"][0], c["B"][0], c["C"][0]))
@pytest.mark.parametrize("naive", [False, True], ids=["fast", "naive"])
def test_gemm_reference_known_answers(case, naive):
    M, N, K = case["M"], case["N"], case["K"]
    la, lb, lc = LAY[case["A"]], LAY[case["B"]], LAY[case["C"]]
    din, dout = DT[case["in"]], DT[case["out"]]
    if naive and M * N * K > 256 ** 3:
        pytest.skip("naive form only on the smaller fixtures")
    A = O.init_matrix(M, K, la, din)
    B = O.init_matrix(K, N, lb, din)
    C = O.gemm(A, B, M, N, K, lc, la, lb, din, dout, naive=naive, threads=4)
    assert O.fnv1a64(C, GOLD["fnv_basis"]) == case["fnv"]
    Cl = O.bits_to_f32(O.logical(C, M, N, lc), dout)
    for key, want in case["elems"].items():
        i, j = map(int, key.split(","))
        assert Cl[i, j] == np.float32(want), (key, Cl[i, j], want)
    if "sum" in case:
        assert abs(float(Cl.astype(np.float64).sum()) - case["sum"]) < 1e-3 * max(1.0, abs(case["sum"])) * 1e-2 + 1e-3
    if "abs_sum" in case:
        assert abs(float(np.abs(Cl.astype(np.float64)).sum()) - case["abs_sum"]) < 0.05


LAYOUTS8 = [(lc, la, lb) for lc in (0, 1) for la in (0, 1) for lb in (0, 1)]


@pytest.mark.parametrize("lc,la,lb", LAYOUTS8)
def test_gemm_identity_and_onehot_pin_every_layout(lc, la, lb):
    M, N, K = 6, 9, 6
    rng = np.random.default_rng(0)
    Bl = rng.integers(-8, 8, size=(K, N)).astype(np.float32)

    def store(mat, lay):
        return np.ascontiguousarray(mat if lay == O.ROW else mat.T).ravel()

    eye = np.eye(M, K, dtype=np.float32)
    C = O.gemm(store(eye, la), store(Bl, lb), M, N, K, lc, la, lb, O.F32, O.F32, threads=2)
    assert np.array_equal(O.logical(C, M, N, lc), Bl)
    # one-hot A(i0,k0): C row i0 is B row k0 and nothing else; a transposed operand
    # or a swapped index would put it elsewhere.
    Al = np.zeros((M, K), dtype=np.float32)
    Al[4, 1] = 2.0
    C = O.logical(O.gemm(store(Al, la), store(Bl, lb), M, N, K, lc, la, lb, O.F32, O.F32), M, N, lc)
    want = np.zeros((M, N), dtype=np.float32)
    want[4] = 2.0 * Bl[1]
    assert np.array_equal(C, want)


@pytest.mark.parametrize("din,dout,K", [(O.F16, O.F16, 2048), (O.BF16, O.BF16, 256), (O.F16, O.F32, 4096)])
def test_gemm_all_ones_is_K(din, dout, K):
    M, N = 3, 70
    one = 0x3C00 if din == O.F16 else 0x3F80
    A = np.full(M * K, one, dtype=np.uint16)
    B = np.full(K * N, one, dtype=np.uint16)
    C = O.bits_to_f32(O.gemm(A, B, M, N, K, O.ROW, O.ROW, O.COL, din, dout), dout)
    assert np.array_equal(C, np.full(M * N, float(K), dtype=np.float32))


@pytest.mark.parametrize("din", [O.F16, O.BF16])
@pytest.mark.parametrize("lc,la,lb", [(0, 0, 1), (1, 1, 0), (0, 1, 1)])
def test_gemm_float64_bruteforce_and_library_matmul(din, lc, la, lb):
    import torch

    M, N, K = 33, 65, 47  # ragged on purpose: exercises the partial column strip
    A = O.init_matrix(M, K, la, din, seed=11)
    B = O.init_matrix(K, N, lb, din, seed=12)
    C, S = O.gemm(A, B, M, N, K, lc, la, lb, din, O.F32, want_scale=True)
    Al = O.bits_to_f32(O.logical(A, M, K, la), din).astype(np.float64)
    Bl = O.bits_to_f32(O.logical(B, K, N, lb), din).astype(np.float64)
    exact = Al @ Bl
    Sx = np.abs(Al) @ np.abs(Bl)
    Cl = O.logical(C, M, N, lc).astype(np.float64)
    assert np.all(np.abs(Cl - exact) <= K * 2.0 ** -24 * Sx)
    assert np.allclose(S.reshape(M, N), Sx, rtol=1e-5)
    tm = torch.matmul(torch.from_numpy(Al.astype(np.float32)), torch.from_numpy(Bl.astype(np.float32))).numpy()
    assert np.all(np.abs(Cl - tm) <= 2 * K * 2.0 ** -24 * Sx)
    # naive and fast forms are the same function, bit for bit
    Cn = O.gemm(A, B, M, N, K, lc, la, lb, din, O.F32, naive=True)
    assert np.array_equal(C, Cn)


def test_gemm_power_of_two_entries_are_order_independent():
    # sums of small integers are exact in fp32, so any k order gives the same bits
    rng = np.random.default_rng(5)
    M, N, K = 16, 24, 512
    Al = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    Bl = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    A = Al.astype(np.float16).view(np.uint16).ravel()
    B = np.ascontiguousarray(Bl.T).astype(np.float16).view(np.uint16).ravel()
    C = O.gemm(A, B, M, N, K, O.ROW, O.ROW, O.COL, O.F16, O.F32)
    assert np.array_equal(C.reshape(M, N), Al @ Bl)


def test_gemm_row_subset_matches_full():
    M, N, K = 40, 50, 64
    A = O.init_matrix(M, K, O.ROW, O.BF16)
    B = O.init_matrix(K, N, O.COL, O.BF16)
    full = O.gemm(A, B, M, N, K, O.ROW, O.ROW, O.COL, O.BF16, O.BF16).reshape(M, N)
    part = O.gemm(A, B, M, N, K, O.ROW, O.ROW, O.COL, O.BF16, O.BF16, rows=(7, 19)).reshape(M, N)
    assert np.array_equal(part[7:19], full[7:19])
    assert not part[:7].any() and not part[19:].any()


def test_col_major_c_is_row_major_of_transposed_problem():
    M, N, K = 12, 20, 32
    A = O.init_matrix(M, K, O.ROW, O.F16, seed=2)
    B = O.init_matrix(K, N, O.ROW, O.F16, seed=3)
    c_col = O.gemm(A, B, M, N, K, O.COL, O.ROW, O.ROW, O.F16, O.F16)
    # C^T (N x M, row-major) = B^T (N x K: the same buffer read column-major) * A^T
    c_t = O.gemm(B, A, N, M, K, O.ROW, O.COL, O.COL, O.F16, O.F16)
    assert np.array_equal(c_col, c_t)


def test_cosine_similarity_cases():
    m, n = 8, 8
    a = O.init_matrix(m, n, O.ROW, O.F16)
    assert abs(O.cosine_similarity(a, a, m, n, O.ROW, O.F16) - 1.0) < 1e-6
    neg = a ^ np.uint16(0x8000)
    assert abs(O.cosine_similarity(a, neg, m, n, O.ROW, O.F16) + 1.0) < 1e-6
    z = np.zeros(m * n, dtype=np.uint16)
    assert O.cosine_similarity(z, z, m, n, O.ROW, O.F16) == 1.0   # both near zero
    assert O.cosine_similarity(z, a, m, n, O.ROW, O.F16) == 0.0   # one zero, one not
    assert O.cosine_threshold(O.F16) == np.float32(0.995)
    assert O.cosine_threshold(O.BF16) == np.float32(0.97)
    # orthogonal vectors
    e1 = np.zeros(m * n, dtype=np.float32); e1[0] = 1
    e2 = np.zeros(m * n, dtype=np.float32); e2[1] = 1
    assert O.cosine_similarity(e1, e2, m, n, O.ROW, O.F32) == 0.0


def test_fnv1a64_known_vectors():
    # published FNV-1a test vectors
    assert O.fnv1a64(np.frombuffer(b"a", dtype=np.uint8)) == "af63dc4c8601ec8c"
    assert O.fnv1a64(np.frombuffer(b"foobar", dtype=np.uint8)) == "85944171f73967e8"


def test_checksums_see_one_wrong_tile():
    """The row/column checksum check of the GPU tests (tests/gemm_harness.py) on the CPU:
    the oracle's own result passes, and so does a result from a different summation order;
    a result with one K tile of 64 missing from one 128 x 128 tile, or with one tile from
    another problem, fails."""
    import sys

    sys.path.insert(0, os.path.dirname(__file__))
    from gemm_harness import checksum_check

    M, N, K = 512, 384, 2048
    for din, dout in [(O.F16, O.F16), (O.BF16, O.F32)]:
        A = O.init_matrix(M, K, O.ROW, din, seed=1)
        B = O.init_matrix(K, N, O.COL, din, seed=2)
        good = O.gemm(A, B, M, N, K, O.ROW, O.ROW, O.COL, din, dout)
        assert checksum_check(good, A, B, M, N, K, O.ROW, O.ROW, O.COL, din, dout) < 0.5
        Af = O.bits_to_f32(A, din).reshape(M, K).astype(np.float64)
        Bf = O.bits_to_f32(B, din).reshape(N, K).T.astype(np.float64)
        exact = Af @ Bf
        def narrow(x):
            if dout == O.F32:
                return x.astype(np.float32).ravel()
            return x.astype(np.float16).view(np.uint16).ravel()
        other_order = narrow(exact)  # float64 sums, rounded once: another legal result
        assert checksum_check(other_order, A, B, M, N, K, O.ROW, O.ROW, O.COL, din, dout) < 0.5
        dropped = exact.copy()
        dropped[128:256, 256:384] -= Af[128:256, 64:128] @ Bf[64:128, 256:384]
        with pytest.raises(AssertionError, match="checksum outside tolerance"):
            checksum_check(narrow(dropped), A, B, M, N, K, O.ROW, O.ROW, O.COL, din, dout)
        swapped = exact.copy()
        swapped[0:128, 0:128] = exact[256:384, 128:256]
        with pytest.raises(AssertionError, match="checksum outside tolerance"):
            checksum_check(narrow(swapped), A, B, M, N, K, O.ROW, O.ROW, O.COL, din, dout)
