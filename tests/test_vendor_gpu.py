"""The vendor wrapper (libvendor_gemm.so: rocBLAS and hipBLASLt behind the GEMM library's
argument conventions) against the CPU oracle, as the reference tests its rocBLAS wrapper
(reference test/rocblas/test.cpp: cosine similarity of the whole of C against hgemm_cpu) --
here for both backends, every layout of A, B and C, the four type pairs and a strided batch.
What is checked is the wrapper's operand mapping; the numbers it is there for are context
lines of the benchmarks."""
import numpy as np
import pytest

import oracle as O
from gemm_harness import LAYOUTS8, TYPE_PAIRS, check_against_oracle, layout_id, make_inputs, to_device, to_host, torch_dtype

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def vendor():
    import torch

    from rocm_wmma_gemm_amd.vendor import VendorGemm

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    torch.cuda.set_device(0)
    v = VendorGemm()
    yield v
    v.close()


@pytest.mark.parametrize("backend", ["rocblas", "hipblaslt"])
@pytest.mark.parametrize("lc,la,lb", LAYOUTS8, ids=[layout_id(*l) for l in LAYOUTS8])
def test_vendor_wrapper_agrees_with_the_oracle(vendor, backend, lc, la, lb):
    import torch

    for tname, (M, N, K) in zip(TYPE_PAIRS, [(256, 128, 192), (320, 448, 256), (128, 384, 512), (192, 64, 320)]):
        din, dout = TYPE_PAIRS[tname]
        A, B = make_inputs(M, N, K, la, lb, din, seed_b=2)
        dA, dB = to_device(A, din), to_device(B, din)
        dC = torch.full((M * N,), float("nan"), dtype=torch_dtype(dout), device="cuda")
        vendor.gemm(backend, dC, dA, dB, M, N, K, lc, la, lb)
        torch.cuda.synchronize()
        gpu = to_host(dC, dout)
        check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
        cpu = O.gemm(A, B, M, N, K, lc, la, lb, din, dout)
        assert O.cosine_similarity(gpu, cpu, M, N, lc, dout) > O.cosine_threshold(dout)


@pytest.mark.parametrize("backend", ["rocblas", "hipblaslt"])
def test_vendor_wrapper_strided_batch(vendor, backend):
    import torch

    M, N, K, batch = 192, 128, 256, 3
    for (lc, la, lb) in [(0, 0, 1), (1, 1, 0)]:
        As = [O.init_matrix(M, K, la, O.F16, seed=1 + b) for b in range(batch)]
        Bs = [O.init_matrix(K, N, lb, O.F16, seed=11 + b) for b in range(batch)]
        dA, dB = to_device(np.concatenate(As), O.F16), to_device(np.concatenate(Bs), O.F16)
        dC = torch.full((M * N * batch,), float("nan"), dtype=torch.float32, device="cuda")
        vendor.gemm(backend, dC, dA, dB, M, N, K, lc, la, lb, batch_count=batch)
        torch.cuda.synchronize()
        gpu = to_host(dC, O.F32)
        for b in range(batch):
            check_against_oracle(gpu[b * M * N:(b + 1) * M * N], As[b], Bs[b], M, N, K, lc, la, lb, O.F16, O.F32)
