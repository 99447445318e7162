"""The tuner's open search space on the GPU: a tuple that the library does not hold is
compiled at run time (csrc/kernel_jit.hip), registered with the loaded library and run
through the tuner hook; its results must agree with the oracle like any compiled variant's
(role of the reference's config/tuner.cpp:237-454, which compiles and times one tuple)."""
import os
import sys

import pytest

import oracle as O
from gemm_harness import TYPE_PAIRS, check_against_oracle, make_inputs, run_gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def loader():
    import torch

    import rocm_wmma_gemm_amd as R

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    torch.cuda.set_device(0)
    return R.Loader()


def test_run_time_compiled_variants_agree_with_the_oracle(loader, tmp_path):
    sys.path.insert(0, os.path.join(ROOT, "rocm_wmma_gemm_amd", "config"))
    import tune as T

    jit = T.JitBuilder(loader._lib, cache_dir=str(tmp_path))
    compiled = {(v.block_m, v.block_n, v.block_k, v.warps_m, v.warps_n, v.pipeline) for v in loader.variants()}
    cases = [  # (tile, type pair, (lc, la, lb), (M, N, K), swizzle, split)
        (T.Tile(128, 256, 32, 2, 2, 1), "f16_f16", (0, 0, 1), (512, 768, 1024), 4, 1),   # ring of 4 x BLOCK_K 32
        (T.Tile(128, 256, 32, 2, 2, 1), "f16_f16", (1, 0, 0), (512, 768, 1024), 4, 2),   # transposed C, split-K
        (T.Tile(256, 128, 64, 2, 4, 3), "f32_bf16", (0, 0, 1), (1024, 512, 512), 8, 1),  # 16x16x32 MFMA, 8 waves
        (T.Tile(128, 256, 64, 2, 2, 3), "bf16_bf16", (0, 1, 0), (384, 768, 320), 1, 1),  # both operands M/N-contiguous
        (T.Tile(64, 128, 64, 1, 2, 0), "f32_f16", (0, 0, 1), (200, 300, 250), 1, 1),     # register-staged, ragged
    ]
    for tile, tname, (lc, la, lb), (M, N, K), sw, sk in cases:
        sig = (tile.block_m, tile.block_n, tile.block_k, tile.warps_m, tile.warps_n, tile.pipeline)
        if sig in compiled:
            continue  # adopted since: covered by the variant sweep of test_gemm_gpu.py
        ak, bk = T.kernel_space_layout(la, lb, lc)
        assert T.tile_feasible(tile, ak, bk), tile
        idx = jit.variant_index(tile, list(TYPE_PAIRS).index(tname), ak, bk)
        assert idx is not None and idx >= len(compiled), (tile, tname)
        din, dout = TYPE_PAIRS[tname]
        A, B = make_inputs(M, N, K, la, lb, din, seed_b=5)
        print(f"run-time compiled {tile} as variant {idx}: {tname} {M}x{N}x{K} layouts(C,A,B)=({lc},{la},{lb})",
              flush=True)
        gpu = run_gpu(loader, A, B, M, N, K, lc, la, lb, din, dout, variant=(idx, sw, sk))
        check_against_oracle(gpu, A, B, M, N, K, lc, la, lb, din, dout)
