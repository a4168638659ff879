"""How the weight-streaming product deals rows of the weight and steps of K to waves: for every size the plan must
name a kernel that exists and sizes that the kernel accepts (no GPU needed)."""
import random

import pytest

from atoma_infer_amd.kernels import gemm_bf16

# (rows of 16 per wave, waves that split K) that csrc/kernels/gemm_bf16.hip instantiates, per entry point
PLAIN = {(1, 1), (2, 1), (4, 1), (1, 4), (2, 4), (4, 4), (1, 8), (2, 8)}
SWIGLU = {(2, 1), (4, 1), (2, 4), (4, 4), (2, 8)}
ROPE = {(1, 1), (2, 1), (1, 4), (2, 4), (1, 8), (2, 8)}


def shapes():
    rnd = random.Random(7)
    fixed = [(n, k) for n in (16, 48, 2048, 3072, 5120, 6144, 16384, 28672, 128256) for k in (32, 96, 2048, 3072, 8192, 14336)]
    return fixed + [(rnd.randrange(1, 40000), 32 * rnd.randrange(1, 500)) for _ in range(300)]


@pytest.mark.parametrize("m", [1, 8, 16, 17, 33, 48, 49, 64])
def test_plans_name_kernels_that_exist(m):
    for n, k in shapes():
        for allow in (False, True):
            rt, wk, slices = gemm_bf16._plan(m, n, k, allow)
            assert (rt, wk) in PLAIN, (m, n, k, allow)
            assert slices >= 1 and (allow or slices == 1)
            assert k % (32 * wk * slices) == 0, (m, n, k, rt, wk, slices)
            if slices > 1:
                assert k // (wk * slices) >= 128          # a wave's share of K stays worth its launch
                groups = -(-(-(-n // 16)) // ((4 if wk == 1 else 1) * rt))
                assert groups * slices <= 1024
        # the fused epilogues adjust the plan to their own kernels
        rt, wk, _ = gemm_bf16._plan(m, n, k, False)
        r2 = rt if rt % 2 == 0 else 2
        if (r2, wk) in SWIGLU:
            assert (r2, wk) != (2, 8) or m <= 48          # eight waves of four row tiles do not exist
        assert (min(rt, 2), wk) in ROPE
        assert (min(rt, 2), wk) != (2, 8) or m <= 48


def test_few_rows_keep_their_two_planes():
    # sizes of Llama-3.2-1B: o and down projections of a decode step
    assert gemm_bf16._plan(8, 2048, 2048, True) == (1, 4, 2)
    assert gemm_bf16._plan(8, 2048, 8192, True) == (1, 4, 2)
    # more rows: about 256 workgroups
    rt, wk, slices = gemm_bf16._plan(64, 2048, 8192, True)
    assert -(-128 // rt) * slices == 256


def test_library_thresholds():
    import torch
    wins = gemm_bf16._library_wins
    assert not wins(64, 3072, 2048, torch.bfloat16) and wins(65, 3072, 2048, torch.bfloat16)
    assert wins(33, 16384, 2048, torch.bfloat16) and not wins(32, 16384, 2048, torch.bfloat16)
    assert wins(17, 128256, 2048, torch.float32) == gemm_bf16._MM_OUT_DTYPE and not wins(16, 128256, 2048, torch.float32)
    # the head: eight waves splitting K up to 8 rows, then 64 rows of W a wave and four waves splitting K
    assert [gemm_bf16._plan(m, 128256, 2048, False) for m in (8, 9, 16)] == [(2, 8, 1), (4, 4, 1), (4, 4, 1)]


# (tiles, waves splitting K, steps a batch of loads, half tiles) of the residual product in csrc/kernels/gemm_bf16.hip
RESID = {(1, 4, 4, 0), (1, 8, 4, 0), (1, 8, 2, 0), (1, 8, 8, 0), (1, 1, 4, 0),
         (1, 4, 4, 1), (1, 4, 8, 1), (1, 8, 4, 1), (1, 8, 8, 1), (1, 8, 2, 1), (1, 1, 4, 1)}


def test_residual_products_name_kernels_that_exist():
    for n, k in shapes():
        for m in (1, 8, 16):
            rt, wk, depth, half = gemm_bf16.resid_plan(m, n, k)
            assert (rt, wk, depth, half) in RESID, (m, n, k)
            assert k % (32 * wk) == 0
            if half:            # a step of half tiles covers 64 values of K, and N is small
                assert k % (64 * wk) == 0 and n <= 2048
    # Llama 1B: 8 rows of the weight a wave; 3B and 8B: whole tiles, and as many steps a batch as K allows
    assert gemm_bf16.resid_plan(8, 2048, 2048) == (1, 8, 4, 1) and gemm_bf16.resid_plan(8, 2048, 8192) == (1, 8, 4, 1)
    assert gemm_bf16.resid_plan(8, 3072, 8192) == (1, 8, 8, 0) and gemm_bf16.resid_plan(8, 4096, 14336) == (1, 8, 8, 0)
    assert gemm_bf16.resid_plan(8, 3072, 3072) == (1, 8, 4, 0)
