"""The library's choice between its bfloat16 product kernels: every kernel says how long it expects to take for a
size (a model fitted to measurements, beside the kernel's code) and the smallest figure wins.  Host functions: no
GPU is needed, only the built library."""
import pytest

from simply_amd.kernels import build


@pytest.fixture(scope="module")
def ops():
    if build.find_library() is None:
        pytest.skip("the kernel library has not been built here")
    from simply_amd.kernels import ops
    return ops


def test_few_rows_stream_through_the_few_rows_kernel_and_many_through_the_wide_one(ops):
    for N, K in ((4096, 2304), (2304, 2048), (3072, 3072), (1024, 1024), (8192, 3584), (2560, 2560)):
        for M in (1, 4, 8):
            assert ops.gemm_plan(M, N, K)[0] == ops.ALGO_SKINNY, (M, N, K)
        for M in (48, 64, 300, 2048):
            assert ops.gemm_plan(M, N, K)[0] == ops.ALGO_WIDE, (M, N, K)


def test_a_long_k_goes_to_the_kernels_that_cut_it(ops):
    """Against a very long K the few-rows kernel's workgroups, a few to a CU, walk all of it at a CU's pace; the wide
    kernel cuts K over workgroups (the 27B down projection: 62 against 76 us at one row)."""
    assert ops.gemm_plan(1, 4608, 36864)[0] == ops.ALGO_WIDE
    assert ops.gemm_plan(16, 2304, 9216)[0] == ops.ALGO_WIDE        # 13 against 17 us
    assert ops.gemm_plan(4, 2304, 9216)[0] == ops.ALGO_SKINNY       # 11 against 14 us
    assert ops.gemm_plan(16, 2048, 16384)[0] == ops.ALGO_WIDE       # a size of no model


def test_the_head_over_a_large_vocabulary(ops):
    """float32 out with a soft-cap: the wide kernel does not take it; up to a few rows the few-rows kernel, then the
    tiled one, whose workgroups do not read the rows of activations once each."""
    import torch
    kw = dict(soft_cap=True, out_dtype=torch.float32)
    kernel, us = ops.gemm_plan(1, 256000, 2304, **kw)
    assert kernel == ops.ALGO_SKINNY and us["wide"] < 0
    assert ops.gemm_plan(16, 256000, 2304, **kw)[0] == ops.ALGO_TILED
    assert ops.gemm_plan(64, 256000, 2304, **kw)[0] == ops.ALGO_TILED


def test_gated_products(ops):
    for N, K in ((9216, 2304), (14336, 3584), (8192, 3072)):
        assert ops.gemm_plan(4, N, K, gated=True)[0] == ops.ALGO_SKINNY
        kernel, us = ops.gemm_plan(32, N, K, gated=True)
        assert kernel == ops.ALGO_WIDE and us["skinny"] < 0      # the few-rows kernel has one block of 16 rows for them


def test_expected_times_grow_with_the_work(ops):
    for name in ("skinny", "tiled", "wide"):
        small, large = ops.gemm_plan(8, 2304, 2048)[1][name], ops.gemm_plan(8, 4608, 36864)[1][name]
        assert 0 < small < large, name
    assert ops.gemm_plan(2048, 2304, 9216)[1]["wide"] > 3 * ops.gemm_plan(256, 2304, 9216)[1]["wide"]
    # what no fast kernel takes (K that is no multiple of 8) is left to the kernel that takes every size
    kernel, us = ops.gemm_plan(4, 100, 100)
    assert kernel == ops.ALGO_GENERIC and all(v < 0 for v in us.values())
