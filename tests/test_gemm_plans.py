"""The launch planner of the staged GEMM kernels (host arithmetic only: no GPU needed).  The products of the headline
train step and of the op suite must keep their single launches; shapes whose tile count leaves the last round of
workgroups mostly empty are cut into a block of whole rounds plus strips, or along k."""
from __future__ import annotations

import pytest

from zigrad_amd.device import gemm_plan


@pytest.mark.parametrize("shape,tile", [
    ((4096, 4096, 4096), (256, 128)),   # the op suite's matmul and five of the wide MLP's eight products
    ((4096, 1024, 4096), (128, 128)),   # last layer forward
    ((1024, 4096, 4096), (128, 128)),   # last layer weight gradient
    ((4096, 4096, 1024), (256, 128)),   # last layer input gradient
    ((512, 512, 512, 32), (256, 128)),  # the op suite's batched product
])
def test_benchmark_products_stay_single_launches(shape, tile):
    p = gemm_plan(*shape)
    assert p["kind"] == "single" and p["tile"] == tile and p["splits"] == 1


def test_off_grid_cubes_are_cut_into_whole_rounds_plus_strips():
    p = gemm_plan(4100, 4100, 4100)   # 4096 x 4096 is two exact rounds; 4 rows and 4 columns are left over
    assert p["kind"] == "parts" and p["main_tiles"] == (16, 32)
    p = gemm_plan(3600, 2308, 1541)
    assert p["kind"] == "parts"


def test_whole_tiles_that_leave_a_round_part_empty_get_their_tail_in_pieces():
    p = gemm_plan(1536, 1536, 1536)   # 576 tiles of 64 x 64: two rounds of 256 whole, 64 tiles in 4 pieces each = 256 pieces
    assert p["kind"] == "tail_in_pieces" and p["tile"] == (64, 64) and p["whole_tiles"] == 512 and p["splits"] == 4
    assert p["k_tiles_per_split"] == 24
    p = gemm_plan(3072, 3072, 3072)   # 576 tiles of 128 x 128
    assert p["kind"] == "tail_in_pieces" and p["tile"] == (128, 128) and p["whole_tiles"] == 512
    for shape in ((1536, 1536, 1234), (2560, 2560, 2560), (3584, 3584, 3584), (2560, 3328, 1024)):
        p = gemm_plan(*shape)
        assert p["kind"] == "tail_in_pieces" and p["whole_tiles"] % 256 == 0 and p["whole_tiles"] > 0
        assert p["k_tiles_per_split"] % 2 == 0 and p["k_tiles_per_split"] >= 8
        assert (p["splits"] - 1) * p["k_tiles_per_split"] * 16 < shape[2] <= p["splits"] * p["k_tiles_per_split"] * 16
    # nothing to gain: a whole number of rounds, fewer tiles than CUs, tiles that end inside C, a batch
    for shape in ((2048, 2048, 2048), (4096, 4096, 4096), (768, 768, 768), (1540, 1536, 1536), (1536, 1536, 1536, 2)):
        assert gemm_plan(*shape)["kind"] != "tail_in_pieces", shape


def test_deep_products_on_few_tiles_are_cut_along_k():
    # first layer of the batch-64 MLP, first layer of the GCN: in the layouts the one-launch kernel for deep products
    # of k-contiguous operands does not take (that kernel is not planned, like the unstaged one for small products)
    for shape in ((64, 128, 784), (2708, 16, 1433)):
        p = gemm_plan(*shape)
        assert p["kind"] == "split_k" and p["tile"] == (64, 64) and p["splits"] >= 2
        assert p["k_tiles_per_split"] % 2 == 0 and p["splits"] * p["k_tiles_per_split"] * 16 >= shape[2]


def test_ranges_of_k_on_few_tiles_get_a_compute_unit_each_and_stay_long():
    # up to 32 tiles of 64 x 64: at most one range per compute unit and at most 16 ranges (256 values of k and more each
    # at k = 4096), and a product of 25 k-tiles is cut once every range has a compute unit to itself
    for shape in ((256, 256, 4096), (64, 64, 4096), (500, 64, 4096), (500, 256, 2048), (1024, 64, 2048), (500, 64, 385)):
        p = gemm_plan(*shape)
        tiles = -(-shape[0] // 64) * -(-shape[1] // 64)
        assert p["kind"] == "split_k" and p["tile"] == (64, 64), shape
        assert 2 <= p["splits"] <= 16 and tiles * p["splits"] <= 256, (shape, p)
        assert (p["splits"] - 1) * p["k_tiles_per_split"] * 16 < shape[2] <= p["splits"] * p["k_tiles_per_split"] * 16
    assert gemm_plan(256, 256, 4096)["k_tiles_per_split"] == 16
    # ranges that would need a second round keep the higher bar: these stay whole
    for shape in ((768, 768, 768), (1024, 500, 512)):
        assert gemm_plan(*shape)["kind"] == "single", shape


def test_plans_are_a_function_of_the_shape_only():
    assert gemm_plan(3072, 3072, 3072) == gemm_plan(3072, 3072, 3072)
    with pytest.raises(Exception):
        gemm_plan(0, 16, 16)
