"""Launch plans of the kernels a record is re-routed to (smelt_hip_plan_qmm / smelt_hip_plan_matvec):
the rules of the choice, checked over a sweep of shapes without a device."""
import itertools

import pytest

from smelt_amd import compiler as cc

CUS, LDS = 256, 160 * 1024
SHAPES = [(9216, 2560), (2560, 9216), (17408, 5120), (5120, 17408), (5120, 5120), (1024, 5120),
          (1000, 6144), (64, 512), (151936, 2560), (24, 1024)]
BATCHES = [1, 2, 7, 8, 9, 16, 31, 32, 33, 64, 127, 128, 129, 200, 256, 512, 1024, 4096]


def ceil_div(a, b):
    return (a + b - 1) // b


def qmt_min_batch(rows, cols, nmat):
    """From how many tokens the token-tile kernel takes a group-64 record: the larger the matrix, the sooner."""
    weights = rows * cols * nmat
    if weights < 5 << 20:
        return 1024 if weights < 2 << 20 else 384
    if weights >= 40 << 20 and rows >= 3584:
        return 33
    return 96 if weights >= 20 << 20 and rows >= 2560 else 128


def test_token_tile_threshold_by_matrix_size():
    for rows, cols, first in [(5120, 25600, 33), (4096, 12288, 33), (8192, 8192, 33), (18944, 3584, 33), (5120, 5120, 96),
                              (9216, 2560, 96), (2560, 9216, 96), (2048, 16384, 128), (4096, 4096, 128), (6144, 1024, 128),
                              (1024, 1024, 1024), (3072, 1024, 384), (2048, 2048, 384)]:
        assert cc.plan_qmm(rows, cols, 64, 1, first - 1, CUS, LDS)["kernel"] == 1, (rows, cols)
        assert cc.plan_qmm(rows, cols, 64, 1, first, CUS, LDS)["kernel"] == 2, (rows, cols)


@pytest.mark.parametrize("nmat", [1, 2])
def test_qmm_plans_cover_the_output_and_fit_the_machine(nmat):
    for (rows, cols), batch in itertools.product(SHAPES, BATCHES):
        p = cc.plan_qmm(rows, cols, 64, nmat, batch, CUS, LDS)
        assert p is not None, (rows, cols, batch)
        assert p["lds"] <= LDS and p["threads"] <= 1024 and p["threads"] % 64 == 0
        if p["kernel"] == 1:       # streaming: 16 * rt rows, 16 tokens per workgroup, no workspace
            assert batch < qmt_min_batch(rows, cols, nmat) or cols % 512
            assert p["grid_x"] * 16 * p["row_tiles"] >= rows > (p["grid_x"] - 1) * 16 * p["row_tiles"]
            assert p["grid_y"] == ceil_div(batch, 16) and p["grid_z"] == 1 and p["workspace"] == 0
            assert p["threads"] == 64 * p["k_waves"]
        else:                      # token tiles: 64 tokens, 32 * rt rows (16 * rt of each matrix when split by wave)
            assert p["kernel"] == 2 and batch >= qmt_min_batch(rows, cols, nmat) and cols % 512 == 0
            bn = (16 if p["per_wave"] else 32) * p["row_tiles"]
            assert p["grid_x"] == ceil_div(rows, bn) and p["grid_y"] == ceil_div(batch, 64)
            assert p["threads"] == 256 * p["k_waves"]
            assert p["per_wave"] == 0 or nmat == 2
            # a K slice is at least six 512-column blocks; a split needs room for its partial sums
            assert 1 <= p["ksplit"] == p["grid_z"] <= max(1, cols // 512 // 6)
            assert (p["workspace"] > 0) == (p["ksplit"] > 1)
            if p["ksplit"] > 1:
                tiles = p["grid_x"] * p["grid_y"]
                assert tiles < 2 * CUS              # only grids that leave the machine short are split
                assert p["workspace"] >= tiles * p["ksplit"] * bn * 64 * 4 * nmat // (2 if p["per_wave"] else 1) // 2


def test_streaming_plan_rows_of_256_column_multiples_and_tall_matrices():
    # rows of a multiple of 256 columns stream at every batch (the token-tile kernel takes multiples of 512 only)
    for batch in (2, 8, 100, 512):
        p = cc.plan_qmm(4096, 11008, 64, 1, batch, CUS, LDS)
        assert p is not None and p["kernel"] == 1 and p["grid_y"] == ceil_div(batch, 16)
    assert cc.plan_qmm(4096, 11008 + 128, 64, 1, 8, CUS, LDS) is None
    # groups of 128 columns stream too (rows of a multiple of 512 columns), at every batch; other groups do not
    for batch in (2, 8, 300):
        p = cc.plan_qmm(4096, 4096, 128, 1, batch, CUS, LDS)
        assert p is not None and p["kernel"] == 1
    p = cc.plan_qmm(16384, 4096, 32, 1, 16, CUS, LDS)       # groups of 32 columns: one row tile per wave
    assert p is not None and p["kernel"] == 1 and p["row_tiles"] == 1
    assert cc.plan_qmm(4096, 11008, 128, 1, 8, CUS, LDS) is None and cc.plan_qmm(4096, 4096, 16, 1, 8, CUS, LDS) is None
    assert cc.plan_qmm(4096, 4096 + 128, 32, 1, 8, CUS, LDS) is None
    # matrices of many rows: about 3500 waves in the launch, at least four per workgroup, none idle
    for rows, cols, want in [(17408, 5120, 4), (14336, 4096, 4), (8192, 8192, 8), (9216, 2560, 5), (4096, 4096, 8), (5120, 5120, 10)]:
        assert cc.plan_qmm(rows, cols, 64, 1, 8, CUS, LDS)["k_waves"] == want, (rows, cols)


def test_qmm_k_split_needs_the_workspace():
    with_ws = cc.plan_qmm(2560, 9216, 64, 1, 512, CUS, LDS)
    assert with_ws["ksplit"] > 1
    without = cc.plan_qmm(2560, 9216, 64, 1, 512, CUS, LDS, workspace_bytes=with_ws["workspace"] - 1)
    assert without["ksplit"] == 1 and without["grid_z"] == 1 and without["workspace"] == 0
    assert {k: without[k] for k in ("kernel", "row_tiles", "k_waves", "grid_x", "grid_y", "lds")} == \
           {k: with_ws[k] for k in ("kernel", "row_tiles", "k_waves", "grid_x", "grid_y", "lds")}


def test_streaming_plan_keeps_two_workgroups_per_unit_when_the_launch_has_them():
    """A long row's scale table takes a large share of LDS: a launch of more workgroups than compute units takes
    fewer waves (more steps each) so that two workgroups fit a unit together; a launch that gives every unit at
    most one workgroup keeps its twelve waves."""
    one_round = cc.plan_qmm(2560, 9216, 64, 1, 16, CUS, LDS)
    assert one_round["kernel"] == 1 and one_round["grid_x"] * one_round["grid_y"] <= CUS
    assert one_round["k_waves"] == 12 and 2 * one_round["lds"] > LDS
    for rows, cols in [(2560, 9216), (5120, 17408), (4096, 14336)]:
        p = cc.plan_qmm(rows, cols, 64, 1, 32, CUS, LDS)
        assert p["kernel"] == 1 and p["grid_x"] * p["grid_y"] > CUS
        assert 2 * p["lds"] <= LDS and 2 <= p["k_waves"] < 12
        # every wave has work: no wave past the last pair of scale groups
        pairs = cols // 128
        steps = ceil_div(pairs, p["k_waves"])
        assert (p["k_waves"] - 1) * steps < pairs
    # short rows never needed it
    assert cc.plan_qmm(9216, 2560, 64, 1, 32, CUS, LDS)["k_waves"] == 5


def test_qmm_plan_rejects_what_no_kernel_takes():
    assert cc.plan_qmm(1024, 1024, 16, 1, 64) is None      # group 16 has no streaming form
    assert cc.plan_qmm(1024, 1024, 32, 1, 257) is None     # groups of 32 stream up to 256 tokens
    assert cc.plan_qmm(1024, 1024, 32, 1, 256) is not None
    assert cc.plan_qmm(1024, 1024, 64, 1, 0) is None
    assert cc.plan_qmm(1024, 1000, 64, 1, 64) is None      # ragged K
    # a small LDS budget: the plan shrinks or gives up, never overshoots
    for limit in (16 << 10, 32 << 10, 64 << 10):
        p = cc.plan_qmm(9216, 2560, 64, 2, 512, CUS, limit)
        assert p is None or p["lds"] <= limit


@pytest.mark.parametrize("layout,group", [(cc.LAYOUT_U4, 64), (cc.LAYOUT_BINARY1, 128), (cc.LAYOUT_TERNARY2, 128),
                                          (cc.LAYOUT_TRIT5, 128)])
def test_matvec_plans(layout, group):
    bytes_per_row = {cc.LAYOUT_U4: lambda c: c // 2, cc.LAYOUT_BINARY1: lambda c: ceil_div(c, 128) * 16,
                     cc.LAYOUT_TERNARY2: lambda c: ceil_div(c, 128) * 32,
                     cc.LAYOUT_TRIT5: lambda c: (ceil_div(c, 5) + 15) // 16 * 16}[layout]
    for rows, cols in SHAPES:
        for nmat in (1, 2):
            p = cc.plan_matvec(layout, rows, cols, group, nmat, LDS, force=True)
            if p is None:
                continue
            segments = ceil_div(bytes_per_row(cols), 128)
            assert p["waves"] <= 16 and p["threads"] == 64 * p["waves"] and p["lds"] <= LDS
            assert p["waves"] * p["segments"] >= segments > (p["waves"] - 1) * p["segments"]
            assert p["workgroups"] == ceil_div(rows, 8)
    # the 27B layer's matrices take the kernel by default in every format
    for rows, cols in [(17408, 5120), (5120, 17408), (5120, 5120)]:
        assert cc.plan_matvec(layout, rows, cols, group) is not None
    # no size threshold in any format; small affine matrices walk few segments per wave, at most eight waves
    small = cc.plan_matvec(layout, 1024, 2560, group)
    assert small is not None
    if layout == cc.LAYOUT_U4:
        assert (small["segments"], small["waves"]) == (2, 5)
        assert cc.plan_matvec(layout, 3584, 1024, group)["segments"] == 1
        assert cc.plan_matvec(layout, 1024, 3584, group)["waves"] <= 8
        assert cc.plan_matvec(layout, 512, 1024, group) is not None
        # 8M to 24M weights: two segments per wave where twelve waves cover the row, else the next that does
        assert (cc.plan_matvec(layout, 9216, 2560, group)["segments"], cc.plan_matvec(layout, 9216, 2560, group)["waves"]) == (2, 5)
        assert (cc.plan_matvec(layout, 2560, 9216, group)["segments"], cc.plan_matvec(layout, 2560, 9216, group)["waves"]) == (3, 12)
        assert cc.plan_matvec(layout, 4096, 4096, group)["segments"] == 2
        # from 24M weights on: a multiple of four waves with next to no idle segments, else the long walk
        for rows, cols, want in [(5120, 5120, (5, 4)), (17408, 5120, (5, 4)), (5120, 17408, (6, 12)), (8192, 8192, (4, 8)),
                                 (14336, 4096, (2, 8)), (4096, 14336, (5, 12)), (8192, 28672, (7, 16))]:
            p = cc.plan_matvec(layout, rows, cols, group)
            assert (p["segments"], p["waves"]) == want, (rows, cols, p)
        # never one segment per wave from 24M weights on; a vocabulary-sized matrix of short rows: one wave per tile
        # (... and two waves per tile for rows of nine to sixteen segments)
        for rows, cols, want in [(16384, 2048, (2, 4)), (65536, 1024, (4, 1)), (151936, 1024, (4, 1)), (151936, 2048, (8, 1)),
                                 (151936, 2560, (5, 2)), (151936, 3072, (6, 2)), (151936, 3584, (7, 2)), (151936, 4096, (8, 2)),
                                 (131072, 5120, (5, 4))]:
            p = cc.plan_matvec(layout, rows, cols, group)
            assert (p["segments"], p["waves"]) == want, (rows, cols, p)
        assert cc.plan_matvec(layout, 64, 32768, group)["segments"] == 8
        assert cc.plan_matvec(layout, 64, 32768 + 256, group) is None      # 129 segments: no single workgroup covers the row
    assert cc.plan_matvec(layout, 256, 2560, group) == cc.plan_matvec(layout, 256, 2560, group, force=True) is not None
    if layout != cc.LAYOUT_U4:
        # the signed formats below the 27B shapes walk one segment per wave (ternary from 8M weights two)
        assert cc.plan_matvec(layout, 2048, 2048, group)["segments"] == 1
        assert cc.plan_matvec(layout, 4096, 4096, group)["segments"] == (2 if layout == cc.LAYOUT_TERNARY2 else 1)
        assert cc.plan_matvec(layout, 17408, 5120, group)["segments"] == 2


def test_matvec_plan_rejects_bad_arguments():
    with pytest.raises(ValueError):
        cc.plan_matvec(7, 1024, 1024, 64)
    with pytest.raises(ValueError):
        cc.plan_matvec(cc.LAYOUT_U4, 1024, 1024, 64, nmat=3)
    with pytest.raises(ValueError):
        cc.plan_qmm(1024, 1024, 64, 0, 64)
    assert cc.plan_matvec(cc.LAYOUT_BINARY1, 8192, 8192, 64) is None     # signed formats are g128 only
    assert cc.plan_matvec(cc.LAYOUT_TRIT5, 8192, 8200, 128) is None      # rows of five-digit bytes: 16-column multiples
    assert cc.plan_matvec(cc.LAYOUT_U4, 8192, 8192, 48) is None
