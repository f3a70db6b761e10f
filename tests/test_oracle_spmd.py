"""Pins the oracle's SPMD plumbing by brute force: ranges cover every block
once, the pid decode is the mixed-radix inverse, the GROUP_SIZE_M swizzle is a
bijection onto the tile grid."""
import itertools

import pytest

from oracle import oracle as orc


@pytest.mark.parametrize("nb,nw", [(0, 4), (1, 4), (97, 8), (4096, 256), (3584, 256), (1000, 7), (5, 5), (6, 5)])
def test_block_ranges_cover_once_and_balance(nb, nw):
    seen = []
    sizes = []
    prev_end = 0
    for w in range(nw):
        s, e = orc.block_range(nb, nw, w)
        assert s == prev_end, "ranges must be contiguous in worker order"
        prev_end = e
        seen.extend(range(s, e))
        sizes.append(e - s)
    assert seen == list(range(nb))
    assert max(sizes) - min(sizes) <= 1
    # the larger ranges come first (w < rem)
    assert sizes == sorted(sizes, reverse=True)


def test_block_range_matches_host_split_of_reference_example():
    # 64x2560x9728 with 64x64 tiles on 40 cores: 1*152 = 152 blocks, 152/40 = 3 rem 32
    # (examples/matmul_tensor_descriptor/matmul_multi_core_tma.cpp:139-158)
    nb, nw = (64 // 64) * (9728 // 64), 40
    sizes = [orc.block_range(nb, nw, w)[1] - orc.block_range(nb, nw, w)[0] for w in range(nw)]
    assert sizes == [4] * 32 + [3] * 8


@pytest.mark.parametrize("gx,gy,gz", [(1, 1, 1), (97, 1, 1), (32, 128, 1), (3, 5, 7)])
def test_pid_decode_is_mixed_radix(gx, gy, gz):
    expect = [(x, y, z) for z in range(gz) for y in range(gy) for x in range(gx)]
    got = [orc.pid_decode(b, gx, gy) for b in range(gx * gy * gz)]
    assert got == expect


@pytest.mark.parametrize("npm,npn,g", [(64, 64, 1), (64, 64, 8), (32, 112, 8), (7, 5, 4), (7, 5, 1), (3, 9, 16), (1, 1, 1)])
def test_group_swizzle_is_a_bijection(npm, npn, g):
    tiles = [orc.tile_of_pid(p, npm, npn, g) for p in range(npm * npn)]
    assert sorted(tiles) == sorted(itertools.product(range(npm), range(npn)))
    if g == 1:
        # GROUP_SIZE_M = 1: row-major over (pid_m, pid_n), so a worker's contiguous
        # chunk reuses one A row-panel
        assert tiles == [(p // npn, p % npn) for p in range(npm * npn)]


def test_group_swizzle_walks_down_columns_inside_a_group():
    # with G=4 the first 4 pids share pid_n=0 and step pid_m
    assert [orc.tile_of_pid(p, 8, 8, 4) for p in range(5)] == [(0, 0), (1, 0), (2, 0), (3, 0), (0, 1)]


def _decode_descriptor(pid, num_pid_m, num_pid_n, GROUP_SIZE_M):
    """09-persistent-matmul.py:118-126, transcribed statement by statement."""
    num_pid_in_group = GROUP_SIZE_M * num_pid_n
    group_id = pid // num_pid_in_group
    first_pid_m = group_id * GROUP_SIZE_M
    group_size_m = min(num_pid_m - first_pid_m, GROUP_SIZE_M)
    pid_m = first_pid_m + (pid % group_size_m)
    pid_n = (pid % num_pid_in_group) // group_size_m
    return pid_m, pid_n


def _decode_pointer(pid, num_pid_m, num_pid_n, GROUP_SIZE_M):
    """03-matrix-multiplication.py:276-282, transcribed statement by statement."""
    num_pid_in_group = GROUP_SIZE_M * num_pid_n
    group_id = pid // num_pid_in_group
    first_pid_m = group_id * GROUP_SIZE_M
    group_size_m = min(num_pid_m - first_pid_m, GROUP_SIZE_M)
    pid_m = first_pid_m + ((pid % num_pid_in_group) % group_size_m)
    pid_n = (pid % num_pid_in_group) // group_size_m
    return pid_m, pid_n


@pytest.mark.parametrize("npm,npn,g", [(5, 3, 3), (7, 5, 4), (64, 64, 8), (3, 9, 16), (9, 7, 5), (1, 1, 1)])
def test_both_decodes_follow_their_sources(npm, npn, g):
    for p in range(npm * npn):
        assert orc.tile_of_pid(p, npm, npn, g) == _decode_descriptor(p, npm, npn, g)
        assert orc.tile_of_pid_pointer(p, npm, npn, g) == _decode_pointer(p, npm, npn, g)
    tiles = [orc.tile_of_pid_pointer(p, npm, npn, g) for p in range(npm * npn)]
    assert sorted(tiles) == sorted(itertools.product(range(npm), range(npn)))


def test_the_two_decodes_differ_in_a_short_last_group():
    # 5 rows of tiles in groups of 3, 3 columns: the last group has 2 rows and starts at program 9, which is odd,
    # so `pid % 2` and `(pid % 9) % 2` disagree (hand-worked: program 9 is the group's first -> row 3 by position)
    assert orc.tile_of_pid_pointer(9, 5, 3, 3) == (3, 0) and orc.tile_of_pid(9, 5, 3, 3) == (4, 0)
    assert orc.tile_of_pid_pointer(10, 5, 3, 3) == (4, 0) and orc.tile_of_pid(10, 5, 3, 3) == (3, 0)
    assert orc.tile_of_pid_pointer(11, 5, 3, 3) == (3, 1) and orc.tile_of_pid(11, 5, 3, 3) == (4, 1)
