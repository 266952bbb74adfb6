"""The host arithmetic that plans launches: key splits of the MFMA attention kernel, and the
workgroups of a product's sweep over its weight tiles."""

import ctypes
from ctypes import c_int

import pytest

from socrates_amd.kernels import MAX_KEY_SPLITS, plan_key_splits


@pytest.mark.parametrize("n_kv_heads", [1, 2, 4, 8])
def test_key_splits_stay_within_what_the_merge_holds(n_kv_heads):
    """Rows 1..64, groups 1..16, contexts up to 131,072 keys: never more splits than the
    kernel takes, one split or a multiple of four (four share a workgroup), splits are whole
    16-key tiles, and together they cover every key (the last may be short; of the last four
    some may be empty, never all)."""
    keys = [1, 15, 16, 17, 255, 256, 257, 1000, 2048, 4096, 16448, 20000, 32768, 65536, 100000, 131072]
    for rows in list(range(1, 18)) + [24, 32, 48, 64]:
        for group in range(1, 17):
            for max_keys in keys:
                split_len, n = plan_key_splits(rows, n_kv_heads, group, max_keys)
                assert 1 <= n <= MAX_KEY_SPLITS, (rows, group, max_keys, n)
                assert split_len % 16 == 0 and split_len >= 16
                assert n == 1 or n % 4 == 0
                assert n * split_len >= max_keys                  # covers the keys
                assert (n - (1 if n == 1 else 4)) * split_len < max_keys    # and no workgroup is empty


def test_key_splits_cases_that_used_to_exceed_the_limit():
    # one decoded token, 4 kv heads, 32,768 keys planned 512 splits of 64; 2 kv heads at 20,000
    # keys planned 313
    assert plan_key_splits(1, 4, 8, 32768) == (128, 256)
    split_len, n = plan_key_splits(1, 2, 4, 20000)
    assert n <= 256 and n * split_len >= 20000
    # a short context is not cut below 64 keys, a full launch is not cut at all
    assert plan_key_splits(1, 8, 4, 100)[1] <= 4
    assert plan_key_splits(128, 8, 4, 4096) == (4096, 1)


def test_a_sweep_shares_the_tiles_out_evenly():
    """At most one workgroup per compute unit (256), every workgroup the same number of weight
    tiles (tile pairs with SwiGLU) up to one, no workgroup without a tile; K beyond 16 waves
    of two halves of 5 steps of 32 is refused. (The plan is host code of the product library; calling it
    needs the library, not a GPU.)"""
    from socrates_amd.kernels.build import load_library
    lib = load_library("gemm")
    lib.soc_gemm_sweep_plan.restype = c_int
    for swiglu in (0, 1):
        for N in (32, 64, 4096, 6144, 8192, 19456, 24576, 51200, 151936, 151968):
            for K in (8, 64, 2560, 4096, 4104, 5120):
                nw, wgs = c_int(0), c_int(0)
                assert lib.soc_gemm_sweep_plan(c_int(N), c_int(K), c_int(swiglu), ctypes.byref(nw), ctypes.byref(wgs)) == 1
                items = N // 32 if swiglu else (N + 15) // 16
                assert nw.value == 16 and 1 <= wgs.value <= min(items, 256)
                most = (items + wgs.value - 1) // wgs.value
                assert most == (items + 255) // 256                        # as few tiles for the busiest as 256 units allow
                assert (most - 1) * wgs.value < items                      # nobody is idle
    nw, wgs = c_int(0), c_int(0)
    for K in (5128, 8192, 9728):
        assert lib.soc_gemm_sweep_plan(c_int(2560), c_int(K), c_int(0), ctypes.byref(nw), ctypes.byref(wgs)) == 0
    # the shapes of a 4B-sized layer: 608 tile pairs as 203 x 3, 384 tiles as 192 x 2
    lib.soc_gemm_sweep_plan(c_int(19456), c_int(2560), c_int(1), ctypes.byref(nw), ctypes.byref(wgs))
    assert wgs.value == 203
    lib.soc_gemm_sweep_plan(c_int(6144), c_int(2560), c_int(0), ctypes.byref(nw), ctypes.byref(wgs))
    assert wgs.value == 192


def test_parts_of_k_fit_the_registers_and_the_gpu():
    """The sweep for 17 to 64 rows: every part of K fits what 16 waves hold (5 steps of 32 for
    up to 32 rows, 3 beyond), parts x groups are at most 256 workgroups, no group is without
    a tile, and the parts cover K. (Host code of the product library: no GPU needed.)"""
    from socrates_amd.kernels.build import load_library
    lib = load_library("gemm")
    lib.soc_gemm_sweep_parts_plan.restype = c_int
    for M in (17, 32, 33, 64):
        for N in (16, 40, 2560, 4096, 5120, 8192):
            for K in (32, 96, 2048, 4096, 9728, 12288, 25600):
                parts, kpw, groups = c_int(0), c_int(0), c_int(0)
                assert lib.soc_gemm_sweep_parts_plan(c_int(M), c_int(N), c_int(K), ctypes.byref(parts),
                                                     ctypes.byref(kpw), ctypes.byref(groups)) == 1
                steps, tiles = (K + 31) // 32, (N + 15) // 16
                per_part = (steps + parts.value - 1) // parts.value
                assert kpw.value % 32 == 0 and kpw.value // 32 <= (5 if M <= 32 else 3)
                assert 16 * (kpw.value // 32) >= per_part                  # 16 waves hold a part
                assert per_part * parts.value >= steps
                assert 1 <= groups.value <= tiles and parts.value * groups.value <= 256
                most = (tiles + groups.value - 1) // groups.value
                assert (most - 1) * groups.value < tiles                   # nobody is idle
    parts, kpw, groups = c_int(0), c_int(0), c_int(0)
    for M, N, K in ((65, 2560, 4096), (0, 2560, 4096), (64, 2560, 16)):
        assert lib.soc_gemm_sweep_parts_plan(c_int(M), c_int(N), c_int(K), ctypes.byref(parts),
                                             ctypes.byref(kpw), ctypes.byref(groups)) == 0
    # the projections of a 4B-sized layer at 64 rows: down as 8 parts x 32 groups of 5 tiles
    lib.soc_gemm_sweep_parts_plan(c_int(64), c_int(2560), c_int(9728), ctypes.byref(parts), ctypes.byref(kpw),
                                  ctypes.byref(groups))
    assert (parts.value, kpw.value, groups.value) == (8, 96, 32)


def test_k_is_split_over_workgroups_only_where_it_pays():
    """The projections with a residual epilogue: one workgroup per tile of 16 outputs unless
    splitting K gives the busiest of 256 compute units enough less to stream to pay for the
    meeting in memory; a split leaves every wave at least 256 elements of K."""
    from socrates_amd.kernels import HipKernels
    rule = HipKernels._addnorm_splits
    for M in (1, 4, 8, 16):
        for tiles in (1, 16, 160, 256, 320, 512, 1000):
            for K in (64, 2560, 4096, 9728, 25600):
                s = rule(tiles, K, M)
                assert s in (1, 2, 4)
                assert s == 1 or K // (s * 8) >= 256
                if tiles % 256 == 0:
                    assert s == 1                     # the GPU is evenly filled as it is
    # 4B-sized layers: the down projection whole up to 8 rows, in four parts from 12 on; the
    # output projection always whole; 32B-sized: four parts for both
    assert [rule(160, 9728, M) for M in (1, 8, 12, 16)] == [1, 1, 4, 4]
    assert {rule(160, 4096, M) for M in (1, 8, 16)} == {1}
    assert rule(320, 25600, 8) == 4 and rule(320, 8192, 8) == 4


def test_key_splits_leave_no_ragged_second_round_of_workgroups():
    """Four splits make a workgroup and a compute unit holds two: a plan a little over a whole
    number of workgroups per compute unit is cut down to that number (8 kv heads, groups of 4:
    6 rows would take 24 splits = 288 workgroups and take 20 = 240; 12 rows take 8 = 192, not
    12 = 288; 24 rows take 4 = 192, not 8 = 384); plans that fill whole rounds stay."""
    def groups(rows, keys):
        return rows * 8 * plan_key_splits(rows, 8, 4, keys)[1] // 4
    for keys in (2048, 8192):
        assert plan_key_splits(6, 8, 4, keys)[1] == 20 and plan_key_splits(12, 8, 4, keys)[1] == 8
        assert plan_key_splits(24, 8, 4, keys)[1] == 4 and plan_key_splits(8, 8, 4, keys)[1] == 16
        for rows in range(1, 65):
            g = groups(rows, keys)
            assert g <= 256 or g % 256 == 0 or (g % 256) * 4 >= 256 * 3 or plan_key_splits(rows, 8, 4, keys)[1] == 4, (rows, keys, g)


def test_weight_rows_of_a_workgroup_in_the_projections_with_a_residual_epilogue():
    """2,560 outputs are 160 tiles of 16 rows, which leave 96 of 256 compute units idle, or 256 of
    10: from 5 rows of x on the lower tile is taken where it divides the width; widths that fill
    the GPU with tiles of 16 keep them; the long K of a 32B-sized down projection stays in four
    parts of 16-row tiles."""
    from socrates_amd.kernels import HipKernels

    class Rules:
        _addnorm_splits = staticmethod(HipKernels._addnorm_splits)
    shape = lambda N, K, M: HipKernels._addnorm_shape(Rules, N, K, M)
    assert shape(2560, 9728, 8) == (10, 1) and shape(2560, 4096, 16) == (10, 1)
    assert shape(2560, 9728, 1) == (16, 1) and shape(2560, 9728, 4)[0] == 16
    assert shape(4096, 4096, 8) == (16, 1) and shape(4096, 12288, 16) == (16, 1)
    assert shape(5120, 8192, 8) == (10, 1) and shape(5120, 25600, 8) == (16, 4)
    for N in (64, 72, 100, 2560, 5000, 151936):
        for M in (1, 5, 16):
            h, s = shape(N, 4096, M)
            assert 8 <= h <= 16 and (h == 16 or N % h == 0) and s in (1, 2, 4)
