"""The host's launch plan for the prefill / multi-row products against what the kernels assume
(rustane_amd/csrc/hipdec_prefill.h): checked on the CPU for every weight format over the shapes of
the bench models, the test models and ragged ones."""
import itertools

import pytest

from rustane_amd import hipdec
from rustane_amd.hipdec import WeightDtype

ROWS = [1, 2, 3, 5, 7, 8, 9, 13, 16, 17, 27, 31, 32, 33, 64, 127, 128, 129, 200, 512, 1000, 1024]
SHAPES = [  # (n, k)
    (4608, 1536), (1536, 1536), (8192, 1536), (1536, 4096), (32000, 1536),          # 600M class
    (12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008), (65536, 4096),       # 5B class
    (896, 384), (384, 384), (2304, 384), (384, 1152), (1000, 384), (50, 128), (70, 640), (28672, 8192), (8192, 28672),
]
STAGE_PAD = 8            # bf16 elements of padding per staged activation row
LDS_LIMIT = 64 * 1024    # dynamic LDS a launch may ask for without an opt-in


def plans():
    for wd, rows, (n, k) in itertools.product(WeightDtype, ROWS, SHAPES):
        if wd == WeightDtype.F32 and rows > 32:
            continue                       # fp32 weights go through the few-row kernel 32 rows at a time
        if wd == WeightDtype.INT4_G128 and k % 128:
            continue
        yield wd, rows, n, k, hipdec.gemm_plan(wd, rows, n, k)


def test_every_split_covers_its_share_and_none_is_empty():
    count = 0
    for wd, rows, n, k, p in plans():
        unit = 32 if p["kernel"].startswith("few_row") else 64
        steps = -(-k // unit)
        s, sps = p["splits"], p["steps_per_split"]
        assert s >= 1 and sps >= 1
        assert s * sps >= steps, (wd, rows, n, k, p)
        assert (s - 1) * sps < steps, (wd, rows, n, k, p)
        count += 1
    assert count > 1500


def test_few_row_kernels_get_the_grid_and_the_lds_they_index():
    for wd, rows, n, k, p in plans():
        if rows <= 32:
            assert p["kernel"].startswith("few_row"), (wd, rows, n, k, p)
        if not p["kernel"].startswith("few_row"):
            continue
        gx, gy, gz = p["grid"]
        rows_per_wg = {"few_row": 32, "few_row_int4": 16 * (p["threads"] // 64), "few_row_e4m3": 16 * (p["threads"] // 64)}[p["kernel"]]
        assert gx == -(-n // rows_per_wg) and gy == p["splits"] and gz == 1, (wd, rows, n, k, p)
        # staged rows: [hi | lo][rows][steps * 32 + pad] bf16
        assert p["lds_bytes"] == 2 * rows * (p["steps_per_split"] * 32 + STAGE_PAD) * 2
        assert p["lds_bytes"] <= LDS_LIMIT, (wd, rows, n, k, p)


def test_four_bit_splits_are_whole_scale_groups_that_fit_one_round_of_loads():
    seen = 0
    for wd, rows, n, k, p in plans():
        if p["kernel"] != "few_row_int4":
            continue
        assert wd == WeightDtype.INT4_G128
        assert p["threads"] == 512
        assert p["steps_per_split"] % 4 == 0, (rows, n, k, p)           # four 32-element steps per 128-element group
        assert p["steps_per_split"] // 4 <= 8, (rows, n, k, p)          # the kernel requests a split's groups at once, 8 slots
        # 16-byte chunks staged per plane: three rounds of 512 threads
        assert rows * p["steps_per_split"] * 4 <= 3 * 512, (rows, n, k, p)
        seen += 1
    assert seen > 100


def test_e4m3_splits_are_whole_blocks_within_the_staging_rounds():
    seen = 0
    for wd, rows, n, k, p in plans():
        if p["kernel"] != "few_row_e4m3":
            continue
        assert wd == WeightDtype.FP8_E4M3 and k % 64 == 0
        assert p["threads"] == 512
        assert p["steps_per_split"] % 2 == 0, (rows, n, k, p)           # two steps per 64-element block
        assert p["steps_per_split"] // 2 <= 8, (rows, n, k, p)          # the kernel requests a split's blocks at once, 8 slots
        assert rows * p["steps_per_split"] * 4 <= 3 * 512, (rows, n, k, p)   # three rounds of 512 threads
        seen += 1
    assert seen > 100


def test_tiled_kernels():
    for wd, rows, n, k, p in plans():
        if p["kernel"].startswith("few_row"):
            continue
        gx, gy, gz = p["grid"]
        assert gz == p["splits"] and gy == -(-rows // 128), (wd, rows, n, k, p)
        if p["kernel"] == "tiled_direct_lds":
            assert wd == WeightDtype.BF16 and rows >= 129 and k % 64 == 0
            assert gx == -(-n // 256) and p["threads"] == 512
        else:
            assert gx == -(-n // (256 if wd == WeightDtype.FP8_E4M3 else 128)) and p["threads"] == 256
            if wd == WeightDtype.INT4_G128:
                assert p["steps_per_split"] % 2 == 0, (rows, n, k, p)   # two 64-element steps per scale group


def test_shapes_the_library_never_launches_are_refused():
    for args in [(WeightDtype.BF16, 8, 64, 48), (WeightDtype.INT4_G128, 8, 64, 96), (WeightDtype.F32, 33, 64, 64),
                 (WeightDtype.BF16, 0, 64, 64), (WeightDtype.BF16, 8, 0, 64)]:
        with pytest.raises(hipdec.HipDecodeError):
            hipdec.gemm_plan(*args)
