"""Decisions that are taken on the host from sizes alone: how a product is split over workgroups."""
from ginfer_amd.parts import linear as L


def test_parts_divide_the_steps_of_k_and_leave_every_wavefront_work():
    for rows in (1, 8, 16, 17, 64):
        for n in (88, 896, 1536, 3584, 8192):
            for k in (64, 520, 1536, 3584, 8960, 18944, 29568):
                nt, parts = L._split_plan(rows, n, k)
                steps = -(-k // 64)
                assert nt in (1, 4) and 1 <= parts <= L.TUNING.max_split_k_parts
                assert parts == 1 or (steps % parts == 0 or k < L.TUNING.split_k_from) and parts * 8 <= max(steps, 8)
                assert nt == 1 or rows > 16


def test_measured_shapes_keep_their_plans():
    """The sizes the plans were measured at (1.5B and 7B shapes) keep what was found best."""
    assert L._split_plan(64, 1536, 8960) == (4, 10)
    assert L._split_plan(8, 1536, 8960) == (1, 5)
    assert L._split_plan(64, 1536, 1536) == (1, 2)
    assert L._split_plan(64, 3584, 18944) == (4, 4)
    assert L._split_plan(64, 3584, 3584) == (4, 4)
    assert L._library_split(256, 1536, 8960) == 5 and L._library_split(64, 1536, 8960) == 1
    assert L._library_split(256, 17920, 1536) == 1
    # the rows of prompt portions: four pieces up to 2,048 rows, one product beyond
    assert L._library_split(512, 1536, 8960) == 4 and L._library_split(2048, 1536, 8960) == 4
    assert L._library_split(4096, 1536, 8960) == 1 and L._library_split(2048, 1536, 1536) == 1


def test_nearest_divisor():
    assert L._nearest_divisor(140, 10.7, 16) == 10
    assert L._nearest_divisor(140, 5.3, 16) == 5
    assert L._nearest_divisor(296, 4.6, 16) == 4
    assert L._nearest_divisor(7, 3.0, 16) == 1          # 1 and 7 are the divisors; 1 is nearer
    assert L._nearest_divisor(24, 100.0, 3) == 3        # never above the cap
