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


def test_a_long_k_of_few_rows_goes_to_the_library_in_pieces():
    """The down projections of larger models at 17 to 256 rows: the library with K in eight pieces (seven where only
    that cuts K into whole steps of 64), also where the streaming kernel could take the rows; the sizes that were
    measured as exceptions keep their own plan; small models are left as they were."""
    plan = lambda rows, n, k: L.linear_plan(rows, n, k, False, False, True, rows <= 64)
    assert plan(64, 2048, 11008) == ("library", 8) and plan(256, 2048, 11008) == ("library", 8)
    assert plan(48, 3584, 18944) == ("library", 8) and plan(256, 3584, 18944) == ("library", 8)
    assert plan(64, 5120, 27648) == ("library", 8) and plan(128, 5120, 13824) == ("library", 8)
    assert plan(64, 8192, 29568) == ("library", 7) and plan(256, 8192, 29568) == ("library", 7)
    # the fewest rows: two pieces where the library is taken anyway and K is very long, else as before
    assert plan(32, 5120, 27648) == ("library", 2) and plan(24, 8192, 29568) == ("library", 2)
    assert plan(32, 5120, 13824) == ("library", 1) and plan(32, 3584, 18944) == ("skinny", 4, 4)
    assert plan(32, 2048, 11008) == ("skinny", 4, 4)
    # about as long as wide
    assert plan(64, 5120, 5120) == ("library", 8) and plan(256, 5120, 5120) == ("library", 8)
    assert plan(64, 8192, 8192) == ("library", 1) and plan(128, 8192, 8192) == ("library", 4)
    assert plan(32, 5120, 5120) == ("library", 1)
    # measured exceptions (the library's own choice of kernel at these very sizes)
    assert plan(64, 3584, 18944) == ("library", 2) and plan(64, 3584, 3584) == ("library", 2)
    assert plan(50, 3584, 18944) == ("library", 2)                  # rows share a plan in classes of 16
    assert L.linear_plan(64, 3584, 18944, False, False, False, True)[0] == "skinny"     # nobody to add parts: no pieces
    assert L.linear_plan(64, 3584, 18944, True, False, True, True)[0] == "skinny"       # a bias: one product
    # the 0.5B and 1.5B shapes: as measured there
    assert plan(64, 1536, 8960) == ("skinny", 4, 10) and plan(256, 1536, 8960) == ("library", 5)
    assert plan(64, 896, 4864) == ("skinny", 1, 4) and plan(64, 1536, 1536) == ("skinny", 1, 2)
    # prompt portions of many columns: a long K in halves up to 1,024 rows
    assert plan(512, 5120, 13824) == ("library", 2) and plan(1024, 8192, 29568) == ("library", 2)
    assert plan(2048, 5120, 13824) == ("library", 1) and plan(512, 8192, 8192) == ("library", 1)
    assert plan(512, 3584, 18944) == ("library", 4) and plan(2048, 2048, 11008) == ("library", 4)
    # decode rows up to 16 fold their norms and never come here in pieces
    assert plan(16, 5120, 27648)[0] == "skinny"
    # every such plan is one the tuner would also try
    for rows, n, k in ((64, 2048, 11008), (64, 8192, 29568), (32, 5120, 27648), (128, 8192, 8192), (64, 3584, 18944)):
        key = ("linear", rows, n, k, False, False, True, rows <= 64)
        assert L.linear_candidates(key)[0] == plan(rows, n, k)


def test_measured_plans_can_be_set_from_json():
    from ginfer_amd.kernels.tuning import Tuning
    t = Tuning()
    t.update({"measured_plans": {"64,1024,8192": ["library", 4]}})
    assert t.measured_plans == {"64,1024,8192": ("library", 4)}


def test_nearest_divisor():
    assert L._nearest_divisor(140, 10.7, 16) == 10
    assert L._nearest_divisor(140, 5.3, 16) == 5
    assert L._nearest_divisor(296, 4.6, 16) == 4
    assert L._nearest_divisor(7, 3.0, 16) == 1          # 1 and 7 are the divisors; 1 is nearer
    assert L._nearest_divisor(24, 100.0, 3) == 3        # never above the cap


def test_rules_as_plans():
    """The rules' decisions as plans, at the sizes they were measured at."""
    # decode rows of the 1.5B shape: the streaming kernel, K in parts where the norm that follows adds them
    assert L.linear_plan(64, 1536, 8960, False, False, True, True) == ("skinny", 4, 10)
    assert L.linear_plan(8, 1536, 8960, False, False, True, True) == ("skinny", 1, 5)
    assert L.linear_plan(8, 1536, 8960, False, False, False, True) == ("skinny", 1, 1)     # nobody to add parts
    assert L.linear_plan(8, 1536, 8960, False, True, True, True) == ("skinny", 1, 1)       # float32 out: no parts
    # wide outputs go to the library from 17 rows on; prompt portions always
    assert L.linear_plan(64, 17920, 1536, False, False, False, True) == ("library", 1)
    assert L.linear_plan(16, 17920, 1536, False, False, False, True) == ("skinny", 1, 1)
    assert L.linear_plan(2048, 1536, 8960, False, False, True, False) == ("library", 4)
    assert L.linear_plan(2048, 1536, 8960, True, False, True, False) == ("library", 1)     # a bias: one product
    assert L.linear_plan(4096, 1536, 8960, False, False, True, False) == ("library", 1)
    assert L.gated_plan(8, 17920, True, True) == ("skinny",)
    assert L.gated_plan(64, 17920, True, True) == ("library",)
    assert L.gated_plan(2048, 17920, False, True) == ("transposed",)
    assert L.gated_plan(2040, 17920, False, True) == ("library",)


def test_candidates_hold_the_rules_plan_first_and_only_plans_that_fit():
    for rows in (1, 8, 16, 17, 64, 128, 256):
        for n, k in ((1536, 8960), (3584, 18944), (8192, 29568), (88, 520), (1536, 1536), (151936, 1536)):
            for has_bias in (False, True):
                for f32 in (False, True):
                    for parts_ok in (False, True):
                        skinny_ok = rows <= 64
                        key = ("linear", rows, n, k, has_bias, f32, parts_ok, skinny_ok)
                        plans = L.linear_candidates(key)
                        assert plans[0] == L.linear_plan(rows, n, k, has_bias, f32, parts_ok, skinny_ok)
                        assert len(set(plans)) == len(plans) and ("library", 1) in plans
                        for plan in plans[1:]:
                            if plan[0] == "skinny":
                                assert skinny_ok and plan[1] in (1, 4) and (plan[1] == 1 or rows > 16)
                                if plan[2] > 1:
                                    assert parts_ok and not f32 and -(-k // 64) % plan[2] == 0 and plan[2] * 8 <= -(-k // 64)
                            else:
                                if plan[1] > 1:
                                    assert parts_ok and not f32 and not has_bias
                                    assert k % plan[1] == 0 and (k // plan[1]) % 8 == 0 and k // plan[1] >= 512
    assert L.gated_candidates(("gated", 64, 17920, 1536, True, True)) == [("library",), ("skinny",), ("transposed",)]
    assert L.gated_candidates(("gated", 2048, 17920, 1536, False, True)) == [("transposed",), ("library",)]
    assert L.gated_candidates(("gated", 100, 17920, 1536, False, False)) == [("library",)]


def test_kept_plans_answer_for_their_class_of_rows():
    from ginfer_amd.kernels import autotune
    assert [autotune.rows_class(r) for r in (1, 7, 16, 17, 32, 33, 64, 65, 200)] == [1, 7, 16, 32, 32, 48, 64, 80, 208]
    assert not autotune.active() and autotune.choose(("linear", 32), ("w",)) is None
    with autotune.collecting() as seen:
        assert autotune.active()
        assert autotune.choose(("linear", 32), ("w0",)) is None and autotune.choose(("linear", 32), ("w1",)) is None
        assert autotune.choose(("gated", 32), ("w2",)) is None
    assert seen == {("linear", 32): [("w0",), ("w1",)], ("gated", 32): [("w2",)]} and not autotune.active()
    table = autotune.Table()
    table[("linear", 32)] = ("library", 2)
    assert not autotune.active() and autotune.choose(("linear", 32), ("w",)) is None      # no table is in use
    with autotune.using(table):
        assert autotune.active() and autotune.choose(("linear", 32), ("w",)) == ("library", 2)
        assert autotune.choose(("linear", 48), ("w",)) is None
        with autotune.using(None):                                                          # a runner without plans
            assert not autotune.active() and autotune.choose(("linear", 32), ("w",)) is None
    assert not autotune.active()


def test_keys_of_a_short_prompt_are_dealt_out_and_those_of_other_steps_are_not(monkeypatch):
    """The rule that deals a tile's keys to several workgroups: one prompt of 2,048 tokens alone in a step (one round of
    workgroups, the last tile walking twice the mean) is split, every part within the mean share, the parts of a tile
    covering its keys once; shorter and longer prompts, and steps of many requests, stay whole."""
    from ginfer_amd.kernels import ops
    tiles = ops.plan_rows([2048], [0], 32)[3]
    assert ops.key_parts(tiles, 32, 0, 4, 2) is None          # switched off in the table of thresholds: it was measured slower
    monkeypatch.setattr(ops.TUNING, "prefill_split_imbalance", 1.5)
    pieces, parts, rows, n = ops.key_parts(tiles, 32, 0, 4, 2)
    assert n == 2 and len(pieces) == len(parts) > len(tiles) and len(rows) % 32 == 0
    share = sum(range(1, 65)) * 4 / 256.0
    assert max((e - b) // 32 for b, e, _, _ in parts) <= 1.15 * share + 2
    by_tile = {}
    for t, (b, e, at, packed) in zip(pieces, parts):
        by_tile.setdefault(t, []).append((b, e, at, packed & 0xffff, packed >> 16))
    assert set(by_tile) == set(tiles)
    for t, ps in by_tile.items():
        ps.sort()
        assert ps[0][0] == 0 and ps[-1][1] == ((t[3] + t[2] - 1) // 32 + 1) * 32
        assert all(x[1] == y[0] for x, y in zip(ps, ps[1:])) and [x[3] for x in ps] == list(range(len(ps)))
        if len(ps) > 1:
            assert all(x[4] == n and x[2] == ps[0][2] for x in ps)
            assert [r[0] for r in rows[ps[0][2]:ps[0][2] + t[2]]] == list(range(t[1], t[1] + t[2]))
        else:
            assert ps[0][2] == -1
    assert [e - b for b, e, _, _ in parts] == sorted((e - b for b, e, _, _ in parts), reverse=True)      # longest walks first
    assert ops.key_parts(ops.plan_rows([1024], [0], 32)[3], 32, 0, 12, 8) is None
    assert ops.key_parts(ops.plan_rows([4096], [0], 32)[3], 32, 0, 4, 2) is None
    assert ops.key_parts(ops.plan_rows([512] * 4, [0] * 4, 32)[3], 32, 0, 4, 2) is None
    # a window bounds every tile's keys: nothing to deal out
    assert ops.key_parts(tiles, 32, 256, 4, 2) is None
