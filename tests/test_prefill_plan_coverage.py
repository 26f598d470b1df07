"""No GPU: the planner's choice of prefill kernel for every benchmark shape, and for a sweep of
other shapes, is an instantiation that a full-size GPU parity case names (tests/prefill_cases.py),
so that a change of the planner cannot move a configuration onto an untested kernel unnoticed."""
import itertools

import prefill_cases as pc
import shainet_amd as sa


def plan_of(H, KV, hd, S, T):
    return sa.describe_plan(H, KV, hd, [S], [T])


def test_cases_name_the_planners_choice():
    for name, H, KV, hd, _norm, S, T, inst in pc.CASES:
        plan = plan_of(H, KV, hd, S, T)
        assert plan["path"] == sa.hip.PATH_PREFILL, name
        assert pc.instantiation(plan) == inst, (name, plan)


def test_every_benchmark_prefill_shape_is_a_case_at_full_size():
    shapes = {(H, KV, hd, S, T) for _, H, KV, hd, _, S, T, _ in pc.CASES}
    for shape in pc.BASELINE_PREFILL_SHAPES:
        assert shape in shapes, shape


def test_bench_prefill_workloads_are_cases():
    # bench.py's prefill workloads (name -> shape) against the table: the bench times nothing
    # whose output no test has looked at
    import bench

    by_name = {name: (H, KV, hd, S, T) for name, H, KV, hd, _, S, T, _ in pc.CASES}
    for name, H, KV, hd, _theta, _norm, lens, T in bench.PREFILL_WORKLOADS:
        if lens is not None and len(lens) == 1:
            assert by_name.get(name) == (H, KV, hd, lens[0], T), name


def test_every_reachable_instantiation_is_covered():
    # (the instantiations for padded tiles, a fifth element in the table, are the same code with the
    # head_dim of the data as a run-time value; the table holds four of them, both tile widths, with
    # and without key chunks, turns and one workgroup per block, and this sweep does not enumerate them)
    covered = {inst for *_, inst in pc.CASES if len(inst) == 4}
    seen = set()
    for hd, KV, g in itertools.product((64, 128), (1, 2, 4, 8), (1, 2, 4, 8)):
        for S in (0, 1000, 4096, 16384, 32768):
            for T in (17, 64, 100, 128, 256, 300, 512, 768, 1024, 1536, 2048, 2560, 3072, 4096, 6144, 8192):
                plan = plan_of(KV * g, KV, hd, S, T)
                if plan["path"] != sa.hip.PATH_PREFILL:
                    continue
                seen.add(pc.instantiation(plan))
    assert seen <= covered, sorted(seen - covered)
    assert seen == covered, sorted(covered - seen)  # and nothing in the table is unreachable


def test_decode_and_generic_paths_are_told_apart():
    assert sa.describe_plan(32, 8, 128, [5000] * 16, [1] * 16)["path"] == sa.hip.PATH_DECODE
    assert sa.describe_plan(32, 8, 128, [5000] * 16, [8] * 16)["path"] == sa.hip.PATH_DECODE  # two entries each
    assert sa.describe_plan(32, 8, 128, [5000] * 16, [9] * 16)["path"] == sa.hip.PATH_PREFILL
    # head dimensions between the tile layouts run in padded tiles: 8 in tiles of 64, 96 in tiles of 128
    small = sa.describe_plan(8, 4, 8, [0], [6])
    assert small["path"] == sa.hip.PATH_DECODE and small["head_dim"] == 64
    assert sa.describe_plan(32, 8, 96, [0], [300])["path"] == sa.hip.PATH_PREFILL
    assert sa.describe_plan(32, 8, 96, [0], [300])["head_dim"] == 128
    assert sa.describe_plan(16, 4, 256, [4096], [1])["head_dim"] == 256
    # what no tile layout holds: not a multiple of 4, or more than 16 rows x heads of head_dim above 128
    assert sa.describe_plan(8, 4, 6, [0], [6])["path"] == sa.hip.PATH_GENERIC
    assert sa.describe_plan(16, 4, 256, [0], [40])["path"] == sa.hip.PATH_GENERIC
    head = sa.describe_plan(32, 8, 128, [5000] * 16, [1] * 16)
    assert head["workgroups"] == 256 and head["units"] * 256 >= 16 * 8 * 313
