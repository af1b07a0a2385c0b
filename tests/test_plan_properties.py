"""Property test of the launch planner: for many random problems, element types, device sizes and
every kind of override, the plan must cover each 16-row tile's k steps exactly once, stay inside
the limits the kernels are compiled for (workgroup size, LDS, 32-bit weight offsets) and leave no
wave along k without work.  The coverage is computed by the library itself, by replaying on the
host the index functions its kernels are compiled from (mgemv_plan_coverage), so this runs
without a GPU.  The reference has one fixed tiling (mixed_gemv_test.cu:67-70) and nothing to test
here; its grid is ceil(m / ThreadBlockShape::kM) (gemv/device/gemv_adaptor.h:190-197)."""
import contextlib

import numpy as np
import pytest

import mixed_gemv_amd as mg

LDS_VALU = 64 * 1024      # the VALU kernel's launches never raise the default limit of dynamic LDS
LDS_DEVICE = 160 * 1024   # what a workgroup can have on gfx950 (the matrix-core launcher raises the limit as needed)
DEVICE_SIZES = (32, 64, 128, 256, 304)


@contextlib.contextmanager
def overrides(split_k=0, tiles_per_wg=0, tiles_per_wave=0, max_workgroups=0, threshold=0, variant=0, stages=0):
    mg.set_launch_override(split_k, tiles_per_wg, tiles_per_wave, max_workgroups)
    mg.set_matrix_core_threshold(threshold)
    mg.set_matrix_core_variant(variant)
    mg.set_prefetch_stages(stages)
    try:
        yield
    finally:
        mg.set_launch_override(0, 0, 0, 0)
        mg.set_matrix_core_threshold(0)
        mg.set_matrix_core_variant(0)
        mg.set_prefetch_stages(0)


def random_problem(rng):
    bits = int(rng.choice((4, 8)))
    # n_out: log-uniform over 4 .. 262144, a multiple of 4; now and then a whole number of tiles
    n_out = int(2.0 ** rng.uniform(2, 18)) // 4 * 4
    if rng.random() < 0.3:
        n_out = max(16, n_out // 16 * 16)
    per_column = rng.random() < 0.25
    if per_column:
        group = 0
        k = int(2.0 ** rng.uniform(3, 16)) // 8 * 8
    else:
        group = int(rng.choice((64, 96, 128, 160, 256, 512, 1024)))
        k = group * int(rng.integers(1, max(2, 32768 // group)))
    k = max(8, k)
    m_batch = int(rng.choice((1, 1, 1, 2, 3, 4, 5, 7, 8, 12, 16)))
    element = "bf16" if rng.random() < 0.3 else "f16"
    return n_out, m_batch, k, bits, group, element


def check_plan(n_out, m_batch, k, bits, group, element, cus, context=""):
    q = mg.query_launch(n_out, m_batch, k, bits, group, element=element, num_compute_units=cus)
    c = mg.plan_coverage(n_out, m_batch, k, bits, group, element=element, num_compute_units=cus)
    what = f"{context} n_out={n_out} m={m_batch} k={k} bits={bits} g={group} {element} cus={cus}: {q} {c}"
    ksteps = -(-k // (512 if bits == 4 else 256))
    assert c["tiles_miscovered"] == 0 and c["bad_waves"] == 0, what
    assert q["threads"] == 64 * q["split_k"] * q["tiles_per_wg"] <= q["max_threads"] <= 1024, what
    assert q["split_k"] * q["steps_per_wave"] >= ksteps > (q["split_k"] - 1) * q["steps_per_wave"], what
    assert 0 < q["workgroups"] < 2 ** 31 and q["workgroups"] % 8 == 0, what
    assert c["max_descriptor_bytes"] < 2 ** 31, what
    assert c["lds_bytes_used"] <= c["lds_bytes"] == q["lds_bytes"] <= (LDS_DEVICE if q["matrix_core"] else LDS_VALU), what
    assert c["busy_waves"] >= 1 and q["stages"] in (1, 2) and q["launches"] == (1 if q["matrix_core"] else -(-m_batch // 4)), what
    if q["matrix_core"] == 0:
        assert c["idle_waves"] < 8 * q["tiles_per_wg"] * q["split_k"] or q["tiles_in_sequence"] == 1, what
        assert c["max_units_per_wave"] <= q["tiles_in_sequence"] * q["steps_per_wave"], what
    return q, c


def test_built_in_plans_cover_every_problem():
    rng = np.random.default_rng(20240607)
    kinds = set()
    for i in range(20000):
        prob = random_problem(rng)
        cus = int(rng.choice(DEVICE_SIZES))
        q, _ = check_plan(*prob, cus)
        kinds.add((q["matrix_core"], q["tiles_in_sequence"] > 1, q["tiles_per_wg"] > 1))
    # the sample reaches every kind of launch: VALU with and without walks and tile pairs, the matrix-core kernels
    assert {k[0] for k in kinds} == {0, 2, 3} or {k[0] for k in kinds} == {0, 1, 2, 3}
    assert (0, True, False) in kinds and (0, False, True) in kinds and (0, True, True) in kinds


def test_every_override_combination_still_covers():
    rng = np.random.default_rng(7)
    checked = 0
    for split_k in (0, 1, 2, 3, 4, 8, 16):
        for tiles_per_wg in (0, 1, 2, 4, 8):
            for tiles_per_wave in (0, 1, 2, 4):
                for max_wg in (0, 1, 100, 256, 512):
                    for threshold, variant in ((0, 0), (17, 0), (1, 1), (1, 2), (2, 0), (1, 3)):
                        stages = int(rng.integers(0, 3))
                        with overrides(split_k, tiles_per_wg, tiles_per_wave, max_wg, threshold, variant, stages):
                            for _ in range(4):
                                prob = random_problem(rng)
                                q, _ = check_plan(*prob, int(rng.choice(DEVICE_SIZES)),
                                                  context=f"sk={split_k} tw={tiles_per_wg} t={tiles_per_wave} "
                                                          f"wg={max_wg} thr={threshold} var={variant} st={stages}")
                                if stages and not q["matrix_core"]:
                                    assert q["stages"] == stages
                                checked += 1
    assert checked >= 14000


def test_largest_problems_stay_in_32_bit_offsets():
    """The benchmark's largest weights and beyond: up to 2 GiB of int8 weights in one matrix."""
    for n_out, k, bits in ((151936, 8192, 4), (262144, 16384, 4), (131072, 16384, 8), (262144, 8192, 8), (16, 32768, 8),
                           (1048576, 2048, 8)):
        for m_batch in (1, 4, 16):
            for cap in (0, 1, 64):
                with overrides(max_workgroups=cap):
                    check_plan(n_out, m_batch, k, bits, 128, "f16", 256, context=f"cap={cap}")


def test_prefetch_stages_knob_and_table_entry():
    base = mg.query_launch(4096, 1, 4096, 4, 128, num_compute_units=256)
    assert base["stages"] == 2
    with overrides(stages=1):
        one = mg.query_launch(4096, 1, 4096, 4, 128, num_compute_units=256)
        assert one["stages"] == 1 and {k: v for k, v in one.items() if k != "stages"} == {k: v for k, v in base.items() if k != "stages"}
        assert mg.query_launch(4096, 8, 4096, 4, 128, num_compute_units=256)["stages"] == 2   # matrix cores: always two
    with pytest.raises(mg.MixedGemvError):
        mg.set_prefetch_stages(3)
    mg.clear_tuned_plans()
    try:
        mg.set_tuned_plan(4096, 4096, 4, 128, 1, stages=1)
        assert mg.query_launch(4096, 1, 4096, 4, 128, num_compute_units=256)["stages"] == 1
        assert mg.query_launch(4096, 1, 4096, 4, 128, element="bf16", num_compute_units=256)["stages"] == 2  # f16 entry only
        mg.set_tuned_plan(4096, 4096, 4, 128, 1, stages=1, element="bf16")
        assert mg.tuned_plan_count() == 2
        mg.erase_tuned_plan(4096, 4096, 4, 128, 1)
        assert mg.tuned_plan_count() == 1
        assert mg.query_launch(4096, 1, 4096, 4, 128, num_compute_units=256)["stages"] == 2
        assert mg.query_launch(4096, 1, 4096, 4, 128, element="bf16", num_compute_units=256)["stages"] == 1
        mg.erase_tuned_plan(4096, 4096, 4, 128, 1)   # erasing what is not there is not an error
        with pytest.raises(mg.MixedGemvError):
            mg.set_tuned_plan(4096, 4096, 4, 128, 1, stages=5)
    finally:
        mg.clear_tuned_plans()
