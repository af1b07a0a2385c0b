"""The k-stationary matrix-core kernel (one wave per k step, the workgroup walks its tiles; activation
operand in registers) against the CPU oracle, and its launch paths against each other: walks shorter
and longer than the workgroup has waves, one and two rounds of the operand through LDS, the 8-byte
and the 2-byte stores, the batched launch, alpha / beta, the dequantiser forms.  The reference has no
such kernel (its own is fixed to one activation row, gemv/threadblock/default_mma_core_simt.h:68-70);
what is pinned is the result of host::reference::MixedGemv (host/mixed_gemv.h:54-107) for each row."""
import numpy as np
import pytest

import mixed_gemv_amd as mg
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, DeviceProblem, Problem, error_report

pytestmark = pytest.mark.gpu
REL_TOL = 2e-3   # max relative error of fp16 outputs against the oracle (floor: helpers.error_report)


class k_stationary:
    """Every row count on the k-stationary kernel, workgroups capped (0 = one per compute unit)."""

    def __init__(self, max_workgroups=0):
        self.cap = max_workgroups

    def __enter__(self):
        mg.set_matrix_core_threshold(1)
        mg.set_matrix_core_variant(mg.MATRIX_CORE_K_STATIONARY)
        mg.set_launch_override(0, 0, 0, self.cap)

    def __exit__(self, *exc):
        mg.set_launch_override(0, 0, 0, 0)
        mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
        mg.set_matrix_core_threshold(0)


CASES = [
    # tag, n_out, k, bits, quant_op, group, rows, bias, workgroup cap, scale range
    ("one_row_16_waves", 512, 8192, 4, SCALE_AND_ZEROS, 128, 1, False, 0, (0.001, 0.02)),
    ("ragged_rows_g64", 1000, 2048, 4, SCALE_AND_ZEROS, 64, 3, True, 0, (0.001, 0.02)),
    ("per_column", 4100, 1024, 4, PER_COLUMN, 0, 5, True, 0, (0.001, 0.02)),
    ("per_column_large_scales", 1040, 1024, 4, PER_COLUMN, 0, 2, False, 16, (0.05, 0.3)),
    ("int8_g64", 2048, 2048, 8, SCALE_AND_ZEROS, 64, 2, False, 0, (0.001, 0.01)),
    ("int8_per_column_16_rows_16_waves", 1024, 4096, 8, PER_COLUMN, 0, 16, True, 0, (0.001, 0.01)),
    ("generic_groups_of_96", 640, 768, 4, SCALE_AND_ZEROS, 96, 7, False, 0, (0.001, 0.02)),
    ("scale_only_two_operand_rounds", 8200, 1536, 4, SCALE_ONLY, 128, 16, True, 0, (0.001, 0.02)),
    ("nine_rows_walks_longer_than_the_waves", 2048, 1024, 4, SCALE_AND_ZEROS, 128, 9, True, 4, (0.001, 0.02)),
    ("one_wave_sums_every_tile", 4096, 512, 4, SCALE_AND_ZEROS, 128, 4, False, 8, (0.001, 0.02)),
    ("k_not_a_multiple_of_the_step", 304, 1000, 4, PER_COLUMN, 0, 6, True, 8, (0.001, 0.02)),
    ("exact_integer_form", 528, 2048, 4, SCALE_AND_ZEROS, 128, 8, False, 8, (0.05, 0.3)),
    ("walks_of_7_like_28672x8192", 7 * 16 * 24, 8192, 4, SCALE_AND_ZEROS, 128, 4, False, 24, (0.001, 0.02)),
    ("a_single_tile", 16, 8192, 4, SCALE_AND_ZEROS, 128, 8, True, 0, (0.001, 0.02)),
    ("four_output_rows", 4, 512, 4, SCALE_AND_ZEROS, 64, 16, True, 0, (0.001, 0.02)),
    ("one_k_step_of_8", 48, 8, 8, PER_COLUMN, 0, 3, False, 0, (0.001, 0.01)),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_parity_with_the_oracle(gpu, case):
    tag, n_out, k, bits, qop, group, rows, bias, cap, srange = case
    prob = Problem("ks_" + tag, n_out, k, bits, qop, group, m_batch=rows, bias=bias, x_dist="normal", scale_range=srange)
    dev = DeviceProblem(prob, gpu)
    with k_stationary(cap):
        plan = mg.query_launch(n_out, rows, k, bits, prob.group_size)
        assert plan["matrix_core"] == 3 and plan["steps_per_wave"] == 1 and plan["threads"] == 64 * plan["split_k"], plan
        if tag in ("nine_rows_walks_longer_than_the_waves", "one_wave_sums_every_tile"):
            assert plan["tiles_in_sequence"] > plan["split_k"], plan      # a wave sums several tiles of the walk
        elif cap:   # (the two above get more workgroups than asked for: the partial sums of a walk must fit the LDS)
            assert plan["workgroups"] == -(-cap // 8) * 8 and plan["tiles_in_sequence"] == -(-(-(-n_out // 16)) // cap), plan
        cov = mg.plan_coverage(n_out, rows, k, bits, prob.group_size)
        assert cov["tiles_miscovered"] == 0 and cov["bad_waves"] == 0, cov
        got = dev.run().copy()
        again = dev.run().copy()
    assert np.array_equal(got.view(np.uint16), again.view(np.uint16))       # run to run: the same bits
    err, rel, _ = error_report(got, prob.oracle_gemv(threads=8))
    assert rel <= REL_TOL, (err, rel)


def test_results_do_not_depend_on_how_the_tiles_are_walked(gpu):
    """One tile per workgroup, walks of 2, 5 and 10 tiles: the k split is the same (one wave per k step), and so
    is every output bit."""
    prob = Problem("ks_walks", 640, 3072, 4, SCALE_AND_ZEROS, 128, m_batch=6, bias=True, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    with k_stationary(0):
        base = dev.run().copy()
    for cap in (20, 8, 4):
        with k_stationary(cap):
            assert mg.query_launch(640, 6, 3072, 4, 128)["tiles_in_sequence"] == -(-40 // cap)
            got = dev.run().copy()
        assert np.array_equal(got.view(np.uint16), base.view(np.uint16)), cap


def test_outputs_that_are_not_8_byte_aligned_take_the_narrow_stores(gpu):
    import torch
    prob = Problem("ks_align", 528, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=3, bias=True)
    dev = DeviceProblem(prob, gpu)
    with k_stationary(0):
        want = dev.run().copy()
        for shift in (1, 2, 3):
            wide = torch.full((3 * 528 + 8,), 0x7e00, dtype=torch.int16, device=gpu)
            y = wide[shift:shift + 3 * 528].view(3, 528)
            assert y.data_ptr() % 8 == 2 * shift
            mg.device_gemv(dev.w, dev.x, dev.scale, dev.zero, dev.bias, y, 1, 528, 3, 2048, 128, SCALE_AND_ZEROS, 4)
            torch.cuda.synchronize()
            host = wide.cpu().numpy().view(np.uint16)
            assert np.array_equal(host[shift:shift + 3 * 528].reshape(3, 528), want.view(np.uint16)), shift
            assert np.all(host[:shift] == 0x7e00) and np.all(host[shift + 3 * 528:] == 0x7e00)   # nothing beside it


def test_batched_launch_and_epilogue_scalars(gpu):
    """Three problems in one launch (gemv/device/gemv_adaptor.h:129-135) give the bits of three launches; alpha and
    beta (gemv_adaptor.h:123) scale the sum and the bias in fp32 before the one rounding."""
    import torch
    n_out, k, rows, batch = 400, 2048, 5, 3
    probs = [Problem("ks_batch", n_out, k, 4, SCALE_AND_ZEROS, 128, m_batch=rows, bias=True, buffer=b) for b in range(batch)]
    devs = [DeviceProblem(p, gpu) for p in probs]
    w = torch.stack([d.w for d in devs]).contiguous()
    s = torch.stack([d.scale for d in devs]).contiguous()
    z = torch.stack([d.zero for d in devs]).contiguous()
    y = torch.zeros((batch, rows, n_out), dtype=torch.int16, device=gpu)
    with k_stationary(0):
        singles = [d.run().copy() for d in devs]
        mg.device_gemv(w, devs[0].x, s, z, devs[0].bias, y, batch, n_out, rows, k, 128, SCALE_AND_ZEROS, 4,
                       batch_strides=(w[0].numel(), 0, s[0].numel(), 0, rows * n_out))
        torch.cuda.synchronize()
        got = y.cpu().numpy().view(np.uint16)
        for b in range(batch):
            assert np.array_equal(got[b], singles[b].view(np.uint16)), b
        # beta = 0 drops the bias, alpha = 0.5 commutes with the rounding (no result here is subnormal after halving)
        d = devs[0]
        nobias = DeviceProblem(Problem("ks_batch", n_out, k, 4, SCALE_AND_ZEROS, 128, m_batch=rows, bias=False, buffer=0), gpu)
        acc16 = nobias.run().copy()

        def run_arguments(alpha, beta):
            d.y.fill_(0x7e00)
            mg.gemv_arguments(d.w, d.x, d.scale, d.zero, d.bias, d.y, n_out, rows, k, 128, SCALE_AND_ZEROS, 4, alpha=alpha, beta=beta)
            torch.cuda.synchronize()
            return d.y.cpu().numpy().view(np.float16)

        assert np.array_equal(run_arguments(1.0, 1.0).view(np.uint16), singles[0].view(np.uint16))
        assert np.array_equal(run_arguments(1.0, 0.0).view(np.uint16), acc16.view(np.uint16))
        big = np.abs(acc16.astype(np.float32)) >= 2.0 ** -13
        assert np.array_equal(run_arguments(0.5, 0.0)[big].view(np.uint16),
                              (acc16[big].astype(np.float32) * 0.5).astype(np.float16).view(np.uint16))
        # general alpha, beta: alpha * acc + beta * bias with one rounding; acc16 is acc rounded to fp16, so allow its half ulp
        got = run_arguments(-1.75, 3.0).astype(np.float64)
    want = -1.75 * acc16.astype(np.float64) + 3.0 * probs[0].bias.astype(np.float64)[None, :]
    tol = 2.0 ** -10 * (1.75 * np.abs(acc16.astype(np.float64)) + np.abs(want)) + 2.0 ** -24
    assert np.all(np.abs(got - want) <= tol)


def test_the_built_in_rule_takes_it_where_it_was_measured_ahead(gpu):
    """2-8 rows, walks of two or more tiles per compute unit (the rule scales with the device): the default launch
    is this kernel, and its result is the oracle's."""
    import torch
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    n_out = 16 * 2 * cus
    for rows, k, walk in ((4, 4096, 2), (8, 2048, 2), (2, 4096, 3)):     # 2 rows: from 2.5 tiles per compute unit
        n_out = 16 * walk * cus
        plan = mg.query_launch(n_out, rows, k, 4, 128, num_compute_units=cus)
        assert plan["matrix_core"] == 3 and plan["workgroups"] == -(-cus // 8) * 8 and plan["tiles_in_sequence"] == walk, plan
        prob = Problem("ks_rule", n_out, k, 4, SCALE_AND_ZEROS, 128, m_batch=rows, bias=True, x_dist="normal")
        _, rel, _ = error_report(DeviceProblem(prob, gpu).run(), prob.oracle_gemv(threads=16))
        assert rel <= REL_TOL, (rows, k, rel)
    n_out = 16 * 2 * cus
    assert mg.query_launch(n_out, 2, 4096, 4, 128, num_compute_units=cus)["matrix_core"] == 0     # 2 rows on walks of 2: VALU
    assert mg.query_launch(n_out, 16, 4096, 4, 128, num_compute_units=cus)["matrix_core"] == 2    # 9-16 rows, filled alike: LDS-staged
    assert mg.query_launch(n_out, 4, 1024, 4, 128, num_compute_units=cus)["matrix_core"] != 3      # 2 k steps: too few waves
    assert mg.query_launch(n_out, 4, 16384, 4, 128, num_compute_units=cus)["matrix_core"] == 2     # 32 k steps: no such launch
    assert mg.query_launch(n_out, 4, 4096, 4, 128, element="bf16", num_compute_units=cus)["matrix_core"] == 2   # fp16 only


def test_measurement_builds(gpu):
    """Arithmetic-only: with walks of one tile every unit is loaded, and the result is the product's, bit for bit.
    Loads-only, and arithmetic-only on longer walks: they run and write every output.  No time-stamped build, and none
    for group sizes that put four groups on a lane's run."""
    import torch
    from mixed_gemv_amd._lib import MixedGemvError
    prob = Problem("ks_probe", 512, 4096, 4, SCALE_AND_ZEROS, 128, m_batch=5, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    trace = torch.zeros((4096, mg.PROBE_TIMELINE_WORDS), dtype=torch.int64, device=gpu)
    with k_stationary(0):
        assert mg.query_launch(512, 5, 4096, 4, 128)["tiles_in_sequence"] == 1
        want = dev.run().copy()
        dev.y.fill_(0x7e00)
        mg.probe_gemv_rows(mg.PROBE_COMPUTE_ONLY, 5, dev.w, dev.x, dev.scale, dev.zero, dev.y, 512, 4096, 128)
        torch.cuda.synchronize()
        assert np.array_equal(dev.y.cpu().numpy().view(np.uint16), want.view(np.uint16))
        dev.y.fill_(0x7e00)
        mg.probe_gemv_rows(mg.PROBE_LOADS_ONLY, 5, dev.w, dev.x, dev.scale, dev.zero, dev.y, 512, 4096, 128)
        torch.cuda.synchronize()
        assert not np.any(dev.y.cpu().numpy().view(np.uint16) == 0x7e00)
    with k_stationary(4):     # walks of 8 tiles: both builds run and write every output
        for kind in (mg.PROBE_LOADS_ONLY, mg.PROBE_COMPUTE_ONLY):
            dev.y.fill_(0x7e00)
            mg.probe_gemv_rows(kind, 5, dev.w, dev.x, dev.scale, dev.zero, dev.y, 512, 4096, 128)
            torch.cuda.synchronize()
            assert not np.any(dev.y.cpu().numpy().view(np.uint16) == 0x7e00)
        with pytest.raises(MixedGemvError):
            mg.probe_gemv(mg.PROBE_TIMELINE, trace, dev.w, dev.x, dev.scale, dev.zero, dev.y, 512, 4096, 128)
        with pytest.raises(MixedGemvError):     # group size 96: four groups per lane run, no measurement build
            mg.probe_gemv_rows(mg.PROBE_LOADS_ONLY, 5, dev.w, dev.x, dev.scale, dev.zero, dev.y, 512, 768, 96)
