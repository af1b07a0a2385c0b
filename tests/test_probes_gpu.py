"""The measurement probes of the library (include/mixed_gemv_probes.h): they run,
the timeline build of the kernel still computes the GEMV, and its timestamps are ordered."""
import numpy as np
import pytest

import mixed_gemv_amd as mg
from helpers import SCALE_AND_ZEROS, DeviceProblem, Problem
from mixed_gemv_amd._lib import MixedGemvError

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_out,k,cap", [(512, 4096, 0), (4096, 2048, 0), (192, 8192, 5)])  # cap: waves walk several tiles
def test_timeline_build_is_the_product_kernel_plus_timestamps(gpu, n_out, k, cap):
    import torch
    prob = Problem("probe", n_out, k, 4, SCALE_AND_ZEROS, 128, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    try:
        mg.set_launch_override(0, 0, 0, cap)
        want = dev.run().copy()
        cus = torch.cuda.get_device_properties(gpu).multi_processor_count
        plan = mg.query_launch(n_out, 1, k, 4, 128, num_compute_units=cus)
        waves = -(-plan["workgroups"] // 8) * 8 * plan["threads"] // 64      # the grid is a multiple of 8 workgroups
        with pytest.raises(MixedGemvError):                                  # a trace that is too small is refused
            mg.probe_gemv(mg.PROBE_TIMELINE, torch.zeros((waves - 1, mg.PROBE_TIMELINE_WORDS), dtype=torch.int64, device=gpu),
                          dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 128)
        trace = torch.zeros((waves, mg.PROBE_TIMELINE_WORDS), dtype=torch.int64, device=gpu)
        dev.y.fill_(0x7e00)
        mg.probe_gemv(mg.PROBE_TIMELINE, trace, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 128)
        torch.cuda.synchronize()
        assert np.array_equal(dev.y.cpu().numpy().view(np.uint16), want.view(np.uint16))
        t = trace.cpu().numpy()
        t = t[t[:, 0] > 0]                                  # workgroups past the last tile leave before stamping
        assert len(t) >= (n_out // 16) * plan["split_k"] // max(plan["tiles_in_sequence"], 1) // 2
        assert np.all(np.diff(t[:, :5], axis=1) >= 0)       # entry <= requested <= arrived <= computed <= stored
        assert (t[:, 4] - t[:, 0]).max() < 100_000          # 10 ns ticks: under a millisecond
        units = plan["steps_per_wave"] * plan["tiles_in_sequence"]
        assert t[:, 11].max() == units and t[:, 11].min() >= 0
        loop = t[t[:, 11] >= 2]                              # waves of two or more units run the loop and time their waits
        assert np.all(loop[:, 5:8].sum(axis=1) <= loop[:, 3] - loop[:, 1])   # waits lie inside the loop
        assert np.all(loop[:, 8] <= loop[:, 5:8].sum(axis=1))
        later = loop[loop[:, 9] > 0]
        assert np.all((later[:, 9] >= later[:, 1]) & (later[:, 9] <= later[:, 3]))
        mg.probe_gemv(mg.PROBE_LOADS_ONLY, None, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 128)
        torch.cuda.synchronize()
    finally:
        mg.set_launch_override(0, 0, 0, 0)


@pytest.mark.parametrize("n_out,k,split", [(640, 512, 0), (320, 2048, 4), (4096, 4096, 0)])
def test_compute_only_build_repeats_the_first_unit(gpu, n_out, k, split):
    """With one unit per wave (one k step, or as many k-split waves as k steps) the arithmetic-only
    build loads everything the product loads: same bits.  With more units per wave it runs and
    writes finite-or-not garbage that must simply not fault."""
    import torch
    prob = Problem("probe_c", n_out, k, 4, SCALE_AND_ZEROS, 128, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    try:
        mg.set_launch_override(split, 0, 0, 0)
        plan = mg.query_launch(n_out, 1, k, 4, 128)
        want = dev.run().copy()
        dev.y.fill_(0x7e00)
        mg.probe_gemv(mg.PROBE_COMPUTE_ONLY, None, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 128)
        torch.cuda.synchronize()
        got = dev.y.cpu().numpy().view(np.uint16)
        if plan["steps_per_wave"] * plan["tiles_in_sequence"] == 1:
            assert np.array_equal(got.reshape(-1), want.view(np.uint16).reshape(-1))
        else:
            assert not np.any(got == 0x7e00)    # every output was written
    finally:
        mg.set_launch_override(0, 0, 0, 0)


@pytest.mark.parametrize("m_batch", [4, 8, 16])
def test_matrix_core_measurement_builds_run(gpu, m_batch):
    """Loads-only and arithmetic-only builds of the LDS-staged matrix-core kernel: they exist for launches
    whose workgroups share a stage between tiles, write every output, and are refused elsewhere."""
    import torch
    n_out, k = 8192, 2048       # 512 tiles: two tiles per workgroup
    prob = Problem("probe_mc", n_out, k, 4, SCALE_AND_ZEROS, 64, m_batch=m_batch, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    mg.set_matrix_core_variant(mg.MATRIX_CORE_LDS_STAGED)    # (up to 8 rows the built-in rule gives this shape to the k-stationary kernel)
    try:
        plan = mg.query_launch(n_out, m_batch, k, 4, 64)
        assert plan["matrix_core"] == 2 and plan["tiles_per_wg"] >= 2
        for kind in (mg.PROBE_LOADS_ONLY, mg.PROBE_COMPUTE_ONLY):
            dev.y.fill_(0x7e00)
            mg.probe_gemv_rows(kind, m_batch, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 64)
            torch.cuda.synchronize()
            assert not np.any(dev.y.cpu().numpy().view(np.uint16) == 0x7e00)
        with pytest.raises(MixedGemvError):     # one tile per workgroup: no measurement build
            mg.probe_gemv_rows(mg.PROBE_LOADS_ONLY, 8, dev.w, dev.x, dev.scale, dev.zero, dev.y, 2048, k, 64)
        with pytest.raises(MixedGemvError):
            mg.probe_gemv_rows(mg.PROBE_TIMELINE, 8, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 64)
    finally:
        mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
    if m_batch <= 8:    # the built-in rule: the k-stationary kernel, whose measurement builds write every output too
        assert mg.query_launch(n_out, m_batch, k, 4, 64)["matrix_core"] == 3
        for kind in (mg.PROBE_LOADS_ONLY, mg.PROBE_COMPUTE_ONLY):
            dev.y.fill_(0x7e00)
            mg.probe_gemv_rows(kind, m_batch, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 64)
            torch.cuda.synchronize()
            assert not np.any(dev.y.cpu().numpy().view(np.uint16) == 0x7e00)
        with pytest.raises(MixedGemvError):
            mg.probe_gemv_rows(mg.PROBE_TIMELINE, m_batch, dev.w, dev.x, dev.scale, dev.zero, dev.y, n_out, k, 64)


def test_stream_read_and_empty_launch_run_and_check_their_arguments(gpu):
    import torch
    buf = torch.zeros(8 << 20, dtype=torch.uint8, device=gpu)
    sink = torch.zeros(1, dtype=torch.int32, device=gpu)
    for wgs, waves, depth in ((256, 4, 2), (64, 16, 4), (8, 1, 8)):
        mg.probe_stream_read(buf, buf.numel(), wgs, waves, depth, sink)
    mg.probe_empty_launch()
    mg.probe_empty_grid(256, 4)
    mg.probe_empty_grid(8016, 1)
    torch.cuda.synchronize()
    for bad in ((0, 4), (256, 0), (256, 17)):
        with pytest.raises(MixedGemvError):
            mg.probe_empty_grid(*bad)
    for bad in ((0, 4, 2), (256, 17, 2), (256, 4, 3), (4096, 16, 2)):   # the last: less than one unit per wave
        with pytest.raises(MixedGemvError):
            mg.probe_stream_read(buf, buf.numel(), *bad, sink)
    with pytest.raises(MixedGemvError):
        mg.probe_gemv(mg.PROBE_TIMELINE, None, buf, buf, buf, buf, buf, 64, 512, 128)   # needs a trace buffer
    with pytest.raises(MixedGemvError):
        mg.probe_gemv(mg.PROBE_LOADS_ONLY, None, buf, buf, buf, buf, buf, 64, 512, 64)  # two groups per run: no probe build
