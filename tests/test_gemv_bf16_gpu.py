"""GPU parity of the bfloat16 entry points (mgemv_gemv_bf16, mgemv_dequantize_bf16), called
through the C-ABI, against the CPU oracle's bf16 functions.

Bars: dequantised weights bit-exact.  Outputs: the oracle's bf16 value or one of its two
neighbours (1 ulp; two correct fp32 sums that differ in their last bits can round to adjacent
bf16 values, and a bf16 ulp is up to 2^-7 relative, so the fp16 bar of 2e-3 cannot be asked),
with at most 1 % of the outputs differing at all."""
import numpy as np
import pytest

import mixed_gemv_amd as mg
import oracle as orc
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, DeviceProblem, Problem, bf16_ulp_report

pytestmark = pytest.mark.gpu

MAX_ULP = 1.0 + 1e-6
MAX_DIFFERING = 0.01


def check(prob, gpu, dequant=True):
    dev = DeviceProblem(prob, gpu)
    if dequant:
        mism = int((dev.dequant() != prob.oracle_dequant()).sum())
        assert mism == 0, f"{mism} dequantised weights differ"
    y = dev.run()
    ref = prob.oracle_gemv(threads=16)
    ulp, differing = bf16_ulp_report(y, ref)
    print(f"{prob.tag}: worst {ulp:.3f} ulp, {100 * differing:.2f} % of outputs differ", flush=True)
    assert np.isfinite(orc.bf16_to_f32_array(y)).all()
    assert ulp <= MAX_ULP and differing <= MAX_DIFFERING
    return dev, y


SMALL = [
    # tag, n_out, k, bits, quant_op, group, m_batch, bias
    ("b_i4_sz_g128", 256, 1024, 4, SCALE_AND_ZEROS, 128, 1, False),
    ("b_i4_sz_g64", 256, 1024, 4, SCALE_AND_ZEROS, 64, 1, True),
    ("b_i4_sz_g256", 64, 2048, 4, SCALE_AND_ZEROS, 256, 2, True),
    ("b_i4_s_g128", 128, 2048, 4, SCALE_ONLY, 128, 1, True),
    ("b_i4_col", 128, 1024, 4, PER_COLUMN, 0, 3, False),
    ("b_i8_col", 256, 1024, 8, PER_COLUMN, 0, 1, True),
    ("b_i8_sz_g64", 128, 512, 8, SCALE_AND_ZEROS, 64, 4, False),
    ("b_i8_s_g96", 32, 576, 8, SCALE_ONLY, 96, 1, False),           # group not a power of two
    ("b_i4_ragged", 100, 1120, 4, SCALE_AND_ZEROS, 160, 1, True),   # n_out % 16 != 0, k % 512 != 0, odd group
    ("b_i4_tiny", 4, 64, 4, SCALE_AND_ZEROS, 64, 1, True),
    ("b_i4_mb7", 64, 1024, 4, SCALE_AND_ZEROS, 64, 7, False),       # two launches of the VALU kernel
    ("b_i8_mb16", 48, 512, 8, PER_COLUMN, 0, 16, True),
    ("b_i4_one_tile_mb7", 16, 512, 4, SCALE_AND_ZEROS, 128, 7, True),   # a single tile: no matrix-core kernel fits
    ("b_i4_two_tiles_mb12", 20, 1024, 4, SCALE_AND_ZEROS, 128, 12, False),
]


@pytest.mark.parametrize("cfg", SMALL, ids=[c[0] for c in SMALL])
@pytest.mark.parametrize("form", ["auto", "general"])
def test_small_parity(gpu, cfg, form):
    tag, n_out, k, bits, qop, g, mb, bias = cfg
    try:
        mg.set_dequant_form(mg.DEQUANT_EXACT_INTEGER if form == "general" else mg.DEQUANT_AUTO)
        check(Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias, element="bf16"), gpu)
    finally:
        mg.set_dequant_form(mg.DEQUANT_AUTO)


@pytest.mark.parametrize("form", ["auto", "general"])
@pytest.mark.parametrize("bits", [4, 8])
def test_dequant_every_finite_scale_bit_exact(gpu, bits, form):
    """Each (row, group) gets its own scale so that ALL finite bf16 scales (subnormals, huge values,
    both signs) meet every int4 weight value (a spread of int8 values), with an additive zero:
    multiply, round, add, round.  Consecutive bit patterns share a tile, so in "auto" the tiles
    whose scales all lie in 0x0d80..0x7aff take the fused form and the others the general one."""
    allbits = np.arange(65536, dtype=np.uint16)
    finite = allbits[(allbits & 0x7F80) != 0x7F80]            # 65280 values
    n_out, g = 64, 64
    groups = finite.size // n_out                              # 1020
    k = groups * g
    prob = Problem(f"b_allscales{bits}", n_out, k, bits, SCALE_AND_ZEROS, g, element="bf16")
    if bits == 4:   # every group of every row holds all 16 values
        q = np.tile(np.arange(-8, 8, dtype=np.int8), n_out * k // 16)
        prob.q, prob.w_raw = q, orc.pack_int4(q)
    prob.scale = finite.reshape(groups, n_out).copy()
    zero = orc.f32_to_bf16_array(orc.fill_uniform_f16(groups * n_out, 99, -0.05, 0.05).astype(np.float32)).reshape(groups, n_out)
    zero[::7, ::3] = 0x0000
    zero[1::7, ::5] = 0x8000
    zero[2::11, :] = np.arange(1, n_out + 1, dtype=np.uint16)          # subnormal additive terms
    prob.zero_add = zero
    try:
        mg.set_dequant_form(mg.DEQUANT_EXACT_INTEGER if form == "general" else mg.DEQUANT_AUTO)
        got = DeviceProblem(prob, gpu).dequant()
    finally:
        mg.set_dequant_form(mg.DEQUANT_AUTO)
    want = prob.oracle_dequant()
    nan = np.isnan(orc.bf16_to_f32_array(want))
    assert np.array_equal(np.isnan(orc.bf16_to_f32_array(got)), nan)   # inf - inf: NaN on both sides
    assert int((got[~nan] != want[~nan]).sum()) == 0


def test_one_hot_activation_is_bit_exact_through_the_gemv_kernel(gpu):
    """y[n] == dq[n, j] bit for bit (up to the sign of a zero): pins the dequantiser inside the GEMV kernel."""
    prob = Problem("b_onehot", 96, 1536, 4, SCALE_AND_ZEROS, 128, element="bf16")
    dq = prob.oracle_dequant()
    dev = DeviceProblem(prob, gpu)
    import torch
    for j in (0, 1, 127, 128, 511, 512, 1000, 1535):
        x = np.zeros((1, prob.k), dtype=np.uint16)
        x[0, j] = 0x3F80
        dev.x = torch.from_numpy(x.view(np.int16)).to(gpu)
        y = dev.run()[0]
        nz = (dq[:, j] & 0x7FFF) != 0
        assert np.array_equal(y[nz], dq[:, j][nz]), j
        assert np.all((y[~nz] & 0x7FFF) == 0), j


@pytest.mark.parametrize("split,tw", [(0, 1), (4, 1), (2, 2), (2, 4), (1, 8)])
@pytest.mark.parametrize("bits", [4, 8])
def test_one_hot_rows_are_bit_exact_through_the_matrix_core_kernel(gpu, bits, split, tw):
    """One-hot activation rows, each at a k of its own, through v_mfma_f32_16x16x32_bf16: y[b][n] == dq[n][k_b]
    bit for bit (up to the sign of a zero), with a stage per wave and with stages shared by 2, 4 and 8 tiles,
    8 and 16 staged rows, the fused and the general dequantiser."""
    import torch
    k = 1536 if bits == 4 else 768
    for m_batch, scale_range in ((5, (1e-4, 0.02)), (8, (1e-4, 0.02)), (16, (1e-4, 0.02)), (13, (1e-4, 0.02))):
        if (8 if m_batch <= 8 else 16) // tw < 2:
            continue
        prob = Problem(f"b_mc_onehot{bits}", 112, k, bits, SCALE_AND_ZEROS, 64, m_batch=m_batch, scale_range=scale_range,
                       element="bf16")
        if m_batch == 13:      # scales outside the fused form's range (negative, tiny): the general dequantiser
            prob.scale[::2, ::3] = 0xBC80
            prob.scale[1::2, 1::3] = 0x0C00
        dq = prob.oracle_dequant()
        dev = DeviceProblem(prob, gpu)
        try:
            mg.set_matrix_core_threshold(1)
            mg.set_launch_override(split, tw, 0, 0)
            plan = mg.query_launch(prob.n_out, m_batch, k, bits, element="bf16")
            assert plan["matrix_core"] == 2 and plan["tiles_per_wg"] == tw, plan
            for trial in range(4):
                hot = [(b * 37 + trial * 131) % k for b in range(m_batch)]
                if trial == 0:
                    hot[:4] = [0, k - 1, 511 if bits == 4 else 255, 512 if bits == 4 else 256][:m_batch]
                x = np.zeros((m_batch, k), dtype=np.uint16)
                x[np.arange(m_batch), hot] = 0x3F80
                dev.x = torch.from_numpy(x.view(np.int16)).to(gpu)
                got = dev.run()
                for b in range(m_batch):
                    want = dq[:, hot[b]]
                    finite = (want & 0x7F80) != 0x7F80
                    nz = ((want & 0x7FFF) != 0) & finite
                    assert np.array_equal(got[b][nz], want[nz]), (m_batch, trial, b, hot[b])
                    assert np.all((got[b][~nz & finite] & 0x7FFF) == 0)
        finally:
            mg.set_matrix_core_threshold(0)
            mg.set_launch_override(0, 0, 0, 0)


def test_split_k_and_tile_walk_invariance(gpu):
    prob = Problem("b_splitk", 192, 8192, 4, SCALE_AND_ZEROS, 128, bias=True, x_dist="normal", element="bf16")
    dev = DeviceProblem(prob, gpu)
    ref = prob.oracle_gemv(threads=16)
    results = {}
    try:
        for sk, tw, cap in ((1, 1, 0), (1, 4, 0), (2, 2, 0), (4, 2, 0), (8, 1, 0), (1, 1, 5), (4, 2, 2)):
            mg.set_launch_override(sk, tw, 0, cap)
            a = dev.run().copy()
            assert np.array_equal(a, dev.run()), "same launch geometry must be bit-reproducible"
            ulp, differing = bf16_ulp_report(a, ref)
            assert ulp <= MAX_ULP and differing <= MAX_DIFFERING, (sk, tw, cap, ulp, differing)
            results[(sk, tw, cap)] = a
    finally:
        mg.set_launch_override(0, 0, 0, 0)
    for other in ((1, 4, 0), (1, 1, 5)):   # the same k split adds in the same order wherever the tiles run
        assert np.array_equal(results[(1, 1, 0)], results[other]), other


@pytest.mark.parametrize("bits,qop,g", [(4, SCALE_AND_ZEROS, 128), (4, SCALE_ONLY, 64), (4, PER_COLUMN, 0),
                                        (8, SCALE_AND_ZEROS, 64), (8, PER_COLUMN, 0), (4, SCALE_AND_ZEROS, 160)])
def test_matrix_core_and_valu_kernels_agree(gpu, bits, qop, g):
    """The same batches through the LDS-staged matrix-core kernel (v_mfma_f32_16x16x32_bf16) at
    several k splits and through the VALU kernel (threshold forced), ragged shape, every mode,
    both dequantiser forms."""
    n_out, k = 100, 1120 if g in (0, 160) else 1024
    for m_batch in (1, 5, 8, 13, 16):
        prob = Problem(f"b_mc{bits}{qop}", n_out, k, bits, qop, g, m_batch=m_batch, bias=True, element="bf16")
        dev = DeviceProblem(prob, gpu)
        ref = prob.oracle_gemv(threads=8)
        results = []
        try:
            for form in (mg.DEQUANT_AUTO, mg.DEQUANT_EXACT_INTEGER):
                mg.set_dequant_form(form)
                mg.set_matrix_core_threshold(1)
                for split, tw in ((0, 0), (1, 2), (2, 2), (4, 1), (2, 4), (1, 8)):   # k-split waves, tiles per workgroup
                    mg.set_launch_override(split, tw, 0, 0)
                    results.append(dev.run().copy())
                    assert np.array_equal(results[-1], dev.run())   # reproducible
                mg.set_launch_override(0, 0, 0, 0)
                mg.set_matrix_core_threshold(17)
                results.append(dev.run().copy())   # VALU kernel
        finally:
            mg.set_matrix_core_threshold(0)
            mg.set_launch_override(0, 0, 0, 0)
            mg.set_dequant_form(mg.DEQUANT_AUTO)
        for y in results:
            ulp, differing = bf16_ulp_report(y, ref)
            assert ulp <= MAX_ULP and differing <= MAX_DIFFERING, (m_batch, ulp, differing)


def test_launch_query_knows_the_bf16_kernels(gpu):
    # 8-wave workgroups at most, and only the LDS-staged matrix-core kernel
    assert mg.query_launch(1024, 1, 8192, 4, 128)["threads"] == 1024
    assert mg.query_launch(1024, 1, 8192, 4, 128, element="bf16")["threads"] == 512
    assert mg.query_launch(16, 7, 512, 4, 128)["matrix_core"] == 1                      # fp16, a single tile: register operand
    assert mg.query_launch(1024, 5, 2048, 4, 128, element="bf16")["matrix_core"] == 2
    assert mg.query_launch(16, 7, 512, 4, 128, element="bf16")["matrix_core"] == 0      # a single tile


def test_batched_launch_with_strides(gpu):
    """batch_count problems in one launch: stacked weights and scales, shared activations."""
    import torch
    n_out, k, g, batch = 64, 1024, 128, 3
    probs = [Problem(f"b_batch{b}", n_out, k, 4, SCALE_AND_ZEROS, g, bias=True, element="bf16") for b in range(batch)]
    devs = [DeviceProblem(p, gpu) for p in probs]
    w = torch.stack([d.w for d in devs]).contiguous()
    s = torch.stack([d.scale for d in devs]).contiguous()
    z = torch.stack([d.zero for d in devs]).contiguous()
    bias = torch.stack([d.bias for d in devs]).contiguous()
    y = torch.zeros((batch, 1, n_out), dtype=torch.int16, device=gpu)
    mg.device_gemv(w, devs[0].x, s, z, bias, y, batch, n_out, 1, k, g, SCALE_AND_ZEROS, 4,
                   batch_strides=(w.stride(0), 0, s.stride(0), bias.stride(0), y.stride(0)), element="bf16")
    torch.cuda.synchronize()
    got = y.cpu().numpy().view(np.uint16)
    for b, p in enumerate(probs):
        p.x = probs[0].x
        ulp, differing = bf16_ulp_report(got[b], p.oracle_gemv(threads=8))
        assert ulp <= MAX_ULP and differing <= MAX_DIFFERING


def test_torch_bfloat16_tensors_select_the_bf16_entry_points(gpu):
    import torch
    prob = Problem("b_torch", 128, 1024, 4, SCALE_AND_ZEROS, 128, bias=True, element="bf16")
    dev = DeviceProblem(prob, gpu)
    want = dev.run()
    x, s, z, b = (t.view(torch.bfloat16) for t in (dev.x, dev.scale, dev.zero, dev.bias))
    y = torch.zeros((1, 128), dtype=torch.bfloat16, device=gpu)
    mg.device_gemv(dev.w, x, s, z, b, y, 1, 128, 1, 1024, 128, SCALE_AND_ZEROS, 4)      # element from the dtype
    torch.cuda.synchronize()
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), want)
    adaptor = mg.GemvAdaptor(SCALE_AND_ZEROS, 4)
    y.zero_()
    adaptor(mg.GemvAdaptor.Arguments((128, 1, 1024), dev.w, x, s, z, b, y, group_size=128))
    torch.cuda.synchronize()
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), want)


FULL = [
    ("b_ns", 4096, 4096, 4, SCALE_AND_ZEROS, 128, 1, False, "uniform"),
    ("b_c1", 4096, 4096, 8, PER_COLUMN, 0, 1, True, "uniform"),
    ("b_c3a", 11008, 4096, 4, SCALE_AND_ZEROS, 128, 1, False, "normal"),
    ("b_c4_m4", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 4, True, "uniform"),
    ("b_c4_m16", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 16, True, "uniform"),   # matrix cores
]


@pytest.mark.parametrize("cfg", FULL, ids=[c[0] for c in FULL])
def test_baseline_shapes_full_size(gpu, cfg):
    tag, n_out, k, bits, qop, g, mb, bias, xd = cfg
    check(Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias, x_dist=xd, element="bf16"), gpu)
