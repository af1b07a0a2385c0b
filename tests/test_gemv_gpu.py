"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle.

Bars: dequantised weights bit-exact; fp16 outputs within max relative error 2e-3 with the
denominator max(|ref|, 2^-7 * rms(ref)) (helpers.error_report explains the floor).  Max abs / max rel errors are printed per case.
"""
import numpy as np
import pytest

import mixed_gemv_amd as mg
import oracle as orc
from helpers import (PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, DeviceProblem, Problem, error_report,
                     float64_bound_violations)

pytestmark = pytest.mark.gpu

REL_TOL = 2e-3


def check(prob, gpu, dequant=True, label=None):
    dev = DeviceProblem(prob, gpu)
    if dequant:
        dq = dev.dequant()
        mism = int((dq.view(np.uint16) != prob.oracle_dequant().view(np.uint16)).sum())
        assert mism == 0, f"{mism} dequantised weights differ"
    y = dev.run()
    ref = prob.oracle_gemv(threads=16)
    abs_err, rel_err, floor = error_report(y, ref)
    print(f"{label or prob.tag}: max_abs={abs_err:.3e} max_rel={rel_err:.3e} (floor {floor:.3e})", flush=True)
    assert np.isfinite(y.astype(np.float32)).all()
    assert rel_err <= REL_TOL
    return dev, y


SMALL = [
    # tag, n_out, k, bits, quant_op, group, m_batch, bias
    ("s_i4_sz_g128", 256, 1024, 4, SCALE_AND_ZEROS, 128, 1, False),
    ("s_i4_sz_g64", 256, 1024, 4, SCALE_AND_ZEROS, 64, 1, True),
    ("s_i4_sz_g256", 64, 2048, 4, SCALE_AND_ZEROS, 256, 1, True),
    ("s_i4_s_g128", 128, 2048, 4, SCALE_ONLY, 128, 1, True),
    ("s_i4_s_g64", 64, 512, 4, SCALE_ONLY, 64, 2, False),
    ("s_i4_col", 128, 1024, 4, PER_COLUMN, 0, 1, False),
    ("s_i8_col", 256, 1024, 8, PER_COLUMN, 0, 1, True),
    ("s_i8_sz_g64", 128, 512, 8, SCALE_AND_ZEROS, 64, 1, False),
    ("s_i8_sz_g128", 64, 768, 8, SCALE_AND_ZEROS, 128, 3, True),
    ("s_i8_s_g128", 128, 512, 8, SCALE_ONLY, 128, 2, True),
    ("s_i8_s_g96", 32, 576, 8, SCALE_ONLY, 96, 1, False),          # group not a power of two
    ("s_i4_ragged", 100, 1120, 4, SCALE_AND_ZEROS, 160, 1, True),  # n_out % 16 != 0, k % 512 != 0, odd group
    ("s_i4_tiny", 4, 64, 4, SCALE_AND_ZEROS, 64, 1, True),         # one partial tile, two chunks
    ("s_i4_one_chunk", 8, 32, 4, PER_COLUMN, 0, 1, False),         # a single 128-bit access per row
    ("s_i8_tiny", 4, 16, 8, PER_COLUMN, 0, 1, True),
    ("s_i4_mb3", 64, 1536, 4, SCALE_AND_ZEROS, 128, 3, True),
    ("s_i4_mb7", 64, 1024, 4, SCALE_AND_ZEROS, 64, 7, False),
    ("s_i4_mb16", 48, 1024, 4, SCALE_AND_ZEROS, 128, 16, True),
    ("s_i8_mb9", 48, 512, 8, PER_COLUMN, 0, 9, True),
    ("s_i4_one_tile_mb7", 16, 512, 4, SCALE_AND_ZEROS, 128, 7, True),   # a single tile: register-operand matrix core
    ("s_i4_two_tiles_mb12", 20, 1024, 4, SCALE_AND_ZEROS, 128, 12, False),
]


@pytest.mark.parametrize("cfg", SMALL, ids=[c[0] for c in SMALL])
def test_small_parity(gpu, cfg):
    tag, n_out, k, bits, qop, g, mb, bias = cfg
    check(Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias), gpu)


def test_reference_zero_convention_int8_zero_points(gpu):
    """The reference's own inputs (mixed_gemv_test.cu:224-239): scales in [0.1, 0.3], int8 zero
    points in [-8, 7] folded on the host; outputs also within the reference's abs 1e-3 per unit scale."""
    prob = Problem("ref_conv", 512, 2048, 4, SCALE_AND_ZEROS, 128, scale_range=(0.1, 0.3), zero_kind="int8")
    dev, y = check(prob, gpu)
    literal = prob.oracle_gemv(threads=16, literal_int8_zero=True)  # host/mixed_gemv.h:92-96 as written
    _, rel, _ = error_report(y, literal)
    assert rel <= REL_TOL


def test_converter_every_16_bit_pattern(gpu):
    """Every 16-bit pattern in both halves of a stored word, scale 1: the kernels' converter must
    return the exact integers (gemv/interleaved_numeric_conversion.h:232-291 contract)."""
    import torch
    h = np.arange(65536, dtype=np.uint32)
    words = (h | ((h[::-1].copy()) << 16)).astype(np.uint32)       # low half ascending, high half descending
    n_out, k = 128, 4096                                           # 65536 words x 8 nibbles
    pre = words.view(np.uint8)
    assert pre.size == mg.preprocessed_size((k, n_out), mg.QuantType.W4_A16)
    raw = mg.unpreprocess_weights(pre, (k, n_out), mg.QuantType.W4_A16)
    scale = np.ones((1, n_out), dtype=np.float16)
    out = torch.zeros((n_out, k), dtype=torch.int16, device=gpu)
    mg.dequantize(torch.from_numpy(pre.copy()).to(gpu), torch.from_numpy(scale.view(np.int16)).to(gpu), None, out, n_out,
                  k, k, PER_COLUMN, 4)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.float16)
    want = orc.unpack_int4(raw).reshape(n_out, k).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))   # also checks that zero is +0
    # int8: all byte values in all four byte positions
    b = np.arange(256, dtype=np.uint32)
    words8 = np.concatenate([b | (b[::-1] << 8) | (np.roll(b, 7) << 16) | (np.roll(b, 101) << 24)] * 4).astype(np.uint32)
    n8, k8 = 16, 256
    pre8 = words8.view(np.uint8)
    assert pre8.size == mg.preprocessed_size((k8, n8), mg.QuantType.W8_A16)
    raw8 = mg.unpreprocess_weights(pre8, (k8, n8), mg.QuantType.W8_A16)
    out8 = torch.zeros((n8, k8), dtype=torch.int16, device=gpu)
    mg.dequantize(torch.from_numpy(pre8.copy()).to(gpu), torch.from_numpy(np.ones((1, n8), np.float16).view(np.int16)).to(gpu),
                  None, out8, n8, k8, k8, PER_COLUMN, 8)
    torch.cuda.synchronize()
    want8 = raw8.view(np.int8).reshape(n8, k8).astype(np.float16)
    assert np.array_equal(out8.cpu().numpy().view(np.uint16), want8.view(np.uint16))


@pytest.fixture
def exact_integer_form():
    """Forces the kernels onto the exact-integer int4 dequantiser for the duration of a test."""
    mg.set_dequant_form(mg.DEQUANT_EXACT_INTEGER)
    yield
    mg.set_dequant_form(mg.DEQUANT_AUTO)


@pytest.mark.parametrize("cfg", [c for c in SMALL if c[3] == 4], ids=[c[0] for c in SMALL if c[3] == 4])
def test_small_parity_exact_integer_form(gpu, exact_integer_form, cfg):
    """The same cases with the one-FMA int4 dequantiser switched off (the default scale range of
    these problems lies below 2^-5, so test_small_parity runs them on the one-FMA form)."""
    tag, n_out, k, bits, qop, g, mb, bias = cfg
    check(Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias), gpu)


def test_one_fma_form_boundaries_bit_exact(gpu):
    """Scales at and around the limits of the one-FMA int4 dequantiser (positive, below 2^-5):
    whole tiles inside the range take it, a tile with a single lane outside must not; all modes."""
    special = np.array([0x0001, 0x0002, 0x03FF, 0x0400, 0x0401, 0x13FF, 0x2000, 0x27FE, 0x27FF,      # inside
                        0x2800, 0x2801, 0x3C00, 0x7BFF, 0x0000, 0x8000, 0x8001, 0xA7FF, 0xFBFF],    # outside
                       dtype=np.uint16)
    n_out, g, k = 16 * special.size * 2, 128, 1024
    groups = k // g
    scale = np.empty((groups, n_out), dtype=np.uint16)
    for t, bits16 in enumerate(special):                 # tile t: every lane has the special value
        scale[:, 16 * t:16 * t + 16] = bits16
    for t, bits16 in enumerate(special):                 # tile size+t: in range, except one lane of one group
        scale[:, 16 * (special.size + t):16 * (special.size + t) + 16] = 0x2400
        scale[t % groups, 16 * (special.size + t) + (5 * t) % 16] = bits16
    q = np.tile(np.arange(-8, 8, dtype=np.int8), n_out * k // 16)
    for qop in (SCALE_AND_ZEROS, SCALE_ONLY, PER_COLUMN):
        prob = Problem(f"edge{qop}", n_out, k, 4, qop, g if qop != PER_COLUMN else 0)
        prob.q, prob.w_raw = q, orc.pack_int4(q)
        prob.scale = (scale if qop != PER_COLUMN else scale[:1]).view(np.float16).copy()
        if qop == SCALE_AND_ZEROS:
            zero = orc.fill_uniform_f16(groups * n_out, 5, -0.01, 0.01).reshape(groups, n_out)
            zero[0, ::2] = np.float16(0.0)
            zero[1, ::3] = np.float16(-0.0)
            prob.zero_add = zero
        for form in (mg.DEQUANT_AUTO, mg.DEQUANT_EXACT_INTEGER):
            mg.set_dequant_form(form)
            try:
                got = DeviceProblem(prob, gpu).dequant().view(np.uint16)
            finally:
                mg.set_dequant_form(mg.DEQUANT_AUTO)
            want = prob.oracle_dequant().view(np.uint16)
            assert int((got != want).sum()) == 0, (qop, form)


@pytest.mark.parametrize("form", ["auto", "exact_integer"])
@pytest.mark.parametrize("bits", [4, 8])
def test_dequant_every_finite_scale_bit_exact(gpu, bits, form, request):
    """Each (row, group) gets its own scale so that ALL finite fp16 scales (subnormals, huge
    values, both signs) meet every weight value, with an additive zero; mul-then-add, two roundings.
    Consecutive bit patterns sit in the same tile, so the tiles whose scales all lie in
    0x0001..0x27ff go through the one-FMA int4 dequantiser in "auto" and every value in that
    range is met by it."""
    if form == "exact_integer":
        request.getfixturevalue("exact_integer_form")
    allbits = np.arange(65536, dtype=np.uint16)
    finite = allbits[(allbits & 0x7C00) != 0x7C00]           # 63488 values
    n_out, g = 64, 64
    groups = finite.size // n_out                              # 992
    k = groups * g
    lo, hi = (-8, 7) if bits == 4 else (-128, 127)
    prob = Problem(f"allscales{bits}", n_out, k, bits, SCALE_AND_ZEROS, g)
    if bits == 4:   # every group of every row holds all 16 values
        q = np.tile(np.arange(lo, hi + 1, dtype=np.int8), n_out * k // 16)
        prob.q, prob.w_raw = q, orc.pack_int4(q)
    prob.scale = finite.reshape(groups, n_out).view(np.float16).copy()
    zero = orc.fill_uniform_f16(groups * n_out, 99, -0.05, 0.05).reshape(groups, n_out)
    zero[::7, ::3] = np.float16(0.0)
    zero[1::7, ::5] = np.float16(-0.0)
    zero[2::11, :] = orc.fill_uniform_f16(n_out, 98, -3e-5, 3e-5)   # subnormal additive terms
    prob.zero_add = zero
    dev = DeviceProblem(prob, gpu)
    got, want = dev.dequant().view(np.uint16), prob.oracle_dequant().view(np.uint16)
    nan = np.isnan(want.view(np.float16))
    assert np.array_equal(np.isnan(got.view(np.float16)), nan)     # inf - inf cases: NaN on both sides
    assert int((got[~nan] != want[~nan]).sum()) == 0


def test_one_hot_activation_is_bit_exact_through_the_gemv_kernel(gpu):
    """y[n] == dq[n, k] bit for bit: pins the dequantiser INSIDE the GEMV kernel (not only the
    debug entry) and the lane-to-k mapping of the DPP broadcast."""
    import torch
    for bits, k, scale_range in ((4, 1024, (1e-4, 0.02)), (4, 1024, (0.02, 0.3)), (8, 512, (1e-4, 0.02))):
        # int4: first range on the one-FMA dequantiser, second (scales beyond 2^-5) on the exact-integer one
        prob = Problem(f"onehot{bits}", 96, k, bits, SCALE_AND_ZEROS, 64, scale_range=scale_range)
        dev = DeviceProblem(prob, gpu)
        dq = prob.oracle_dequant().view(np.uint16)
        for kk in list(range(0, 40)) + [63, 64, 127, 128, 255, 256, 511, k - 33, k - 1]:
            x = np.zeros((1, k), dtype=np.float16)
            x[0, kk] = 1.0
            dev.x.copy_(torch.from_numpy(x.view(np.int16)))
            got = dev.run().view(np.uint16)[0]
            want = dq[:, kk]
            nz = (want & 0x7FFF) != 0
            assert np.array_equal(got[nz], want[nz]), (bits, kk)
            assert np.all((got[~nz] & 0x7FFF) == 0)


# (matrix-core variant, k-split waves, tiles per workgroup): the LDS-staged kernel with a stage per wave
# (one tile per workgroup) and with stages shared by 2, 4 and 8 tiles, and the register-operand kernel
MATRIX_CORE_LAUNCHES = [("lds_own_stages", "lds", 0, 1), ("lds_own_stages_split4", "lds", 4, 1), ("lds_shared_by_2", "lds", 2, 2),
                        ("lds_shared_by_4", "lds", 2, 4), ("lds_shared_by_8", "lds", 1, 8), ("register_operand", "reg", 0, 0),
                        ("k_stationary", "kstat", 0, 0)]


@pytest.mark.parametrize("launch", MATRIX_CORE_LAUNCHES, ids=[c[0] for c in MATRIX_CORE_LAUNCHES])
@pytest.mark.parametrize("bits", [4, 8])
def test_one_hot_rows_are_bit_exact_through_the_matrix_core_kernels(gpu, bits, launch):
    """Every activation row is a one-hot vector at a k of its own: y[b][n] == dq[n][k_b] bit for bit (up
    to the sign of a zero) through v_mfma_f32_16x16x32_f16 -- a product with 1 and sums with zeros are
    exact in the matrix core too.  Pins the dequantiser inside the matrix-core kernels and which
    lane's weights meet which activation (the LDS stage's layout, 8 and 16 staged rows, shared and
    own stages, the register operand's loads, the k-stationary kernel's operand turned round through
    LDS in one and two rounds), which a tolerance against the VALU kernel does not."""
    import torch
    _, variant, split, tw = launch
    k = 1536 if bits == 4 else 768
    rng = np.random.default_rng(bits * 100 + split * 10 + tw)
    for m_batch, scale_range in ((5, (1e-4, 0.02)), (8, (0.02, 0.3)), (16, (1e-4, 0.02)), (13, (0.02, 0.3))):
        if variant == "lds" and tw and (8 if m_batch <= 8 else 16) // tw < 2:
            continue    # that many tiles cannot share a stage of 8 rows
        prob = Problem(f"mc_onehot{bits}", 112, k, bits, SCALE_AND_ZEROS, 64, m_batch=m_batch, scale_range=scale_range)
        dev = DeviceProblem(prob, gpu)
        dq = prob.oracle_dequant().view(np.uint16)
        try:
            mg.set_matrix_core_threshold(1)
            mg.set_matrix_core_variant({"lds": mg.MATRIX_CORE_LDS_STAGED, "reg": mg.MATRIX_CORE_REGISTER_OPERAND,
                                        "kstat": mg.MATRIX_CORE_K_STATIONARY}[variant])
            mg.set_launch_override(split, tw, 0, 3 if variant == "kstat" else 0)   # k-stationary: walks of 2 and 3 tiles
            plan = mg.query_launch(prob.n_out, m_batch, k, bits)
            assert plan["matrix_core"] == {"lds": 2, "reg": 1, "kstat": 3}[variant], plan
            if variant == "lds" and tw:
                assert plan["tiles_per_wg"] == tw, plan
            for trial in range(6):
                # first trials: k positions that exercise every lane group, block and word of a unit
                hot = ([(b * 37 + trial * 131) % k for b in range(m_batch)] if trial < 4
                       else list(rng.integers(0, k, m_batch)))
                if trial == 0:
                    hot[:4] = [0, k - 1, 511 if bits == 4 else 255, 512 if bits == 4 else 256][:m_batch]
                x = np.zeros((m_batch, k), dtype=np.float16)
                x[np.arange(m_batch), hot] = 1.0
                dev.x.copy_(torch.from_numpy(x.view(np.int16)))
                got = dev.run().view(np.uint16)
                for b in range(m_batch):
                    want = dq[:, hot[b]]
                    nz = (want & 0x7FFF) != 0
                    assert np.array_equal(got[b][nz], want[nz]), (m_batch, trial, b, hot[b])
                    assert np.all((got[b][~nz] & 0x7FFF) == 0)
        finally:
            mg.set_matrix_core_threshold(0)
            mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
            mg.set_launch_override(0, 0, 0, 0)


def test_bias_only_and_output_fully_written(gpu):
    import torch
    prob = Problem("biasonly", 200, 640, 4, SCALE_AND_ZEROS, 128, m_batch=2, bias=True)
    dev = DeviceProblem(prob, gpu)
    dev.x.zero_()
    y = dev.run().view(np.uint16)
    assert np.array_equal(y[0], prob.bias.view(np.uint16)) and np.array_equal(y[1], prob.bias.view(np.uint16))


def test_split_k_invariance_and_determinism(gpu):
    prob = Problem("splitk", 192, 8192, 4, SCALE_AND_ZEROS, 128, bias=True, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    ref = prob.oracle_gemv(threads=16)
    results = {}
    try:
        # (k-split waves, tile sequences per workgroup, workgroup cap): with a cap below the 12
        # tiles every wave walks several tiles in a row
        for sk, tw, cap in ((1, 1, 0), (1, 4, 0), (2, 2, 0), (3, 1, 0), (4, 4, 0), (8, 2, 0), (16, 1, 0),
                            (1, 1, 5), (4, 1, 5), (4, 2, 2), (2, 1, 1), (16, 1, 8), (1, 1, 1)):
            mg.set_launch_override(sk, tw, 0, cap)
            a = dev.run().copy()
            b = dev.run().copy()
            assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), "same launch geometry must be bit-reproducible"
            _, rel, _ = error_report(a, ref)
            assert rel <= REL_TOL, (sk, tw, cap, rel)
            results[(sk, tw, cap)] = a
    finally:
        mg.set_launch_override(0, 0, 0, 0)
    # different arrangements of the tiles over workgroups and waves add in the same order
    for same in (((1, 1, 0), (1, 4, 0), (1, 1, 5), (1, 1, 1)), ((4, 4, 0), (4, 1, 5)), ((16, 1, 0), (16, 1, 8))):
        for other in same[1:]:
            assert np.array_equal(results[same[0]].view(np.uint16), results[other].view(np.uint16)), (same[0], other)


def test_tuned_plan_equals_the_same_override_bit_for_bit(gpu):
    from mixed_gemv_amd import autotune
    prob = Problem("tuned", 192, 4096, 4, SCALE_AND_ZEROS, 128, bias=True, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    autotune.clear()
    try:
        builtin = dev.run().copy()
        for sk, tw, cap in ((8, 2, 0), (2, 1, 3)):
            mg.set_launch_override(sk, tw, 0, cap)
            forced = dev.run().copy()
            mg.set_launch_override(0, 0, 0, 0)
            mg.set_tuned_plan(192, 4096, 4, 128, 1, kernel=mg.KERNEL_VALU, split_k=sk, tiles_per_wg=tw, max_workgroups=cap)
            tuned = dev.run().copy()
            assert np.array_equal(forced.view(np.uint16), tuned.view(np.uint16))
        autotune.clear()
        assert np.array_equal(builtin.view(np.uint16), dev.run().view(np.uint16))
    finally:
        autotune.clear()
        mg.set_launch_override(0, 0, 0, 0)


@pytest.mark.parametrize("m_batch", [1, 6])
def test_tuner_measures_installs_and_keeps_parity(gpu, m_batch):
    """The tuner on a small problem: every candidate it keeps is a distinct geometry, the overrides
    it sweeps are gone afterwards, and whatever it installed still meets the parity bar."""
    from mixed_gemv_amd import autotune
    prob = Problem("tuner", 1024, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=m_batch, bias=True)
    autotune.clear()
    try:
        cus = 256
        before = mg.query_launch(1024, m_batch, 2048, 4, 128, num_compute_units=cus)
        # an entry left by an earlier run (a poor one) must neither pass for the built-in plan nor survive
        mg.set_tuned_plan(1024, 2048, 4, 128, m_batch, kernel=mg.KERNEL_VALU, split_k=1, tiles_per_wg=1, max_workgroups=1)
        assert mg.query_launch(1024, m_batch, 2048, 4, 128, num_compute_units=cus) != before
        lines = []
        res = autotune.tune(1024, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=m_batch, bias=True, launches=64, rounds=1,
                            min_gain=0.0, cold_bytes=8 << 20, log=lines.append)
        print("\n".join(lines), flush=True)
        assert len(res["measurements"]) >= 4 and all(us > 0 for us, _ in res["measurements"])
        assert res["entry"] is None or res["entry"]["us"] < res["entry"]["builtin_us"]
        assert res["builtin_geometry"] == before
        after = mg.query_launch(1024, m_batch, 2048, 4, 128, num_compute_units=cus)
        if res["entry"] is None:
            assert after == before and mg.tuned_plan_count() == 0
        else:
            assert after == res["best_geometry"] and mg.tuned_plan_count() == 1 and res["entry"]["element"] == "f16"
        assert mg.query_launch(2048, m_batch, 2048, 4, 128) == mg.query_launch(2048, m_batch, 2048, 4, 0)
        check(prob, gpu, dequant=False)
    finally:
        autotune.clear()


def test_reconfirm_measures_an_entry_against_the_built_in_plan_and_leaves_no_override(gpu):
    from mixed_gemv_amd import autotune
    entry = dict(n_out=2048, k=4096, weight_bits=4, group_size=128, m_batch=1, element="f16", kernel=mg.KERNEL_VALU,
                 split_k=1, tiles_per_wg=1, max_workgroups=8)     # a poor plan: 8 workgroups walk everything
    before = mg.query_launch(2048, 1, 4096, 4, 128)
    gain = autotune.reconfirm(entry, launches=64, rounds=2, cold_bytes=8 << 20)
    assert entry["confirmations"] == [gain] and gain < -20.0, gain        # clearly behind the built-in plan
    assert not autotune.confirmed(entry)
    assert mg.query_launch(2048, 1, 4096, 4, 128) == before and mg.tuned_plan_count() == 0


@pytest.mark.parametrize("tag,n_out,k,bits,qop,g,m_batch,cap", [
    ("st_ns", 4096, 4096, 4, SCALE_AND_ZEROS, 128, 1, 0),        # four waves of two units
    ("st_walk", 1024, 8192, 4, SCALE_AND_ZEROS, 128, 1, 8),      # walks of eight tiles
    ("st_rows", 512, 6144, 4, SCALE_ONLY, 64, 3, 0),
    ("st_i8", 768, 4096, 8, PER_COLUMN, 0, 2, 5),
    ("st_bf16", 640, 5120, 4, SCALE_AND_ZEROS, 128, 1, 3),
])
def test_single_stage_loop_gives_the_same_bits(gpu, tag, n_out, k, bits, qop, g, m_batch, cap):
    """kStages = 1 against 2 (gemv/threadblock/default_dq_mma_simt.h:224-234, 394-404): the same
    arithmetic in the same order, only without a load in flight beside it."""
    prob = Problem(tag, n_out, k, bits, qop, g, m_batch=m_batch, bias=True, x_dist="normal",
                   element="bf16" if tag.endswith("bf16") else "f16")
    dev = DeviceProblem(prob, gpu)
    try:
        mg.set_launch_override(0, 0, 0, cap)
        mg.set_matrix_core_threshold(17)
        two = dev.run().copy()
        mg.set_prefetch_stages(1)
        assert mg.query_launch(n_out, m_batch, k, bits, g, element=prob.element, num_compute_units=256)["stages"] == 1
        one = dev.run().copy()
    finally:
        mg.set_prefetch_stages(0)
        mg.set_matrix_core_threshold(0)
        mg.set_launch_override(0, 0, 0, 0)
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))
    if prob.element == "f16":   # (the bf16 two-stage result is pinned to the oracle by the bf16 tests)
        _, rel, _ = error_report(one, prob.oracle_gemv(threads=8))
        assert rel <= REL_TOL


WALKS = [
    # tag, n_out, k, bits, quant_op, group, m_batch, bias
    ("w_i4_sz_g64", 208, 2048, 4, SCALE_AND_ZEROS, 64, 1, True),     # two groups per lane run
    ("w_i4_sz_g160", 100, 1120, 4, SCALE_AND_ZEROS, 160, 1, True),   # generic group lookup, ragged rows and k
    ("w_i4_col", 176, 1536, 4, PER_COLUMN, 0, 2, False),
    ("w_i4_s_g128_mb3", 144, 1024, 4, SCALE_ONLY, 128, 3, True),
    ("w_i8_sz_g128", 112, 768, 8, SCALE_AND_ZEROS, 128, 1, False),
    ("w_i8_col_mb4", 96, 512, 8, PER_COLUMN, 0, 4, True),
]


@pytest.mark.parametrize("cfg", WALKS, ids=[c[0] for c in WALKS])
def test_tile_walks_match_one_tile_per_wave(gpu, cfg):
    """Every kernel variant with waves that walk several tiles in a row (fewer workgroups than
    tiles): same bits as the one-tile-per-wave launch with the same k split, and parity with the oracle."""
    tag, n_out, k, bits, qop, g, mb, bias = cfg
    prob = Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias)
    dev = DeviceProblem(prob, gpu)
    ref = prob.oracle_gemv(threads=16)
    try:
        for sk in (1, 2):
            mg.set_launch_override(sk, 1, 0, 0)
            base = dev.run().copy()
            _, rel, _ = error_report(base, ref)
            assert rel <= REL_TOL, (sk, rel)
            for tw, cap in ((1, 3), (2, 2), (1, 1)):
                mg.set_launch_override(sk, tw, 0, cap)
                assert mg.query_launch(n_out, mb, k, bits)["tiles_in_sequence"] > 1
                got = dev.run().copy()
                assert np.array_equal(got.view(np.uint16), base.view(np.uint16)), (sk, tw, cap)
    finally:
        mg.set_launch_override(0, 0, 0, 0)


@pytest.mark.parametrize("m_batch", [4, 7, 11])
def test_each_activation_row_equals_the_single_row_result(gpu, m_batch):
    """Rows of a batch are independent GEMVs.  Up to 4 rows the VALU kernel adds every row in
    the single-row order (bit-identical); from 5 rows the matrix-core kernel takes over, whose
    fp32 sums are grouped differently (within tolerance, and reproducible run to run)."""
    prob = Problem("rows", 80, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=m_batch, bias=True)
    dev = DeviceProblem(prob, gpu)
    y_all = dev.run().copy()
    assert np.array_equal(y_all.view(np.uint16), dev.run().view(np.uint16))
    assert mg.query_launch(80, m_batch, 2048, 4)["matrix_core"] == (0 if m_batch < 5 else 2)   # LDS-staged from 2 tiles
    assert mg.query_launch(16, 7, 2048, 4)["matrix_core"] == 1    # a single tile: register operand
    assert mg.query_launch(8192, 7, 2048, 4)["matrix_core"] == 3    # two tiles per compute unit: k-stationary
    assert mg.query_launch(4096, 7, 2048, 4)["matrix_core"] == 2
    single = Problem("rows", 80, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=1, bias=True)
    for b in range(m_batch):
        single.x = prob.x[b:b + 1].copy()
        y1 = DeviceProblem(single, gpu).run()
        if m_batch <= 4:
            assert np.array_equal(y1.view(np.uint16)[0], y_all.view(np.uint16)[b]), b
        else:
            _, rel, _ = error_report(y_all[b], y1[0])
            assert rel <= REL_TOL, (b, rel)


@pytest.mark.parametrize("bits,qop,g", [(4, SCALE_AND_ZEROS, 128), (4, SCALE_ONLY, 64), (4, PER_COLUMN, 0),
                                        (8, SCALE_AND_ZEROS, 64), (8, PER_COLUMN, 0), (4, SCALE_AND_ZEROS, 160)])
def test_matrix_core_and_valu_kernels_agree(gpu, bits, qop, g):
    """The same batches through the three matrix-core kernels (LDS-staged at several k splits, register
    operand, k-stationary) and the VALU kernel (threshold forced), ragged shape, every mode."""
    n_out, k = 100, 1120 if g in (0, 160) else 1024
    for m_batch in (1, 5, 8, 13, 16):
        prob = Problem(f"mc{bits}{qop}", n_out, k, bits, qop, g, m_batch=m_batch, bias=True)
        dev = DeviceProblem(prob, gpu)
        ref = prob.oracle_gemv(threads=8)
        results = []
        try:
            mg.set_matrix_core_threshold(1)
            # (variant, k-split waves, tiles per workgroup): 1-8 tiles share an activation stage of 8 or 16
            # rows; 7 tiles do not divide by 2, 4 or 8, so some waves of the last workgroup have no tile
            for variant, split, tw in ((mg.MATRIX_CORE_LDS_STAGED, 0, 0), (mg.MATRIX_CORE_LDS_STAGED, 1, 2),
                                       (mg.MATRIX_CORE_LDS_STAGED, 2, 2), (mg.MATRIX_CORE_LDS_STAGED, 4, 1),
                                       (mg.MATRIX_CORE_LDS_STAGED, 2, 4), (mg.MATRIX_CORE_LDS_STAGED, 1, 8),
                                       (mg.MATRIX_CORE_REGISTER_OPERAND, 0, 0), (mg.MATRIX_CORE_K_STATIONARY, 0, 0)):
                mg.set_matrix_core_variant(variant)
                mg.set_launch_override(split, tw, 0, 0)
                plan = mg.query_launch(n_out, m_batch, k, bits)
                assert plan["matrix_core"] == {mg.MATRIX_CORE_LDS_STAGED: 2, mg.MATRIX_CORE_REGISTER_OPERAND: 1,
                                               mg.MATRIX_CORE_K_STATIONARY: 3}[variant]
                if variant == mg.MATRIX_CORE_LDS_STAGED and tw and (8 if m_batch <= 8 else 16) // tw >= 2:
                    assert plan["tiles_per_wg"] == tw, plan
                results.append(dev.run().copy())
                assert np.array_equal(results[-1].view(np.uint16), dev.run().view(np.uint16))   # reproducible
            mg.set_matrix_core_threshold(17)
            results.append(dev.run().copy())   # VALU kernel
        finally:
            mg.set_matrix_core_threshold(0)
            mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
            mg.set_launch_override(0, 0, 0, 0)
        for y in results:
            _, rel, _ = error_report(y, ref)
            assert rel <= REL_TOL, (m_batch, rel)


def test_batched_launch_with_strides(gpu):
    """batch_count problems in one launch (gemv/device/gemv_adaptor.h:129-135): expert-stacked
    weights and scales, shared activations, per-problem outputs."""
    import torch
    e, n_out, k, g = 3, 64, 1024, 128
    probs = [Problem(f"batch{i}", n_out, k, 4, SCALE_AND_ZEROS, g, bias=True) for i in range(e)]
    raw = np.concatenate([p.w_raw for p in probs])
    pre = mg.MixedGemvWeightPreprocessor.run(raw, (e, k, n_out), mg.LayoutType.kColumnMajor, mg.QuantType.W4_A16)
    one = mg.preprocessed_size((k, n_out), mg.QuantType.W4_A16)

    def stack(name):
        return torch.from_numpy(np.stack([getattr(p, name) for p in probs]).view(np.int16)).to(gpu)

    w = torch.from_numpy(pre).to(gpu)
    scale, zero, bias = stack("scale"), stack("zero_add"), stack("bias")
    x = torch.from_numpy(probs[0].x.view(np.int16)).to(gpu)
    y = torch.full((e, n_out), 0x7E00, dtype=torch.int16, device=gpu)
    groups = k // g
    results = []
    try:
        # default geometry, then one workgroup per problem (every wave walks all four tiles in a row)
        for cap in (0, 1):
            mg.set_launch_override(0, 0, 0, cap)
            y.fill_(0x7E00)
            mg.device_gemv(w, x, scale, zero, bias, y, e, n_out, 1, k, g, SCALE_AND_ZEROS, 4,
                           batch_strides=(one, 0, groups * n_out, n_out, n_out))
            torch.cuda.synchronize()
            results.append(y.cpu().numpy().view(np.float16).copy())
    finally:
        mg.set_launch_override(0, 0, 0, 0)
    assert mg.query_launch(n_out, 1, k, 4)["tiles_in_sequence"] == 1
    for got in results:
        for i, p in enumerate(probs):
            p.x = probs[0].x
            _, rel, _ = error_report(got[i], p.oracle_gemv(threads=8)[0])
            assert rel <= REL_TOL, i
    assert np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))   # same k split, same sums


def test_adaptor_mirror_runs(gpu):
    import torch
    prob = Problem("adaptor", 128, 1024, 4, SCALE_ONLY, 128, bias=True)
    dev = DeviceProblem(prob, gpu)
    op = mg.GemvAdaptor(mg.WeightOnlyQuantOp.FINEGRAINED_SCALE_ONLY, 4)
    # ref_zero_point is ignored outside the scale+zero mode (mixed_gemv_test.cu:145-147)
    op(mg.GemvAdaptor.Arguments((128, 1, 1024), dev.w, dev.x, dev.scale, dev.scale, dev.bias, dev.y, group_size=128))
    torch.cuda.synchronize()
    _, rel, _ = error_report(dev.y.cpu().numpy().view(np.float16), prob.oracle_gemv())
    assert rel <= REL_TOL


FULL = [
    # the benchmark configurations at their real sizes
    ("c1_int8_percol", 4096, 4096, 8, PER_COLUMN, 0, 1, True, "uniform", (0.001, 0.01)),
    ("c2_int4_g128_scale", 4096, 4096, 4, SCALE_ONLY, 128, 1, True, "uniform", (0.001, 0.02)),
    ("ns_int4_g128_sz", 4096, 4096, 4, SCALE_AND_ZEROS, 128, 1, False, "uniform", (0.001, 0.02)),
    ("c3a_mlp_up", 11008, 4096, 4, SCALE_AND_ZEROS, 128, 1, False, "normal", (0.001, 0.02)),
    ("c3b_mlp_down", 4096, 11008, 4, SCALE_AND_ZEROS, 128, 1, False, "normal", (0.001, 0.02)),
    ("c4_m1", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 1, True, "uniform", (0.001, 0.02)),
    ("c4_m2", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 2, True, "uniform", (0.001, 0.02)),
    ("c4_m4", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 4, True, "uniform", (0.001, 0.02)),
    ("c4_m8", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 8, True, "uniform", (0.001, 0.02)),
    ("c4_m16", 8192, 8192, 4, SCALE_AND_ZEROS, 64, 16, True, "uniform", (0.001, 0.02)),
    ("c5_70b_up", 28672, 8192, 4, SCALE_AND_ZEROS, 128, 1, False, "normal", (0.001, 0.02)),
]


# Shapes that take the other branches of the launch heuristic (one four-wave workgroup per compute
# unit with 4 / 2 / 1 tile sequences, with and without several tiles per sequence, with remainders).
FIT = [
    ("fit_tw4_two_tiles_each", 32032, 4096, 4, SCALE_AND_ZEROS, 128, 1, False, "normal", (0.001, 0.02)),
    ("fit_tw2_long_k", 8192, 28672, 4, SCALE_AND_ZEROS, 128, 1, True, "normal", (0.001, 0.02)),
    ("fit_tw1_seven_tiles", 28672, 6144, 4, SCALE_AND_ZEROS, 128, 1, False, "normal", (0.001, 0.02)),
    ("fit_int8_tw2", 8192, 4096, 8, PER_COLUMN, 0, 2, True, "uniform", (0.001, 0.01)),
]


@pytest.mark.parametrize("cfg", FIT, ids=[c[0] for c in FIT])
def test_exact_fit_launches_full_size(gpu, cfg):
    tag, n_out, k, bits, qop, g, mb, bias, xd, sr = cfg
    plan = mg.query_launch(n_out, mb, k, bits)
    assert plan["workgroups"] == 256 and plan["threads"] == 256, plan
    prob = Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias, x_dist=xd, scale_range=sr)
    check(prob, gpu, dequant=False)


def test_vocabulary_projection_one_tile_per_workgroup(gpu):
    """128256 x 4096 (8016 tiles): an exact fit would mean walks of 8 tiles, which measured slower than one
    tile per workgroup, so this shape launches one single-wave workgroup per tile."""
    plan = mg.query_launch(128256, 1, 4096, 4)
    assert plan["tiles_in_sequence"] == 1 and plan["workgroups"] == 8016, plan
    prob = Problem("vocab", 128256, 4096, 4, SCALE_AND_ZEROS, 128, x_dist="normal")
    check(prob, gpu, dequant=False)


# Shapes on which the remaining launch rules were measured, each with the plan field that shows the
# rule took effect: whole-k single-wave workgroups, one-unit waves at 5-8 k steps (in and over the
# usual wave count), paired tiles, the four-wave limit of long reductions, matrix cores from 3 rows, the tile count per activation stage and the balanced
# k split of the LDS-staged kernel.
RULES = [
    ("whole_k_m1", 13824, 5120, 1, dict(matrix_core=0, threads=64, split_k=1, steps_per_wave=10)),
    ("whole_k_m2", 13824, 8704, 2, dict(matrix_core=0, threads=64, split_k=1)),   # (17 k steps: out of the k-stationary kernel's reach)
    ("one_unit_waves_m2", 6144, 4096, 2, dict(matrix_core=0, split_k=8, steps_per_wave=1)),
    ("one_unit_waves_11008_waves", 22016, 4096, 1, dict(matrix_core=0, split_k=8, workgroups=1376)),
    ("paired_tiles", 5120, 5120, 1, dict(matrix_core=0, tiles_per_wg=2, split_k=2, workgroups=160)),
    ("paired_tiles_m2_long_k", 7168, 14336, 2, dict(matrix_core=0, tiles_per_wg=2, split_k=2, steps_per_wave=14)),
    ("four_waves_from_16_k_steps", 9216, 8192, 1, dict(matrix_core=0, tiles_per_wg=1, split_k=4, steps_per_wave=4)),
    ("matrix_cores_at_3_rows", 5120, 4096, 3, dict(matrix_core=2, variant="lds_staged")),
    ("two_tiles_even_split", 5120, 5120, 8, dict(matrix_core=2, tiles_per_wg=2, split_k=2, steps_per_wave=5, variant="lds_staged")),
    ("two_tiles_592_workgroups", 18944, 3584, 8, dict(matrix_core=2, tiles_per_wg=2, workgroups=592, variant="lds_staged")),
    ("k_stationary_walks_of_5", 18944, 3584, 8, dict(matrix_core=3, workgroups=256, split_k=7, tiles_in_sequence=5)),
    ("k_stationary_walks_of_3_16_waves", 12288, 8192, 3, dict(matrix_core=3, workgroups=256, split_k=16, tiles_in_sequence=3)),
    ("k_stationary_two_rows", 22016, 4096, 2, dict(matrix_core=3, workgroups=256, split_k=8, tiles_in_sequence=6)),
    ("four_tiles_160_workgroups", 10240, 8192, 8, dict(matrix_core=2, tiles_per_wg=4, workgroups=160, variant="lds_staged")),
    ("k_stationary_better_filled", 10240, 8192, 8, dict(matrix_core=3, workgroups=256, tiles_in_sequence=3)),
    ("k_stationary_walks_of_2", 5120, 4096, 3, dict(matrix_core=3, workgroups=256, tiles_in_sequence=2)),
    # long reductions on many tiles (17 k steps, 1025 / 1792 tiles): about two workgroups per compute unit
    ("long_k_two_tiles_split_in_two", 16400, 8704, 5, dict(matrix_core=2, tiles_per_wg=2, split_k=2, workgroups=520)),
    ("long_k_two_tiles_whole_k", 16400, 8704, 12, dict(matrix_core=2, tiles_per_wg=2, split_k=1, workgroups=520)),
    ("long_k_four_tiles_of_two_rows_each", 28672, 8704, 3, dict(matrix_core=2, tiles_per_wg=4, split_k=1, workgroups=448)),
    ("two_rows_on_uneven_walks", 21024, 7808, 2, dict(matrix_core=3, workgroups=256, tiles_in_sequence=6)),
]


@pytest.mark.parametrize("cfg", RULES, ids=[c[0] for c in RULES])
def test_launch_rule_shapes_full_size(gpu, cfg):
    tag, n_out, k, mb, want = cfg
    want = dict(want)
    # variant: the rule of the LDS-staged kernel on a shape that the k-stationary kernel now takes
    mg.set_matrix_core_variant(mg.MATRIX_CORE_LDS_STAGED if want.pop("variant", None) else mg.MATRIX_CORE_AUTO)
    try:
        plan = mg.query_launch(n_out, mb, k, 4, 128)
        assert {key: plan[key] for key in want} == want, plan
        prob = Problem(tag, n_out, k, 4, SCALE_AND_ZEROS, 128, m_batch=mb, bias=(mb % 2 == 0), x_dist="normal")
        check(prob, gpu, dequant=False)
    finally:
        mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)


@pytest.mark.parametrize("cfg", FULL, ids=[c[0] for c in FULL])
def test_baseline_configs_full_size(gpu, cfg):
    tag, n_out, k, bits, qop, g, mb, bias, xd, sr = cfg
    prob = Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias, x_dist=xd, scale_range=sr)
    # dequantised weights of the whole matrix, bit for bit (skipped for the M > 1 repeats of the same matrix)
    check(prob, gpu, dequant=(mb == 1))


def test_hip_graph_replays_match_eager_launches(gpu):
    """The entry points neither allocate nor synchronise, so a caller may capture them; every replay of
    a graph holding a VALU launch, the three matrix-core launches and a bf16 launch must reproduce the eager
    results bit for bit, with eager work and synchronisations between the replays."""
    import torch
    probs = [Problem("g_valu", 320, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=2, bias=True),
             Problem("g_reg", 16, 2048, 4, SCALE_AND_ZEROS, 64, m_batch=6, bias=True),       # one tile: register-operand matrix core
             Problem("g_lds", 320, 2048, 8, PER_COLUMN, 0, m_batch=16, bias=False),          # LDS-staged, 16 rows staged
             Problem("g_kstat", 8192, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=3, bias=True),   # walks of 2 tiles: k-stationary
             Problem("g_bf16", 320, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=1, bias=True, element="bf16")]
    devs = [DeviceProblem(p, gpu) for p in probs]
    assert [mg.query_launch(p.n_out, p.m_batch, 2048, p.bits)["matrix_core"] for p in probs[:4]] == [0, 1, 2, 3]
    eager = [d.run().copy() for d in devs]

    def launch_all():
        for d in devs:
            p = d.p
            mg.device_gemv(d.w, d.x, d.scale, d.zero, d.bias, d.y, 1, p.n_out, p.m_batch, p.k, p.group_size,
                           p.quant_op, p.bits, element=p.element)

    launch_all()   # anything lazy (function attributes for large LDS) happens before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launch_all()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(4):
        for d in devs:
            d.y.fill_(0x7e00)                     # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for d, want in zip(devs, eager):
            got = d.y.cpu().numpy().view(want.dtype)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (replay, d.p.tag)


def test_reference_shipped_shape(gpu):
    """The problem the reference's main() ships with (mixed_gemv_test.cu:187-191) at full size:
    out = 151936, K = 2048, int4 g128 scale+zero, its own scale range and int8 zero points."""
    prob = Problem("ref_main", 151936, 2048, 4, SCALE_AND_ZEROS, 128, scale_range=(0.1, 0.3), zero_kind="int8")
    dev, y = check(prob, gpu, dequant=False)
    ref = prob.oracle_gemv(threads=16)
    abs_err = np.abs(y.astype(np.float64) - ref.astype(np.float64))
    # The reference prints rows whose abs error exceeds 1e-3 (mixed_gemv_test.cu:296-300).  With its
    # own scale range the outputs are O(10..100), where one fp16 ulp is already 0.008-0.06, so that
    # threshold is restated in units of the output's ulp (taken at the error metric's floor for
    # outputs that cancel to almost zero).
    _, _, floor = error_report(y, ref)
    ulp = np.spacing(np.maximum(np.abs(ref), floor).astype(np.float16)).astype(np.float64)
    assert np.all(abs_err <= 2 * ulp)
    bad, worst = float64_bound_violations(prob, y, rows_per_chunk=8192)
    assert bad == 0, (bad, worst)


# tag, n_out, k, group, activation rows run (each on the first rows of one set of activations), bias, x
BOUND_CASES = [
    ("c5", 28672, 8192, 128, (1,), False, "normal"),
    ("c4", 8192, 8192, 64, (1, 2, 4, 8, 16), True, "uniform"),
    ("vocab", 128256, 4096, 128, (1,), False, "normal"),
]


@pytest.mark.parametrize("cfg", BOUND_CASES, ids=[c[0] for c in BOUND_CASES])
def test_full_size_outputs_within_the_float64_bound(gpu, cfg):
    """At BASELINE's full sizes, every output of the kernel -- VALU at 1-2 rows, matrix cores from 4 --
    lies within the fp32-accumulation bound around the exactly accumulated sum of the dequantised
    weights (helpers.float64_bound_violations): the property the oracle's own HOST_CHECK loop is held
    to (test_oracle_gemv.py), which needs no denominator floor."""
    tag, n_out, k, g, rows, bias, xd = cfg
    prob = Problem(tag + "_bound", n_out, k, 4, SCALE_AND_ZEROS, g, m_batch=max(rows), bias=bias, x_dist=xd)
    dev = DeviceProblem(prob, gpu)
    full_x, full_rows = prob.x, prob.m_batch
    dq = prob.oracle_dequant()
    for m in rows:
        prob.m_batch, prob.x = m, full_x[:m]
        dev.y.fill_(0x7e00)
        mg.device_gemv(dev.w, dev.x, dev.scale, dev.zero, dev.bias, dev.y, 1, n_out, m, k, g, SCALE_AND_ZEROS, 4)
        import torch
        torch.cuda.synchronize()
        y = dev.y.cpu().numpy().view(np.float16)[:m]
        bad, worst = float64_bound_violations(prob, y, dq=dq)
        # ... and the kernel is as close to the exact sum as the reference's own ascending-k loop is
        host_check_bad, host_check_worst = float64_bound_violations(prob, prob.oracle_gemv(threads=16), dq=dq)
        print(f"{tag} M={m}: largest error / bound = {worst:.3f} (HOST_CHECK loop: {host_check_worst:.3f})", flush=True)
        assert bad == 0 and host_check_bad == 0, (m, bad, worst)
        assert worst <= 1.25 * host_check_worst, (m, worst, host_check_worst)
    prob.m_batch, prob.x = full_rows, full_x
