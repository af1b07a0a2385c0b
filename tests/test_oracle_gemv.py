"""Pins the oracle's dequantiser and HOST_CHECK GEMV (host/mixed_gemv.h:82-104) against an
independent numpy restatement, closed forms and special cases chosen so that a dropped term,
a wrong group index, a transposed scale table or a fused rounding each fail a test."""
import numpy as np
import pytest

import np_restate
import oracle as orc
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, Problem

FINITE = np.arange(65536, dtype=np.uint16)
FINITE = FINITE[(FINITE & 0x7C00) != 0x7C00]


def _q_matrix(prob):
    return prob.q.reshape(prob.n_out, prob.k).astype(np.int32)


CASES = [
    ("o_i4_sz", 24, 256, 4, SCALE_AND_ZEROS, 64, 1, True, "int8"),
    ("o_i4_sz_f16", 16, 384, 4, SCALE_AND_ZEROS, 128, 2, False, "f16"),
    ("o_i4_s", 12, 256, 4, SCALE_ONLY, 128, 1, True, "f16"),
    ("o_i4_col", 8, 192, 4, PER_COLUMN, 0, 3, False, "f16"),
    ("o_i8_col", 16, 128, 8, PER_COLUMN, 0, 1, True, "f16"),
    ("o_i8_sz", 8, 256, 8, SCALE_AND_ZEROS, 64, 2, True, "int8"),
]


@pytest.mark.parametrize("cfg", CASES, ids=[c[0] for c in CASES])
def test_dequant_and_gemv_match_numpy_restatement(cfg):
    tag, n, k, bits, qop, g, mb, bias, zk = cfg
    prob = Problem(tag, n, k, bits, qop, g, m_batch=mb, bias=bias, zero_kind=zk)
    q = _q_matrix(prob)
    for literal in ([False, True] if zk == "int8" else [False]):
        zero = None
        if qop == SCALE_AND_ZEROS:
            zero = prob.zeros_i8 if literal else prob.zero_add
        ref_dq = np_restate.dequantize(q, prob.scale, zero, prob.group_size, int8_zero=literal)
        got_dq = orc.dequantize(prob.w_raw, prob.scale, zero, n, k, prob.group_size, qop, bits)
        assert np.array_equal(got_dq.view(np.uint16), ref_dq.view(np.uint16))
        ref_y = np_restate.gemv(ref_dq, prob.x, prob.bias)
        got_y = orc.gemv(prob.w_raw, prob.x, prob.scale, zero, prob.bias, n, mb, k, prob.group_size, qop, bits)
        assert np.array_equal(got_y.view(np.uint16), ref_y.view(np.uint16))


def test_int8_zero_and_folded_zero_conventions_agree():
    """host/mixed_gemv.h takes int8 zeros, the device the folded -z*s; same values except -0/+0."""
    prob = Problem("o_conv", 32, 256, 4, SCALE_AND_ZEROS, 64, zero_kind="int8")
    a = orc.dequantize(prob.w_raw, prob.scale, prob.zeros_i8, 32, 256, 64, SCALE_AND_ZEROS, 4).view(np.uint16)
    b = orc.dequantize(prob.w_raw, prob.scale, prob.zero_add, 32, 256, 64, SCALE_AND_ZEROS, 4).view(np.uint16)
    diff = a != b
    assert np.all((a[diff] & 0x7FFF) == 0) and np.all((b[diff] & 0x7FFF) == 0)


def test_dequant_exhaustive_q_times_all_scales():
    # one row per q value, one "group" per scale: every (q, s) product once, no zero
    for bits, qs in ((4, np.arange(-8, 8)), (8, np.array([-128, -127, -77, -3, -1, 0, 1, 2, 5, 100, 127]))):
        chunk = 2048
        for start in range(0, FINITE.size, chunk):
            s = FINITE[start:start + chunk]
            groups, n = s.size, qs.size
            k = groups * 64
            q = np.repeat(qs[:, None], k, axis=1).astype(np.int8)
            w = orc.pack_int4(q.reshape(-1)) if bits == 4 else q.reshape(-1).view(np.uint8)
            scale = np.repeat(s[:, None], n, axis=1)
            got = orc.dequantize(w, scale, None, n, k, 64, SCALE_ONLY, bits).view(np.uint16)
            with np.errstate(over="ignore"):
                ref = (qs[:, None].astype(np.float16) * s.view(np.float16)[None, :]).astype(np.float16).view(np.uint16)
            assert np.array_equal(got[:, ::64], ref)


def test_group_index_and_scale_table_orientation():
    """scale[g*n_out + n] with g = k / group_size: scales that identify (g, n) make any slip gross."""
    n, k, g = 8, 512, 128
    q = np.ones((n, k), dtype=np.int8)
    groups = k // g
    scale = (np.arange(groups)[:, None] * 16 + np.arange(n)[None, :] + 1).astype(np.float16)  # distinct integers
    dq = orc.dequantize(orc.pack_int4(q.reshape(-1)), scale, None, n, k, g, SCALE_ONLY, 4).astype(np.float32)
    for row in range(n):
        for kk in (0, g - 1, g, 2 * g + 5, k - 1):
            assert dq[row, kk] == scale[kk // g, row]
    # per-column mode ignores group_size and uses one scale per output row (mixed_gemv_test.cu:142-143)
    dq = orc.dequantize(orc.pack_int4(q.reshape(-1)), scale[:1], None, n, k, 64, PER_COLUMN, 4).astype(np.float32)
    assert np.array_equal(dq, np.repeat(scale[0].astype(np.float32)[:, None], k, axis=1))


def test_one_hot_activation_returns_dequantised_column_bit_exactly():
    prob = Problem("o_onehot", 32, 256, 4, SCALE_AND_ZEROS, 64)
    dq = prob.oracle_dequant()
    for kk in (0, 63, 64, 200, 255):
        x = np.zeros((1, 256), dtype=np.float16)
        x[0, kk] = 1.0
        y = orc.gemv(prob.w_raw, x, prob.scale, prob.zero_add, None, 32, 1, 256, 64, SCALE_AND_ZEROS, 4)
        got, want = y.view(np.uint16)[0], dq.view(np.uint16)[:, kk]
        nz = (want & 0x7FFF) != 0  # a zero column entry comes back as +0 from the fp32 sum
        assert np.array_equal(got[nz], want[nz])
        assert np.all((got[~nz] & 0x7FFF) == 0)


def test_unit_weights_sum_the_activations_in_ascending_order():
    n, k = 4, 1024
    q = np.ones((n, k), dtype=np.int8)
    scale = np.ones((k // 128, n), dtype=np.float16)
    x = orc.fill_uniform_f16(k, 77, -1.0, 1.0).reshape(1, k)
    y = orc.gemv(orc.pack_int4(q.reshape(-1)), x, scale, None, None, n, 1, k, 128, SCALE_ONLY, 4)
    acc = np.float32(0)
    for v in x[0].astype(np.float32):
        acc = np.float32(acc + v)
    assert np.all(y.view(np.uint16) == np.float16(acc).view(np.uint16))
    # and the mathematically exact sum is close
    assert abs(float(acc) - float(np.sum(x.astype(np.float64)))) < 1e-3


def test_bias_only_and_bias_rounding():
    n, k = 16, 128
    prob = Problem("o_bias", n, k, 4, SCALE_ONLY, 128, bias=True)
    x = np.zeros((1, k), dtype=np.float16)
    y = orc.gemv(prob.w_raw, x, prob.scale, None, prob.bias, n, 1, k, 128, SCALE_ONLY, 4)
    assert np.array_equal(y.view(np.uint16)[0], prob.bias.view(np.uint16))
    # acc + bias is ONE fp32 add then ONE rounding: acc = 2048; +1 -> tie 2049 -> 2048 (even); +3 -> tie 2051 -> 2052;
    # -1 -> 2047 exact; +0.5 -> 2048
    q = np.ones((4, 128), dtype=np.int8)
    scale = np.full((1, 4), 16.0, dtype=np.float16)
    x = np.ones((1, 128), dtype=np.float16)
    bias = np.array([1.0, 3.0, -1.0, 0.5], dtype=np.float16)
    y = orc.gemv(orc.pack_int4(q.reshape(-1)), x, scale, None, bias, 4, 1, 128, 128, SCALE_ONLY, 4).astype(np.float32)
    assert np.array_equal(y[0], np.array([2048.0, 2052.0, 2047.0, 2048.0], dtype=np.float32))


def test_float64_bound_and_batch_rows_and_threads():
    prob = Problem("o_big", 64, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=3, bias=True, x_dist="normal")
    y1 = prob.oracle_gemv(threads=1)
    y8 = prob.oracle_gemv(threads=8)
    assert np.array_equal(y1.view(np.uint16), y8.view(np.uint16))
    dq = prob.oracle_dequant().astype(np.float64)
    exact = prob.x.astype(np.float64) @ dq.T + prob.bias.astype(np.float64)[None, :]
    # fp32 accumulation of 2048 terms plus one fp16 rounding
    mag = np.abs(prob.x.astype(np.float64)) @ np.abs(dq.T)
    bound = mag * 2048 * 2.0 ** -24 + np.abs(exact) * 2.0 ** -11 + 2.0 ** -24
    assert np.all(np.abs(y1.astype(np.float64) - exact) <= bound)
    # each activation row is an independent GEMV
    for b in range(3):
        yb = orc.gemv(prob.w_raw, prob.x[b:b + 1], prob.scale, prob.zero_add, prob.bias, 64, 1, 2048, 128,
                      SCALE_AND_ZEROS, 4)
        assert np.array_equal(yb.view(np.uint16)[0], y1.view(np.uint16)[b])


def test_generator_is_deterministic_and_in_range():
    a = orc.fill_int8(100000, 42, -8, 7)
    assert np.array_equal(a, orc.fill_int8(100000, 42, -8, 7))
    assert not np.array_equal(a, orc.fill_int8(100000, 43, -8, 7))
    assert a.min() == -8 and a.max() == 7
    counts = np.bincount(a.astype(np.int32) + 8, minlength=16)
    assert counts.min() > 100000 / 16 * 0.9
    # a prefix of a longer stream is the shorter stream (counter-based)
    assert np.array_equal(orc.fill_int8(1000, 42, -8, 7), a[:1000])
    u = orc.fill_uniform_f16(100000, 7, 0.001, 0.02).astype(np.float64)
    assert u.min() >= 0.001 - 1e-6 and u.max() <= 0.02 + 1e-5
    g = orc.fill_normal_clipped_f16(200000, 9, 4.0).astype(np.float64)
    assert abs(g.mean()) < 0.02 and abs(g.std() - 1.0) < 0.02 and np.abs(g).max() <= 4.0
