"""Pins the oracle's bfloat16 arithmetic and its bf16 dequantiser / GEMV.

The reference holds no bf16 vector or test (its bf16 instantiation is rejected at compile time,
gemv/threadblock/default_dq_mma_simt.h:133-134), so these functions are pinned by what the
mathematics fixes: conversions against torch.bfloat16 (different code: torch's c10::BFloat16)
and against exact rational arithmetic, the element operations against exact rational
arithmetic, the matrix functions against a torch.bfloat16 restatement and closed forms."""
from fractions import Fraction

import numpy as np
import pytest
import torch

import mixed_gemv_amd as mg
import oracle as orc
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, Problem
from torch_restate import as_torch_bf16, sequential_gemv, torch_bits, torch_dequantize

ALL = np.arange(65536, dtype=np.uint16)
FINITE = ALL[(ALL & 0x7F80) != 0x7F80]


def exact(bits):
    """Exact value of a finite bf16 bit pattern."""
    b = int(bits)
    sign = -1 if b & 0x8000 else 1
    e, m = (b >> 7) & 0xFF, b & 0x7F
    if e == 0:
        return sign * Fraction(m, 1 << 7) * Fraction(2) ** -126
    return sign * (1 + Fraction(m, 1 << 7)) * Fraction(2) ** (e - 127)


def round_exact(v):
    """Correctly rounded (nearest, ties to even) bf16 bit pattern of a rational, by search over
    the ordered finite patterns -- shares nothing with the oracle's bit manipulation."""
    if v == 0:
        return None  # sign of zero is the operation's business; callers skip it
    sign = 0x8000 if v < 0 else 0
    a = abs(v)
    lo, hi = 0, 0x7F7F  # magnitudes are ordered like their bit patterns
    while lo < hi:
        mid = (lo + hi + 1) // 2
        if exact(mid) <= a:
            lo = mid
        else:
            hi = mid - 1
    if lo == 0x7F7F:
        top = exact(0x7F7F)
        half_step = Fraction(2) ** (127 - 8)
        return sign | (0x7F80 if a >= top + half_step else 0x7F7F)
    down, up = exact(lo), exact(lo + 1)
    if a - down < up - a:
        return sign | lo
    if a - down > up - a:
        return sign | (lo + 1)
    return sign | (lo if lo % 2 == 0 else lo + 1)


def test_conversions_every_pattern_and_random_floats():
    f = orc.bf16_to_f32_array(ALL)
    assert np.array_equal(f.view(np.uint32), ALL.astype(np.uint32) << 16)
    assert np.array_equal(orc.f32_to_bf16_array(f[FINITE]), FINITE)      # exact values survive
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 1 << 32, 4_000_000, dtype=np.uint64).astype(np.uint32)
    bits = bits[(bits & 0x7F800000) != 0x7F800000]                        # finite
    vals = bits.view(np.float32)
    assert np.array_equal(orc.f32_to_bf16_array(vals), torch_bits(vals))
    # every tie (low half exactly 0x8000) over a sweep of upper halves, and the overflow boundary
    ties = ((FINITE.astype(np.uint32) << 16) | 0x8000).view(np.float32)
    got = orc.f32_to_bf16_array(ties)
    want = FINITE + (FINITE & 1)                                          # to even; 0x7f7f + tie -> inf
    assert np.array_equal(got, want.astype(np.uint16))
    assert np.array_equal(got, torch_bits(ties))
    edge = np.array([3.3895314e38, 3.3961775e38, 3.4028235e38, 1e-45, 4.6e-41, 9.1e-41, 9.2e-41], dtype=np.float32)
    assert np.array_equal(orc.f32_to_bf16_array(edge), torch_bits(edge))
    for v in edge.tolist() + vals[:3000].tolist():
        r = round_exact(Fraction(v))
        if r is not None:
            assert int(orc.f32_to_bf16_array(np.array([v], dtype=np.float32))[0]) == r, v


def test_mul_and_add_are_correctly_rounded():
    rng = np.random.default_rng(11)
    a = rng.choice(FINITE, 6000)
    b = rng.choice(FINITE, 6000)
    # exponents near each other, so that sums cancel and carry
    near = (a & 0x807F) | (np.clip(((b >> 7) & 0xFF).astype(np.int32) + rng.integers(-9, 10, 6000), 0, 254) << 7).astype(np.uint16)
    small = rng.choice(FINITE[((FINITE >> 7) & 0xFF) < 12], 2000)          # subnormal results
    pairs = [(a, b), (near, b), (np.concatenate([small, small]), rng.choice(FINITE, 4000))]
    for x, y in pairs:
        mul = orc.bf16_mul_array(x, y)
        add = orc.bf16_add_array(x, y)
        for i in range(0, x.size, 3):
            ex, ey = exact(x[i]), exact(y[i])
            for got, v in ((mul[i], ex * ey), (add[i], ex + ey)):
                want = round_exact(v)
                if want is not None:
                    assert int(got) == want, (hex(int(x[i])), hex(int(y[i])), hex(int(got)), hex(want))
    # torch computes the same operations in its own code
    ta, tb = as_torch_bf16(a), as_torch_bf16(b)
    assert np.array_equal(orc.bf16_mul_array(a, b), (ta * tb).view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(orc.bf16_add_array(near, b), (as_torch_bf16(near) + tb).view(torch.int16).numpy().view(np.uint16))


def test_zero_fold_every_zero_point_times_every_finite_scale():
    z = np.arange(-128, 128, dtype=np.int8)
    for start in range(0, FINITE.size, 8192):
        s = FINITE[start:start + 8192]
        zz, ss = np.meshgrid(z, s, indexing="ij")
        got = orc.fold_zero_points_bf16(ss, zz)
        want = (torch.from_numpy((-zz.astype(np.int32)).astype(np.float32)).bfloat16() * as_torch_bf16(ss))   # utils/preprocess.h:99: the int is negated
        want = want.view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got, want)
        assert np.array_equal(mg.ZeroPointPreprocessor.neg_zero_point_multiplies_scale(ss, zz, element="bf16"), got)


CASES = [
    ("b_i4_sz", 24, 256, 4, SCALE_AND_ZEROS, 64, 1, True, "int8"),
    ("b_i4_sz_f", 16, 384, 4, SCALE_AND_ZEROS, 128, 2, False, "f16"),
    ("b_i4_s", 12, 256, 4, SCALE_ONLY, 128, 1, True, "f16"),
    ("b_i4_col", 8, 192, 4, PER_COLUMN, 0, 3, False, "f16"),
    ("b_i8_col", 16, 128, 8, PER_COLUMN, 0, 1, True, "f16"),
    ("b_i8_sz", 8, 256, 8, SCALE_AND_ZEROS, 64, 2, True, "int8"),
]


@pytest.mark.parametrize("cfg", CASES, ids=[c[0] for c in CASES])
def test_dequant_and_gemv_match_torch_restatement(cfg):
    tag, n, k, bits, qop, g, mb, bias, zk = cfg
    prob = Problem(tag, n, k, bits, qop, g, m_batch=mb, bias=bias, zero_kind=zk, element="bf16")
    q = prob.q.reshape(n, k).astype(np.int32)
    ref_dq = torch_dequantize(q, prob.scale, prob.zero_add, prob.group_size)
    got_dq = prob.oracle_dequant()
    assert np.array_equal(got_dq, ref_dq.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(prob.oracle_gemv(threads=1), sequential_gemv(ref_dq, prob.x, prob.bias))
    assert np.array_equal(prob.oracle_gemv(threads=4), prob.oracle_gemv(threads=1))
    if zk == "int8":   # host/mixed_gemv.h:92-96 as written: the int8 zero folded on the fly
        lit = orc.dequantize_bf16(prob.w_raw, prob.scale, prob.zeros_i8, n, k, prob.group_size, qop, bits)
        diff = lit != got_dq
        assert np.all((lit[diff] & 0x7FFF) == 0) and np.all((got_dq[diff] & 0x7FFF) == 0)   # -0 / +0 only


def test_dequant_every_weight_value_times_every_finite_scale():
    for bits, qs in ((4, np.arange(-8, 8)), (8, np.array([-128, -127, -77, -3, -1, 0, 1, 2, 5, 100, 127]))):
        n = qs.size
        for start in range(0, FINITE.size, 4096):
            s = FINITE[start:start + 4096]
            groups = s.size
            k = groups * 64
            q = np.repeat(qs[:, None], k, axis=1).astype(np.int8)
            w = orc.pack_int4(q.reshape(-1)) if bits == 4 else q.view(np.uint8).reshape(-1)
            scale = np.repeat(s[:, None], n, axis=1)
            got = orc.dequantize_bf16(w, scale, None, n, k, 64, SCALE_ONLY, bits)[:, ::64]
            want = (torch.from_numpy(qs.astype(np.float32)).bfloat16()[:, None] * as_torch_bf16(s)[None, :])
            assert np.array_equal(got, want.view(torch.int16).numpy().view(np.uint16))


def test_closed_forms_one_hot_unit_weights_bias_only():
    prob = Problem("b_hot", 16, 256, 4, SCALE_AND_ZEROS, 64, element="bf16")
    dq = prob.oracle_dequant()
    for j in (0, 63, 64, 255):
        x = np.zeros((1, 256), dtype=np.uint16)
        x[0, j] = 0x3F80                                                  # 1.0
        y = orc.gemv_bf16(prob.w_raw, x, prob.scale, prob.zero_add, None, 16, 1, 256, 64, SCALE_AND_ZEROS, 4)
        assert np.array_equal(y[0] & 0x7FFF, dq[:, j] & 0x7FFF) and np.array_equal(y[0][dq[:, j] & 0x7FFF != 0], dq[:, j][dq[:, j] & 0x7FFF != 0])
    # weights 1, scale 1, no zero: the output is the ascending fp32 sum of the activations
    q = np.ones((4, 128), dtype=np.int8)
    w = orc.pack_int4(q.reshape(-1))
    one = np.full((1, 4), 0x3F80, dtype=np.uint16)
    x = orc.f32_to_bf16_array(np.random.default_rng(3).standard_normal((1, 128)).astype(np.float32))
    acc = np.float32(0)
    for v in orc.bf16_to_f32_array(x[0]):
        acc = np.float32(acc + v)
    y = orc.gemv_bf16(w, x, one, None, None, 4, 1, 128, 128, PER_COLUMN, 4)
    assert np.all(y == torch_bits(np.array([acc]))[0])
    # zero activations: the bias comes back
    bias = orc.f32_to_bf16_array(np.array([0.5, -1.25, 3.0, 1e-3], dtype=np.float32))
    y = orc.gemv_bf16(w, np.zeros((1, 128), dtype=np.uint16), one, None, bias, 4, 1, 128, 128, PER_COLUMN, 4)
    assert np.array_equal(y[0], bias)
