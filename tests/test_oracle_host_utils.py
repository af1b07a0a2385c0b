"""Pins the oracle's restatement of the reference's host utilities: int4 packing
(utils/preprocess.h:41-84), zero folding (:94-101), the reference's own device layout
(:292-348, 393-455) and converter (gemv/interleaved_numeric_conversion.h:62-81, 232-291)."""
import numpy as np
import pytest

import np_restate
import oracle as orc


def test_pack_closed_form_exhaustive_pairs():
    # all 16 x 16 pairs of int4 values: element 2i -> low nibble, 2i+1 -> high nibble
    lo, hi = np.meshgrid(np.arange(-8, 8), np.arange(-8, 8), indexing="ij")
    vals = np.stack([lo.reshape(-1), hi.reshape(-1)], axis=1).astype(np.int8).reshape(-1)
    packed = orc.pack_int4(vals)
    expect = ((lo.reshape(-1) & 0xF) | ((hi.reshape(-1) & 0xF) << 4)).astype(np.uint8)
    assert np.array_equal(packed, expect)
    assert np.array_equal(orc.unpack_int4(packed), vals)


def test_unpack_every_byte_and_independent_restatement():
    every = np.arange(256, dtype=np.uint8)
    got = orc.unpack_int4(every)
    assert np.array_equal(got, np_restate.unpack_int4(every))
    assert got.min() == -8 and got.max() == 7
    assert np.array_equal(orc.pack_int4(got), every)


def test_pack_truncates_like_the_reference():
    # the reference's range check is dead code (`<` && `>`), values are masked to 4 bits
    vals = np.array([17, -9, 8, 7], dtype=np.int8)
    assert np.array_equal(orc.pack_int4(vals), np.array([(17 & 0xF) | ((-9 & 0xF) << 4), (8 & 0xF) | (7 << 4)], np.uint8))


def test_fold_zero_points_exhaustive_against_numpy_half():
    bits = np.arange(65536, dtype=np.uint16)
    finite = bits[(bits & 0x7C00) != 0x7C00]
    for z in list(range(-8, 8)) + [-128, -127, 127, 100, -77]:
        zz = np.full(finite.shape, z, dtype=np.int8)
        got = orc.fold_zero_points(finite.view(np.float16), zz).view(np.uint16)
        with np.errstate(over="ignore"):
            ref = (np.float16(-z) * finite.view(np.float16)).view(np.uint16)
        assert np.array_equal(got, ref), z
        # host/mixed_gemv.h:92-93 computes -(s * half(z)); identical except for the sign of zero
        with np.errstate(over="ignore"):
            alt = (-(finite.view(np.float16) * np.float16(z))).view(np.uint16)
        differ = got != alt
        assert np.all((got[differ] & 0x7FFF) == 0) and np.all((alt[differ] & 0x7FFF) == 0)


def _words(seed, n):
    return np.random.default_rng(seed).integers(0, 2 ** 32, size=n, dtype=np.uint64).astype(np.uint32)


def test_reference_layout_is_inverted_by_reference_converter():
    """convert(preprocess(W)) == W: the invariant the reference's kernel relies on."""
    rows, cols = 8, 64
    q = orc.fill_int8(rows * cols, 5, -8, 7)
    pre = orc.ref_preprocess_int4(orc.pack_int4(q), rows, cols).view(np.uint32)
    qm = q.reshape(rows, cols)
    C = cols // 8
    for r in range(rows):
        for c in range(C):
            # utils/preprocess.h:341-343: word (r, c) lands at (r/4)*4C + 4c + r%4
            w = int(pre[(r // 4) * 4 * C + 4 * c + (r % 4)])
            vals = orc.ref_convert_u4x8(w).astype(np.float32)
            assert np.array_equal(vals, qm[r, 8 * c: 8 * c + 8].astype(np.float32)), (r, c)


def test_reference_int4_converter_all_nibble_values_exact_integers():
    # every nibble value in every position: result is the exact integer u - 8 as fp16, zero is +0
    for pos in range(8):
        for u in range(16):
            w = u << (4 * pos)
            out = orc.ref_convert_u4x8(w)
            # stored order [e7 e5 e3 e1 e6 e4 e2 e0]: position p holds element 2p (p<4) or 2(p-4)+1
            elem = 2 * pos if pos < 4 else 2 * (pos - 4) + 1
            expect = np.full(8, -8.0, dtype=np.float32)
            expect[elem] = u - 8
            assert np.array_equal(out.astype(np.float32), expect)
            assert np.all(out.view(np.uint16)[out == 0] == 0)


def test_reference_int8_converter():
    # biased bytes laid out [e3 e1 e2 e0] (utils/preprocess.h:387-390) come back as e0..e3 = u - 128
    r = np.random.default_rng(9)
    for _ in range(2000):
        e = r.integers(-128, 128, size=4)
        b = (e + 128).astype(np.uint32)
        w = int(b[0] | (b[2] << 8) | (b[1] << 16) | (b[3] << 24))
        out = orc.ref_convert_u8x4(w).astype(np.float32)
        # halves come out as (b0, b2) then (b1, b3) of the stored word = e0, e1, e2, e3
        assert np.array_equal(out, e.astype(np.float32))


def test_reference_preprocess_rejects_bad_shapes():
    with pytest.raises(ValueError):
        orc.ref_preprocess_int4(np.zeros(3 * 8 // 2, np.uint8), 3, 8)
    with pytest.raises(ValueError):
        orc.ref_preprocess_int4(np.zeros(4 * 12 // 2, np.uint8), 4, 12)
