"""Host side of the library (no GPU needed): packing, zero folding, the gfx950 weight
preprocessor, error codes, and that the shared library exports every symbol the header declares."""
import ctypes
import os
import re

import numpy as np
import pytest

import mixed_gemv_amd as mg
import oracle as orc
from mixed_gemv_amd import _lib
from mixed_gemv_amd._lib import MixedGemvError

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
W4, W8 = mg.QuantType.W4_A16, mg.QuantType.W8_A16
COL, ROW = mg.LayoutType.kColumnMajor, mg.LayoutType.kRowMajor


# least significant bit of the stored 4-bit field of element e of a 32-bit int4 word (wraps at 32)
INT4_FIELD_SHIFT = (7, 23, 3, 19, 15, 31, 11, 27)

def test_library_exports_every_declared_symbol():
    # the boundary (mixed_gemv.h) and the measurement probes (mixed_gemv_probes.h) are one library
    header = "".join(open(os.path.join(REPO, "include", h)).read() for h in ("mixed_gemv.h", "mixed_gemv_probes.h"))
    declared = set(re.findall(r"MGEMV_API\s+[\w\s\*]+?\b(mgemv_\w+)\s*\(", header))
    assert len(declared) >= 12
    boundary = open(os.path.join(REPO, "include", "mixed_gemv.h")).read()
    assert "mgemv_probe_" not in boundary, "measurement entries belong in mixed_gemv_probes.h"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in include/ but not exported"
    assert declared == set(_lib.SIGNATURES), "python binding and header disagree"
    assert _lib.lib().mgemv_version() >= 100
    for code in range(0, 17):
        assert _lib.lib().mgemv_status_string(code) not in (None, b"", b"unknown status")


def test_pack_unpack_and_fold_equal_the_oracle():
    q = orc.fill_int8(4096, 3, -8, 7)
    packed = mg.SubBytePacker.pack(q)
    assert np.array_equal(packed, orc.pack_int4(q))
    assert np.array_equal(mg.SubBytePacker.unpack(packed), q)
    every = np.arange(256, dtype=np.uint8)
    assert np.array_equal(mg.SubBytePacker.unpack(every), orc.unpack_int4(every))
    # all finite scales x a spread of zero points
    bits = np.arange(65536, dtype=np.uint16)
    finite = bits[(bits & 0x7C00) != 0x7C00]
    for z in (-128, -8, -1, 0, 1, 7, 127):
        zz = np.full(finite.shape, z, dtype=np.int8)
        got = mg.ZeroPointPreprocessor.neg_zero_point_multiplies_scale(finite.view(np.float16), zz)
        assert np.array_equal(got.view(np.uint16), orc.fold_zero_points(finite.view(np.float16), zz).view(np.uint16))


def _expected_offset(n, k0, k, bits):
    """Layout closed form restated independently of csrc/tile_layout.h."""
    chunk = 128 // bits
    run, step = 4 * chunk, 16 * chunk
    ksteps = -(-k // step)
    tile, r = divmod(n, 16)
    s, kk = divmod(k0, step)
    slice_, rem = divmod(kk, run)
    blk = rem // chunk
    return (tile * ksteps + s) * 4096 + blk * 1024 + (slice_ * 16 + r) * 16


@pytest.mark.parametrize("bits,n_out,k", [(4, 16, 512), (4, 20, 544), (4, 100, 1120), (8, 16, 256), (8, 36, 400)])
def test_preprocess_layout_closed_form_and_round_trip(bits, n_out, k):
    lo, hi = (-8, 7) if bits == 4 else (-128, 127)
    q = orc.fill_int8(n_out * k, 100 + n_out, lo, hi).reshape(n_out, k)
    raw = orc.pack_int4(q.reshape(-1)) if bits == 4 else q.reshape(-1).view(np.uint8)
    qt = W4 if bits == 4 else W8
    pre = mg.MixedGemvWeightPreprocessor.run(raw, (k, n_out), COL, qt)
    assert pre.size == mg.preprocessed_size((k, n_out), qt)
    assert pre.size == -(-n_out // 16) * -(-k // (2048 // bits)) * 4096
    chunk = 128 // bits
    touched = np.zeros(pre.size, dtype=bool)
    for n in range(n_out):
        for k0 in range(0, k, chunk):
            off = _expected_offset(n, k0, k, bits)
            words = pre[off:off + 16].view(np.uint32)
            touched[off:off + 16] = True
            vals = q[n, k0:k0 + chunk].astype(np.int32)
            for j in range(4):
                w = int(words[j])
                if bits == 4:
                    for e in range(8):
                        # pair (e, e+1) sits at the same bits of the two 16-bit halves: bits 7-10 or 3-6,
                        # directly (e < 4) or after an 8-bit right rotation (e >= 4)
                        shift = INT4_FIELD_SHIFT[e]
                        rot = ((w >> shift) | (w << (32 - shift))) & 0xFFFFFFFF
                        assert (rot & 0xF) == vals[8 * j + e] + 8
                else:
                    for e in range(4):
                        assert ((w >> (8 * e)) & 0xFF) == vals[4 * j + e] + 128
    assert not pre[~touched].any(), "padding must be zero"
    back = mg.unpreprocess_weights(pre, (k, n_out), qt)
    assert np.array_equal(back, raw)


def test_int4_field_positions_tile_the_word():
    # the eight 4-bit fields cover each of the 32 bits exactly once, and the two elements of a
    # k-adjacent pair sit 16 bits apart
    covered = np.zeros(32, dtype=int)
    for e, shift in enumerate(INT4_FIELD_SHIFT):
        for b in range(4):
            covered[(shift + b) % 32] += 1
        if e % 2:
            assert shift == INT4_FIELD_SHIFT[e - 1] + 16
    assert (covered == 1).all()
    # after the rotation that the kernels apply, every field sits at bits 7-10 or 3-6 of a half-word
    for e, shift in enumerate(INT4_FIELD_SHIFT):
        pos = (shift - (8 if e >= 4 else 0)) % 32
        assert pos % 16 in (7, 3)


def test_preprocess_is_a_bijection_on_nibbles():
    n_out, k = 32, 1024
    # every nibble distinct-ish: use a counter pattern so that a collision or a dropped chunk shows
    raw = (np.arange(n_out * k // 2, dtype=np.uint32) * 2654435761 >> 7).astype(np.uint8)
    pre = mg.MixedGemvWeightPreprocessor.run(raw, (k, n_out), COL, W4)
    words = pre.view(np.uint32).astype(np.uint64)
    fields = np.concatenate([(((words >> s) | (words << (32 - s))) & 0xF) for s in INT4_FIELD_SHIFT]).astype(np.int8)
    assert np.array_equal(np.sort(fields), np.sort(mg.SubBytePacker.unpack(raw ^ 0x88).astype(np.int8) & 0xF))
    assert np.array_equal(mg.unpreprocess_weights(pre, (k, n_out), W4), raw)


@pytest.mark.parametrize("bits", [4, 8])
def test_row_major_input_equals_transposed_column_major(bits):
    n_out, k = 48, 320
    lo, hi = (-8, 7) if bits == 4 else (-128, 127)
    q = orc.fill_int8(n_out * k, 55, lo, hi).reshape(n_out, k)          # [n_out][k]
    qt = W4 if bits == 4 else W8
    to_raw = (lambda a: orc.pack_int4(a.reshape(-1))) if bits == 4 else (lambda a: a.reshape(-1).view(np.uint8).copy())
    col = mg.MixedGemvWeightPreprocessor.run(to_raw(q), (k, n_out), COL, qt)
    row = mg.MixedGemvWeightPreprocessor.run(to_raw(np.ascontiguousarray(q.T)), (k, n_out), ROW, qt)
    assert np.array_equal(col, row)


def test_three_dimensional_shape_is_per_expert():
    e, n_out, k = 3, 20, 96
    q = orc.fill_int8(e * n_out * k, 66, -8, 7).reshape(e, n_out, k)
    raw = orc.pack_int4(q.reshape(-1))
    pre = mg.MixedGemvWeightPreprocessor.run(raw, (e, k, n_out), COL, W4)
    one = mg.preprocessed_size((k, n_out), W4)
    assert pre.size == e * one
    for i in range(e):
        single = mg.MixedGemvWeightPreprocessor.run(orc.pack_int4(q[i].reshape(-1)), (k, n_out), COL, W4)
        assert np.array_equal(pre[i * one:(i + 1) * one], single)
    assert np.array_equal(mg.unpreprocess_weights(pre, (e, k, n_out), W4), raw)


def test_preprocess_error_codes():
    buf = np.zeros(1 << 16, dtype=np.uint8)
    cases = [
        ((64,), COL, W4, 2),            # rank 1          utils/preprocess.h:486-489
        ((1, 2, 64, 64), COL, W4, 2),   # rank 4
        ((64, 6), COL, W4, 3),          # rows % 4        utils/preprocess.h:319-322
        ((36, 64), COL, W4, 4),         # k % 8           utils/preprocess.h:324-327
        ((20, 64), COL, W8, 4),
        ((64, 64), COL, mg.QuantType.W4_AFP8, 7),
        ((64, 64), 5, W4, 9),
        ((0, 64), COL, W4, 10),
    ]
    for shape, layout, qt, status in cases:
        with pytest.raises(MixedGemvError) as ei:
            mg.MixedGemvWeightPreprocessor.run(buf, shape, layout, qt)
        assert ei.value.status == status, (shape, ei.value.status)
    assert mg.preprocessed_size((64,), W4) == 0
    lib = _lib.lib()
    shape = (ctypes.c_size_t * 2)(64, 64)
    assert lib.mgemv_preprocess_weights(None, None, shape, 2, 1, 1) == 1
    assert lib.mgemv_pack_int4(None, None, 8) == 1
    assert lib.mgemv_pack_int4(None, None, 0) == 0
    three = np.zeros(3, dtype=np.int8)
    assert lib.mgemv_pack_int4(ctypes.c_void_p(buf.ctypes.data), ctypes.c_void_p(three.ctypes.data), 3) == 10  # odd count
    assert lib.mgemv_fold_zero_points(None, None, None, 4) == 1


def test_gemv_argument_checks_return_codes_without_launching():
    """Every condition on which the reference prints and exits is a status code here; all of
    these return before anything touches a GPU."""
    lib = _lib.lib()
    p = ctypes.c_void_p(0x1000)  # never dereferenced: the checks below all fail first

    def gemv(n_out=64, m=1, k=512, g=128, qop=3, bits=4, w=p, x=p, s=p, z=p, y=p):
        return lib.mgemv_gemv(w, x, s, z, None, y, n_out, m, k, g, qop, bits, None)

    assert gemv(qop=0) == 6 and gemv(qop=4) == 6          # gemv/weight_only_quant_op.h:12-18
    assert gemv(bits=5) == 7
    assert gemv(m=0) == 8 and gemv(m=17) == 8              # the reference accepts N == 1 only (host/mixed_gemv.h:72-75)
    assert gemv(n_out=0) == 10 and gemv(k=-4) == 10
    assert gemv(n_out=66) == 3
    assert gemv(k=516) == 4                                 # k % 8 (utils/preprocess.h:324-327)
    assert gemv(k=520, qop=1) != 4                          # a multiple of 8 passes the shape checks (per-column mode)
    assert gemv(g=32) == 5                                  # gemv/device/gemv_adaptor.h:199-203
    assert gemv(g=96, k=512) == 5                           # does not divide k
    assert gemv(g=80, k=640) == 5                           # not a multiple of 32
    assert gemv(w=None) == 1 and gemv(s=None) == 1 and gemv(z=None) == 1 and gemv(x=None) == 1 and gemv(y=None) == 1
    assert gemv(w=ctypes.c_void_p(0x1008)) == 13
    assert gemv(x=ctypes.c_void_p(0x1002)) == 13
    assert lib.mgemv_gemv_batched(p, p, p, p, None, p, 0, 64, 1, 512, 128, 3, 4, 0, 0, 0, 0, 0, None) == 8
    assert lib.mgemv_dequantize(p, p, p, None, 64, 512, 128, 3, 4, None) == 1
    # routed launch: the route is required, its stack extent positive, its address a multiple of 4
    routed = lambda r, extent, fn=lib.mgemv_gemv_routed: fn(p, p, p, p, None, p, r, extent, 2, 64, 1, 512, 128, 3, 4,  # noqa: E731
                                                            0, 0, 0, 0, 0, None)
    assert routed(None, 4) == 1 and routed(None, 4, lib.mgemv_gemv_routed_bf16) == 1
    assert routed(p, 0) == 8 and routed(p, -3, lib.mgemv_gemv_routed_bf16) == 8
    assert routed(ctypes.c_void_p(0x1002), 4) == 13
    assert lib.mgemv_dequantize(p, p, p, p, 64, 512, 16, 2, 4, None) == 5
    # per-column mode ignores group_size entirely (mixed_gemv_test.cu:142-143): 16 would be rejected otherwise
    assert lib.mgemv_dequantize(p, p, None, None, 64, 512, 16, 1, 4, None) == 1
    out = (ctypes.c_int * 8)()
    assert lib.mgemv_query_launch(4096, 1, 4096, 4, 128, ctypes.byref(out)) == 0
    assert out[0] % 8 == 0 and out[1] % 64 == 0 and out[2] * out[4] >= 8
    assert lib.mgemv_query_launch(4096, 1, 4096, 3, 128, ctypes.byref(out)) == 7
    assert lib.mgemv_query_launch(4096, 1, 4096, 4, -1, ctypes.byref(out)) == 5
    assert lib.mgemv_set_launch_override(-1, 0, 0, 0) == 10
    assert lib.mgemv_set_launch_override(0, 0, 3, 0) == 10
    assert lib.mgemv_set_matrix_core_threshold(18) == 8
    assert lib.mgemv_set_matrix_core_variant(4) == 10 and lib.mgemv_set_matrix_core_variant(0) == 0
    assert lib.mgemv_set_dequant_form(2) == 10 and lib.mgemv_set_dequant_form(0) == 0


@pytest.mark.parametrize("bits,n_out,k", [(4, 20, 40), (4, 64, 8), (4, 36, 1000), (8, 12, 24), (8, 32, 520)])
def test_k_that_is_a_multiple_of_8_only_round_trips(bits, n_out, k):
    """utils/preprocess.h:324-327 asks for k % 8 == 0, not for whole 128-bit chunks: the last chunk
    of a row may be partly padding."""
    qt = W4 if bits == 4 else W8
    raw = orc.fill_int8(n_out * k * bits // 8, 11, -128, 127).view(np.uint8)
    pre = mg.MixedGemvWeightPreprocessor.run(raw, (k, n_out), COL, qt)
    assert pre.size == mg.preprocessed_size((k, n_out), qt)
    assert np.array_equal(mg.unpreprocess_weights(pre, (k, n_out), qt), raw)
    # row-major input of the same matrix gives the same buffer
    q = mg.SubBytePacker.unpack(raw) if bits == 4 else raw.view(np.int8)
    qt_rm = np.ascontiguousarray(q.reshape(n_out, k).T)
    raw_rm = mg.SubBytePacker.pack(qt_rm.reshape(-1)) if bits == 4 else qt_rm.view(np.uint8).reshape(-1)
    assert np.array_equal(mg.MixedGemvWeightPreprocessor.run(raw_rm, (k, n_out), ROW, qt), pre)


def test_arguments_entry_refuses_operands_that_are_not_dense():
    """GemvAdaptor::Arguments carries leading dimensions (gemv/device/gemv_adaptor.h:116-122); only the
    dense values are taken, everything else is a status, before anything touches a GPU."""
    from mixed_gemv_amd.api import _Arguments
    lib = _lib.lib()
    n, m, k = 64, 1, 512

    def call(**over):
        f = dict(n_out=n, m_batch=m, k=k, weights=0x1000, lda=4 * k, x=0x1000, ldb=0, scale=0x1000, ld_scale=n,
                 zero_add=0x1000, ld_zero=n, bias=0, ldc=n, y=0x1000, ldd=n, alpha=1.0, beta=1.0, group_size=128,
                 batch_count=1, batch_stride_weights=0, batch_stride_x=0, batch_stride_scale=0, batch_stride_bias=0,
                 batch_stride_y=0, quant_op=3, weight_bits=4, element=0)
        f.update(over)
        a = _Arguments(**f)
        return lib.mgemv_gemv_arguments(ctypes.byref(a), None)

    assert lib.mgemv_gemv_arguments(None, None) == 1
    for field, bad in (("lda", 2 * k), ("ldb", k + 8), ("ld_scale", n + 4), ("ld_zero", 2 * n), ("ldc", 1), ("ldd", n + 64)):
        assert call(**{field: bad}) == 14, field
    assert call(m_batch=2, ldb=0) == 14          # stride-0 activations are the reference's single row only
    assert call(element=2) == 7
    # dense operands pass the leading-dimension checks and fail later, on the missing device or not at all
    assert call() in (0, 12)
    assert call(lda=0, ldb=k, ld_scale=0, ld_zero=0, ldc=0, ldd=0) in (0, 12)
    assert call(k=516, lda=0) == 4 and call(group_size=32) == 5      # the checks of mgemv_gemv still apply


def test_device_entry_points_report_a_missing_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = _lib.lib()
    p = ctypes.c_void_p(0x1000)
    assert lib.mgemv_gemv(p, p, p, p, None, p, 64, 1, 512, 128, 3, 4, None) == 12
    assert lib.mgemv_dequantize(p, p, p, p, 64, 512, 128, 3, 4, None) == 12


@pytest.mark.parametrize("entry", ["mgemv_host_gemv", "mgemv_host_gemv_static"])
def test_host_gemv_checks_its_arguments_before_touching_the_device(entry):
    lib = _lib.lib()
    w = np.zeros(64 * 512 // 2, dtype=np.uint8)
    h = np.zeros(64 * 512, dtype=np.uint16)
    z = np.zeros(64 * 4, dtype=np.int8)
    ptr = lambda a: ctypes.c_void_p(a.ctypes.data)  # noqa: E731

    def call(batch=1, n=64, m=1, k=512, g=128, ww=w, x=h, s=h, zz=z, y=h, qop=3, bits=4):
        return getattr(lib, entry)(batch, n, m, k, g, ptr(ww) if ww is not None else None, ptr(x), ptr(s),
                                   ptr(zz) if zz is not None else None, None, ptr(y), qop, bits)

    assert call(batch=2) == 8                      # host/mixed_gemv.h:77-80
    assert call(m=0) == 8 and call(m=17) == 8      # host/mixed_gemv.h:72-75 takes N == 1 only; here up to 16 rows
    assert call(ww=None) == 1 and call(zz=None) == 1
    assert call(qop=0) == 6 and call(bits=3) == 7
    assert call(g=100) == 5
    assert call(n=66) == 3 and call(k=516, g=516) == 4


def test_static_scratch_limit_is_checked_on_the_host():
    """mgemv_host_gemv_static refuses a problem whose staging exceeds its static arrays before it
    looks for a device; the size query agrees with the layout both host-pointer entries use."""
    lib = _lib.lib()
    limit = mg.STATIC_SCRATCH_BYTES
    assert limit == 16 << 20
    # weights + activations + scales + folded zeros + outputs, each piece rounded up to 256 bytes
    need = mg.static_scratch_bytes_needed(4096, 1, 4096, 128)
    assert need == 4096 * 4096 // 2 + 4096 * 2 + 2 * (32 * 4096 * 2) + 4096 * 2
    assert mg.static_scratch_bytes_needed(4096, 1, 4096, 128, has_bias=True) == need + 4096 * 2
    assert mg.static_scratch_bytes_needed(100, 3, 1120, 160) == (
        7 * 3 * 4096 + 6912 + 2 * 1536 + 768)   # 7 tiles x 3 k steps; 3 x 1120 x 2 = 6720 -> 6912; 7 x 100 x 2 = 1400 -> 1536; 600 -> 768
    assert mg.static_scratch_bytes_needed(4096, 1, 4096, 100) == 0 and mg.static_scratch_bytes_needed(4096, 17, 4096, 128) == 0
    n_out, k = 8192, 8192
    assert mg.static_scratch_bytes_needed(n_out, 1, k, 128) > limit
    dummy = np.zeros(16, dtype=np.uint16)   # never read: the size check comes first
    p = ctypes.c_void_p(dummy.ctypes.data)
    assert lib.mgemv_host_gemv_static(1, n_out, 1, k, 128, p, p, p, p, None, p, 3, 4) == 16
    assert b"static scratch" in lib.mgemv_status_string(16)


def test_tuned_plan_table_steers_exactly_its_problem(tmp_path):
    from mixed_gemv_amd import autotune
    autotune.clear()
    try:
        builtin = mg.query_launch(4096, 1, 4096, 4, 128)
        other = mg.query_launch(8192, 1, 8192, 4, 64)
        mg.set_tuned_plan(4096, 4096, 4, 128, 1, kernel=mg.KERNEL_VALU, split_k=8, tiles_per_wg=2)
        assert mg.tuned_plan_count() == 1
        tuned = mg.query_launch(4096, 1, 4096, 4, 128)
        assert (tuned["split_k"], tuned["tiles_per_wg"], tuned["matrix_core"]) == (8, 2, 0) and tuned != builtin
        # other group size, batch size, weight width or shape: untouched
        assert mg.query_launch(4096, 1, 4096, 4, 64) == builtin
        assert mg.query_launch(4096, 2, 4096, 4, 128) == mg.query_launch(4096, 2, 4096, 4, 0)
        assert mg.query_launch(8192, 1, 8192, 4, 64) == other
        # an entry for any group size; the exact one still wins where it exists
        mg.set_tuned_plan(4096, 4096, 4, 0, 1, kernel=mg.KERNEL_VALU, split_k=2, tiles_per_wg=1)
        assert mg.query_launch(4096, 1, 4096, 4, 64)["split_k"] == 2
        assert mg.query_launch(4096, 1, 4096, 4, 128)["split_k"] == 8
        # replacing a key keeps the count; kernel choice for a small batch
        mg.set_tuned_plan(4096, 4096, 4, 128, 1, kernel=mg.KERNEL_VALU, split_k=4, tiles_per_wg=1)
        assert mg.tuned_plan_count() == 2 and mg.query_launch(4096, 1, 4096, 4, 128)["split_k"] == 4
        mg.set_tuned_plan(4096, 4096, 4, 128, 4, kernel=mg.KERNEL_MATRIX_CORE_LDS_STAGED)
        assert mg.query_launch(4096, 4, 4096, 4, 128)["matrix_core"] == 2
        mg.set_tuned_plan(4096, 4096, 4, 128, 8, kernel=mg.KERNEL_MATRIX_CORE_REGISTER_OPERAND, tiles_per_wave=2)
        q = mg.query_launch(4096, 8, 4096, 4, 128)
        assert q["matrix_core"] == 1 and q["tiles_per_wave"] == 2
        mg.set_tuned_plan(4096, 4096, 4, 128, 16, kernel=mg.KERNEL_VALU)
        assert mg.query_launch(4096, 16, 4096, 4, 128)["matrix_core"] == 0
        # a process-wide override takes precedence over the table
        mg.set_launch_override(8, 1, 0, 0)
        assert mg.query_launch(4096, 1, 4096, 4, 128)["split_k"] == 8
        mg.set_launch_override(0, 0, 0, 0)
        assert mg.query_launch(4096, 1, 4096, 4, 128)["split_k"] == 4
        # the JSON table carries entries from one process to the next
        autotune.install(dict(n_out=11008, k=4096, weight_bits=4, group_size=128, m_batch=1, kernel=mg.KERNEL_VALU,
                              split_k=2, tiles_per_wg=2, max_workgroups=256))
        want = mg.query_launch(11008, 1, 4096, 4, 128)
        autotune.save_table(tmp_path / "plans.json")
        autotune.clear()
        assert mg.tuned_plan_count() == 0 and mg.query_launch(4096, 1, 4096, 4, 128) == builtin
        assert autotune.load_table(tmp_path / "plans.json") == 1
        assert mg.query_launch(11008, 1, 4096, 4, 128) == want
        # argument checks
        for bad, code in ((dict(weight_bits=5), 7), (dict(n_out=0), 10), (dict(group_size=-1), 5), (dict(m_batch=0), 8),
                          (dict(m_batch=17), 8), (dict(kernel=5), 10), (dict(tiles_per_wave=3), 10), (dict(split_k=-1), 10)):
            args = dict(n_out=64, k=512, weight_bits=4, group_size=128, m_batch=1)
            args.update(bad)
            with pytest.raises(MixedGemvError) as ei:
                mg.set_tuned_plan(**args)
            assert ei.value.status == code
        assert _lib.lib().mgemv_tuned_plan_set(None) == 1
    finally:
        autotune.clear()
        mg.set_launch_override(0, 0, 0, 0)


def test_tuned_plan_table_is_safe_under_concurrent_writers_and_readers():
    import threading
    from mixed_gemv_amd import autotune
    autotune.clear()
    errors = []

    def writer(t):
        try:
            for i in range(300):
                mg.set_tuned_plan(64 * (1 + i % 50), 512 * (1 + t), 4, 128, 1, kernel=mg.KERNEL_VALU, split_k=1 + i % 4)
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    def reader():
        try:
            for i in range(600):
                q = mg.query_launch(64 * (1 + i % 50), 1, 512 * (1 + i % 4), 4, 128)
                assert q["threads"] % 64 == 0 and q["workgroups"] >= 1
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=writer, args=(t,)) for t in range(4)] + [threading.Thread(target=reader) for _ in range(4)]
    try:
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors
        assert mg.tuned_plan_count() == 4 * 50
    finally:
        autotune.clear()


def test_adaptor_mirror_rejects_small_groups_like_the_reference():
    args = mg.GemvAdaptor.Arguments((64, 1, 512), 0x1000, 0x1000, 0x1000, 0x1000, None, 0x1000, group_size=32)
    with pytest.raises(MixedGemvError) as ei:
        mg.GemvAdaptor().initialize(args)
    assert ei.value.status == 5


# (n_out, m_batch, k) -> expected fields of the built-in plan, int4 group 128.  Each row is a shape
# on which the rule that produces it was measured against its alternatives on an MI355X; the
# test pins the rules, so a change to plan_launch that moves one of them shows up here.
BUILTIN_PLANS = [
    # exact fit: one 4-wave workgroup per compute unit, every wave walking 7 tiles
    ((28672, 1, 8192), dict(matrix_core=0, workgroups=256, threads=256, split_k=4, tiles_in_sequence=7)),
    ((57344, 1, 8192), dict(matrix_core=0)),                   # a single row never goes to the matrix cores
    ((8192, 1, 8192), dict(matrix_core=0, workgroups=256, threads=256)),
    # an even fit of the tiles is not enough for one four-wave workgroup per compute unit: the k steps must divide
    # over its waves too, and there must be more than four of them
    ((12288, 1, 3072), dict(matrix_core=0, workgroups=768, split_k=6, steps_per_wave=1, tiles_in_sequence=1)),
    ((12288, 1, 2048), dict(matrix_core=0, workgroups=768, split_k=4, steps_per_wave=1, tiles_in_sequence=1)),
    ((12288, 1, 5120), dict(matrix_core=0, workgroups=768, split_k=10, steps_per_wave=1, tiles_in_sequence=1)),
    ((28672, 1, 5120), dict(matrix_core=0, workgroups=1792, split_k=1, steps_per_wave=10)),
    ((12288, 1, 6144), dict(matrix_core=0, workgroups=256, split_k=4, steps_per_wave=3, tiles_in_sequence=3)),
    # at most one workgroup per compute unit: four k-split waves
    ((4096, 1, 4096), dict(matrix_core=0, workgroups=256, split_k=4, steps_per_wave=2)),
    ((4096, 1, 14336), dict(matrix_core=0, workgroups=256, split_k=4, steps_per_wave=7)),
    # few tiles and a short reduction: one unit per wave
    ((1024, 1, 4096), dict(matrix_core=0, split_k=8, steps_per_wave=1)),
    # more than one workgroup per compute unit and 5-8 k steps: one unit per wave, at one and two rows
    ((6144, 1, 4096), dict(matrix_core=0, workgroups=384, split_k=8, steps_per_wave=1)),
    ((6144, 2, 4096), dict(matrix_core=0, workgroups=384, split_k=8, steps_per_wave=1)),
    ((22016, 1, 4096), dict(matrix_core=0, workgroups=1376, split_k=8, steps_per_wave=1)),
    # 288-512 tiles and 9 or more k steps: two tiles per workgroup with two waves each (four up to 384 tiles from 20 k steps)
    ((7168, 1, 14336), dict(matrix_core=0, workgroups=224, tiles_per_wg=2, split_k=2, steps_per_wave=14)),
    ((7680, 1, 4096), dict(matrix_core=0, workgroups=480, tiles_per_wg=1, split_k=8)),
    ((5120, 1, 5120), dict(matrix_core=0, workgroups=160, tiles_per_wg=2, split_k=2, steps_per_wave=5)),
    ((6144, 2, 8192), dict(matrix_core=0, workgroups=192, tiles_per_wg=2, split_k=2, steps_per_wave=8)),
    ((5120, 1, 14336), dict(matrix_core=0, workgroups=160, tiles_per_wg=2, split_k=4, steps_per_wave=7)),
    ((4160, 1, 8192), dict(matrix_core=0, tiles_per_wg=1, split_k=4)),
    # above 512 tiles and from 16 k steps: at most four k-split waves
    ((9216, 1, 14336), dict(matrix_core=0, workgroups=576, tiles_per_wg=1, split_k=4, steps_per_wave=7)),
    # one wave per unit would not fit and one wave per tile fills the SIMDs: whole-k waves
    ((13824, 1, 5120), dict(matrix_core=0, workgroups=864, threads=64, split_k=1, steps_per_wave=10)),
    ((128256, 1, 4096), dict(matrix_core=0, workgroups=8016, threads=64, split_k=1)),
    # ... and with a poor fit the k split stays
    ((17408, 1, 5120), dict(matrix_core=0, workgroups=1088, split_k=5, steps_per_wave=2)),
    # matrix cores: from 5 rows anywhere, from 3 rows on more than 256 tiles, from 2 rows on many tiles
    ((4096, 3, 4096), dict(matrix_core=0)),
    ((4096, 4, 4096), dict(matrix_core=0, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((4096, 5, 4096), dict(matrix_core=2, tiles_per_wg=1, split_k=4, variant=mg.MATRIX_CORE_LDS_STAGED)),
    # at most one tile per compute unit: the k-stationary kernel at 4-7 rows with 5-8 k steps, at 3-7 with 9-14
    ((4096, 4, 4096), dict(matrix_core=3, workgroups=256, split_k=8, tiles_in_sequence=1)),
    ((4096, 7, 4096), dict(matrix_core=3)),
    ((2560, 4, 2560), dict(matrix_core=3, workgroups=160, split_k=5)),
    ((2048, 3, 5120), dict(matrix_core=3, workgroups=128, split_k=10)),
    ((4096, 6, 7168), dict(matrix_core=3)),
    ((4096, 6, 7680), dict(matrix_core=2)),                    # 15 k steps: only up to 4 rows
    ((4096, 4, 7680), dict(matrix_core=3)),
    ((4096, 3, 8192), dict(matrix_core=0)),                    # 16 waves without a walk lose
    ((4096, 4, 8192), dict(matrix_core=2)),
    ((1024, 4, 6144), dict(matrix_core=0)),                    # fewer tiles than half the compute units: not measured
    ((16, 8, 4096), dict(matrix_core=1)),                      # a single tile: the register-operand kernel
    ((4096, 8, 4096), dict(matrix_core=2, tiles_per_wg=1, split_k=4)),
    ((5120, 3, 4096), dict(matrix_core=2, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((5120, 3, 4096), dict(matrix_core=3, workgroups=256, tiles_in_sequence=2)),
    ((4096, 3, 14336), dict(matrix_core=0)),
    ((4096, 4, 14336), dict(matrix_core=2, tiles_per_wg=1)),   # 4 rows, up to 256 tiles, from 16 k steps
    ((2048, 4, 8192), dict(matrix_core=2, tiles_per_wg=1)),    # ... on few tiles as well (6.5 us against 6.7; 1536x8960 7.4 / 8.2)
    ((2048, 3, 8192), dict(matrix_core=0)),
    ((1024, 4, 7680), dict(matrix_core=0)),                    # 15 k steps, fewer tiles than half the compute units
    ((10240, 2, 8192), dict(matrix_core=0, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((28672, 2, 8192), dict(matrix_core=2, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((50304, 2, 2048), dict(matrix_core=0)),
    ((151936, 2, 2048), dict(matrix_core=2)),
    # 2-8 rows on the k-stationary kernel: walks of 2 tiles or more with up to 8 k steps (2 rows: 8 k steps), of 3 or
    # more with 9-16, that fill their last round; one workgroup per compute unit, one wave per k step
    ((28672, 2, 8192), dict(matrix_core=3, workgroups=256, split_k=16, tiles_in_sequence=7)),
    ((11008, 3, 4096), dict(matrix_core=3, workgroups=256, split_k=8, tiles_in_sequence=3)),
    ((8192, 8, 4096), dict(matrix_core=3, workgroups=256, split_k=8, tiles_in_sequence=2)),
    ((8192, 7, 2048), dict(matrix_core=3, workgroups=256, split_k=4, tiles_in_sequence=2)),
    ((22016, 2, 4096), dict(matrix_core=3, workgroups=256, split_k=8, tiles_in_sequence=6)),
    ((12288, 3, 8192), dict(matrix_core=3, workgroups=256, split_k=16, tiles_in_sequence=3)),
    ((10240, 8, 8192), dict(matrix_core=3, tiles_in_sequence=3)),    # 640 tiles: better filled than 160 workgroups of 4 tiles
    ((10240, 2, 8192), dict(matrix_core=3, tiles_in_sequence=3)),
    ((5120, 8, 5120), dict(matrix_core=3, tiles_in_sequence=2)),     # 10 k steps, walks of 2
    ((8192, 4, 8192), dict(matrix_core=3, tiles_in_sequence=2)),     # 3-4 rows: walks of 2 and 3, or tiles that divide evenly
    ((16384, 4, 8192), dict(matrix_core=3, tiles_in_sequence=4)),
    ((13312, 4, 8192), dict(matrix_core=2)),                   # walks of 4 that neither divide evenly nor fill better: no
    ((8192, 8, 8192), dict(matrix_core=2)),                    # 5-8 rows, 16 k steps, filled alike: no
    ((16384, 8, 8192), dict(matrix_core=2)),
    ((14336, 8, 8192), dict(matrix_core=2)),
    ((8192, 2, 8192), dict(matrix_core=0)),                    # 2 rows on walks of 2: the VALU kernel
    ((6144, 2, 4096), dict(matrix_core=0)),
    ((4608, 4, 2048), dict(matrix_core=0)),                    # 4 k steps: from 1.5 tiles per compute unit
    ((32768, 4, 1024), dict(matrix_core=2)),                   # 2 k steps, 2 waves per compute unit: no
    # 9-16 rows: only where it fills the machine better than the LDS-staged kernel's workgroups of up to 8 tiles and the
    # partial sums of a walk fit the LDS; with up to 8 k steps only on walks of up to 6 tiles
    ((28672, 9, 8192), dict(matrix_core=3, workgroups=256, tiles_in_sequence=7)),
    ((28672, 16, 8192), dict(matrix_core=3, workgroups=256, tiles_in_sequence=7)),
    ((11008, 16, 4096), dict(matrix_core=3, tiles_in_sequence=3)),
    ((28672, 16, 4096), dict(matrix_core=2)),
    ((32768, 16, 8192), dict(matrix_core=2)),
    ((8192, 16, 6144), dict(matrix_core=2)),
    ((128256, 8, 4096), dict(matrix_core=3, workgroups=1024, tiles_in_sequence=8)),   # the partial sums of a walk must fit the LDS
    # tiles that share an activation stage: as few as give at most 256 workgroups ...
    ((5120, 8, 5120), dict(matrix_core=2, tiles_per_wg=2, workgroups=160, split_k=2, steps_per_wave=5, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((8192, 16, 8192), dict(matrix_core=2, tiles_per_wg=2, workgroups=256, split_k=4)),
    ((10240, 8, 8192), dict(matrix_core=2, tiles_per_wg=4, workgroups=160, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((28672, 16, 8192), dict(matrix_core=2, tiles_per_wg=8, workgroups=224, split_k=1, variant=mg.MATRIX_CORE_LDS_STAGED)),
    # ... or, when that cannot be had, a count whose last round of 256 is well filled
    ((28672, 8, 8192), dict(matrix_core=2, tiles_per_wg=4, workgroups=448, variant=mg.MATRIX_CORE_LDS_STAGED)),
    ((18944, 8, 3584), dict(matrix_core=2, tiles_per_wg=2, workgroups=592, split_k=1, variant=mg.MATRIX_CORE_LDS_STAGED)),
    # an uneven k split is halved only while the workgroup keeps four waves
    ((4096, 8, 6656), dict(matrix_core=2, tiles_per_wg=1, split_k=4, steps_per_wave=4)),
    ((8192, 8, 6656), dict(matrix_core=2, tiles_per_wg=2, split_k=2, steps_per_wave=7)),
]


@pytest.mark.parametrize("shape,want", BUILTIN_PLANS,
                         ids=[f"{s[0]}x{s[2]}_m{s[1]}" + ("_lds_staged" if "variant" in w else "") for s, w in BUILTIN_PLANS])
def test_builtin_launch_rules_on_the_shapes_they_were_measured_on(shape, want):
    """variant: the rules of the named matrix-core kernel, on a shape that the k-stationary kernel now takes."""
    n_out, m_batch, k = shape
    want = dict(want)
    mg.set_default_plans(False)   # the rules themselves, without the built-in table of measured exceptions
    mg.set_matrix_core_variant(want.pop("variant", mg.MATRIX_CORE_AUTO))
    try:
        got = mg.query_launch(n_out, m_batch, k, 4, 128)
    finally:
        mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
        mg.set_default_plans(True)
    assert {key: got[key] for key in want} == want, got
    # every plan covers every tile and every k step, within the workgroup size the kernels allow
    tiles, ksteps = -(-n_out // 16), -(-k // 512)
    assert got["split_k"] * got["steps_per_wave"] >= ksteps > (got["split_k"] - 1) * got["steps_per_wave"]
    assert got["threads"] <= 1024 and got["threads"] % 64 == 0
    per_workgroup = got["tiles_per_wg"] * got["tiles_per_wave"] * got["tiles_in_sequence"]
    assert got["workgroups"] * per_workgroup >= tiles


def test_group_sizes_that_do_not_divide_the_k_step_stay_off_the_k_stationary_rule():
    """With one scale / zero lookup per block (groups of 96, 160, 192 ...) the k-stationary kernel measured 10-17 %
    behind the LDS-staged one (11008x3072 g96 at 4 rows 10.98 against 9.61 us; 28672x8064 g96 36.5 against 33.1;
    8192x6144 g192 12.3 against 10.8): the rule leaves such launches where they were; naming the kernel still works."""
    for n_out, rows, k, group in [(11008, 4, 3072, 96), (28672, 2, 8064, 96), (8192, 4, 6144, 192), (20480, 3, 5120, 160)]:
        assert mg.query_launch(n_out, rows, k, 4, 128 if k % 128 == 0 else 64)["matrix_core"] == 3, (n_out, k)
        assert mg.query_launch(n_out, rows, k, 4, group)["matrix_core"] in (0, 2), (n_out, k, group)
        mg.set_matrix_core_variant(mg.MATRIX_CORE_K_STATIONARY)
        try:
            assert mg.query_launch(n_out, rows, k, 4, group)["matrix_core"] == 3
        finally:
            mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
    # per-column mode passes the reduction length as its group: regular
    assert mg.query_launch(11008, 4, 4096, 4, 4096)["matrix_core"] == 3


def test_k_stationary_clauses_found_by_the_audits_of_random_shapes():
    q = lambda n, m, k: mg.query_launch(n, m, k, 4, 128)["matrix_core"]  # noqa: E731
    # tile counts that leave the LDS-staged kernel no grouping (1055 and 1088 tiles; 2275 at 16 staged rows)
    assert [q(16880, m, 5376) for m in (3, 5, 8)] == [3, 3, 3] and [q(17408, m, 8192) for m in (3, 8)] == [3, 3]
    assert q(36400, 16, 5376) == 3
    # walks of 4: up to 5 rows and 15 k steps; walks of 5 and more: also at 6-8 rows
    assert [q(15360, m, 6144) for m in (3, 5, 6, 8)] == [3, 3, 2, 2] and q(13312, 3, 8192) == 2
    assert [q(13584, m, 5632) for m in (3, 6, 8)] == [3, 3, 3]          # 11 k steps: up to 8 rows
    assert q(22944, 4, 7680) == 3                                        # walks of 6 at 3-4 rows too
    assert [q(22144, m, 7936) for m in (5, 6, 8)] == [3, 3, 3]
    # two rows: walks of 3 and more with 9-16 k steps, 2.5 tiles per compute unit with 6-8
    assert q(21024, 2, 7808) == 3 and q(8192, 2, 8192) == 0 and q(12288, 2, 3072) == 3 and q(12288, 2, 2560) == 0
    # 9-12 rows on walks of 2
    assert [q(5120, m, 5120) for m in (9, 12, 13, 16)] == [3, 3, 2, 2]
    # five waves on four SIMDs: not on walks of 4 and more
    assert q(26208, 3, 2176) == 2 and q(14240, 8, 2560) == 2 and q(6912, 3, 2432) == 3


def test_bf16_launch_rules_differ_where_they_were_measured_to():
    """The bfloat16 kernels are bound by arithmetic: no tile walks, no whole-k single-wave workgroups,
    no two-unit waves; at most 8 waves per workgroup."""
    q = lambda n, m, k: mg.query_launch(n, m, k, 4, 128, element="bf16")
    c5 = q(28672, 1, 8192)
    assert (c5["workgroups"], c5["split_k"], c5["tiles_in_sequence"]) == (1792, 4, 1), c5
    assert mg.query_launch(28672, 1, 8192, 4, 128)["tiles_in_sequence"] == 7       # fp16 walks 7 tiles
    mlp = q(13824, 1, 5120)
    assert mlp["split_k"] > 1 and mlp["steps_per_wave"] != 2, mlp
    assert mg.query_launch(13824, 1, 5120, 4, 128)["split_k"] == 1                 # fp16: whole-k waves
    assert q(28672, 2, 8192)["matrix_core"] == 0 and q(28672, 3, 8192)["matrix_core"] == 2   # 2 rows stay on the VALU kernel
    assert q(8192, 1, 8192)["workgroups"] == 256                                   # one tile per sequence: kept
    for n, m, k in [(4096, 1, 4096), (1024, 1, 8192), (22016, 1, 4096), (5120, 2, 5120), (4096, 16, 4096)]:
        assert q(n, m, k)["threads"] <= 512, (n, m, k)
        assert q(n, m, k)["matrix_core"] in (0, 2)                                 # no register-operand kernel for bf16


def test_int8_weights_keep_two_to_four_rows_on_the_valu_kernel():
    q = lambda n, m, k: mg.query_launch(n, m, k, 8, 128)["matrix_core"]
    assert [q(8192, m, 8192) for m in (2, 3, 4, 5)] == [0, 0, 0, 2]
    assert [q(4096, m, 11008) for m in (3, 4, 5)] == [0, 0, 2]
    assert [q(28672, m, 8192) for m in (2, 3, 4)] == [0, 2, 2]
    # ... unless the k-stationary kernel takes the launch: 8-16 k steps of 256, 3-8 rows, more tiles than compute units
    assert [q(8192, m, 4096) for m in (2, 3, 4, 8)] == [0, 3, 3, 3]
    assert q(28672, 3, 4096) == 3 and q(28672, 2, 4096) == 0 and q(8192, 4, 1536) == 0 and q(4096, 8, 4096) == 2
    # ... and at 9-16 rows wherever there are more tiles than compute units and the partial sums of a walk fit the LDS
    assert [q(8192, m, 4096) for m in (9, 12, 16)] == [3, 3, 3]
    assert q(11008, 16, 1024) == 3 and q(18944, 12, 3584) == 3
    assert q(4096, 12, 4096) == 2                     # at most one tile per compute unit
    assert q(32000, 16, 4096) == 2 and q(32000, 10, 4096) == 3 and q(50304, 16, 2048) == 2   # walks of 8 and 13 tiles
    assert q(8192, 12, 8192) == 2                     # 32 k steps of 256: more than a workgroup has waves


def test_default_plan_table_is_the_shipped_json_and_applies_to_256_compute_units_only():
    import json
    import os
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "..", "default_plans.json")
    with open(path) as f:
        table = json.load(f)
    assert table["format"] == 1 and mg.default_plan_count() == len(table["plans"]) >= 1
    kinds = {0: 0, 1: 0, 2: 1, 3: 2, 4: 3}   # MGEMV_KERNEL_* -> what query_launch reports as matrix_core
    for e in table["plans"]:
        key = (e["n_out"], e["m_batch"], e["k"], e["weight_bits"], e["group_size"])
        got = mg.query_launch(*key, element=e["element"], num_compute_units=256)
        mg.set_default_plans(False)
        try:
            rules = mg.query_launch(*key, element=e["element"], num_compute_units=256)
        finally:
            mg.set_default_plans(True)
        assert got != rules, "an entry that changes nothing has no business in the table"
        if e.get("split_k"):
            assert got["split_k"] == e["split_k"]
        if e.get("tiles_per_wg"):
            assert got["tiles_per_wg"] == e["tiles_per_wg"]
        if e.get("max_workgroups"):
            assert got["workgroups"] <= -(-e["max_workgroups"] // 8) * 8
        if e.get("kernel"):
            assert got["matrix_core"] == kinds[e["kernel"]]
        assert e["us"] < e["builtin_us"] * 0.98
        # ... and the gain was seen again on at least two separate leases, and the entry was never behind
        from mixed_gemv_amd import autotune
        assert autotune.confirmed(e), e.get("confirmations")
        # the entry covers the problem like any plan
        cov = mg.plan_coverage(*key, element=e["element"], num_compute_units=256)
        assert cov["tiles_miscovered"] == 0 and cov["bad_waves"] == 0
        # other device sizes, the other element type, a caller's table entry and any override: not this entry
        assert mg.query_launch(*key, element=e["element"], num_compute_units=128) == \
            _with_defaults_off(lambda: mg.query_launch(*key, element=e["element"], num_compute_units=128))
        other = "bf16" if e["element"] == "f16" else "f16"
        assert mg.query_launch(*key, element=other, num_compute_units=256) == \
            _with_defaults_off(lambda: mg.query_launch(*key, element=other, num_compute_units=256))
        mg.set_prefetch_stages(2)
        try:
            assert {k: v for k, v in mg.query_launch(*key, element=e["element"], num_compute_units=256).items()} == rules
        finally:
            mg.set_prefetch_stages(0)


def _with_defaults_off(fn):
    mg.set_default_plans(False)
    try:
        return fn()
    finally:
        mg.set_default_plans(True)


def test_an_entry_ships_only_after_two_confirmations():
    from mixed_gemv_amd import autotune
    assert not autotune.confirmed({})
    assert not autotune.confirmed({"confirmations": [3.1]})
    assert not autotune.confirmed({"confirmations": [3.1, 0.4, 1.9]})
    assert autotune.confirmed({"confirmations": [3.1, 0.4, 2.0]})
    assert not autotune.confirmed({"confirmations": [3.1, 2.4, -2.2]})      # behind once by as much as it gains
    assert autotune.confirmed({"confirmations": [5.0, 4.0]}, min_gain=0.04) and not autotune.confirmed({"confirmations": [5.0, 4.0]}, leases=3)


def test_the_library_is_loaded_behind_pytorch():
    """PyTorch brings its own HIP runtime; loaded in front of it, the library would bind to the system's runtime
    instead and know nothing of the tensors' memory.  The loader therefore imports torch first."""
    import subprocess
    import sys
    code = ("import sys, mixed_gemv_amd as mg; assert 'torch' not in sys.modules; mg.set_default_plans(True); "
            "assert 'torch' in sys.modules; print('ok')")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300,
                         cwd=os.path.join(os.path.dirname(__file__), ".."))
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stderr[-2000:]
