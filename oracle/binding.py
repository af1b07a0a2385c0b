"""ctypes binding of the plain-C oracle (oracle/mgemv_oracle.c)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmgemv_oracle.so")

ZERO_NONE, ZERO_INT8, ZERO_FOLDED_F16 = 0, 1, 2
PER_COLUMN_SCALE_ONLY, FINEGRAINED_SCALE_ONLY, FINEGRAINED_SCALE_AND_ZEROS = 1, 2, 3

_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        h = ctypes.CDLL(LIB_PATH)
        c = ctypes
        vp = c.c_void_p
        h.orc_f16_to_f32.restype = c.c_float
        h.orc_f16_to_f32.argtypes = [c.c_uint16]
        h.orc_f32_to_f16.restype = c.c_uint16
        h.orc_f32_to_f16.argtypes = [c.c_float]
        for name in ("orc_h_mul", "orc_h_add"):
            getattr(h, name).restype = c.c_uint16
            getattr(h, name).argtypes = [c.c_uint16, c.c_uint16]
        h.orc_h_fma.restype = c.c_uint16
        h.orc_h_fma.argtypes = [c.c_uint16] * 3
        for name, nargs in (("orc_f16_to_f32_n", 2), ("orc_f32_to_f16_n", 2), ("orc_h_mul_n", 3), ("orc_h_add_n", 3),
                            ("orc_h_fma_n", 4)):
            getattr(h, name).argtypes = [vp] * nargs + [c.c_size_t]
        h.orc_pack_int4.argtypes = [vp, vp, c.c_size_t]
        h.orc_unpack_int4.argtypes = [vp, vp, c.c_size_t]
        h.orc_fold_zero_points.argtypes = [vp, vp, vp, c.c_size_t]
        h.orc_ref_preprocess_int4.restype = c.c_int
        h.orc_ref_preprocess_int4.argtypes = [vp, vp, c.c_size_t, c.c_size_t]
        h.orc_ref_convert_u4x8.argtypes = [vp, c.c_uint32]
        h.orc_ref_convert_u8x4.argtypes = [vp, c.c_uint32]
        h.orc_dequantize.restype = c.c_int
        h.orc_dequantize.argtypes = [vp, vp, vp, vp] + [c.c_int] * 6
        h.orc_gemv.restype = c.c_int
        h.orc_gemv.argtypes = [vp, vp, vp, vp, vp, vp] + [c.c_int] * 8
        h.orc_dequantize_bf16.restype = c.c_int
        h.orc_dequantize_bf16.argtypes = h.orc_dequantize.argtypes
        h.orc_gemv_bf16.restype = c.c_int
        h.orc_gemv_bf16.argtypes = h.orc_gemv.argtypes
        h.orc_fold_zero_points_bf16.argtypes = [vp, vp, vp, c.c_size_t]
        h.orc_bf16_to_f32.restype = c.c_float
        h.orc_bf16_to_f32.argtypes = [c.c_uint16]
        h.orc_f32_to_bf16.restype = c.c_uint16
        h.orc_f32_to_bf16.argtypes = [c.c_float]
        for name in ("orc_bf16_mul", "orc_bf16_add"):
            getattr(h, name).restype = c.c_uint16
            getattr(h, name).argtypes = [c.c_uint16, c.c_uint16]
        for name, nargs in (("orc_bf16_to_f32_n", 2), ("orc_f32_to_bf16_n", 2), ("orc_bf16_mul_n", 3),
                            ("orc_bf16_add_n", 3)):
            getattr(h, name).argtypes = [vp] * nargs + [c.c_size_t]
        h.orc_max_threads.restype = c.c_int
        h.orc_fill_int8.argtypes = [vp, c.c_size_t, c.c_uint64, c.c_int, c.c_int]
        h.orc_fill_uniform_f16.argtypes = [vp, c.c_size_t, c.c_uint64, c.c_float, c.c_float]
        h.orc_fill_normal_clipped_f16.argtypes = [vp, c.c_size_t, c.c_uint64, c.c_float]
        _lib = h
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _u16(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


# ---- scalars ----------------------------------------------------------------------------

def f16_to_f32(bits):
    return float(lib().orc_f16_to_f32(int(bits)))


def f32_to_f16(value):
    return int(lib().orc_f32_to_f16(float(value)))


def h_mul(a, b):
    return int(lib().orc_h_mul(int(a), int(b)))


def h_add(a, b):
    return int(lib().orc_h_add(int(a), int(b)))


def h_fma(a, b, c):
    return int(lib().orc_h_fma(int(a), int(b), int(c)))


def f16_to_f32_array(bits):
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().orc_f16_to_f32_n(_p(out), _p(b), b.size)
    return out


def f32_to_f16_array(values):
    v = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(v.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_n(_p(out), _p(v), v.size)
    return out


def _binary(fn, a, b):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    assert a.shape == b.shape
    out = np.empty(a.shape, dtype=np.uint16)
    fn(_p(out), _p(a), _p(b), a.size)
    return out


def h_mul_array(a, b):
    return _binary(lib().orc_h_mul_n, a, b)


def h_add_array(a, b):
    return _binary(lib().orc_h_add_n, a, b)


def h_fma_array(a, b, c):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    c = np.ascontiguousarray(c, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().orc_h_fma_n(_p(out), _p(a), _p(b), _p(c), a.size)
    return out


# ---- bfloat16 (bit patterns travel as uint16 arrays; numpy has no such dtype) --------------

def bf16_to_f32_array(bits):
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().orc_bf16_to_f32_n(_p(out), _p(b), b.size)
    return out


def f32_to_bf16_array(values):
    v = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(v.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16_n(_p(out), _p(v), v.size)
    return out


def bf16_mul_array(a, b):
    return _binary(lib().orc_bf16_mul_n, a, b)


def bf16_add_array(a, b):
    return _binary(lib().orc_bf16_add_n, a, b)


def fold_zero_points_bf16(scales, zeros):
    s = np.ascontiguousarray(scales, dtype=np.uint16)
    z = np.ascontiguousarray(zeros, dtype=np.int8)
    out = np.empty(s.shape, dtype=np.uint16)
    lib().orc_fold_zero_points_bf16(_p(out), _p(s), _p(z), s.size)
    return out


def dequantize_bf16(W, scale, zero, n_out, k, group_size, quant_op, bits):
    """As dequantize, with bf16 bit patterns (uint16) for scale / folded zero / result."""
    W = np.ascontiguousarray(W)
    s = np.ascontiguousarray(scale, dtype=np.uint16)
    z, zk = _zero_args(zero, quant_op)
    out = np.empty((n_out, k), dtype=np.uint16)
    rc = lib().orc_dequantize_bf16(_p(out), _p(W), _p(s), _p(z), zk, n_out, k, group_size, quant_op, bits)
    assert rc == 0
    return out


def gemv_bf16(W, x, scale, zero, bias, n_out, m_batch, k, group_size, quant_op, bits, threads=1):
    """HOST_CHECK GEMV with bfloat16 elements; every 16-bit operand and the result are uint16 bit patterns."""
    W = np.ascontiguousarray(W)
    xx = np.ascontiguousarray(x, dtype=np.uint16)
    s = np.ascontiguousarray(scale, dtype=np.uint16)
    z, zk = _zero_args(zero, quant_op)
    b = np.ascontiguousarray(bias, dtype=np.uint16) if bias is not None else None
    y = np.empty((m_batch, n_out), dtype=np.uint16)
    rc = lib().orc_gemv_bf16(_p(y), _p(W), _p(xx), _p(s), _p(z), _p(b), zk, n_out, m_batch, k, group_size, quant_op,
                             bits, threads)
    assert rc == 0
    return y


# ---- host utilities ----------------------------------------------------------------------

def pack_int4(unpacked):
    u = np.ascontiguousarray(unpacked, dtype=np.int8).reshape(-1)
    out = np.empty(u.size // 2, dtype=np.uint8)
    lib().orc_pack_int4(_p(out), _p(u), u.size)
    return out


def unpack_int4(packed):
    pk = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    out = np.empty(pk.size * 2, dtype=np.int8)
    lib().orc_unpack_int4(_p(out), _p(pk), pk.size)
    return out


def fold_zero_points(scales, zeros):
    s = _u16(scales)
    z = np.ascontiguousarray(zeros, dtype=np.int8)
    out = np.empty(s.shape, dtype=np.uint16)
    lib().orc_fold_zero_points(_p(out), _p(s), _p(z), s.size)
    return out.view(np.float16)


def ref_preprocess_int4(packed, rows, cols):
    src = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    out = np.empty_like(src)
    rc = lib().orc_ref_preprocess_int4(_p(out), _p(src), rows, cols)
    if rc:
        raise ValueError("rows % 4 or cols % 8")
    return out


def ref_convert_u4x8(word):
    out = np.empty(8, dtype=np.uint16)
    lib().orc_ref_convert_u4x8(_p(out), int(word))
    return out.view(np.float16)


def ref_convert_u8x4(word):
    out = np.empty(4, dtype=np.uint16)
    lib().orc_ref_convert_u8x4(_p(out), int(word))
    return out.view(np.float16)


# ---- the path ----------------------------------------------------------------------------

def _zero_args(zero, quant_op):
    if zero is None or quant_op != FINEGRAINED_SCALE_AND_ZEROS:
        return None, ZERO_NONE
    z = np.ascontiguousarray(zero)
    if z.dtype == np.int8:
        return z, ZERO_INT8
    return _u16(z), ZERO_FOLDED_F16


def dequantize(W, scale, zero, n_out, k, group_size, quant_op, bits):
    """W: raw weights [n_out][k] (int4 packed uint8, or int8).  Returns float16 [n_out][k]."""
    W = np.ascontiguousarray(W)
    s = _u16(scale)
    z, zk = _zero_args(zero, quant_op)
    out = np.empty((n_out, k), dtype=np.uint16)
    rc = lib().orc_dequantize(_p(out), _p(W), _p(s), _p(z), zk, n_out, k, group_size, quant_op, bits)
    assert rc == 0
    return out.view(np.float16)


def gemv(W, x, scale, zero, bias, n_out, m_batch, k, group_size, quant_op, bits, threads=1):
    """HOST_CHECK GEMV.  x: [m_batch][k] fp16.  Returns float16 [m_batch][n_out]."""
    W = np.ascontiguousarray(W)
    xx = _u16(x)
    s = _u16(scale)
    z, zk = _zero_args(zero, quant_op)
    b = _u16(bias) if bias is not None else None
    y = np.empty((m_batch, n_out), dtype=np.uint16)
    rc = lib().orc_gemv(_p(y), _p(W), _p(xx), _p(s), _p(z), _p(b), zk, n_out, m_batch, k, group_size, quant_op,
                        bits, threads)
    assert rc == 0
    return y.view(np.float16)


def max_threads():
    return int(lib().orc_max_threads())


# ---- seeded inputs -----------------------------------------------------------------------

def fill_int8(n, seed, lo, hi):
    out = np.empty(n, dtype=np.int8)
    lib().orc_fill_int8(_p(out), n, seed, lo, hi)
    return out


def fill_uniform_f16(n, seed, lo, hi):
    out = np.empty(n, dtype=np.uint16)
    lib().orc_fill_uniform_f16(_p(out), n, seed, lo, hi)
    return out.view(np.float16)


def fill_normal_clipped_f16(n, seed, clip=4.0):
    out = np.empty(n, dtype=np.uint16)
    lib().orc_fill_normal_clipped_f16(_p(out), n, seed, clip)
    return out.view(np.float16)
