"""An independent numpy restatement of the reference arithmetic, used only to cross-check the
C oracle on small cases.  numpy's float16 operations are correctly rounded binary16
operations computed by different code (numpy's half implementation)."""
import numpy as np


def unpack_int4(packed):
    p = np.asarray(packed, dtype=np.uint8).reshape(-1)
    lo = (p & 0xF).astype(np.int16)
    hi = (p >> 4).astype(np.int16)
    lo = np.where(lo >= 8, lo - 16, lo)
    hi = np.where(hi >= 8, hi - 16, hi)
    out = np.empty(p.size * 2, dtype=np.int8)
    out[0::2] = lo  # utils/vector_subbyte.h:150-156: element i in bits 4*(i%2) of byte i/2
    out[1::2] = hi
    return out


def dequantize(q, scale, zero, group_size, int8_zero):
    """q: int [n][k]; scale [groups][n] float16; zero: int8 or float16 [groups][n] or None."""
    n, k = q.shape
    g = np.arange(k) // group_size                     # host/mixed_gemv.h:88
    s = scale[g, :].T.astype(np.float16)               # [n][k]
    with np.errstate(over="ignore", invalid="ignore"):
        p = (q.astype(np.float16) * s).astype(np.float16)   # host/mixed_gemv.h:95-96, first rounding
        if zero is None:
            return p
        if int8_zero:
            sz = -(s * zero[g, :].T.astype(np.float16)).astype(np.float16)  # host/mixed_gemv.h:92-93
        else:
            sz = zero[g, :].T.astype(np.float16)                             # warp_dequantizer.h:57
        return (p + sz).astype(np.float16)


def gemv(dq, x, bias):
    """dq [n][k] float16, x [m][k] float16; fp32 accumulation in ascending k (host/mixed_gemv.h:84-98)."""
    n, k = dq.shape
    m = x.shape[0]
    out = np.empty((m, n), dtype=np.float16)
    d32 = dq.astype(np.float32)
    for b in range(m):
        acc = np.zeros(n, dtype=np.float32)
        xb = x[b].astype(np.float32)
        with np.errstate(over="ignore", invalid="ignore"):
            for kk in range(k):
                acc = (acc + (xb[kk] * d32[:, kk]).astype(np.float32)).astype(np.float32)
            if bias is not None:
                acc = (acc + bias.astype(np.float32)).astype(np.float32)   # host/mixed_gemv.h:102-103
            out[b] = acc.astype(np.float16)
    return out
