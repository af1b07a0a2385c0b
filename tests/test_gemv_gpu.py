"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle.

Bars: dequantised weights bit-exact; fp16 outputs within max relative error 2e-3
(denominator max(|ref|, 2^-10 rms(ref))).
"""
import numpy as np
import pytest

from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, DeviceProblem, Problem, error_report

pytestmark = pytest.mark.gpu

REL_TOL = 2e-3

SMALL = [
    # tag, n_out, k, bits, quant_op, group, m_batch, bias
    ("s_i4_sz_g128", 256, 1024, 4, SCALE_AND_ZEROS, 128, 1, False),
    ("s_i4_sz_g64", 256, 1024, 4, SCALE_AND_ZEROS, 64, 1, True),
    ("s_i4_s_g128", 128, 2048, 4, SCALE_ONLY, 128, 1, True),
    ("s_i4_col", 128, 1024, 4, PER_COLUMN, 0, 1, False),
    ("s_i8_col", 256, 1024, 8, PER_COLUMN, 0, 1, True),
    ("s_i8_sz_g64", 128, 512, 8, SCALE_AND_ZEROS, 64, 1, False),
    ("s_i8_s_g128", 128, 512, 8, SCALE_ONLY, 128, 2, True),
    ("s_i4_ragged", 100, 1120, 4, SCALE_AND_ZEROS, 160, 1, True),   # n_out % 16 != 0, k % 512 != 0, odd group
    ("s_i4_mb3", 64, 1536, 4, SCALE_AND_ZEROS, 128, 3, True),
    ("s_i4_mb7", 64, 1024, 4, SCALE_AND_ZEROS, 64, 7, False),
]


@pytest.mark.parametrize("cfg", SMALL, ids=[c[0] for c in SMALL])
def test_small_parity(gpu, cfg):
    tag, n_out, k, bits, qop, g, mb, bias = cfg
    prob = Problem(tag, n_out, k, bits, qop, g, m_batch=mb, bias=bias)
    dev = DeviceProblem(prob, gpu)
    dq = dev.dequant()
    ref_dq = prob.oracle_dequant()
    mism = int((dq.view(np.uint16) != ref_dq.view(np.uint16)).sum())
    assert mism == 0, f"{mism} dequantised weights differ"
    y = dev.run()
    ref = prob.oracle_gemv()
    abs_err, rel_err, floor = error_report(y, ref)
    print(f"{tag}: max_abs={abs_err:.3e} max_rel={rel_err:.3e} floor={floor:.3e}")
    assert np.isfinite(y.astype(np.float32)).all()
    assert rel_err <= REL_TOL
