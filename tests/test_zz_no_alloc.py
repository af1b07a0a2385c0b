"""The allocation-free host-pointer entry (mgemv_host_gemv_static): same arguments and, bit for bit,
the same results as mgemv_host_gemv, with its device staging in a static device array.  Two calls in
a row, the second on a smaller problem that leaves most of the first call's data in the array; then a
larger one again, other modes, and the size limit.  Through the C-ABI (ctypes)."""
import numpy as np
import pytest

import mixed_gemv_amd as mg
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, Problem, error_report

pytestmark = pytest.mark.gpu
REL_TOL = 2e-3  # fp16 outputs within max relative error 2e-3 of the CPU oracle (denominator floor: helpers.error_report)


def both(prob, bias=True):
    args = (prob.w_raw, prob.x, prob.scale, prob.zeros_i8, prob.bias if bias else None, 1, prob.n_out, prob.m_batch,
            prob.k, prob.group_size, prob.quant_op, prob.bits)
    return mg.host_gemv(*args), mg.host_gemv(*args, static_scratch=True)


def test_static_scratch_entry_matches_the_allocating_one_on_consecutive_calls(gpu):
    big = Problem("na_big", 4096, 4096, 4, SCALE_AND_ZEROS, 128, bias=True, scale_range=(0.1, 0.3), zero_kind="int8")
    small = Problem("na_small", 100, 1120, 4, SCALE_AND_ZEROS, 160, bias=True, scale_range=(0.1, 0.3), zero_kind="int8")
    rows = Problem("na_rows", 512, 2048, 4, SCALE_ONLY, 64, m_batch=3, bias=True, scale_range=(0.1, 0.3), zero_kind="int8")
    i8 = Problem("na_i8", 1024, 1024, 8, PER_COLUMN, 0, bias=False, scale_range=(0.01, 0.03), zero_kind="int8")
    assert mg.static_scratch_bytes_needed(4096, 1, 4096, 128, has_bias=True) <= mg.STATIC_SCRATCH_BYTES
    for prob in (big, small, big, rows, i8, small):   # the second call is the smaller one; later ones grow and shrink again
        want, got = both(prob, bias=prob.bias is not None)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), prob.tag
        _, rel, _ = error_report(got, prob.oracle_gemv(threads=8, literal_int8_zero=True))
        assert rel <= REL_TOL, prob.tag


def test_static_scratch_entry_refuses_what_does_not_fit(gpu):
    n_out, k = 8192, 8192
    assert mg.static_scratch_bytes_needed(n_out, 1, k, 128) > mg.STATIC_SCRATCH_BYTES
    w = np.zeros(n_out * k // 2, dtype=np.uint8)
    x = np.zeros(k, dtype=np.float16)
    s = np.ones((k // 128, n_out), dtype=np.float16)
    z = np.zeros((k // 128, n_out), dtype=np.int8)
    with pytest.raises(mg.MixedGemvError) as err:
        mg.host_gemv(w, x, s, z, None, 1, n_out, 1, k, 128, static_scratch=True)
    assert err.value.status == 16 and "static scratch" in str(err.value)
    # and the call before and after it are unaffected
    small = Problem("na_after", 256, 1024, 4, SCALE_AND_ZEROS, 128, bias=True, scale_range=(0.1, 0.3), zero_kind="int8")
    want, got = both(small)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_static_scratch_entry_from_several_threads(gpu):
    """All callers share one device array and one host array; the library serialises them.  Four threads,
    different problems, three calls each: every result equals the allocating entry's."""
    import threading
    probs = [Problem(f"na_t{i}", 128 * (i + 1), 1024 + 512 * i, 4, SCALE_AND_ZEROS, 128, bias=True, scale_range=(0.1, 0.3),
                     zero_kind="int8") for i in range(4)]
    want = [mg.host_gemv(p.w_raw, p.x, p.scale, p.zeros_i8, p.bias, 1, p.n_out, 1, p.k, p.group_size, p.quant_op, p.bits)
            for p in probs]
    failures = []

    def worker(i):
        p = probs[i]
        for _ in range(3):
            got = mg.host_gemv(p.w_raw, p.x, p.scale, p.zeros_i8, p.bias, 1, p.n_out, 1, p.k, p.group_size, p.quant_op,
                               p.bits, static_scratch=True)
            if not np.array_equal(got.view(np.uint16), want[i].view(np.uint16)):
                failures.append(i)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures
