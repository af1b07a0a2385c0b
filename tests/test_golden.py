"""The committed vectors (tests/golden/gemv_cases.npz): the oracle and the library's host
utilities must reproduce them on the CPU, the HIP path on the GPU."""
import os

import numpy as np
import pytest

import mixed_gemv_amd as mg
import oracle as orc
from helpers import error_report

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemv_cases.npz")


def _cases():
    data = np.load(GOLDEN, allow_pickle=False)
    tags = sorted({key.split("/")[0] for key in data.files})
    return data, tags


DATA, TAGS = _cases()


def _get(tag, name):
    key = f"{tag}/{name}"
    return DATA[key] if key in DATA.files else None


@pytest.mark.parametrize("tag", TAGS)
def test_oracle_reproduces_golden(tag):
    n, k, bits, qop, g, mb = (int(v) for v in _get(tag, "meta"))
    zero = _get(tag, "zero_add")
    zero = zero.view(np.float16) if zero is not None else None
    bias = _get(tag, "bias")
    bias = bias.view(np.float16) if bias is not None else None
    dq = orc.dequantize(_get(tag, "w_raw"), _get(tag, "scale").view(np.float16), zero, n, k, g, qop, bits)
    assert np.array_equal(dq.view(np.uint16), _get(tag, "dequant"))
    y = orc.gemv(_get(tag, "w_raw"), _get(tag, "x").view(np.float16), _get(tag, "scale").view(np.float16), zero, bias,
                 n, mb, k, g, qop, bits)
    assert np.array_equal(y.view(np.uint16), _get(tag, "y"))
    zi = _get(tag, "zeros_i8")
    if zi is not None:  # the folded term in the file is what the library's folding produces
        folded = mg.ZeroPointPreprocessor.neg_zero_point_multiplies_scale(_get(tag, "scale").view(np.float16), zi)
        assert np.array_equal(folded.view(np.uint16), _get(tag, "zero_add"))


@pytest.mark.gpu
@pytest.mark.parametrize("tag", TAGS)
def test_hip_path_reproduces_golden(gpu, tag):
    import torch
    n, k, bits, qop, g, mb = (int(v) for v in _get(tag, "meta"))
    qt = mg.QuantType.W4_A16 if bits == 4 else mg.QuantType.W8_A16
    pre = mg.MixedGemvWeightPreprocessor.run(_get(tag, "w_raw"), (k, n), mg.LayoutType.kColumnMajor, qt)

    def dev(name):
        a = _get(tag, name)
        return torch.from_numpy(a.view(np.int16)).to(gpu) if a is not None else None

    w = torch.from_numpy(pre).to(gpu)
    x, scale, zero, bias = dev("x"), dev("scale"), dev("zero_add"), dev("bias")
    dq = torch.zeros((n, k), dtype=torch.int16, device=gpu)
    mg.dequantize(w, scale, zero, dq, n, k, g, qop, bits)
    y = torch.full((mb, n), 0x7E00, dtype=torch.int16, device=gpu)
    mg.device_gemv(w, x, scale, zero, bias, y, 1, n, mb, k, g, qop, bits)
    torch.cuda.synchronize()
    assert np.array_equal(dq.cpu().numpy().view(np.uint16), _get(tag, "dequant")), "dequantised weights must be bit-exact"
    got = y.cpu().numpy().view(np.float16)
    abs_err, rel_err, _ = error_report(got, _get(tag, "y").view(np.float16))
    assert rel_err <= 2e-3, (abs_err, rel_err)


# ---- bfloat16 vectors (tests/golden/gemv_cases_bf16.npz) ---------------------------------------

GOLDEN_BF16 = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemv_cases_bf16.npz")
DATA_B = np.load(GOLDEN_BF16, allow_pickle=False)
TAGS_B = sorted({key.split("/")[0] for key in DATA_B.files})


def _getb(tag, name):
    key = f"{tag}/{name}"
    return DATA_B[key] if key in DATA_B.files else None


@pytest.mark.parametrize("tag", TAGS_B)
def test_oracle_reproduces_golden_bf16(tag):
    n, k, bits, qop, g, mb = (int(v) for v in _getb(tag, "meta"))
    dq = orc.dequantize_bf16(_getb(tag, "w_raw"), _getb(tag, "scale"), _getb(tag, "zero_add"), n, k, g, qop, bits)
    assert np.array_equal(dq, _getb(tag, "dequant"))
    y = orc.gemv_bf16(_getb(tag, "w_raw"), _getb(tag, "x"), _getb(tag, "scale"), _getb(tag, "zero_add"),
                      _getb(tag, "bias"), n, mb, k, g, qop, bits)
    assert np.array_equal(y, _getb(tag, "y"))
    zi = _getb(tag, "zeros_i8")
    if zi is not None:
        folded = mg.ZeroPointPreprocessor.neg_zero_point_multiplies_scale(_getb(tag, "scale"), zi, element="bf16")
        assert np.array_equal(folded, _getb(tag, "zero_add"))


@pytest.mark.gpu
@pytest.mark.parametrize("tag", TAGS_B)
def test_hip_path_reproduces_golden_bf16(gpu, tag):
    import torch
    from helpers import bf16_ulp_report
    n, k, bits, qop, g, mb = (int(v) for v in _getb(tag, "meta"))
    qt = mg.QuantType.W4_A16 if bits == 4 else mg.QuantType.W8_A16
    pre = mg.MixedGemvWeightPreprocessor.run(_getb(tag, "w_raw"), (k, n), mg.LayoutType.kColumnMajor, qt)

    def dev(name):
        a = _getb(tag, name)
        return torch.from_numpy(a.view(np.int16)).to(gpu) if a is not None else None

    w = torch.from_numpy(pre).to(gpu)
    x, scale, zero, bias = dev("x"), dev("scale"), dev("zero_add"), dev("bias")
    dq = torch.zeros((n, k), dtype=torch.int16, device=gpu)
    mg.dequantize(w, scale, zero, dq, n, k, g, qop, bits, element="bf16")
    y = torch.full((mb, n), 0x7FC0, dtype=torch.int16, device=gpu)
    mg.device_gemv(w, x, scale, zero, bias, y, 1, n, mb, k, g, qop, bits, element="bf16")
    torch.cuda.synchronize()
    assert np.array_equal(dq.cpu().numpy().view(np.uint16), _getb(tag, "dequant")), "dequantised weights must be bit-exact"
    ulp, differing = bf16_ulp_report(y.cpu().numpy().view(np.uint16), _getb(tag, "y"))
    assert ulp <= 1.0 + 1e-6 and differing <= 0.02, (ulp, differing)
