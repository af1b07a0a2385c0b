"""The rest of the drop-in boundary on the GPU, all through the C-ABI: the HOST_CHECK-shaped entry
(host/mixed_gemv.h:60-70), the Arguments-struct entry with the epilogue's alpha / beta
(gemv/device/gemv_adaptor.h:114-178), reductions that are a multiple of 8 but not of a 128-bit
chunk (utils/preprocess.h:324-327), and weights preprocessed from row-major input
(utils/preprocess.h:507-511)."""
import numpy as np
import pytest

import mixed_gemv_amd as mg
import oracle as orc
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, DeviceProblem, Problem, error_report

pytestmark = pytest.mark.gpu
REL_TOL = 2e-3  # fp16 outputs within max relative error 2e-3 of the CPU oracle (denominator floor: helpers.error_report)


@pytest.mark.parametrize("tag,n_out,k,bits,qop,g,m_batch,bias", [
    ("h_i4_sz", 512, 2048, 4, SCALE_AND_ZEROS, 128, 1, True),     # the one instantiation the reference defines (host/mixed_gemv.h:23-42)
    ("h_i4_sz_nobias", 100, 1120, 4, SCALE_AND_ZEROS, 160, 1, False),
    ("h_i4_sz_rows", 256, 1024, 4, SCALE_AND_ZEROS, 64, 3, True),
    ("h_i4_s", 128, 1024, 4, SCALE_ONLY, 128, 1, True),
    ("h_i8_col", 256, 1024, 8, PER_COLUMN, 0, 1, True),
])
def test_host_gemv_is_the_host_check_call_site_on_the_gpu(gpu, tag, n_out, k, bits, qop, g, m_batch, bias):
    """Un-preprocessed weights and int8 zero points in, result out: against the oracle's literal
    int8-zero path (host/mixed_gemv.h:92-96 as written)."""
    prob = Problem(tag, n_out, k, bits, qop, g, m_batch=m_batch, bias=bias, scale_range=(0.1, 0.3), zero_kind="int8")
    y = mg.host_gemv(prob.w_raw, prob.x, prob.scale, prob.zeros_i8, prob.bias, 1, n_out, m_batch, k, prob.group_size,
                     qop, bits)
    ref = prob.oracle_gemv(threads=8, literal_int8_zero=True)
    _, rel, _ = error_report(y, ref)
    assert rel <= REL_TOL
    # the same numbers as the device entry fed by hand
    dev = DeviceProblem(prob, gpu)
    assert np.array_equal(dev.run().view(np.uint16), y.view(np.uint16))


def _run_arguments(dev, prob, alpha=1.0, beta=1.0, leading_dims=None):
    import torch
    dev.y.fill_(0x7e00)
    mg.gemv_arguments(dev.w, dev.x, dev.scale, dev.zero, dev.bias, dev.y, prob.n_out, prob.m_batch, prob.k,
                      prob.group_size, prob.quant_op, prob.bits, alpha=alpha, beta=beta, leading_dims=leading_dims,
                      element=prob.element)
    torch.cuda.synchronize()
    return dev.y.cpu().numpy().view(np.float16)


@pytest.mark.parametrize("m_batch", [1, 3, 8])   # VALU kernel, VALU with several rows, matrix cores
def test_arguments_entry_alpha_beta(gpu, m_batch):
    prob = Problem("a_ab", 256, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=m_batch, bias=True, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    plain = dev.run().copy()
    # alpha = beta = 1 with the reference's own leading dimensions (mixed_gemv_test.cu:136-140) is the plain entry, bit for bit
    lds = (4 * prob.k, prob.k if m_batch > 1 else 0, prob.n_out, prob.n_out, prob.n_out, prob.n_out)
    assert np.array_equal(_run_arguments(dev, prob, leading_dims=lds).view(np.uint16), plain.view(np.uint16))
    # beta = 0 drops the bias: equals the launch without one
    nobias = DeviceProblem(Problem("a_ab", 256, 2048, 4, SCALE_AND_ZEROS, 128, m_batch=m_batch, bias=False,
                                   x_dist="normal"), gpu)
    acc16 = nobias.run().copy()
    assert np.array_equal(_run_arguments(dev, prob, beta=0.0).view(np.uint16), acc16.view(np.uint16))
    # a power of two commutes with the final rounding (no result here is subnormal after halving)
    half = _run_arguments(dev, prob, alpha=0.5, beta=0.0)
    big = np.abs(acc16.astype(np.float32)) >= 2.0 ** -13
    assert np.array_equal(half[big].view(np.uint16), (acc16[big].astype(np.float32) * 0.5).astype(np.float16).view(np.uint16))
    # general alpha, beta: alpha * acc + beta * bias with one rounding; acc16 is acc rounded to fp16, so allow its half ulp
    got = _run_arguments(dev, prob, alpha=-1.75, beta=3.0).astype(np.float64)
    want = -1.75 * acc16.astype(np.float64) + 3.0 * prob.bias.astype(np.float64)[None, :]
    tol = 2.0 ** -10 * (1.75 * np.abs(acc16.astype(np.float64)) + np.abs(want)) + 2.0 ** -24
    assert np.all(np.abs(got - want) <= tol)


@pytest.mark.parametrize("element", ["f16", "bf16"])
def test_arguments_entry_batched_with_strides_and_epilogue(gpu, element):
    """The whole argument struct at once (gemv/device/gemv_adaptor.h:114-178): three problems per launch
    through their batch strides, either element type, alpha = 2 and beta = 0.5.  Doubling commutes with
    the final rounding of both types (no result here is near overflow), so the launch must equal, bit for
    bit, twice the accumulator-only result plus the exactly halved bias whenever that sum is exact; it is
    checked against the plain batched entry through the closed form for alpha alone, and against fp64
    within half an ulp for both."""
    import torch
    e, n_out, k, g = 3, 96, 1536, 128
    probs = [Problem(f"argb{i}", n_out, k, 4, SCALE_AND_ZEROS, g, bias=True, x_dist="normal", element=element)
             for i in range(e)]
    raw = np.concatenate([p.w_raw for p in probs])
    pre = mg.MixedGemvWeightPreprocessor.run(raw, (e, k, n_out), mg.LayoutType.kColumnMajor, mg.QuantType.W4_A16)
    one = mg.preprocessed_size((k, n_out), mg.QuantType.W4_A16)

    def stack(name):
        return torch.from_numpy(np.stack([np.asarray(getattr(p, name)).view(np.uint16) for p in probs]).view(np.int16)).to(gpu)

    w = torch.from_numpy(pre).to(gpu)
    scale, zero, bias = stack("scale"), stack("zero_add"), stack("bias")
    x = torch.from_numpy(np.asarray(probs[0].x).view(np.uint16).view(np.int16)).to(gpu)
    y = torch.full((e, n_out), 0x7E00, dtype=torch.int16, device=gpu)
    strides = (one, 0, (k // g) * n_out, n_out, n_out)

    def run(alpha, beta, with_bias=True):
        y.fill_(0x7E00)
        mg.gemv_arguments(w, x, scale, zero, bias if with_bias else None, y, n_out, 1, k, g, SCALE_AND_ZEROS, 4,
                          alpha=alpha, beta=beta, batch_count=e, batch_strides=strides, element=element)
        torch.cuda.synchronize()
        return y.cpu().numpy().view(np.uint16).copy()

    def to_f64(bits):
        if element == "bf16":
            return orc.bf16_to_f32_array(bits).astype(np.float64)
        return bits.view(np.float16).astype(np.float64)

    # alpha = beta = 1 is the batched entry, bit for bit
    y.fill_(0x7E00)
    mg.device_gemv(w, x, scale, zero, bias, y, e, n_out, 1, k, g, SCALE_AND_ZEROS, 4, batch_strides=strides, element=element)
    torch.cuda.synchronize()
    assert np.array_equal(run(1.0, 1.0), y.cpu().numpy().view(np.uint16))
    # alpha = 2 without a bias: exactly twice the accumulator-only result
    acc = run(1.0, 0.0, with_bias=False)
    assert np.array_equal(to_f64(run(2.0, 0.0, with_bias=False)), 2.0 * to_f64(acc))
    # alpha = 2, beta = 0.5: one rounding of 2 acc + bias / 2; acc is only known rounded, so allow its ulp
    got = to_f64(run(2.0, 0.5))
    bias64 = to_f64(np.stack([np.asarray(p.bias).view(np.uint16) for p in probs]))
    want = 2.0 * to_f64(acc) + 0.5 * bias64
    ulp = 2.0 ** (-7 if element == "bf16" else -10)
    assert np.all(np.abs(got - want) <= ulp * (2.0 * np.abs(to_f64(acc)) + np.abs(want)) + 2.0 ** -24)


def test_arguments_entry_bias_term_alone_is_exact(gpu):
    """x = 0: y = fp16(beta * bias) exactly (epilogue/threadblock/epilogue.h:64)."""
    import torch
    prob = Problem("a_bias", 128, 1024, 4, SCALE_AND_ZEROS, 128, bias=True)
    dev = DeviceProblem(prob, gpu)
    dev.x = torch.zeros_like(dev.x)
    for alpha, beta in ((1.0, 1.0), (5.0, 0.37), (0.0, -2.0)):
        y = _run_arguments(dev, prob, alpha=alpha, beta=beta)[0]
        want = (np.float32(beta) * prob.bias.astype(np.float32)).astype(np.float16)
        assert np.array_equal(y.view(np.uint16), want.view(np.uint16)), (alpha, beta)


@pytest.mark.parametrize("bits,k", [(4, 4104), (4, 520), (4, 8), (8, 1048), (8, 264)])
@pytest.mark.parametrize("m_batch", [1, 4, 8])
def test_reduction_length_a_multiple_of_8_only(gpu, bits, k, m_batch):
    """Per-column mode with k % 8 == 0 but not a whole 128-bit chunk per row: the preprocessor pads
    the last chunk, the kernels never multiply the padding by a non-zero activation."""
    prob = Problem(f"k8_{bits}_{k}", 96, k, bits, PER_COLUMN, 0, m_batch=m_batch, bias=True, x_dist="normal")
    dev = DeviceProblem(prob, gpu)
    assert np.array_equal(dev.dequant().view(np.uint16), prob.oracle_dequant().view(np.uint16))
    y = dev.run()
    _, rel, _ = error_report(y, prob.oracle_gemv(threads=8))
    assert rel <= REL_TOL


@pytest.mark.parametrize("bits,k", [(4, 4104), (4, 520), (4, 8), (8, 264)])
@pytest.mark.parametrize("m_batch", [5, 8, 16])
def test_reduction_length_a_multiple_of_8_only_register_operand_kernel(gpu, bits, k, m_batch):
    """The same through the register-operand matrix-core kernel, which loads its activation operand
    in 8-element pieces of its own: a single tile (the only shape that kernel serves by itself),
    and a larger matrix with the kernel forced."""
    for n_out, force in ((16, False), (96, True)):
        prob = Problem(f"k8r_{bits}_{k}", n_out, k, bits, PER_COLUMN, 0, m_batch=m_batch, bias=True, x_dist="normal")
        dev = DeviceProblem(prob, gpu)
        try:
            if force:
                mg.set_matrix_core_variant(mg.MATRIX_CORE_REGISTER_OPERAND)
            assert mg.query_launch(n_out, m_batch, k, bits)["matrix_core"] == 1
            y = dev.run()
        finally:
            mg.set_matrix_core_variant(mg.MATRIX_CORE_AUTO)
        _, rel, _ = error_report(y, prob.oracle_gemv(threads=8))
        assert rel <= REL_TOL, (n_out, rel)


@pytest.mark.parametrize("bits,qop,g", [(4, SCALE_AND_ZEROS, 128), (8, PER_COLUMN, 0)])
def test_weights_preprocessed_from_row_major_input(gpu, bits, qop, g):
    """utils/preprocess.h:507-511: a [k][n_out] row-major matrix is transposed first.  The buffer the
    kernels consume must be the one the column-major route produces, and the GEMV over it must pass."""
    import torch
    n_out, k = 320, 1536
    prob = Problem(f"rm_{bits}", n_out, k, bits, qop, g, bias=True)
    q = prob.q.reshape(n_out, k)
    qt = mg.QuantType.W4_A16 if bits == 4 else mg.QuantType.W8_A16
    q_rm = np.ascontiguousarray(q.T)                                   # [k][n_out]
    raw_rm = orc.pack_int4(q_rm.reshape(-1)) if bits == 4 else q_rm.view(np.uint8).reshape(-1)
    pre = mg.MixedGemvWeightPreprocessor.run(raw_rm, (k, n_out), mg.LayoutType.kRowMajor, qt)
    dev = DeviceProblem(prob, gpu)
    assert np.array_equal(pre, dev.w.cpu().numpy())
    dev.w = torch.from_numpy(pre).to(gpu)
    assert np.array_equal(dev.dequant().view(np.uint16), prob.oracle_dequant().view(np.uint16))
    _, rel, _ = error_report(dev.run(), prob.oracle_gemv(threads=8))
    assert rel <= REL_TOL
