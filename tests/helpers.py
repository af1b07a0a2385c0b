"""Shared test helpers: seeded problems (from the oracle's generator) and error metrics."""
import numpy as np

import oracle as orc

PER_COLUMN, SCALE_ONLY, SCALE_AND_ZEROS = 1, 2, 3


def seed_of(tag, tensor, buffer=0):
    """One documented 64-bit seed per (problem tag, tensor, buffer)."""
    h = 1469598103934665603
    for ch in f"{tag}/{tensor}/{buffer}".encode():
        h = ((h ^ ch) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


class Problem:
    """Raw (un-preprocessed) operands of one GEMV, as numpy arrays."""

    def __init__(self, tag, n_out, k, bits, quant_op, group_size, m_batch=1, bias=False, x_dist="uniform",
                 scale_range=(0.001, 0.02), zero_kind="f16", zero_range=(-0.05, 0.05), buffer=0, element="f16"):
        """element="bf16": the same draws rounded to bfloat16; x / scale / zero_add / bias are then
        uint16 arrays of bf16 bit patterns (numpy has no such dtype)."""
        self.element = element
        self.tag, self.n_out, self.k, self.bits, self.quant_op = tag, n_out, k, bits, quant_op
        self.group_size = k if quant_op == PER_COLUMN else group_size
        self.m_batch = m_batch
        groups = k // self.group_size
        lo, hi = (-8, 7) if bits == 4 else (-128, 127)
        self.q = orc.fill_int8(n_out * k, seed_of(tag, "w", buffer), lo, hi)
        self.w_raw = orc.pack_int4(self.q) if bits == 4 else self.q.view(np.uint8).copy()
        if x_dist == "uniform":
            self.x = orc.fill_uniform_f16(m_batch * k, seed_of(tag, "x"), -1.0, 1.0).reshape(m_batch, k)
        else:
            self.x = orc.fill_normal_clipped_f16(m_batch * k, seed_of(tag, "x"), 4.0).reshape(m_batch, k)
        self.scale = orc.fill_uniform_f16(groups * n_out, seed_of(tag, "s", buffer), *scale_range).reshape(groups, n_out)
        self.zeros_i8 = None
        self.zero_add = None
        if quant_op == SCALE_AND_ZEROS:
            if zero_kind == "int8":
                self.zeros_i8 = orc.fill_int8(groups * n_out, seed_of(tag, "z", buffer), -8, 7).reshape(groups, n_out)
                self.zero_add = orc.fold_zero_points(self.scale, self.zeros_i8)
            else:
                self.zero_add = orc.fill_uniform_f16(groups * n_out, seed_of(tag, "z", buffer), *zero_range).reshape(
                    groups, n_out)
        self.bias = orc.fill_uniform_f16(n_out, seed_of(tag, "b"), -0.1, 0.1) if bias else None
        if element == "bf16":
            to_bf16 = lambda a: None if a is None else orc.f32_to_bf16_array(a.astype(np.float32))  # noqa: E731
            self.x, self.scale, self.bias = to_bf16(self.x), to_bf16(self.scale), to_bf16(self.bias)
            if self.zeros_i8 is not None:
                self.zero_add = orc.fold_zero_points_bf16(self.scale, self.zeros_i8)
            else:
                self.zero_add = to_bf16(self.zero_add)

    def oracle_dequant(self):
        if self.element == "bf16":
            return orc.dequantize_bf16(self.w_raw, self.scale, self.zero_add, self.n_out, self.k, self.group_size,
                                       self.quant_op, self.bits)
        return orc.dequantize(self.w_raw, self.scale, self.zero_add, self.n_out, self.k, self.group_size,
                              self.quant_op, self.bits)

    def oracle_gemv(self, threads=8, literal_int8_zero=False):
        zero = self.zeros_i8 if (literal_int8_zero and self.zeros_i8 is not None) else self.zero_add
        if self.element == "bf16":
            return orc.gemv_bf16(self.w_raw, self.x, self.scale, zero, self.bias, self.n_out, self.m_batch, self.k,
                                 self.group_size, self.quant_op, self.bits, threads=threads)
        return orc.gemv(self.w_raw, self.x, self.scale, zero, self.bias, self.n_out, self.m_batch, self.k,
                        self.group_size, self.quant_op, self.bits, threads=threads)


REL_FLOOR_FRACTION = 2.0 ** -7


def error_report(got, ref):
    """max abs error, and max relative error with denominator max(|ref|, 2^-7 * rms(ref)).

    Why a floor, and why this one: an output that happens to be almost zero is a sum of
    thousands of cancelling terms, and its ABSOLUTE error is set by the order in which fp32
    adds them (a few 1e-5 for k = 8192 with outputs of rms 3).  The reference's own ascending-k
    HOST_CHECK loop differs from the exactly accumulated, once-rounded result by 2.8e-3
    relative when the floor is 2^-10 * rms, i.e. it would fail a 2e-3 bar against the truth;
    from 2^-7 * rms upwards its deviation is the half-ulp rounding level (9.7e-4), so that is
    the smallest floor under which "within 2e-3 of HOST_CHECK" is a statement about the kernel
    and not about summation order."""
    g = np.asarray(got, dtype=np.float64).reshape(-1)
    r = np.asarray(ref, dtype=np.float64).reshape(-1)
    rms = float(np.sqrt(np.mean(r * r))) if r.size else 0.0
    floor = max(rms * REL_FLOOR_FRACTION, 2.0 ** -24)
    abs_err = np.abs(g - r)
    rel = abs_err / np.maximum(np.abs(r), floor)
    return float(abs_err.max(initial=0.0)), float(rel.max(initial=0.0)), floor


def bf16_ulp_report(got_bits, ref_bits):
    """For bf16 outputs (uint16 bit patterns): the largest |got - ref| in units of the bf16 ulp of
    max(|ref|, 2^-7 * rms(ref)), and the fraction of outputs whose bits differ.  One ulp is 2^-7
    relative at the bottom of a binade, so "within 2e-3" cannot be asked of a bf16 result: two
    correct fp32 sums that differ in their last bits can round to adjacent bf16 values."""
    g = orc.bf16_to_f32_array(got_bits).astype(np.float64).reshape(-1)
    r = orc.bf16_to_f32_array(ref_bits).astype(np.float64).reshape(-1)
    rms = float(np.sqrt(np.mean(r * r))) if r.size else 0.0
    floor = max(rms * REL_FLOOR_FRACTION, 2.0 ** -100)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(r), floor))) - 7)
    worst = float((np.abs(g - r) / ulp).max(initial=0.0))
    differing = float(np.mean(np.asarray(got_bits).reshape(-1) != np.asarray(ref_bits).reshape(-1)))
    return worst, differing


class DeviceProblem:
    """Uploads a Problem through the library's own preprocessor."""

    def __init__(self, prob, device):
        import torch
        import mixed_gemv_amd as mg
        self.p = prob
        qt = mg.QuantType.W4_A16 if prob.bits == 4 else mg.QuantType.W8_A16
        pre = mg.MixedGemvWeightPreprocessor.run(prob.w_raw, (prob.k, prob.n_out), mg.LayoutType.kColumnMajor, qt)
        self.w = torch.from_numpy(pre).to(device)
        self.x = torch.from_numpy(prob.x.view(np.int16)).to(device)
        self.scale = torch.from_numpy(prob.scale.view(np.int16)).to(device)
        self.zero = torch.from_numpy(prob.zero_add.view(np.int16)).to(device) if prob.zero_add is not None else None
        self.bias = torch.from_numpy(prob.bias.view(np.int16)).to(device) if prob.bias is not None else None
        self.y = torch.zeros((prob.m_batch, prob.n_out), dtype=torch.int16, device=device)

    def run(self):
        import torch
        import mixed_gemv_amd as mg
        p = self.p
        self.y.fill_(0x7e00)  # NaN pattern: every output must be overwritten
        mg.device_gemv(self.w, self.x, self.scale, self.zero, self.bias, self.y, 1, p.n_out, p.m_batch, p.k,
                       p.group_size, p.quant_op, p.bits, element=p.element)
        torch.cuda.synchronize()
        out = self.y.cpu().numpy()
        return out.view(np.uint16) if p.element == "bf16" else out.view(np.float16)

    def dequant(self):
        import torch
        import mixed_gemv_amd as mg
        p = self.p
        out = torch.zeros((p.n_out, p.k), dtype=torch.int16, device=self.w.device)
        mg.dequantize(self.w, self.scale, self.zero, out, p.n_out, p.k, p.group_size, p.quant_op, p.bits,
                      element=p.element)
        torch.cuda.synchronize()
        out = out.cpu().numpy()
        return out.view(np.uint16) if p.element == "bf16" else out.view(np.float16)


def float64_bound_violations(prob, y, rows_per_chunk=2048, dq=None):
    """How many outputs lie outside what the mathematics allows ANY correct kernel: with the
    (bit-exact) dequantised weights dq, the exactly accumulated sum  x . dq[n] + bias[n]  in float64,
    and around it the classical bound for k products (exact in fp32) summed in fp32 in any order,
    k * 2^-24 * sum |x| |dq|, plus one rounding to fp16 (2^-11 relative, 2^-24 absolute for
    subnormal results).  Unlike a relative error against HOST_CHECK this needs no floor: outputs
    that cancel to almost zero are bounded by the magnitude of what cancelled.
    dq: the oracle's dequantised weights if the caller already has them.
    Returns (violations, largest error / bound)."""
    dq = prob.oracle_dequant() if dq is None else dq
    x = prob.x.astype(np.float64)
    y = np.asarray(y).astype(np.float64).reshape(prob.m_batch, prob.n_out)
    bias = prob.bias.astype(np.float64) if prob.bias is not None else np.zeros(prob.n_out)
    bad, worst = 0, 0.0
    for r0 in range(0, prob.n_out, rows_per_chunk):
        d = dq[r0:r0 + rows_per_chunk].astype(np.float64)
        exact = x @ d.T + bias[None, r0:r0 + rows_per_chunk]
        mag = np.abs(x) @ np.abs(d.T) + np.abs(bias[None, r0:r0 + rows_per_chunk])
        bound = mag * (prob.k + 1) * 2.0 ** -24 + np.abs(exact) * 2.0 ** -11 + 2.0 ** -24
        err = np.abs(y[:, r0:r0 + rows_per_chunk] - exact)
        bad += int((err > bound).sum())
        worst = max(worst, float((err / bound).max()))
    return bad, worst
