"""An independent restatement of the bfloat16 arithmetic with torch.bfloat16 (torch's own
c10::BFloat16 code), used only to cross-check the C oracle on small cases and to gate the golden
vectors.  bf16 values travel as uint16 bit patterns (numpy has no such dtype)."""
import numpy as np
import torch

import oracle as orc


def torch_bits(values_f32):
    return torch.from_numpy(np.ascontiguousarray(values_f32, dtype=np.float32)).bfloat16().view(torch.int16).numpy().view(np.uint16)


def as_torch_bf16(bits):
    return torch.from_numpy(np.ascontiguousarray(bits, dtype=np.uint16).view(np.int16)).view(torch.bfloat16)


def torch_dequantize(q, scale_bits, zero_bits, group_size):
    n, k = q.shape
    g = torch.arange(k) // group_size
    s = as_torch_bf16(scale_bits)[g, :].T
    p = torch.from_numpy(q.astype(np.float32)).bfloat16() * s            # first rounding
    if zero_bits is not None:
        p = p + as_torch_bf16(zero_bits)[g, :].T                         # second rounding
    return p


def sequential_gemv(dq_bf16, x_bits, bias_bits):
    """fp32 accumulation in ascending k (host/mixed_gemv.h:84-98), one rounding to bf16."""
    d = dq_bf16.float().numpy()
    x = orc.bf16_to_f32_array(x_bits)
    out = np.empty((x.shape[0], d.shape[0]), dtype=np.uint16)
    for b in range(x.shape[0]):
        acc = np.zeros(d.shape[0], dtype=np.float32)
        for kk in range(d.shape[1]):
            acc = (acc + (x[b, kk] * d[:, kk]).astype(np.float32)).astype(np.float32)
        if bias_bits is not None:
            acc = (acc + orc.bf16_to_f32_array(bias_bits)).astype(np.float32)
        out[b] = torch_bits(acc)
    return out
