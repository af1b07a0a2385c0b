#!/usr/bin/env python3
"""Writes tests/golden/gemv_cases.npz and gemv_cases_bf16.npz: small seeded problems with their
expected dequantised weights and outputs (fp16 and bfloat16 elements).

The reference ships no vectors of its own (its only test draws from std::random_device and
prints differences), and its host code cannot be compiled here (it needs NVIDIA CUTLASS
v3.4.1 and CUDA headers), so the expected values are produced by the C oracle and, before
they are written, required to be bit-identical to the independent numpy restatement in
tests/np_restate.py (fp16) or the torch.bfloat16 restatement in tests/torch_restate.py (bf16).
The files pin both against silent drift.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import np_restate  # noqa: E402
import oracle as orc  # noqa: E402
from helpers import PER_COLUMN, SCALE_AND_ZEROS, SCALE_ONLY, Problem  # noqa: E402

CASES = [
    # tag, n_out, k, bits, quant_op, group, m_batch, bias, zero kind, x distribution
    ("g_i4_sz_g128", 48, 512, 4, SCALE_AND_ZEROS, 128, 1, False, "f16", "normal"),
    ("g_i4_sz_g64_int8z", 32, 256, 4, SCALE_AND_ZEROS, 64, 2, True, "int8", "uniform"),
    ("g_i4_s_g128", 32, 384, 4, SCALE_ONLY, 128, 1, True, "f16", "uniform"),
    ("g_i4_col", 20, 160, 4, PER_COLUMN, 0, 1, False, "f16", "uniform"),
    ("g_i8_col", 32, 272, 8, PER_COLUMN, 0, 1, True, "f16", "uniform"),
    ("g_i8_sz_g64", 16, 192, 8, SCALE_AND_ZEROS, 64, 3, False, "f16", "normal"),
]


def build(case, element="f16"):
    tag, n, k, bits, qop, g, mb, bias, zk, xd = case
    return Problem(tag, n, k, bits, qop, g, m_batch=mb, bias=bias, zero_kind=zk, x_dist=xd, element=element)


def main_bf16():
    import torch
    import torch_restate
    out = {}
    for case in CASES:
        tag = "b" + case[0][1:]
        p = build((tag,) + case[1:], element="bf16")
        dq = p.oracle_dequant()
        y = p.oracle_gemv(threads=1)
        q = p.q.reshape(p.n_out, p.k).astype(np.int32)
        ref_dq = torch_restate.torch_dequantize(q, p.scale, p.zero_add, p.group_size)
        ref_y = torch_restate.sequential_gemv(ref_dq, p.x, p.bias)
        assert np.array_equal(dq, ref_dq.view(torch.int16).numpy().view(np.uint16)), tag
        assert np.array_equal(y, ref_y), tag
        out[f"{tag}/w_raw"] = p.w_raw
        out[f"{tag}/x"] = p.x
        out[f"{tag}/scale"] = p.scale
        if p.zero_add is not None:
            out[f"{tag}/zero_add"] = p.zero_add
        if p.zeros_i8 is not None:
            out[f"{tag}/zeros_i8"] = p.zeros_i8
        if p.bias is not None:
            out[f"{tag}/bias"] = p.bias
        out[f"{tag}/dequant"] = dq
        out[f"{tag}/y"] = y
        out[f"{tag}/meta"] = np.array([p.n_out, p.k, p.bits, p.quant_op, p.group_size, p.m_batch], dtype=np.int64)
    path = os.path.join(HERE, "gemv_cases_bf16.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


def main():
    out = {}
    for case in CASES:
        tag = case[0]
        p = build(case)
        dq = p.oracle_dequant()
        y = p.oracle_gemv(threads=1)
        q = p.q.reshape(p.n_out, p.k).astype(np.int32)
        ref_dq = np_restate.dequantize(q, p.scale, p.zero_add, p.group_size, int8_zero=False)
        ref_y = np_restate.gemv(ref_dq, p.x, p.bias)
        assert np.array_equal(dq.view(np.uint16), ref_dq.view(np.uint16)), tag
        assert np.array_equal(y.view(np.uint16), ref_y.view(np.uint16)), tag
        out[f"{tag}/w_raw"] = p.w_raw
        out[f"{tag}/x"] = p.x.view(np.uint16)
        out[f"{tag}/scale"] = p.scale.view(np.uint16)
        if p.zero_add is not None:
            out[f"{tag}/zero_add"] = p.zero_add.view(np.uint16)
        if p.zeros_i8 is not None:
            out[f"{tag}/zeros_i8"] = p.zeros_i8
        if p.bias is not None:
            out[f"{tag}/bias"] = p.bias.view(np.uint16)
        out[f"{tag}/dequant"] = dq.view(np.uint16)
        out[f"{tag}/y"] = y.view(np.uint16)
        out[f"{tag}/meta"] = np.array([p.n_out, p.k, p.bits, p.quant_op, p.group_size, p.m_batch], dtype=np.int64)
    path = os.path.join(HERE, "gemv_cases.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
    main_bf16()
