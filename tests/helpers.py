"""Shared test helpers: fixture loading, synthetic inputs, comparisons."""
import os

import numpy as np
import torch

from oracle import nvf_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# GEMM tolerance of this build: max |out - ref| <= 1e-2 * max |ref| against the fp32
# dequantize+matmul oracle.  bf16 rounding of the output alone contributes up to 2^-9 = 2e-3.
GEMM_MAX_REL = 1e-2


def golden(name):
    return np.load(os.path.join(GOLDEN, name))


def all_bf16_as_f32():
    return (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)


def max_rel(out, ref):
    out = out.float().cpu()
    return ((out - ref).abs().max() / ref.abs().max()).item()


def gs_of(x):
    """Encode global scale 448*6 / amax (tests/python/direct/test_cutlass_nvfp4_gemm.py:70-76)."""
    return float(2688.0 / x.float().abs().max())


def start_offsets(sizes):
    out = [0]
    for s in sizes[:-1]:
        out.append(out[-1] + s)
    return torch.tensor(out, dtype=torch.int32)


def fp4(t):
    return t.view(torch.float4_e2m1fn_x2)


def e4m3(t):
    return t.view(torch.float8_e4m3fn)


def e8m0(t):
    return t.view(torch.float8_e8m0fnu)


def valid_scales(sf_swizzled_u8, rows, cols):
    return O.swizzled_to_linear_128_4(sf_swizzled_u8, rows, cols)
