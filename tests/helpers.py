"""Shared test helpers: fixture loading, synthetic inputs, comparisons."""
import os

import numpy as np
import torch

from oracle import nvf_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# GEMM tolerance of this build: 1e-2 "max-rel" against the fp32 dequantize+matmul oracle, where max-rel is
# max |out - ref| / max |ref| -- over the whole output (max_rel) or, stricter, row by row (max_rel_rowwise: an
# error confined to a row of small magnitude cannot hide behind a large element elsewhere).  It is not an
# element-wise relative error: elements near zero have none.  bf16 rounding of the output alone contributes
# up to 2^-9 = 2e-3; observed values are 2-4e-3.
GEMM_MAX_REL = 1e-2


def golden(name):
    return np.load(os.path.join(GOLDEN, name))


def all_bf16_as_f32():
    return (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)


def max_rel(out, ref):
    out = out.float().cpu()
    return ((out - ref).abs().max() / ref.abs().max()).item()


def max_rel_rowwise(out, ref):
    out = out.float().cpu()
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    return ((out - ref).abs() / scale).max().item()


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
