"""Eager counterparts of the reference's quantization graph ops.

Same names, argument order and defaults as ``fd.ops.nv_block_quantize``,
``fd.ops.nv_grouped_block_quantize`` and ``fd.ops.preprocess_grouped_matmul_input_sf``
(python/python_direct/ops.cpp:3521-3607, :3179-3212); each is one launch of a HIP kernel.
"""
import torch

from . import _C


def nv_block_quantize(input, global_scale=None, swizzle_block_scales=False, block_size=16,
                      dtype=torch.float4_e2m1fn_x2):
    """-> (quantized, block_scales).

    dtype float4_e2m1fn_x2: NVFP4 (block 16, e4m3 scales, optional 0-dim fp32 ``global_scale``);
    quantized is [.., K/2].  dtype float8_e4m3fn: MXFP8 (block 32, e8m0 scales).
    With ``swizzle_block_scales`` the scales come back in the 128x4 layout with the padded shape
    (roundUp(M,128), roundUp(K/block,4)) that the scaled GEMMs expect.
    """
    return _C.nv_block_quantize(input, global_scale, swizzle_block_scales, block_size, dtype)


def nv_grouped_block_quantize(input, input_offsets, output_offsets, global_scale=None, block_size=16,
                              dtype=torch.float4_e2m1fn_x2):
    """-> (quantized [M, K/2], block_scales [M + 127*G, roundUp(K/16,4)]) with every group's scales
    128x4-swizzled on its own, starting at row ``output_offsets[g]``."""
    return _C.nv_grouped_block_quantize(input, input_offsets, output_offsets, global_scale, block_size, dtype)


def preprocess_grouped_matmul_input_sf(input, input_offsets, output_offsets):
    """Copies linear block scales [M, C] into the per-group padded 128x4 layout."""
    return _C.preprocess_grouped_matmul_input_sf(input, input_offsets, output_offsets)


def silu_mul_nv_grouped_block_quantize(gate, up, input_offsets, output_offsets, global_scale=None):
    """``nv_grouped_block_quantize(torch.nn.functional.silu(gate) * up, ...)`` in one kernel: the product is
    formed in registers with the eager chain's roundings (silu and product each rounded to the inputs'
    bf16 / f16 type) and never written to memory."""
    return _C.silu_mul_nv_grouped_block_quantize(gate, up, input_offsets, output_offsets, global_scale)


def compute_nvfp4_global_scale(tensor):
    """0-dim fp32 device tensor ``448 * 6 / max|tensor|`` (1.0 for an all-zero tensor, clamped to the fp32
    maximum), as tests/python/direct/test_narrow_precision.py:138-156 defines the NVFP4 global scale, computed
    on the device without a host round trip; pass it as ``global_scale`` to the quantizers."""
    return _C.compute_nvfp4_global_scale(tensor)
