"""``torch.library`` surface of the NVFP4 grouped GEMM for MoE layers.

Importing this module registers ``torch.ops.nvf_cutlass.f16a_nvfp4weight_scaled_grouped_mm`` with the
signature of the reference's inference benchmark layers
(benchmarks/python/layers_for_inference_benchmark.py:217-279), so that ``NVFP4InferenceGroupedLinear`` /
``NVFP4InferenceGroupedSwiGLU`` (:375-524 there) run on this package unchanged.  The op computes what the
reference's nvFuser translation of it computes (benchmarks/python/benchmark_inference.py:139-174):

    fp4_act, act_scales = nv_grouped_block_quantize(activation, offsets, blockscale_offsets)
    out = cutlass_nvfp4_grouped_mm(fp4_act, fp4_weight, act_scales, weight_scaling_factor,
                                   weight_global_scale, problem_sizes, offsets, blockscale_offsets, bf16)

i.e. the activations are quantized to NVFP4 on the fly, per group, without a global scale, and
``weight_global_scale`` [G] is the per-expert alpha.  (The reference's eager definition of the op is a
slow dequantize-the-weights stand-in for machines without the kernel; it is not what runs in the benchmark.)

It is not imported by ``fuser_amd/__init__.py``: a process that also imports the reference's layer file
would register the same op name twice.
"""
import torch

from . import _C, ops

__all__ = ["f16a_nvfp4weight_scaled_grouped_mm", "compute_auxiliary_tensors"]


@torch.library.custom_op("nvf_cutlass::f16a_nvfp4weight_scaled_grouped_mm", mutates_args=())
def f16a_nvfp4weight_scaled_grouped_mm(
    activation: torch.Tensor,
    fp4_weight: torch.Tensor,
    weight_scaling_factor: torch.Tensor,
    weight_global_scale: torch.Tensor,
    offsets: torch.Tensor,
    blockscale_offsets: torch.Tensor,
    problem_sizes: torch.Tensor,
) -> torch.Tensor:
    """activation [.., K] bf16/f16; fp4_weight [G, K/2, N] (transposed view of [G, N, K/2]);
    weight_scaling_factor [G, N, K/16] e4m3, every expert 128x4-swizzled; weight_global_scale [G] fp32;
    offsets int32 [G] start row of every group; blockscale_offsets int32 [G] start row of every group's
    scale slab (rows rounded up to 128); problem_sizes int32 [G, 3] = (rows, N, K).  -> [.., N] bf16."""
    a2d = activation.reshape(-1, activation.size(-1))
    if not a2d.is_contiguous():
        a2d = a2d.contiguous()
    fp4_act, act_scales = ops.nv_grouped_block_quantize(a2d, offsets, blockscale_offsets)
    out = _C.callers.cutlass_nvfp4_grouped_mma(
        fp4_act, fp4_weight, act_scales, weight_scaling_factor, weight_global_scale,
        problem_sizes, offsets, blockscale_offsets, torch.bfloat16)
    return out.reshape(activation.shape[:-1] + (out.size(-1),))


@torch.library.register_fake("nvf_cutlass::f16a_nvfp4weight_scaled_grouped_mm")
def _(activation, fp4_weight, weight_scaling_factor, weight_global_scale, offsets, blockscale_offsets, problem_sizes):
    # same contract as the reference's fake (layers_for_inference_benchmark.py:243-279)
    if activation.ndim == 0:
        raise ValueError(f"Expected activation to have at least 1 dimension, got {activation.ndim}")
    tensors = (activation, fp4_weight, weight_scaling_factor, weight_global_scale, offsets, blockscale_offsets, problem_sizes)
    if len({t.device for t in tensors}) != 1:
        raise ValueError("Expected all inputs to be on the same device.")
    return torch.empty(activation.shape[:-1] + (fp4_weight.size(2),), device=activation.device, dtype=torch.bfloat16)


def compute_auxiliary_tensors(hidden_states, offsets, out_features):
    """-> (blockscale_offsets int32 [G], problem_sizes [G, 3]) from the groups' start rows, as
    ``NVFP4InferenceGroupedLinear.compute_auxiliary_tensors`` derives them
    (layers_for_inference_benchmark.py:395-424): rows per group from neighbouring starts (the last group
    ends at the last row), scale slabs of whole 128-row tiles laid end to end."""
    total = torch.tensor([hidden_states.size(0)], device=offsets.device, dtype=offsets.dtype)
    rows = torch.diff(torch.cat([offsets, total]))
    problem_sizes = torch.stack(
        [rows, torch.full_like(rows, out_features), torch.full_like(rows, hidden_states.size(1))], dim=1)
    slab_rows = (rows + 127) // 128 * 128
    blockscale_offsets = (torch.cumsum(slab_rows, 0, dtype=torch.int32) - slab_rows.to(torch.int32))
    return blockscale_offsets, problem_sizes
