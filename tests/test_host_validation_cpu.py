"""Host-forcible failures of the at::Tensor entry points, checked on CPU tensors: the same
conditions and messages as the reference's validators (cutlass/nvf_cutlass.cpp:13-234,
cutlass/group_mm.cu:417-497, cutlass/nvfp4_scaled_group_mm.cu:570-688).  pybind turns the thrown
nvfError into RuntimeError, as in the reference."""
import pytest
import torch

from fuser_amd import nvf_cutlass, ops
from helpers import e4m3, e8m0, fp4


def _nvfp4_args(m=128, n=128, k=64):
    a = fp4(torch.zeros(m, k // 2, dtype=torch.uint8))
    b = fp4(torch.zeros(n, k // 2, dtype=torch.uint8))
    sa = e4m3(torch.zeros((m + 127) // 128 * 128, (k // 16 + 3) // 4 * 4, dtype=torch.uint8))
    sb = e4m3(torch.zeros((n + 127) // 128 * 128, (k // 16 + 3) // 4 * 4, dtype=torch.uint8))
    return a, b, sa, sb, torch.tensor(1.0)


def test_nvfp4_validator_returns_mnk_with_skip_checks():
    a, b, sa, sb, alpha = _nvfp4_args(128, 256, 64)
    assert nvf_cutlass.validate_inputs_nvfp4_scaled_mm(a, b, sa, sb, alpha, skip_checks=True) == (128, 256, 64)
    a8 = torch.zeros(16, 64, dtype=torch.uint8).view(torch.float8_e4m3fn)
    assert nvf_cutlass.validate_inputs_mxfp8_scaled_mm(a8, a8, sa, sb, alpha, skip_checks=True) == (16, 16, 64)


def test_dense_validators_reject_cpu_tensors_and_bad_ranks():
    a, b, sa, sb, alpha = _nvfp4_args()
    with pytest.raises(RuntimeError, match="must be a CUDA tensor and contiguous"):
        nvf_cutlass.nvfp4_scaled_mm(a, b, sa, sb, alpha, torch.bfloat16)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor and contiguous"):
        nvf_cutlass.nvfp4_scaled_mm_blockscale(a, b, sa, sb, alpha, torch.tensor(2.0))
    with pytest.raises(RuntimeError, match="Operand A must be a matrix"):
        nvf_cutlass.validate_inputs_nvfp4_scaled_mm(a[0], b, sa, sb, alpha)
    with pytest.raises(RuntimeError, match="cannot be multiplied"):
        nvf_cutlass.validate_inputs_nvfp4_scaled_mm(a, fp4(torch.zeros(128, 16, dtype=torch.uint8)), sa, sb, alpha)
    a8 = torch.zeros(16, 64, dtype=torch.uint8).view(torch.float8_e4m3fn)
    s8 = e8m0(torch.zeros(128, 4, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor and contiguous"):
        nvf_cutlass.mxfp8_scaled_mm(a8, a8, s8, s8, alpha, torch.float16)


def test_grouped_entry_points_reject_cpu_tensors():
    a = torch.zeros(8, 64, dtype=torch.bfloat16)
    b = torch.zeros(2, 16, 64, dtype=torch.bfloat16)
    i64 = torch.zeros(2, dtype=torch.int64)
    ps = torch.zeros(2, 3, dtype=torch.int32)
    eo = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="Expected CUDA tensor for Operand A"):
        nvf_cutlass.grouped_mm(a, b, i64, i64, ps, eo)
    with pytest.raises(RuntimeError, match="Expected CUDA tensor for Operand A"):
        nvf_cutlass.nvfp4_scaled_grouped_mm(fp4(torch.zeros(8, 32, dtype=torch.uint8)), fp4(torch.zeros(2, 16, 32, dtype=torch.uint8)),
                                            e4m3(torch.zeros(128, 4, dtype=torch.uint8)), e4m3(torch.zeros(2, 16, 4, dtype=torch.uint8)),
                                            torch.ones(2), i64, i64, ps, eo, eo, torch.bfloat16)


def test_quantizer_entry_points_reject_cpu_tensors_and_bad_block_size():
    x = torch.zeros(4, 32, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ops.nv_block_quantize(x)
    with pytest.raises(RuntimeError, match="Block size must be 16"):
        ops.nv_block_quantize(x, None, False, 32)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ops.nv_grouped_block_quantize(x, torch.zeros(1, dtype=torch.int32), torch.zeros(1, dtype=torch.int32))
