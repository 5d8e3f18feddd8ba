"""GPU parity of the steps fused either side of the NVFP4 quantizer: the global (per-tensor) scale
(tests/python/direct/test_narrow_precision.py:138-156) and silu(gate) * up ahead of the grouped quantizer
(benchmarks/python/layers_for_inference_benchmark.py:504)."""
import math

import pytest
import torch

from helpers import start_offsets
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("numel,skip", [(1, 0), (7, 0), (1000, 0), (4099, 3), ((1 << 20) + 5, 1), (3 << 20, 0)])
def test_global_scale_equals_the_host_formula(dev, dtype, numel, skip):
    """bit-equal fp32 scale for sizes below / across / far above one 16-byte vector per thread, and for a
    view that does not start on a 16-byte boundary"""
    from fuser_amd import ops

    gen = torch.Generator().manual_seed(numel)
    base = (torch.randn(numel + skip, generator=gen) * 3).to(dtype)
    base[(numel + skip) // 2] = -11.5  # the maximum is negative and away from the ends
    x = base[skip:]
    got = ops.compute_nvfp4_global_scale(base.to(dev)[skip:])
    assert got.dim() == 0 and got.dtype == torch.float32 and got.device.type == "cuda"
    want = torch.tensor(O.compute_nvfp4_global_scale(x), dtype=torch.float32)
    assert got.cpu().view(torch.int32) == want.view(torch.int32)


def test_global_scale_special_tensors_and_use_by_the_quantizer(dev):
    from fuser_amd import ops

    f32max = torch.finfo(torch.float32).max
    assert ops.compute_nvfp4_global_scale(torch.zeros(300, device=dev)).item() == 1.0
    assert ops.compute_nvfp4_global_scale(torch.zeros(0, device=dev)).item() == 1.0
    assert ops.compute_nvfp4_global_scale(torch.tensor([1e-40, 0.0], device=dev)).item() == f32max
    assert ops.compute_nvfp4_global_scale(torch.tensor([1.0, float("-inf")], device=dev)).item() == 0.0
    assert math.isnan(ops.compute_nvfp4_global_scale(torch.tensor([1.0, float("nan"), 5.0], device=dev).bfloat16()).item())
    # twice on the same output type: the reduction cell is re-initialised by every call
    x = torch.randn(256, 512, generator=torch.Generator().manual_seed(1)).bfloat16()
    gs = ops.compute_nvfp4_global_scale(x.to(dev))
    assert torch.equal(gs, ops.compute_nvfp4_global_scale(x.to(dev)))
    q, sf = ops.nv_block_quantize(x.to(dev), gs, True, 16)
    rq, rsf = O.block_quantize_nvfp4(x, O.compute_nvfp4_global_scale(x), True)
    assert torch.equal(q.view(torch.uint8).cpu(), rq)
    assert torch.equal(O.swizzled_to_linear_128_4(sf.view(torch.uint8).cpu(), 256, 32), O.swizzled_to_linear_128_4(rsf, 256, 32))


def _valid_scales(sf, sizes, so, cols):
    sf = sf.view(torch.uint8).cpu()
    return [O.swizzled_to_linear_128_4(sf[int(so[e]) : int(so[e]) + O.round_up(t, 128)], t, cols // 16) for e, t in enumerate(sizes) if t]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("use_gs", [False, True])
def test_silu_mul_quantizer_returns_the_bytes_of_the_eager_chain(dev, dtype, use_gs):
    """fused kernel == grouped quantizer applied to torch's own silu(gate) * up on the GPU (bit-exact:
    same formula, same roundings), and == the CPU oracle chain except where fp32 exp differs by an ulp
    at a rounding tie of the 16-bit intermediate (bounded fraction of bytes)."""
    from fuser_amd import ops

    sizes = [130, 0, 77, 1, 300]
    m, k = sum(sizes), 2048 + 64
    gen = torch.Generator().manual_seed(7)
    gate = (torch.randn(m, k, generator=gen) * 2).to(dtype)
    up = torch.randn(m, k, generator=gen).to(dtype)
    gate[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, -200.0, 88.0, 1e-3, -1e-3]).to(dtype)  # exp under / overflow
    eo = start_offsets(sizes)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    gd, ud, eod, sod = gate.to(dev), up.to(dev), eo.to(dev), so.to(dev)
    gs = ops.compute_nvfp4_global_scale(torch.nn.functional.silu(gd) * ud) if use_gs else None
    q, sf = ops.silu_mul_nv_grouped_block_quantize(gd, ud, eod, sod, gs)
    assert q.shape == (m, k // 2) and sf.shape == (m + 127 * len(sizes), k // 16)
    q2, sf2 = ops.nv_grouped_block_quantize(torch.nn.functional.silu(gd) * ud, eod, sod, gs, 16)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8))
    for a, b in zip(_valid_scales(sf, sizes, so, k), _valid_scales(sf2, sizes, so, k)):
        assert torch.equal(a, b)
    rq, rsf = O.grouped_block_quantize_nvfp4(O.silu_mul(gate, up), eo, so, None if gs is None else float(gs.item()))
    assert (q.view(torch.uint8).cpu() != rq).float().mean().item() <= 1e-3


def test_silu_mul_quantizer_nonfinite_inputs_follow_the_chain(dev):
    from fuser_amd import ops

    m, k = 8, 64
    gate = torch.randn(m, k, generator=torch.Generator().manual_seed(3)).bfloat16()
    up = torch.ones(m, k).bfloat16()
    gate[1, 3], gate[2, 17], gate[3, 40] = float("inf"), float("-inf"), float("nan")
    up[4, 5], up[5, 6] = float("inf"), float("nan")
    off = torch.zeros(1, dtype=torch.int32, device=dev)
    q, sf = ops.silu_mul_nv_grouped_block_quantize(gate.to(dev), up.to(dev), off, off, None)
    q2, sf2 = ops.nv_grouped_block_quantize(torch.nn.functional.silu(gate.to(dev)) * up.to(dev), off, off, None, 16)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(O.swizzled_to_linear_128_4(sf.view(torch.uint8).cpu()[:128], m, k // 16),
                       O.swizzled_to_linear_128_4(sf2.view(torch.uint8).cpu()[:128], m, k // 16))


def test_fused_producers_through_the_c_abi(dev):
    from fuser_amd import capi, ops

    m, k = 200, 512
    gen = torch.Generator().manual_seed(11)
    gate, up = torch.randn(m, k, generator=gen).bfloat16().to(dev), torch.randn(m, k, generator=gen).bfloat16().to(dev)
    prod = torch.nn.functional.silu(gate) * up
    scale = torch.empty((), dtype=torch.float32, device=dev)
    capi.check(capi.lib().nvf_nvfp4_global_scale(prod.data_ptr(), capi.BF16, prod.numel(), scale.data_ptr(), None))
    assert scale.item() == torch.tensor(O.compute_nvfp4_global_scale(prod.cpu()), dtype=torch.float32).item()
    # input_offsets == NULL: ungrouped, 128x4 layout with zero-filled padding rows
    q = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
    sf = torch.full((256, k // 16), 0x55, dtype=torch.uint8, device=dev)
    capi.check(capi.lib().nvf_nvfp4_silu_mul_block_quantize(gate.data_ptr(), up.data_ptr(), capi.BF16, m, k, None, None, 0,
                                                            scale.data_ptr(), q.data_ptr(), sf.data_ptr(), None))
    q2, sf2 = ops.nv_block_quantize(prod, scale, True, 16)
    assert torch.equal(q, q2.view(torch.uint8)) and torch.equal(sf, sf2.view(torch.uint8))
    with pytest.raises(capi.NvfError):
        capi.check(capi.lib().nvf_nvfp4_silu_mul_block_quantize(gate.data_ptr(), up.data_ptr(), capi.F32, m, k, None, None, 0, None,
                                                                q.data_ptr(), sf.data_ptr(), None))
