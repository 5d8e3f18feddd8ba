"""Pins of the two oracle helpers for the steps either side of the quantizer (global scale, silu * up)."""
import math

import torch

from oracle import nvf_oracle as O


def test_global_scale_closed_forms():
    assert O.compute_nvfp4_global_scale(torch.tensor([0.5, -2688.0, 3.0])) == 1.0
    assert O.compute_nvfp4_global_scale(torch.tensor([1.0, -0.25])) == 2688.0
    assert O.compute_nvfp4_global_scale(torch.zeros(5)) == 1.0
    assert O.compute_nvfp4_global_scale(torch.tensor([1e-40])) == torch.finfo(torch.float32).max
    assert O.compute_nvfp4_global_scale(torch.tensor([float("inf"), 1.0])) == 0.0
    assert math.isnan(O.compute_nvfp4_global_scale(torch.tensor([float("nan"), 1.0])))
    x = torch.tensor([3.0, -7.0], dtype=torch.bfloat16)
    assert O.compute_nvfp4_global_scale(x) == 384.0


def test_silu_mul_matches_torch_and_known_values():
    # silu(0) = 0, silu(x) -> x for large x, -> -0 for very negative x; ln 3: silu = ln3 * 3/4
    g = torch.tensor([0.0, 20.0, -100.0, math.log(3.0)], dtype=torch.float32).bfloat16()
    u = torch.tensor([5.0, 0.5, 3.0, 2.0]).bfloat16()
    out = O.silu_mul(g, u)
    assert out[0] == 0 and out[1] == 10.0 and out[2] == 0
    g3 = float(g[3])
    assert out[3] == torch.tensor(g3 / (1 + math.exp(-g3))).bfloat16() * 2
    # against torch's own CPU kernels on random data: same roundings, exp may differ by an ulp of fp32,
    # which the rounding to bf16 / f16 hides except in rare ties
    gen = torch.Generator().manual_seed(0)
    for dt in (torch.bfloat16, torch.float16):
        gg = (torch.randn(1 << 16, generator=gen) * 3).to(dt)
        uu = torch.randn(1 << 16, generator=gen).to(dt)
        ref = torch.nn.functional.silu(gg) * uu
        mism = (O.silu_mul(gg, uu) != ref).float().mean().item()
        assert mism <= 1e-3, (dt, mism)
