"""Writes the golden fixtures under tests/golden/.

The reference ships no golden-vector files for this path (all of its oracles are computed at test
time on a Blackwell GPU), so these vectors are derived from what pins the semantics independently
of both the C oracle and the HIP kernels:

  e2m1_of_bf16.npy        e2m1 code of every non-NaN bf16 value: closed-form round-half-even on the
                          grid {0,.5,1,1.5,2,3,4,6} with numpy's own rounding
                          (cvt.rn.satfinite.e2m1x2.f32 of runtime/casts.cu:1074-1111)
  e4m3_of_bf16.npy        e4m3 code of every non-NaN bf16 value: torch's float8_e4m3fn cast after
                          clamping to +-448 (satfinite)
  swizzle_256x8.npy       the 128x4 layout of arange(256*8) built with reshape/transpose
                          (tests/python/direct_utils/narrow_precision.py:27-43)
  grouped_layout_m512_k9.npz   the fixture of tests/cpp/test_layout_op.cpp:125-133 (m=512, k=9,
                          input arange, offsets {0,100,250}, sf offsets {0,128,384}); expected buffer
                          built per group with pad + reshape/transpose
  nvfp4_quant_128x512.npz seeded bf16 input with payload and scales computed by a torch-op pipeline
                          in the kernel's operation order (runtime/block_quantization_kernels.cu:194-263),
                          using torch's fp8 cast and the closed-form e2m1 rounding
  mxfp8_quant_64x256.npz  same for the MXFP8 recipe (:142-186), e8m0 by ceil(log2)

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
GRID = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def e2m1_closed_form(x: np.ndarray) -> np.ndarray:
    """Round-half-even onto the e2m1 grid, saturating, sign kept (also for -0)."""
    x = x.astype(np.float32)
    sign = np.signbit(x).astype(np.uint8) << 3
    a = np.minimum(np.abs(x.astype(np.float64)), 6.0)
    e = np.maximum(np.floor(np.log2(np.maximum(a, 1e-300))), 0.0)  # spacing 0.5 below 2, then 1, then 2
    ulp = 2.0 ** (e - 1.0)
    r = np.round(a / ulp) * ulp  # numpy rounds half to even
    code = np.searchsorted(GRID, r).astype(np.uint8)
    assert np.all(GRID[code] == r)
    return code | sign


def e4m3_torch(x: torch.Tensor) -> torch.Tensor:
    return x.float().clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)


def swizzle_by_reshape(sf: torch.Tensor) -> torch.Tensor:
    m, c = sf.shape
    mp, cp = (m + 127) // 128 * 128, (c + 3) // 4 * 4
    padded = torch.zeros(mp, cp, dtype=sf.dtype)
    padded[:m, :c] = sf
    return padded.reshape(mp // 128, 4, 32, cp // 4, 4).transpose(1, 3).reshape(mp, cp).contiguous()


def nvfp4_by_torch_ops(x: torch.Tensor, gs):
    m, k = x.shape
    xf = x.float().reshape(m, k // 16, 16)
    amax = xf.abs().amax(dim=-1)
    s = amax / 6.0
    if gs is not None:
        s = s * gs
    s = torch.clamp(s, max=torch.finfo(torch.float32).max)
    q8 = e4m3_torch(s)
    sf = q8.view(torch.float8_e4m3fn).float()
    if gs is not None:
        r = 1.0 / (sf * (torch.tensor(1.0) / gs))
    else:
        r = 1.0 / sf
    r = torch.clamp(r, max=torch.finfo(torch.float32).max)
    y = (xf * r.unsqueeze(-1)).reshape(m, k)
    codes = e2m1_closed_form(y.numpy())
    payload = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    return payload, q8.numpy()


def mxfp8_by_torch_ops(x: torch.Tensor):
    m, k = x.shape
    xf = x.float().reshape(m, k // 32, 32)
    amax = xf.abs().amax(dim=-1)
    t = (amax * torch.tensor(1.0 / 448, dtype=torch.float32)).double()
    e = torch.where(t > 0, torch.ceil(torch.log2(t.clamp(min=1e-300))) + 127, torch.zeros_like(t)).clamp(0, 254)
    inv = torch.where(e == 0, torch.ones_like(e), torch.exp2(127 - e)).float()
    y = xf * inv.unsqueeze(-1)
    return e4m3_torch(y.reshape(m, k)).numpy(), e.to(torch.uint8).numpy()


def main():
    bits = np.arange(65536, dtype=np.uint32) << 16
    vals = bits.view(np.float32)
    ok = ~np.isnan(vals)
    e2 = np.full(65536, 0xFF, dtype=np.uint8)  # 0xFF marks "NaN input, not covered"
    e2[ok] = e2m1_closed_form(vals[ok])
    np.save(os.path.join(HERE, "e2m1_of_bf16.npy"), e2)
    e4 = np.full(65536, 0xFF, dtype=np.uint8)  # 0xFF never occurs for non-NaN inputs (satfinite)
    e4[ok] = e4m3_torch(torch.from_numpy(vals[ok].copy())).numpy()
    np.save(os.path.join(HERE, "e4m3_of_bf16.npy"), e4)

    sw = swizzle_by_reshape(torch.arange(256 * 8, dtype=torch.int32).reshape(256, 8))
    np.save(os.path.join(HERE, "swizzle_256x8.npy"), sw.numpy())

    m, k = 512, 9
    inp = torch.arange(m * k, dtype=torch.float32).reshape(m, k)
    offs, sf_offs = [0, 100, 250], [0, 128, 384]
    expected = torch.full((768, 12), -1.0)  # -1 marks bytes no group writes
    valid = torch.zeros(768, 12, dtype=torch.bool)
    ends = offs[1:] + [m]
    for o, e, so in zip(offs, ends, sf_offs):
        grp = swizzle_by_reshape(inp[o:e])
        mask = swizzle_by_reshape(torch.ones(e - o, k)) > 0
        expected[so : so + grp.shape[0]] = torch.where(mask, grp, expected[so : so + grp.shape[0]])
        valid[so : so + grp.shape[0]] = mask
    np.savez_compressed(os.path.join(HERE, "grouped_layout_m512_k9.npz"), expected=expected.numpy(), valid=valid.numpy(),
                        offsets=np.array(offs, dtype=np.int32), sf_offsets=np.array(sf_offs, dtype=np.int32))

    gen = torch.Generator().manual_seed(1234)
    x = torch.randn(128, 512, generator=gen).bfloat16()
    x[3, 32:48] = 0  # an all-zero block
    x[5, 0:16] = torch.tensor([6.0 * 2.0**-3] + [2.0**-3 * v for v in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)] + [0.0] * 8)
    gs = np.float32(2688.0) / x.float().abs().max().numpy()
    p_gs, s_gs = nvfp4_by_torch_ops(x, torch.tensor(gs))
    p_no, s_no = nvfp4_by_torch_ops(x, None)
    np.savez_compressed(os.path.join(HERE, "nvfp4_quant_128x512.npz"), x_bits=x.view(torch.int16).numpy(), gs=gs,
                        payload_gs=p_gs, scales_gs=s_gs, payload_nogs=p_no, scales_nogs=s_no)

    x8 = (torch.randn(64, 256, generator=gen) * torch.exp(torch.randn(64, 1, generator=gen) * 3)).bfloat16()
    q8, e8 = mxfp8_by_torch_ops(x8)
    np.savez_compressed(os.path.join(HERE, "mxfp8_quant_64x256.npz"), x_bits=x8.view(torch.int16).numpy(), payload=q8, scales=e8)
    print("golden fixtures written to", HERE)


if __name__ == "__main__":
    main()
