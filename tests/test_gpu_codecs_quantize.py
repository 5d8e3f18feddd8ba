"""GPU parity of the narrow casts and the block quantizers against the CPU oracle: every payload
byte and every scale byte must be identical (runtime/block_quantization_kernels.cu, runtime/casts.cu)."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import all_bf16_as_f32, golden, gs_of, start_offsets, valid_scales
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def _cast(kind, x, dev):
    from fuser_amd import capi

    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev)
    out = torch.empty(t.numel(), dtype=torch.uint8, device=dev)
    fn = getattr(capi.lib(), f"nvf_cast_f32_to_{kind}")
    capi.check(fn(t.data_ptr(), t.numel(), out.data_ptr(), None))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _cast_inputs():
    rng = np.random.default_rng(7)
    edges = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 448.0, 464.0, 2.0**-6, 2.0**-9, 2.0**-10, 2.0**-127, 1.0], dtype=np.float32)
    near = np.concatenate([np.nextafter(edges, np.float32(np.inf)), np.nextafter(edges, np.float32(0)), edges])
    specials = np.array([0.0, -0.0, np.inf, -np.inf, 3.4e38, -3.4e38, 1e-45, -1e-45, 1.17e-38], dtype=np.float32)
    wide = (rng.standard_normal(1 << 20) * np.exp(rng.uniform(-30, 12, 1 << 20))).astype(np.float32)
    bf = all_bf16_as_f32()
    return np.concatenate([near, -near, specials, wide, bf[~np.isnan(bf)]])


def test_casts_match_oracle_bit_for_bit(dev):
    x = _cast_inputs()
    assert np.array_equal(_cast("e2m1", x, dev), O.f32_to_e2m1(x))
    assert np.array_equal(_cast("e4m3", x, dev), O.f32_to_e4m3(x))
    assert np.array_equal(_cast("e8m0", x, dev), O.f32_to_e8m0_rp(x))
    nan = np.array([np.nan, -np.nan], dtype=np.float32)  # unpinned in the reference; oracle's choice
    assert np.array_equal(_cast("e2m1", nan, dev), O.f32_to_e2m1(nan))
    assert np.array_equal(_cast("e4m3", nan, dev), O.f32_to_e4m3(nan))
    assert np.array_equal(_cast("e8m0", nan, dev), O.f32_to_e8m0_rp(nan))


def test_casts_match_golden_tables(dev):
    bf = all_bf16_as_f32()
    ok = ~np.isnan(bf)
    assert np.array_equal(_cast("e2m1", bf[ok], dev), golden("e2m1_of_bf16.npy")[ok])
    assert np.array_equal(_cast("e4m3", bf[ok], dev), golden("e4m3_of_bf16.npy")[ok])


def _quantize_gpu(x, gs, swizzle, dev, block=16, dtype=torch.float4_e2m1fn_x2):
    from fuser_amd import ops

    gst = None if gs is None else torch.tensor(gs, dtype=torch.float32, device=dev)
    q, s = ops.nv_block_quantize(x.to(dev), gst, swizzle, block, dtype)
    torch.cuda.synchronize()
    return q.view(torch.uint8).cpu(), s.view(torch.uint8).cpu()


# sizes of tests/cpp/test_low_precision_recipe.cpp:1459-1470 plus ragged ones
SIZES = [(1024, 1024), (128, 64), (2048, 128), (2048, 2048), (1000, 208), (5, 16), (129, 4112), (4096, 4096)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("use_gs", [True, False])
@pytest.mark.parametrize("swizzle", [True, False])
def test_nvfp4_quantizer_bytes_equal_oracle(dev, dtype, use_gs, swizzle):
    gen = torch.Generator().manual_seed(11)
    for m, k in SIZES:
        x = torch.randn(m, k, generator=gen).to(dtype)
        gs = gs_of(x) if use_gs else None
        rq, rs = O.block_quantize_nvfp4(x, gs, swizzle)
        q, s = _quantize_gpu(x, gs, swizzle, dev)
        assert q.shape == (m, k // 2)
        assert torch.equal(q, rq), f"payload differs at {m}x{k}"
        if swizzle:
            assert s.shape == (O.round_up(m, 128), O.round_up(k // 16, 4))
            assert torch.equal(valid_scales(s, m, k // 16), valid_scales(rs, m, k // 16)), f"scales differ at {m}x{k}"
            assert torch.equal(s, rs), "padding bytes of touched tiles must be zero"
        else:
            assert torch.equal(s, rs), f"scales differ at {m}x{k}"


def test_nvfp4_quantizer_golden_fixture(dev):
    d = golden("nvfp4_quant_128x512.npz")
    x = torch.from_numpy(d["x_bits"]).view(torch.bfloat16)
    q, s = _quantize_gpu(x, float(d["gs"]), False, dev)
    assert np.array_equal(q.numpy(), d["payload_gs"]) and np.array_equal(s.numpy(), d["scales_gs"])
    q, s = _quantize_gpu(x, None, False, dev)
    assert np.array_equal(q.numpy(), d["payload_nogs"]) and np.array_equal(s.numpy(), d["scales_nogs"])


def test_nvfp4_quantizer_special_values(dev):
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(64, 1024, generator=gen)
    x[0, :16] = 0
    x[1, 5] = float("inf")
    x[2, 17] = float("-inf")
    x[3, 40] = float("nan")       # NaN results are unpinned in the reference; the oracle's choice is tested
    x[4, 64:80] = float("nan")
    x[5, :] = 1e-30
    x[6, :] = 3e38
    x[7, 100] = -0.0
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        xd = x.to(dtype)
        for gs in (None, 3.0, 1e-3):
            rq, rs = O.block_quantize_nvfp4(xd, gs, True)
            q, s = _quantize_gpu(xd, gs, True, dev)
            assert torch.equal(q, rq) and torch.equal(s, rs), (dtype, gs)


def test_nvfp4_quantizer_large_rank_and_properties(dev):
    """BASELINE config 5 activation size (65536 x 7168): too big for the scalar oracle in a test, so
    check a row sample against it and size-independent properties on the whole result."""
    from fuser_amd import ops

    m, k = 65536, 7168
    gen = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    q, s = ops.nv_block_quantize(x, None, True, 16)
    q2, s2 = ops.nv_block_quantize(x, None, True, 16)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s.view(torch.uint8), s2.view(torch.uint8))  # deterministic
    rows = torch.randint(0, m, (256,), generator=torch.Generator().manual_seed(1))
    rows[:4] = torch.tensor([0, 127, 128, m - 1])
    xs = x[rows.to(dev)].cpu()
    rq, rs = O.block_quantize_nvfp4(xs, None, False)
    assert torch.equal(q.view(torch.uint8)[rows.to(dev)].cpu(), rq)
    # gather the sampled rows' scales out of the swizzled buffer with the index formula
    cols = torch.arange(k // 16)
    pc = k // 16
    off = ((rows // 128) * pc * 128 + (rows % 32) * 16 + ((rows % 128) // 32) * 4).view(-1, 1) + ((cols // 4) * 512 + cols % 4).view(1, -1)
    got = s.view(torch.uint8).reshape(-1)[off.to(dev)].cpu()
    assert torch.equal(got, rs)
    # every block keeps at least one element of magnitude >= 4 (amax maps into [4,6] after scaling) unless all-zero
    codes = q.view(torch.uint8)[:4096]
    mag = torch.maximum(codes & 7, (codes >> 4) & 7).reshape(4096, k // 16, 8).amax(-1)
    assert (mag >= 6).all()


def test_nvfp4_quantizer_rank3_input_and_linear_scales(dev):
    x = torch.randn(3, 40, 64).bfloat16()
    q, s = _quantize_gpu(x, None, False, dev)
    rq, rs = O.block_quantize_nvfp4(x.reshape(120, 64), None, False)
    assert q.shape == (3, 40, 32) and s.shape == (3, 40, 4)
    assert torch.equal(q.reshape(120, 32), rq) and torch.equal(s.reshape(120, 4), rs)


@pytest.mark.parametrize("sizes", [[115, 144, 8, 757], [5, 7, 9, 246], [0, 300, 0, 212], [128, 128], [1]])
def test_grouped_quantizer_bytes_equal_oracle(dev, sizes):
    from fuser_amd import ops

    m = sum(sizes)
    for k in (256, 144, 7168 if m < 400 else 512):
        x = torch.randn(m, k).bfloat16()
        io = start_offsets(sizes)
        oo = start_offsets([O.round_up(t, 128) for t in sizes])
        for gs in (None, gs_of(x)):
            gst = None if gs is None else torch.tensor(gs, dtype=torch.float32, device=dev)
            q, s = ops.nv_grouped_block_quantize(x.to(dev), io.to(dev), oo.to(dev), gst, 16)
            torch.cuda.synchronize()
            assert s.shape == (m + 127 * len(sizes), O.round_up(k // 16, 4))
            rq, rs = O.grouped_block_quantize_nvfp4(x, io, oo, gs)
            assert torch.equal(q.view(torch.uint8).cpu(), rq)
            s = s.view(torch.uint8).cpu()
            for g, t in enumerate(sizes):
                if t == 0:
                    continue
                o = int(oo[g])
                p = O.round_up(t, 128)
                assert torch.equal(valid_scales(s[o : o + p], t, k // 16), valid_scales(rs[o : o + p], t, k // 16))


def test_preprocess_grouped_sf_fixture(dev):
    # tests/cpp/test_layout_op.cpp:125-133
    from fuser_amd import ops

    d = golden("grouped_layout_m512_k9.npz")
    inp = torch.arange(512 * 9, dtype=torch.float32).reshape(512, 9)
    out = ops.preprocess_grouped_matmul_input_sf(inp.to(dev), torch.from_numpy(d["offsets"]).to(dev), torch.from_numpy(d["sf_offsets"]).to(dev))
    torch.cuda.synchronize()
    assert out.shape == (512 + 3 * 127, 12)
    got = out.cpu().numpy()[:768]
    assert np.array_equal(got[d["valid"]], d["expected"][d["valid"]])
    # k = 144 variant of test_layout_op.cpp:396-404, one-byte elements, against the oracle
    sf = torch.randint(0, 255, (512, 144), dtype=torch.uint8)
    io, oo = torch.from_numpy(d["offsets"]), torch.from_numpy(d["sf_offsets"])
    out8 = ops.preprocess_grouped_matmul_input_sf(sf.to(dev), io.to(dev), oo.to(dev)).cpu()
    ref8 = O.preprocess_grouped_sf(sf, io, oo)
    for g, (o, t) in enumerate(zip([0, 128, 384], [100, 150, 262])):
        p = O.round_up(t, 128)
        assert torch.equal(valid_scales(out8[o : o + p], t, 144), valid_scales(ref8[o : o + p], t, 144))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_mxfp8_quantizer_bytes_equal_oracle(dev, dtype):
    gen = torch.Generator().manual_seed(13)
    for m, k in [(1024, 1024), (2048, 128), (128, 64), (100, 96), (7, 32), (2048, 2048)]:
        x = (torch.randn(m, k, generator=gen) * torch.exp(torch.randn(m, 1, generator=gen) * 2)).to(dtype)
        rq, rs = O.block_quantize_mxfp8(x)
        q, s = _quantize_gpu(x, None, False, dev, 32, torch.float8_e4m3fn)
        assert torch.equal(q, rq) and torch.equal(s, rs), (m, k)
        q, s = _quantize_gpu(x, None, True, dev, 32, torch.float8_e4m3fn)
        assert torch.equal(q, rq) and torch.equal(s, O.linear_to_swizzled_128_4(rs)), (m, k)
    d = golden("mxfp8_quant_64x256.npz")
    x = torch.from_numpy(d["x_bits"]).view(torch.bfloat16)
    q, s = _quantize_gpu(x, None, False, dev, 32, torch.float8_e4m3fn)
    assert np.array_equal(q.numpy(), d["payload"]) and np.array_equal(s.numpy(), d["scales"])
    xs = torch.randn(8, 64)
    xs[0, 0], xs[1, 1], xs[2, :32] = float("inf"), float("nan"), 0.0
    rq, rs = O.block_quantize_mxfp8(xs)
    q, s = _quantize_gpu(xs, None, False, dev, 32, torch.float8_e4m3fn)
    assert torch.equal(q, rq) and torch.equal(s, rs)


def test_quantizer_through_raw_c_abi_on_a_side_stream(dev):
    from fuser_amd import capi

    x = torch.randn(300, 160).bfloat16()
    rq, rs = O.block_quantize_nvfp4(x, 2.5, True)
    xd = x.to(dev)
    gs = torch.tensor(2.5, device=dev)
    q = torch.empty(300, 80, dtype=torch.uint8, device=dev)
    s = torch.full((384, 12), 0xAA, dtype=torch.uint8, device=dev)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    capi.check(capi.lib().nvf_nvfp4_block_quantize(xd.data_ptr(), capi.BF16, 300, 160, gs.data_ptr(), 1, q.data_ptr(), s.data_ptr(),
                                                   ctypes.c_void_p(stream.cuda_stream)))
    stream.synchronize()
    assert torch.equal(q.cpu(), rq) and torch.equal(s.cpu(), rs)


def test_quantizer_division_shortcuts_equal_true_division_for_every_operand(dev):
    """amax / 6 and 1 / x inside the NVFP4 quantizer are a reciprocal plus one fused correction step; the library's
    self-check compares both with true fp32 division on the device for every fp32 pattern with biased exponent in
    [2, 250] (2.09e9 operands each) -- the range for which the kernel uses them."""
    from fuser_amd import capi

    res = torch.full((4,), 7, dtype=torch.int32, device=dev)
    capi.check(capi.lib().nvf_selftest_fast_division(res.data_ptr(), None))
    torch.cuda.synchronize()
    bad_rcp, first_rcp, bad_div, first_div = [int(v) & 0xFFFFFFFF for v in res.cpu().tolist()]
    assert bad_rcp == 0 and first_rcp == 0xFFFFFFFF, f"1/x differs for {bad_rcp} operands, first {first_rcp:#010x}"
    assert bad_div == 0 and first_div == 0xFFFFFFFF, f"x/6 differs for {bad_div} operands, first {first_div:#010x}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_nvfp4_quantizer_zero_and_tiny_blocks_next_to_ordinary_ones(dev, dtype):
    """All-zero blocks (padded or sparse activations) take the quantizer's ordinary path; blocks whose amax is
    denormal or whose scale underflows to zero sit in the same wavefronts as N(0,1) blocks: bytes equal the oracle."""
    from fuser_amd import ops

    gen = torch.Generator().manual_seed(12)
    x = torch.randn(256, 2048, generator=gen)
    blocks = x.view(256, 128, 16)
    blocks[::3, ::2] = 0.0                       # zero blocks interleaved with ordinary ones
    blocks[1::7, 1::5] *= 1e-30                  # tiny amax: the scale rounds to zero
    if dtype == torch.float32:
        blocks[2::11, 3::9] *= 1e-42             # fp32 denormals
    blocks[5, 7] = 0.0
    blocks[5, 7, 3] = 2.0 ** -20
    x = x.to(dtype)
    for gs in (None, 2688.0 / 4.5, 1e-3):
        gst = None if gs is None else torch.tensor(gs, device=dev)
        for swz in (False, True):
            q, s = ops.nv_block_quantize(x.to(dev), gst, swz, 16)
            rq, rs = O.block_quantize_nvfp4(x, gs, swz)
            assert torch.equal(q.view(torch.uint8).cpu(), rq), (gs, swz)
            assert torch.equal(s.view(torch.uint8).cpu(), rs), (gs, swz)
