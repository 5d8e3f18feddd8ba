"""Pins the oracle's 128x4 layout, block quantizers and dequantisation against the golden fixtures,
closed-form special cases and invariants."""
import numpy as np
import pytest
import torch

from helpers import golden, gs_of, start_offsets
from oracle import nvf_oracle as O


# ----------------------------------------------------------------------------- 128x4 layout
def test_swizzle_formula_matches_reshape_transpose_golden():
    gold = golden("swizzle_256x8.npy")  # built with reshape/transpose
    lin = torch.arange(256 * 8, dtype=torch.int32).reshape(256, 8)
    assert np.array_equal(O.linear_to_swizzled_128_4(lin).numpy(), gold)
    flat = gold.reshape(-1)
    for r, c in [(0, 0), (1, 0), (31, 3), (32, 0), (127, 7), (128, 0), (255, 7), (100, 5)]:
        assert flat[O.swizzle_offset(r, c, 8)] == r * 8 + c


def test_swizzle_round_trip_with_padding():
    for m, c in [(1, 1), (5, 9), (129, 3), (300, 13)]:
        lin = torch.randint(0, 255, (m, c), dtype=torch.uint8)
        sw = O.linear_to_swizzled_128_4(lin)
        assert sw.shape == (O.round_up(m, 128), O.round_up(c, 4))
        assert torch.equal(O.swizzled_to_linear_128_4(sw, m, c), lin)
        # brute-force the index formula
        flat = sw.reshape(-1)
        pc = sw.shape[1]
        for r in range(0, m, max(1, m // 7)):
            for cc in range(c):
                assert flat[O.swizzle_offset(r, cc, pc)] == lin[r, cc]


def test_grouped_layout_fixture_m512_k9():
    # tests/cpp/test_layout_op.cpp:125-133
    d = golden("grouped_layout_m512_k9.npz")
    inp = torch.arange(512 * 9, dtype=torch.float32).reshape(512, 9)
    out = O.preprocess_grouped_sf(inp, torch.from_numpy(d["offsets"]), torch.from_numpy(d["sf_offsets"]))
    assert out.shape == (768, 12)
    assert np.array_equal(out.numpy()[d["valid"]], d["expected"][d["valid"]])
    assert np.all(out.numpy()[~d["valid"]] == 0)  # nothing else written


# ----------------------------------------------------------------------------- NVFP4 quantizer
def test_nvfp4_quantizer_against_torch_op_golden():
    d = golden("nvfp4_quant_128x512.npz")
    x = torch.from_numpy(d["x_bits"]).view(torch.bfloat16)
    q, s = O.block_quantize_nvfp4(x, float(d["gs"]), False)
    assert np.array_equal(q.numpy(), d["payload_gs"]) and np.array_equal(s.numpy(), d["scales_gs"])
    q, s = O.block_quantize_nvfp4(x, None, False)
    assert np.array_equal(q.numpy(), d["payload_nogs"]) and np.array_equal(s.numpy(), d["scales_nogs"])
    # swizzled output = same bytes, other place
    q2, s2 = O.block_quantize_nvfp4(x, None, True)
    assert torch.equal(q2, q) and torch.equal(O.swizzled_to_linear_128_4(s2, 128, 32), s)


def test_nvfp4_quantizer_closed_form_blocks():
    x = torch.zeros(4, 16)
    # row 0: all zero -> scale 0, payload 0
    # row 1: amax = 6 * 2^-2 -> scale exactly 2^-2 (0x28), payload = x / 2^-2 rounded
    x[1] = torch.tensor([1.5, -1.5, 0.25, 0.5, 0.75, 1.0, 0.125, -0.125, 0.0625, 0.1875, 0.3125, 0.4375, 0, 0, 0, -0.0])
    # row 2: one huge element -> scale saturates at 448, that element becomes +-6
    x[2, 3] = -1e30
    x[2, 4] = 1.0
    # row 3: no-global-scale scale rounding: amax = 1 -> s = 1/6 -> e4m3(0.16667) = 0.171875 = 2^-3 * (1 + 3/8) (0x23)
    x[3, 0] = 1.0
    q, s = O.block_quantize_nvfp4(x, None, False)
    assert s.flatten().tolist() == [0x00, 0x28, 0x7E, 0x23]
    assert q[0].tolist() == [0] * 8
    # 1.5/.25=6 -> 7 ; .25/.25=1 -> 2 ; .5/.25=2 -> 4 ; .75/.25=3 -> 5 ; 1/.25=4 -> 6 ; .125/.25=.5 -> 1
    # .0625/.25=.25 -> tie -> 0 ; .1875/.25=.75 -> tie -> 1.0 (2) ; .3125/.25=1.25 -> 1.0 (2) ; .4375/.25=1.75 -> 2.0 (4)
    codes = [7, 15, 2, 4, 5, 6, 1, 9, 0, 2, 2, 4, 0, 0, 0, 8]
    assert q[1].tolist() == [codes[2 * j] | (codes[2 * j + 1] << 4) for j in range(8)]
    assert q[2].tolist() == [0, 0xF0, 0, 0, 0, 0, 0, 0]  # 1/448 -> 0 ; -1e30 -> -6
    # row 3: 1 / 0.171875 = 5.818 -> 6
    assert q[3, 0].item() == 0x07


def test_nvfp4_quantizer_global_scale_path_order_of_operations():
    # scale = e4m3(amax/6*gs); r = 1/(sf*(1/gs)); pick gs with an inexact reciprocal
    gs = 2688.0 / 3.7
    x = torch.zeros(1, 16)
    x[0, :4] = torch.tensor([3.7, 1.0, -2.2, 0.3])
    q, s = O.block_quantize_nvfp4(x, gs, False)
    g32 = np.float32(gs)
    sc = np.float32(np.float32(np.float32(3.7) / np.float32(6.0)) * g32)
    q8 = torch.tensor([min(sc, 448.0)], dtype=torch.float32).to(torch.float8_e4m3fn)
    assert s.item() == q8.view(torch.uint8).item() == 0x7E
    sf = np.float32(q8.float().item())
    r = np.float32(1.0) / np.float32(sf * np.float32(np.float32(1.0) / g32))
    y = (np.array([3.7, 1.0, -2.2, 0.3], dtype=np.float32) * r).astype(np.float32)
    expect = O.f32_to_e2m1(y)
    assert q[0, 0].item() == (expect[0] | (expect[1] << 4)) and q[0, 1].item() == (expect[2] | (expect[3] << 4))
    assert expect.tolist() == [7, 3, 14, 1]  # 6.0000005 -> 6 ; 1.62 -> 1.5 ; -3.57 -> -4 ; 0.486 -> 0.5


def test_nvfp4_quantizer_ignores_nan_in_amax_and_handles_inf():
    x = torch.ones(1, 32)
    x[0, 3] = float("nan")
    x[0, 20] = float("inf")
    q, s = O.block_quantize_nvfp4(x, None, False)
    # block 0: amax ignores the NaN -> same scale as an all-ones block ; NaN element -> +6 (unpinned choice)
    qr, sr = O.block_quantize_nvfp4(torch.ones(1, 32), None, False)
    assert s[0, 0] == sr[0, 0]
    assert q[0, 1].item() == ((qr[0, 1].item() & 0x0F) | 0x70)
    # block 1: inf -> scale saturates to 448, inf element -> 6, ones -> 1/448 -> 0
    assert s[0, 1].item() == 0x7E
    assert q[0, 10].item() == 0x07 and q[0, 8].item() == 0


def test_grouped_quantizer_equals_per_group_quantizer():
    sizes = [100, 0, 150, 262]
    m, k = sum(sizes), 96  # k/16 = 6 -> padded to 8
    x = torch.randn(m, k).bfloat16()
    io = start_offsets(sizes)
    oo = start_offsets([O.round_up(s, 128) for s in sizes])
    gs = gs_of(x)
    q, sf = O.grouped_block_quantize_nvfp4(x, io, oo, gs)
    assert sf.shape == (128 + 0 + 256 + 384, 8)
    row = 0
    for g, sz in enumerate(sizes):
        if sz == 0:
            continue
        qg, sg = O.block_quantize_nvfp4(x[row : row + sz], gs, True)
        assert torch.equal(q[row : row + sz], qg)
        assert torch.equal(sf[int(oo[g]) : int(oo[g]) + O.round_up(sz, 128)], sg)
        row += sz


def test_group_lookup_with_empty_groups_matches_linear_scan():
    # runtime/block_quantization_kernels.cu:387-393: first i in 1..G-1 with row < offsets[i] -> i-1, else G-1
    offsets = [0, 5, 5, 5, 9]
    x = torch.arange(12 * 16, dtype=torch.float32).reshape(12, 16)
    oo = torch.tensor([0, 128, 256, 384, 512], dtype=torch.int32)
    _, sf = O.grouped_block_quantize_nvfp4(x, torch.tensor(offsets, dtype=torch.int32), oo, None, padded_rows=640)
    _, lin = O.block_quantize_nvfp4(x, None, False)
    owner = [0] * 5 + [3] * 4 + [4] * 3
    for r in range(12):
        g = owner[r]
        assert sf.reshape(-1)[int(oo[g]) * 4 + O.swizzle_offset(r - offsets[g], 0, 4)] == lin[r, 0]


# ----------------------------------------------------------------------------- MXFP8 quantizer
def test_mxfp8_quantizer_against_torch_op_golden():
    d = golden("mxfp8_quant_64x256.npz")
    x = torch.from_numpy(d["x_bits"]).view(torch.bfloat16)
    q, s = O.block_quantize_mxfp8(x)
    assert np.array_equal(q.numpy(), d["payload"]) and np.array_equal(s.numpy(), d["scales"])


def test_mxfp8_quantizer_closed_form():
    x = torch.zeros(3, 32)
    x[1, 0] = 448.0  # amax/448 = 1 -> e = 127 -> payload 448 (0x7E)
    x[1, 1] = -224.0
    x[2, 0] = 449.0  # amax*(1/448) slightly > 1 -> round up to 2 -> e = 128 ; 449/2 = 224.5 -> 224 (0x76)
    q, s = O.block_quantize_mxfp8(x)
    assert s.flatten().tolist() == [0, 127, 128]
    assert q[0].tolist() == [0] * 32
    assert q[1, 0].item() == 0x7E and q[1, 1].item() == 0xF6
    assert q[2, 0].item() == 0x76


# ----------------------------------------------------------------------------- dequantise + matmul
def test_dequantize_scalar_and_vectorised_paths_agree_and_bound_the_error():
    torch.manual_seed(77)
    x = torch.randn(130, 160).bfloat16()
    gs = gs_of(x)
    q, s = O.block_quantize_nvfp4(x, gs, True)
    d1 = O.dequantize_nvfp4(q, s, 1.0 / gs)
    d2 = O.dequantize_nvfp4_fast(q, s, 1.0 / gs)
    assert torch.equal(d1, d2)
    # e2m1 has a relative step of at most 1/3 above 0.5*scale: the block-wise error is bounded by amax/6*... loose check
    err = (d1 - x.float()).abs().reshape(130, 10, 16).amax(-1)
    amax = x.float().abs().reshape(130, 10, 16).amax(-1)
    assert torch.all(err <= amax * 0.26)
    x8 = torch.randn(40, 96).bfloat16()
    q8, s8 = O.block_quantize_mxfp8(x8)
    sw = O.linear_to_swizzled_128_4(s8)
    assert torch.equal(O.dequantize_mxfp8(q8, sw), O.dequantize_mxfp8_fast(q8, sw))
    # e4m3 rounds to half an ulp: 2^-4 relative for normals, 2^-10 absolute (times the block scale) below 2^-6
    step = torch.exp2(s8.float() - 127.0).repeat_interleave(32, dim=1) * 2.0**-10
    bound = torch.maximum(x8.float().abs() * 2.0**-4, step)
    assert ((O.dequantize_mxfp8(q8, sw) - x8.float()).abs() <= bound).all()


def test_reference_matmul_against_python_loops():
    a = torch.randint(0, 256, (3, 16), dtype=torch.uint8)  # 3 x 32 fp4
    b = torch.randint(0, 256, (2, 16), dtype=torch.uint8)
    sa = O.linear_to_swizzled_128_4(torch.tensor([[0x38, 0x30], [0x40, 0x28], [0x3C, 0x38]], dtype=torch.uint8))
    sb = O.linear_to_swizzled_128_4(torch.tensor([[0x38, 0x38], [0x34, 0x44]], dtype=torch.uint8))
    out = O.ref_nvfp4_scaled_mm(a, b, sa, sb, 0.5, fast=False)
    lut, e4 = O.e2m1_table(), O.e4m3_table()
    sal, sbl = O.swizzled_to_linear_128_4(sa, 3, 2), O.swizzled_to_linear_128_4(sb, 2, 2)
    for i in range(3):
        for j in range(2):
            acc = 0.0
            for kk in range(32):
                av = lut[(int(a[i, kk // 2]) >> (4 * (kk & 1))) & 15] * e4[int(sal[i, kk // 16])]
                bv = lut[(int(b[j, kk // 2]) >> (4 * (kk & 1))) & 15] * e4[int(sbl[j, kk // 16])]
                acc += float(av) * float(bv)
            assert abs(out[i, j].item() - 0.5 * acc) <= 1e-5 * max(1.0, abs(acc))


def test_grouped_references_slice_like_the_pointer_rule():
    sizes = [3, 0, 5]
    a = torch.randn(8, 16).bfloat16()
    b = torch.randn(3, 8, 16).bfloat16()
    ps = torch.tensor([[s, 8, 16] for s in sizes], dtype=torch.int32)
    eo = start_offsets(sizes)
    out = O.ref_grouped_mm(a, b, ps, eo)
    assert torch.allclose(out[:3], a[:3].float() @ b[0].float().t())
    assert torch.allclose(out[3:], a[3:].float() @ b[2].float().t())
