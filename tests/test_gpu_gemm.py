"""GPU parity of the dense block-scaled GEMMs against the fp32 dequantize+matmul oracle.
Tolerance (stated by this build's target): max |out - ref| <= 1e-2 * max |ref|.  The shapes of the
reference's own tests (tests/python/direct/test_cutlass_nvfp4_gemm.py:55-100,
test_cutlass_mxfp8_gemm.py:92-124) are included verbatim with the reference's tolerances as well."""
import ctypes

import pytest
import torch

from helpers import GEMM_MAX_REL, e4m3, e8m0, fp4, gs_of, max_rel, max_rel_rowwise
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def _nvfp4_operand(rows, k, std, gen):
    x = (torch.randn(rows, k, generator=gen) * std).bfloat16()
    gs = gs_of(x)
    q, s = O.block_quantize_nvfp4(x, gs, True)
    return q, s, gs


def _run_nvfp4(a, b, sa, sb, alpha, dtype, dev):
    from fuser_amd import nvf_cutlass

    out = nvf_cutlass.nvfp4_scaled_mm(fp4(a.to(dev)), fp4(b.to(dev)), e4m3(sa.to(dev)), e4m3(sb.to(dev)),
                                      torch.tensor(alpha, dtype=torch.float32, device=dev), dtype)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(128, 128, 64), (128, 128, 128), (256, 128, 64), (128, 256, 128)])
def test_nvfp4_gemm_reference_shapes(dev, dtype, shape):
    m, n, packed_k = shape
    k = packed_k * 2
    gen = torch.Generator().manual_seed(0)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 1.0, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    out = _run_nvfp4(a, b, sa, sb, alpha, dtype, dev)
    assert out.dtype == dtype and out.shape == (m, n)
    torch.testing.assert_close(out.cpu(), ref.to(dtype), atol=1e-1, rtol=1e-1)  # the reference's own bar
    assert max_rel(out, ref) <= GEMM_MAX_REL and max_rel_rowwise(out, ref) <= GEMM_MAX_REL


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(128, 128, 64), (128, 128, 128), (256, 128, 64), (128, 256, 128)])
def test_nvfp4_gemm_epilogue_reference_shapes(dev, dtype, shape):
    """tests/python/direct/test_cutlass_nvfp4_gemm.py:103-175 with its own tolerances: operands quantized
    from `dtype` data, the expectation is the NVFP4 quantization (global scale 2) of the product rounded to
    `dtype`; then the tighter statement against the fp32 product."""
    from fuser_amd import nvf_cutlass

    m, n, packed_k = shape
    k = packed_k * 2
    gen = torch.Generator().manual_seed(0)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 1.0, gen)
    alpha = 1.0 / (ga * gb)
    norm = 2.0
    q, sf = nvf_cutlass.nvfp4_scaled_mm_blockscale(fp4(a.to(dev)), fp4(b.to(dev)), e4m3(sa.to(dev)), e4m3(sb.to(dev)),
                                                   torch.tensor(alpha, dtype=torch.float32, device=dev),
                                                   torch.tensor(norm, dtype=torch.float32, device=dev))
    torch.cuda.synchronize()
    assert q.dtype == torch.float4_e2m1fn_x2 and q.shape == (m, n // 2)
    assert sf.dtype == torch.float8_e4m3fn and sf.shape == (m, O.round_up(n // 16, 4))
    q, sf = q.view(torch.uint8).cpu(), sf.view(torch.uint8).cpu()
    lut, e4 = torch.from_numpy(O.e2m1_table()), torch.from_numpy(O.e4m3_table())

    def unpack(p):
        return torch.stack([lut[(p & 15).long()], lut[(p >> 4).long()]], dim=-1).reshape(p.shape[0], -1)

    prod = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    eq, esf = O.block_quantize_nvfp4(prod.to(dtype), norm, True)  # the reference test's expectation
    diff = (unpack(q) - unpack(eq)).abs()
    assert diff.max() <= 2.0 and (diff != 0).float().mean() < 0.1
    torch.testing.assert_close(e4[sf.long()], e4[esf.long()], atol=2e-3, rtol=0.125)
    # against the fp32 product: only a summation-order ulp can flip a code or a scale
    eq, esf = O.ref_nvfp4_scaled_mm_blockscale(a, b, sa, sb, alpha, norm)
    assert (unpack(q) != unpack(eq)).float().mean() < 2e-3 and (sf != esf).float().mean() < 2e-3


@pytest.mark.parametrize("shape", [(200, 160, 192), (4096, 3072, 256), (1920, 4096, 384), (1024, 2048, 384), (300, 544, 608), (64, 96, 64),
                                   (2176, 2048, 256), (4096, 4128, 128), (2100, 4096, 256), (4000 + 77, 2048, 384),
                                   (16, 4096, 512), (100, 14336, 256), (128, 2048, 1024), (300, 4096, 2048), (48, 1056, 384), (1000, 14336, 256),
                                   (200, 14336, 256), (100, 28672, 128)])
def test_nvfp4_gemm_epilogue_quantizes_its_own_fp32_product_bit_exactly(dev, shape):
    """Through the C ABI.  The result is quantized in the GEMM's epilogue; with a workspace the call also dumps the
    fp32 product it quantized: that agrees with the oracle product to fp32 summation noise, and payload and scales
    are bit-identical to the oracle quantizer applied to exactly that product (rows not a multiple of 128 and
    padded scale columns on the 64x64, 128x128 and 256x256 tile kernels; shapes on the persistent kernel with
    256x256 and with 128x256 tiles; the last two: M not a multiple of 128, cut into a part for the persistent kernel
    and the remaining rows for the tile kernels, whose payload and scale tiles follow the first part's; the six before the last two:
    shapes that the 16-bit op streams - one to eight activation row tiles, one to four weight tiles per workgroup, one
    and several slabs, and 104 rows streamed behind 896 on the persistent kernel - where the weight-streaming kernel's
    last stage quantizes the summed product; the two after those: the same on its form with 4 wavefronts)."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(11)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 1.0, gen)
    alpha, norm = 1.0 / (ga * gb), 2688.0 / 40.0
    d = [t.to(dev) for t in (a, b, sa, sb)]
    al, nc = torch.tensor(alpha, dtype=torch.float32, device=dev), torch.tensor(norm, dtype=torch.float32, device=dev)
    q = torch.zeros(m, n // 2, dtype=torch.uint8, device=dev)
    sf = torch.full((O.round_up(m, 128), O.round_up(n // 16, 4)), 0x55, dtype=torch.uint8, device=dev)
    ws = torch.zeros(m, n, dtype=torch.float32, device=dev)
    capi.check(capi.lib().nvf_nvfp4_scaled_mm_blockscale(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), al.data_ptr(),
                                                         nc.data_ptr(), q.data_ptr(), sf.data_ptr(), ws.data_ptr(), m, n, k, None))
    torch.cuda.synchronize()
    prod = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    assert max_rel(ws, prod) <= 1e-5
    eq, esf = O.block_quantize_nvfp4(ws.cpu(), norm, True)
    assert torch.equal(q.cpu(), eq)
    assert torch.equal(sf.cpu(), esf)  # the padding bytes of the last 128x4 tiles are zero as well
    # without the dump (what the at::Tensor layer calls): the same bytes from the one fused launch
    q2 = torch.zeros_like(q)
    sf2 = torch.full_like(sf, 0x55)
    capi.check(capi.lib().nvf_nvfp4_scaled_mm_blockscale(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), al.data_ptr(),
                                                         nc.data_ptr(), q2.data_ptr(), sf2.data_ptr(), None, m, n, k, None))
    torch.cuda.synchronize()
    assert torch.equal(q2, q) and torch.equal(sf2, sf)


def test_nvfp4_gemm_epilogue_random_shapes_and_codes(dev):
    """Sixty seeded cases over every tile kernel: arbitrary payload bytes (all sixteen e2m1 codes, both signs),
    scale codes over 2^-10..2^1, all-zero rows, several alpha and norm constants.  Payload and scales equal the
    oracle quantizer applied to the dumped fp32 product, byte for byte, padding of the scale layout included."""
    import random

    from fuser_amd import capi

    rnd = random.Random(5)
    lib = capi.lib()
    for case in range(60):
        kind = ("persistent", "half_tiles", "ragged", "tiny")[case % 4]
        if kind == "persistent":
            m, n, k = 256 * rnd.randint(1, 8), 256 * rnd.randint(1, 8), 128 * rnd.randint(2, 6)
        elif kind == "half_tiles":
            m, n, k = 128 * rnd.randint(1, 16), 256 * rnd.randint(1, 8), 128 * rnd.randint(2, 5)
        elif kind == "ragged":
            m, n, k = rnd.randint(1, 700), 32 * rnd.randint(1, 40), 32 * rnd.randint(1, 20)
        else:
            m, n, k = rnd.randint(1, 64), 32 * rnd.randint(1, 6), 32 * rnd.randint(1, 8)
        g = torch.Generator(device=dev).manual_seed(case)
        a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=dev, generator=g)
        b = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=g)
        sa = torch.randint(0x28, 0x48, (O.round_up(m, 128), O.round_up(k // 16, 4)), dtype=torch.uint8, device=dev, generator=g)
        sb = torch.randint(0x28, 0x48, (O.round_up(n, 128), O.round_up(k // 16, 4)), dtype=torch.uint8, device=dev, generator=g)
        if case % 5 == 0:
            a[rnd.randrange(m)] = 0  # a row of zero blocks
        alpha, norm = rnd.choice([1.0, 0.37, 2.0**-8]), rnd.choice([1.0, 2.0, 26.88, 1e-3])
        al, nc = torch.tensor(alpha, dtype=torch.float32, device=dev), torch.tensor(norm, dtype=torch.float32, device=dev)
        q = torch.zeros(m, n // 2, dtype=torch.uint8, device=dev)
        sf = torch.full((O.round_up(m, 128), O.round_up(n // 16, 4)), 0x55, dtype=torch.uint8, device=dev)
        ws = torch.zeros(m, n, dtype=torch.float32, device=dev)
        capi.check(lib.nvf_nvfp4_scaled_mm_blockscale(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), al.data_ptr(), nc.data_ptr(),
                                                      q.data_ptr(), sf.data_ptr(), ws.data_ptr(), m, n, k, None))
        torch.cuda.synchronize()
        eq, esf = O.block_quantize_nvfp4(ws.cpu(), norm, True)
        assert torch.equal(q.cpu(), eq) and torch.equal(sf.cpu(), esf), (kind, m, n, k, alpha, norm)
        if case % 6 == 0:  # the dumped product itself, against the oracle GEMM
            ref = O.ref_nvfp4_scaled_mm(a.cpu(), b.cpu(), sa.cpu(), sb.cpu(), alpha)
            assert max_rel(ws, ref) <= 1e-5, (kind, m, n, k)


def test_config1_quantize_then_gemm(dev):
    """BASELINE config 1: A [256,1024], B [1024,1024] N(0,1) bf16, quantized on the GPU, C = A B^T bf16."""
    from fuser_amd import nvf_cutlass, ops

    gen = torch.Generator().manual_seed(0)
    a = torch.randn(256, 1024, generator=gen).bfloat16()
    b = torch.randn(1024, 1024, generator=gen).bfloat16()
    ga, gb = gs_of(a), gs_of(b)
    qa, sa = ops.nv_block_quantize(a.to(dev), torch.tensor(ga, device=dev), True, 16)
    qb, sb = ops.nv_block_quantize(b.to(dev), torch.tensor(gb, device=dev), True, 16)
    rqa, rsa = O.block_quantize_nvfp4(a, ga, True)
    rqb, rsb = O.block_quantize_nvfp4(b, gb, True)
    assert torch.equal(qa.view(torch.uint8).cpu(), rqa) and torch.equal(sa.view(torch.uint8).cpu(), rsa)
    assert torch.equal(qb.view(torch.uint8).cpu(), rqb) and torch.equal(sb.view(torch.uint8).cpu(), rsb)
    alpha = 1.0 / (ga * gb)
    out = nvf_cutlass.nvfp4_scaled_mm(qa, qb, sa, sb, torch.tensor(alpha, device=dev), torch.bfloat16)
    ref = O.ref_nvfp4_scaled_mm(rqa, rqb, rsa, rsb, alpha)
    assert max_rel(out, ref) <= GEMM_MAX_REL
    # the quantized product also approximates the unquantized one (quantization noise ~ 10 % per element)
    full = a.float() @ b.float().t()
    assert ((out.float().cpu() - full).norm() / full.norm()).item() < 0.2


# BASELINE config 3 (dense-LLM shapes) and ragged / small cases
@pytest.mark.parametrize("shape", [(16, 4096, 4096), (128, 4096, 4096), (2048, 4096, 4096), (16, 14336, 4096),
                                   (128, 14336, 4096), (2048, 14336, 4096), (16, 4096, 14336), (128, 4096, 14336),
                                   (2048, 4096, 14336),  # the nine shapes of config 3
                                   (1, 32, 32), (300, 544, 608), (129, 96, 2080), (257, 1056, 96)])
def test_nvfp4_gemm_llm_and_ragged_shapes(dev, shape):
    from fuser_amd import ops

    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 7 + n)
    w, sw, gw = _nvfp4_operand(n, k, 0.02, gen)          # pre-quantized weights N(0, 0.02)
    x = torch.randn(m, k, generator=gen).bfloat16()
    gx = gs_of(x)
    qx, sx = ops.nv_block_quantize(x.to(dev), torch.tensor(gx, device=dev), True, 16)  # on-the-fly activations
    rqx, rsx = O.block_quantize_nvfp4(x, gx, True)
    assert torch.equal(qx.view(torch.uint8).cpu(), rqx)
    assert torch.equal(O.swizzled_to_linear_128_4(sx.view(torch.uint8).cpu(), m, k // 16), O.swizzled_to_linear_128_4(rsx, m, k // 16))
    alpha = 1.0 / (gx * gw)
    ref = O.ref_nvfp4_scaled_mm(rqx, w, rsx, sw, alpha)
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(qx.view(torch.uint8).cpu(), w, sx.view(torch.uint8).cpu(), sw, alpha, dtype, dev)
        assert max_rel(out, ref) <= GEMM_MAX_REL, (shape, dtype)
        assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype)


@pytest.mark.parametrize("shape", [(1, 32, 128), (7, 96, 256), (16, 32, 128), (17, 64, 384), (33, 160, 1152),
                                   (64, 4096, 512), (65, 2048, 256), (127, 224, 640), (128, 16384, 128),
                                   (9, 288, 384), (16, 64, 8192), (5, 13056, 1152), (20, 13120, 640), (3, 6560, 2304),
                                   (32, 6592, 128), (25, 6560, 256), (40, 6560, 384), (50, 13056, 256),
                                   (100, 13056, 384), (128, 6560, 1152), (81, 96, 2048), (129, 64, 256), (200, 6560, 384),
                                   (256, 96, 1152), (192, 512, 2048), (100, 1024, 256), (250, 2048, 384), (150, 1024, 640),
                                   (60, 160, 512), (250, 4096, 256),
                                   (16, 13056, 4352), (31, 6592, 4224), (12, 256, 6272), (32, 13120, 2176), (2, 64, 256)])
def test_nvfp4_gemm_decode_sized_activations(dev, shape):
    """M <= 256 (in one launch of slabs of 128, 64 or 32 rows, the last one ragged) with K % 128 == 0 and N % 16 == 0 takes the kernel that streams the
    weights once and splits K over the wavefronts of a workgroup, the tiles travelling through a per-wavefront ring in LDS:
    every count of 16-row activation tiles, activation rows that do not fill a tile, 1 / 2 / 4 weight-row
    tiles per workgroup with one- and two-slot rings, all four scale row groups, 1 to 8 chunks per
    wavefront (odd and even counts, wavefronts without work), poisoned scale padding, both output types,
    run-to-run determinism of the in-workgroup reduction."""
    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 31 + n)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p = sa.clone()  # NaN code in every scale byte of the padding rows
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev)
        assert out.shape == (m, n) and max_rel(out, ref) <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev))


@pytest.mark.parametrize("shape", [(200, 14336, 256), (100, 28672, 128), (256, 14336, 640), (300, 8256, 512), (256, 16384, 4096)])
def test_nvfp4_gemm_streaming_form_with_four_wavefronts(dev, shape):
    """More workgroups (128-row slabs x 64 weight rows) than compute units: the streaming kernel runs with 4 wavefronts
    per workgroup, two workgroups to a compute unit.  Ragged last slabs (72, 100 and 44 of 128 rows), K of one to five
    chunks (wavefronts without any chunk add zeros) and 32; every element compared, both output types, NaN codes in the
    scale padding of the activations, run-to-run bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p = sa.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    plan = capi.describe_dispatch("nvfp4_scaled_mm", m, n, k)
    assert plan.startswith("nvfp4_skinny_ring_kernel<RT=4,TT=8,W=4>") and ";" not in plan, plan
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev)
        assert out.shape == (m, n) and max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev))


@pytest.mark.parametrize("nk", [(1024, 2048), (2048, 4096), (4096, 2048), (6144, 2176), (4096, 7168), (8192, 1152), (14336, 640)])
def test_nvfp4_gemm_slab_height_and_weight_tiles_by_cost(dev, nk):
    """33..256 rows: the weight-streaming kernel runs as slabs of 128, 64 or 32 rows with 1, 2 or 4 weight tiles per
    workgroup, picked by a cost estimate.  Row counts on both sides of the slab heights (ragged last slabs), shapes that
    select each of the nine forms; every element compared, both output types, run-to-run bit equality."""
    from fuser_amd import capi

    n, k = nk
    gen = torch.Generator().manual_seed(n + k)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    forms = set()
    for m in (33, 48, 64, 65, 96, 100, 128, 129, 192, 200, 256):
        plan = capi.describe_dispatch("nvfp4_scaled_mm", m, n, k)
        assert plan.startswith("nvfp4_skinny_ring_kernel<"), plan
        forms.add(plan.split(" ")[0])
        a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
        alpha = 1.0 / (ga * gb)
        ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
        for dtype in (torch.bfloat16, torch.float16):
            out = _run_nvfp4(a, b, sa, sb, alpha, dtype, dev)
            assert out.shape == (m, n) and max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (m, n, k, dtype, plan)
            assert torch.equal(out, _run_nvfp4(a, b, sa, sb, alpha, dtype, dev))
    assert len(forms) >= 2, forms


@pytest.mark.parametrize("shape", [(300, 2048, 2048), (512, 1536, 2304), (384, 3072, 4096), (640, 544, 2176), (1000, 288, 2560),
                                   (257, 32, 2048), (1024, 768, 2048), (2100, 96, 4096), (512, 4096, 4096), (640, 2048, 2048),
                                   (1024, 2048, 4096), (384, 8192, 2048), (640, 8192, 2176)])
def test_nvfp4_gemm_many_rows_small_n_deep_k(dev, shape):
    """More than 256 rows with K >= 2048 and an N small enough that the workgroups of the kernel for decode-sized
    activations (one per 128 rows x 16 columns) cover the compute units at most two or three times: all slabs
    (of 128, 64 or 32 rows, 3 to 33 of them, the last one ragged: 44, 104, 1, 52 rows or whole) go side by side in
    one launch.  Every output element is compared with the oracle, with poisoned scale padding, both output
    types and run-to-run determinism."""
    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 31 + n)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p = sa.clone()  # NaN code in every scale byte of the padding rows
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev)
        assert out.shape == (m, n) and max_rel(out, ref) <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev))


@pytest.mark.parametrize("shape", [(2100, 4096, 2048), (2504, 2048, 2048), (1000, 14336, 2048), (2304 + 255, 4096, 2048), (4300, 2048, 2048), (1000, 2048, 256),
                                   (2100, 4096, 2080), (2504, 2048, 2144), (1000, 14336, 2080), (4300, 2048, 2080)])
def test_dense_gemms_with_m_not_a_multiple_of_128(dev, shape):
    """A prefill of any token count, M > 128 and not a multiple of 128.  K % 128 == 0: one launch of the persistent
    kernel whose last row tile holds fewer rows.  K % 128 != 0 (the last four shapes): MXFP8 the same with a short last
    K step as well; NVFP4 (that variant of its kernel wants whole row tiles) cut at a multiple of 128 or 256; the rows before the cut go to the persistent kernel, the 1..255
    rows after it to the weight-streaming kernel in a launch of its own, which reads its activation scales a whole
    number of 128-row scale tiles further on.  Both ops, both output types, every element against the oracle, poisoned
    scale padding, rows of the two launches next to the cut compared like all others, run-to-run bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    plans = []
    # NVFP4
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p = sa.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    plans.append(capi.describe_dispatch("nvfp4_scaled_mm", m, n, k))
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev)
        assert out.shape == (m, n) and max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype, plans[-1])
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb, alpha, dtype, dev))
    # MXFP8
    a8, sa8 = _mxfp8_operand(m, k, gen, 1.0)
    b8, sb8 = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a8, b8, sa8, sb8, 0.75)
    sa8_p = sa8.clone()
    sa8_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    plans.append(capi.describe_dispatch("mxfp8_scaled_mm", m, n, k))
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a8, b8, sa8_p, sb8, 0.75, dtype, dev)
        assert out.shape == (m, n)
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype, plans[-1])
        assert torch.equal(out, _run_mxfp8(a8, b8, sa8_p, sb8, 0.75, dtype, dev))
    if k % 128 != 0:  # NVFP4: the cut; MXFP8: one launch of the variant with a short last K step and a short last row tile
        assert "; " in plans[0] and "ragged_k" in plans[0] and "ragged_k,ragged_m" in plans[1] and "; " not in plans[1], plans
    elif shape != (1000, 2048, 256):  # (too few tiles for the persistent kernel)
        assert all("ragged_m" in p and "; " not in p for p in plans), plans


@pytest.mark.parametrize("shape", [(2048, 2432, 256), (2100, 2368, 384), (1536, 4128, 256), (640, 4224, 2048), (2048, 4224, 2048),
                                   (100, 16512, 512), (200, 12352, 512), (200, 32896, 2048)])
def test_dense_gemms_with_n_not_a_multiple_of_256(dev, shape):
    """N > 256 and not a multiple of 256: the columns up to the last multiple of 256 go to the persistent kernel, the
    remaining 32..224 columns to a launch of their own (tile kernel or weight-streaming kernel) that writes into the same
    rows of the result at the full row pitch; the second shape is cut along M as well (K % 128 != 0), the last three
    have a short last row tile in the main part (100 rows: MXFP8 only, NVFP4 streams; the last: both ops).  Both ops,
    both output types, every element against the oracle (a launch writing at the wrong pitch would show), run-to-run
    bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    plans = [capi.describe_dispatch("nvfp4_scaled_mm", m, n, k)]
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa, sb, alpha, dtype, dev)
        assert out.shape == (m, n) and max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype, plans[-1])
        assert torch.equal(out, _run_nvfp4(a, b, sa, sb, alpha, dtype, dev))
    a8, sa8 = _mxfp8_operand(m, k, gen, 1.0)
    b8, sb8 = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a8, b8, sa8, sb8, 0.75)
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    plans.append(capi.describe_dispatch("mxfp8_scaled_mm", m, n, k))
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a8, b8, sa8, sb8, 0.75, dtype, dev)
        assert out.shape == (m, n)
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype, plans[-1])
        assert torch.equal(out, _run_mxfp8(a8, b8, sa8, sb8, 0.75, dtype, dev))
    assert any("; " in p for p in plans), plans


@pytest.mark.parametrize("shape", [(2048, 2048, 2880), (512, 4096, 288), (1024, 2048, 416), (1024, 1536, 352), (4096, 5120, 2880)])
def test_mxfp8_gemm_k_not_a_multiple_of_128_on_the_persistent_kernel(dev, shape):
    """K % 128 = 32, 64 or 96 (2880 = 22 x 128 + 64): the persistent kernel's last K step is short; the bytes past the end
    of a row are the next row's and must not count, and the padding columns of the scale layout (NaN codes here, rows
    and columns) must not be read as scales.  Every element against the oracle, run-to-run bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a8, sa8 = _mxfp8_operand(m, k, gen, 1.0)
    b8, sb8 = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a8, b8, sa8, sb8, 0.75)
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    sa8_p, sb8_p = sa8.clone(), sb8.clone()
    sa8_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    sb8_p[O.linear_to_swizzled_128_4(torch.ones(n, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    plan = capi.describe_dispatch("mxfp8_scaled_mm", m, n, k)
    assert "mxfp8_gemm_256_kernel" in plan and "ragged_k" in plan, plan
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a8, b8, sa8_p, sb8_p, 0.75, dtype, dev)
        assert out.shape == (m, n) and torch.isfinite(out.float()).all()
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype, plan)
        assert torch.equal(out, _run_mxfp8(a8, b8, sa8_p, sb8_p, 0.75, dtype, dev))


@pytest.mark.parametrize("shape", [(16, 4096, 2880), (128, 5760, 2880), (300, 4096, 2880), (64, 512, 96), (7, 256, 32), (100, 1024, 4192),
                                   (33, 2048, 160), (2048, 5760, 2880)])
def test_mxfp8_gemm_k_not_a_multiple_of_128_on_the_streaming_kernel(dev, shape):
    """The same on the weight-streaming kernel (decode sizes, ragged M, and - last shape - the columns that the persistent
    kernel leaves over): the last 128-deep chunk of a row is short.  NaN codes in all scale padding."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a8, sa8 = _mxfp8_operand(m, k, gen, 1.0)
    b8, sb8 = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a8, b8, sa8, sb8, 0.75)
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    sa8_p, sb8_p = sa8.clone(), sb8.clone()
    sa8_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    sb8_p[O.linear_to_swizzled_128_4(torch.ones(n, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    plan = capi.describe_dispatch("mxfp8_scaled_mm", m, n, k)
    assert "mxfp8_skinny_kernel" in plan, plan
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a8, b8, sa8_p, sb8_p, 0.75, dtype, dev)
        assert out.shape == (m, n) and torch.isfinite(out.float()).all()
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype, plan)
        assert torch.equal(out, _run_mxfp8(a8, b8, sa8_p, sb8_p, 0.75, dtype, dev))


@pytest.mark.parametrize("shape", [(16, 4096, 2880), (128, 5760, 2880), (300, 4096, 2880), (64, 512, 96), (7, 256, 32), (100, 1024, 4192),
                                   (128, 1024, 8224), (100, 256, 8224), (200, 512, 10272), (65, 160, 9248), (300, 2048, 14368)])
def test_nvfp4_gemm_k_not_a_multiple_of_128_on_the_streaming_kernel(dev, shape):
    """K % 128 = 32, 64 or 96 on the weight-streaming kernel (all of its forms: 1, 2, 4 and 8 row tiles, several slabs,
    ragged M): the last 128-deep chunk of a row is short; the bytes past the end of a row are the next row's and the
    scale column tile past K may not exist.  NaN codes in all scale padding; every element against the oracle, both
    output types, run-to-run bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p, sb_p = sa.clone(), sb.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    sb_p[O.linear_to_swizzled_128_4(torch.ones(n, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    plan = capi.describe_dispatch("nvfp4_scaled_mm", m, n, k)
    assert plan.startswith("nvfp4_skinny_ring_kernel<") and ";" not in plan, plan
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb_p, alpha, dtype, dev)
        assert out.shape == (m, n) and torch.isfinite(out.float()).all()
        assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype, plan)
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb_p, alpha, dtype, dev))


@pytest.mark.parametrize("shape", [(2048, 4096, 4160), (2048, 4096, 2976), (4096, 5120, 2880), (4096, 4096, 1504), (2048, 5760, 2880),
                                   (2100, 4096, 2880)])
def test_nvfp4_gemm_k_not_a_multiple_of_128_on_the_persistent_kernel(dev, shape):
    """K % 128 = 32, 64 or 96 on the persistent kernel (128x256 and 256x256 tiles, an odd and an even number of spans;
    the last two shapes are cut along N and along M as well): a tile's last span is short.  NaN codes in all scale
    padding; every element against the oracle, both output types, run-to-run bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p, sb_p = sa.clone(), sb.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    sb_p[O.linear_to_swizzled_128_4(torch.ones(n, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    plan = capi.describe_dispatch("nvfp4_scaled_mm", m, n, k)
    assert "nvfp4_gemm_256_kernel<" in plan and "ragged_k" in plan, plan
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb_p, alpha, dtype, dev)
        assert out.shape == (m, n) and torch.isfinite(out.float()).all()
        assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype, plan)
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb_p, alpha, dtype, dev))


@pytest.mark.parametrize("shape", [(300, 14336, 512), (264, 12288, 256), (520, 14336, 512), (640, 14336, 384), (700, 12288, 256),
                                   (2049, 4096, 512), (390, 28672, 384), (200, 49152, 2048)])
def test_nvfp4_gemm_last_row_tile_with_fewer_rows_on_the_persistent_kernel(dev, shape):
    """M no multiple of the tile height, N % 256 == K % 128 == 0 and enough tiles: the persistent kernel's variant whose
    last row tile reads the rows past M as zero (the range of its buffer ends with the last row) and does not store
    them.  128-row tiles with 44 and 8 rows in the last one, 256-row tiles with 8 rows (the scale tile of the tile's
    second half does not exist and is not read), 128 (M % 256 == 128), 188, 1 and 134 rows, and a single 256-row tile row
    with 200 rows; 2 to 16 spans.
    NaN code in all scale padding, both output types, every element against the oracle, run-to-run bit equality; through
    the C ABI into the first M rows of a larger buffer, whose other rows keep their contents."""
    from fuser_amd import capi

    m, n, k = shape
    plan = capi.describe_dispatch("nvfp4_scaled_mm", m, n, k)
    assert plan.startswith("nvfp4_gemm_256_kernel<") and "ragged_m" in plan and ";" not in plan, plan
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    sa_p, sb_p = sa.clone(), sb.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    sb_p[O.linear_to_swizzled_128_4(torch.ones(n, k // 16, dtype=torch.uint8)) == 0] = 0x7F
    for dtype in (torch.bfloat16, torch.float16):
        out = _run_nvfp4(a, b, sa_p, sb_p, alpha, dtype, dev)
        assert out.shape == (m, n) and torch.isfinite(out.float()).all()
        assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL, (shape, dtype, plan)
        assert torch.equal(out, _run_nvfp4(a, b, sa_p, sb_p, alpha, dtype, dev))
    buf = torch.full((m + 130, n), 7.0, dtype=torch.bfloat16, device=dev)
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa_p.to(dev), sb_p.to(dev)
    al = torch.tensor(float(alpha), dtype=torch.float32, device=dev)
    capi.check(capi.lib().nvf_nvfp4_scaled_mm(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), al.data_ptr(), buf.data_ptr(),
                                              m, n, k, capi.BF16, None))
    torch.cuda.synchronize()
    assert max_rel_rowwise(buf[:m], ref) <= GEMM_MAX_REL
    assert bool((buf[m:] == 7.0).all())


@pytest.mark.parametrize("shape", [(384, 6176, 8224), (512, 5152, 8224), (640, 4224, 12320), (512, 3104, 12320),
                                   (80, 6144, 8192), (70, 8192, 7168), (72, 4736, 10752), (65, 4096, 14336)])
def test_nvfp4_gemm_split_k_with_workspace(dev, shape):
    """Fewer 128x128 output tiles than compute units and a deep K where the weight-streaming kernel (more than 256 rows in
    too many rounds of workgroups) and the persistent kernel behind a cut of N are estimated slower: with the scratch memory
    that nvf_nvfp4_scaled_mm_workspace_bytes asks for, K is split over workgroups of the tile kernel and fp32 partial
    tiles are added in a fixed order.  Ragged N / K (splits that do not divide the spans), both
    output types, against the oracle; run-to-run bit equality; a workspace that is too small, NULL or misaligned falls
    back to the kernels without one.  The last four shapes (one slab of 65..96 rows, N / 64 workgroups covering half
    the chip or less, K % 128 == 0, 28+ chunks per split, 48 Mi weights or more) split K over workgroups of the
    weight-streaming kernel instead: 2, 2, 3 and 4 splits, with 64, 56, 84 and 112 chunks, five activation row tiles."""
    from fuser_amd import capi

    m, n, k = shape
    if shape in ((80, 6144, 8192), (70, 8192, 7168), (72, 4736, 10752), (65, 4096, 14336)):
        assert "nvfp4_skinny_ring_kernel<RT=4,TT=8>" in capi.describe_dispatch("nvfp4_scaled_mm", m, n, k, 1, capi.BF16, 1 << 30)
    gen = torch.Generator().manual_seed(m + k)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    need = capi.lib().nvf_nvfp4_scaled_mm_workspace_bytes(m, n, k)
    assert need >= 2 * m * n * 4 and need % (m * n * 4) == 0
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    al = torch.tensor(alpha, dtype=torch.float32, device=dev)
    ws = torch.empty(need + 16, dtype=torch.uint8, device=dev)

    def run(dt, ws_ptr, ws_bytes):
        out = torch.full((m, n), 7.0, dtype=dt, device=dev)
        code = capi.BF16 if dt == torch.bfloat16 else capi.F16
        capi.check(capi.lib().nvf_nvfp4_scaled_mm_ws(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), al.data_ptr(),
                                                     out.data_ptr(), m, n, k, code, ws_ptr, ws_bytes, None))
        torch.cuda.synchronize()
        return out

    for dt in (torch.bfloat16, torch.float16):
        ws.fill_(0xFF)  # NaN patterns: every partial that is read must have been written
        out = run(dt, ws.data_ptr(), need)
        assert max_rel(out, ref) <= GEMM_MAX_REL, (shape, dt)
        assert torch.equal(out, run(dt, ws.data_ptr(), need))
        for ptr, size in ((None, 0), (ws.data_ptr(), need - 1), (ws.data_ptr() + 4, need)):
            assert max_rel(run(dt, ptr, size), ref) <= GEMM_MAX_REL, (shape, dt, size)
    # the at::Tensor entry point allocates the scratch itself
    assert torch.equal(_run_nvfp4(a, b, sa, sb, alpha, torch.bfloat16, dev), run(torch.bfloat16, ws.data_ptr(), need))
    # shapes that fill the chip or are served by the weight-streaming kernel ask for nothing
    assert capi.lib().nvf_nvfp4_scaled_mm_workspace_bytes(4096, 4096, 4096) == 0
    assert capi.lib().nvf_nvfp4_scaled_mm_workspace_bytes(16, 4096, 4096) == 0


def test_nvfp4_gemm_ignores_scale_padding_and_is_deterministic(dev):
    gen = torch.Generator().manual_seed(9)
    m, n, k = 100, 160, 96  # k/16 = 6 -> padded to 8 ; rows padded to 128 / 256
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 1.0, gen)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, 1.0)
    # poison the padding bytes (the reference leaves them uninitialised): NaN code 0x7F everywhere unused
    sa_p, sb_p = torch.full_like(sa, 0x7F), torch.full_like(sb, 0x7F)
    lin_a, lin_b = O.swizzled_to_linear_128_4(sa, m, k // 16), O.swizzled_to_linear_128_4(sb, n, k // 16)
    for dst, lin, rows in ((sa_p, lin_a, m), (sb_p, lin_b, n)):
        flat = dst.reshape(-1)
        for r in range(rows):
            for c in range(k // 16):
                flat[O.swizzle_offset(r, c, 8)] = lin[r, c]
    o1 = _run_nvfp4(a, b, sa_p, sb_p, 1.0, torch.bfloat16, dev)
    o2 = _run_nvfp4(a, b, sa_p, sb_p, 1.0, torch.bfloat16, dev)
    assert torch.equal(o1, o2)
    assert max_rel(o1, ref) <= GEMM_MAX_REL


def test_nvfp4_gemm_exact_on_small_integers(dev):
    """With unit scales and few terms every partial sum is an exact fp32 / bf16 number: bit-exact output."""
    m, n, k = 128, 128, 64
    gen = torch.Generator().manual_seed(4)
    a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=gen)
    b = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=gen)
    a, b = a & 0xBB, b & 0xBB  # codes with magnitude in {0, .5, 1, 1.5} -> sums are multiples of 1/4 below 2^8
    one = torch.full((128, 4), 0x38, dtype=torch.uint8)  # e4m3 1.0
    ref = O.ref_nvfp4_scaled_mm(a, b, one, one, 1.0, fast=False)
    out = _run_nvfp4(a, b, one, one, 1.0, torch.float16, dev)
    assert torch.equal(out.float().cpu(), ref)


def _mxfp8_operand(rows, k, gen, spread=1.0):
    x = (torch.randn(rows, k, generator=gen) * torch.exp(torch.randn(rows, 1, generator=gen) * spread)).bfloat16()
    q, s = O.block_quantize_mxfp8(x)
    return q, O.linear_to_swizzled_128_4(s)


def _run_mxfp8(a, b, sa, sb, alpha, dtype, dev):
    from fuser_amd import nvf_cutlass

    out = nvf_cutlass.mxfp8_scaled_mm(a.to(dev).view(torch.float8_e4m3fn), b.to(dev).view(torch.float8_e4m3fn), e8m0(sa.to(dev)),
                                      e8m0(sb.to(dev)), torch.tensor(alpha, dtype=torch.float32, device=dev), dtype)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(128, 128, 128), (128, 128, 256), (256, 128, 128), (128, 256, 256)])
def test_mxfp8_gemm_reference_shapes(dev, dtype, shape):
    m, n, k = shape
    gen = torch.Generator().manual_seed(1)
    a, sa = _mxfp8_operand(m, k, gen, 0.0)
    b, sb = _mxfp8_operand(n, k, gen, 0.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 1.0)
    out = _run_mxfp8(a, b, sa, sb, 1.0, dtype, dev)
    # The reference's test uses assert_close's defaults (fp16: rtol 1e-3, atol 1e-5), which only hold when
    # both sides accumulate in the same order; an independent kernel differs by a rounding step of the
    # output type on a few elements.  Bar here: 2 output ulps relative, plus 1e-3 of the largest output.
    ulp2 = 2.0**-9 if dtype == torch.float16 else 2.0**-6
    torch.testing.assert_close(out.float().cpu(), ref, rtol=ulp2, atol=1e-3 * ref.abs().max().item())
    assert max_rel(out, ref) <= GEMM_MAX_REL


@pytest.mark.parametrize("shape", [(512, 384, 1024), (100, 48, 160), (1, 16, 32), (1024, 1024, 1024), (300, 272, 96), (2048, 2048, 4096)])
def test_mxfp8_gemm_ragged_shapes_alpha_and_scale_spread(dev, shape):
    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa = _mxfp8_operand(m, k, gen, 3.0)  # rows with very different magnitudes -> wide range of e8m0 codes
    b, sb = _mxfp8_operand(n, k, gen, 3.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 0.37)
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a, b, sa, sb, 0.37, dtype, dev)
        # rows differ by orders of magnitude: compare row-normalised
        scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        err = ((out.float().cpu() - ref).abs() / scale).max().item()
        assert err <= GEMM_MAX_REL, (shape, dtype, err)


@pytest.mark.parametrize("shape", [(4096, 3072, 512), (3328, 3840, 384), (2048, 6144, 256), (8192, 1536, 1152),
                                   (4096, 8192, 256), (8192, 4096, 384), (4608, 5120, 128 * 5),
                                   (4096, 2048, 512), (4352, 4096, 384), (1920, 4096, 256), (1024, 2048, 384),
                                   (4096, 1536, 256), (2048, 3840, 256), (4096, 1280, 256)])
def test_nvfp4_gemm_persistent_256_tile_kernel_full_compare(dev, shape):
    """Dense shapes with M % 128 == N % 256 == K % 128 == 0 take the persistent kernel that converts the
    operands to fp16 between its MFMAs, with 256x256 tiles (192, 195, 192, 192, 512, 512 and 360 tiles on 256
    compute units: blocked and unblocked tile grids, one and several tiles per workgroup with two, three, five
    and nine 128-deep spans per tile) or with 128x256 tiles where those fill the compute units better
    ((4096, 2048): 256 tiles; (4352, 4096): 544, i.e. two and three per workgroup; (1920, 4096): 240, M no
    multiple of 256); (1024, 2048) with 64 such tiles falls to the 128x128 tile kernel; the last three: 6, 15 and 5
    n-tiles, i.e. blocks of 8 (m) x 2, 3 and 1 (n) after the 8 x 4 blocks of the tile walk.  Every output element
    is compared with the oracle."""
    m, n, k = shape
    gen = torch.Generator().manual_seed(k + 1)
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 0.02, gen)
    alpha = 1.0 / (ga * gb)
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    out = _run_nvfp4(a, b, sa, sb, alpha, torch.bfloat16, dev)
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL
    assert torch.equal(out, _run_nvfp4(a, b, sa, sb, alpha, torch.bfloat16, dev))
    out16 = _run_nvfp4(a, b, sa, sb, alpha, torch.float16, dev)
    assert ((out16.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL


@pytest.mark.parametrize("n_cols", [6144, 4096])  # 256x256 persistent kernel, 128x128 tile kernel
@pytest.mark.parametrize("scale_range", [(0x01, 0x0F), (0x01, 0x7E), (0x70, 0x7E)])
def test_nvfp4_gemm_persistent_kernel_every_scale_code_is_decoded_exactly(dev, scale_range, n_cols):
    """Random payload bytes and random e4m3 scale bytes, including the subnormal codes 0x01..0x07 and the
    largest finite ones: each e2m1 x e4m3 product is exactly representable in fp16, so the only error
    left is the fp32 summation order and the bf16 rounding of the output."""
    m, n, k = 2048, n_cols, 256
    gen = torch.Generator().manual_seed(scale_range[0] * 131 + scale_range[1])
    a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=gen)
    b = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=gen)
    lo, hi = scale_range
    sa = O.linear_to_swizzled_128_4(torch.randint(lo, hi + 1, (m, k // 16), dtype=torch.uint8, generator=gen))
    sb = O.linear_to_swizzled_128_4(torch.randint(lo, hi + 1, (n, k // 16), dtype=torch.uint8, generator=gen))
    alpha = 2.0 ** -12 if hi > 0x40 else 1.0
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    out = _run_nvfp4(a, b, sa, sb, alpha, torch.bfloat16, dev)
    # row-wise: 2^-8 (half a bf16 ulp) of the largest magnitude plus fp32 summation noise
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-38)
    assert ((out.float().cpu() - ref).abs() / scale).max().item() <= 2.0 ** -7


@pytest.mark.parametrize("shape", [(1, 16, 128), (7, 96, 256), (16, 48, 384), (17, 304, 1152), (32, 6560, 128), (33, 160, 2048),
                                   (64, 4096, 512), (5, 6592, 1152), (20, 6560, 640), (50, 6560, 256), (16, 64, 8192),
                                   (9, 288, 3200), (48, 144, 1024), (100, 96, 384), (128, 6560, 256), (200, 64, 1152),
                                   (256, 160, 512), (129, 32, 128), (100, 13056, 128), (192, 512, 2048), (100, 1024, 256),
                                   (250, 2048, 384), (150, 1024, 640), (128, 13120, 256)])
def test_mxfp8_gemm_decode_sized_activations(dev, shape):
    """M <= 256 (in one launch of slabs of 128, 64 or 32 rows, the last one ragged; height and weight tiles per workgroup
    by a cost estimate) with K % 128 == 0 and N % 16 == 0 takes the kernel that streams the weights once through
    per-wavefront LDS rings into v_mfma_scale_f32_16x16x128_f8f6f4: 1 / 2 / 4 / 8 activation tiles, 1 / 2 / 4
    weight-row tiles per workgroup (rings of 3, 2 and 1 slots), activation rows that do not fill a tile,
    all four scale row groups, 1 to 8 chunks per wavefront (wavefronts without work, ring wrap), scales
    spread over many octaves, poisoned scale padding, both output types, run-to-run determinism."""
    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 31 + n)
    a, sa = _mxfp8_operand(m, k, gen, 1.0)
    b, sb = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 0.75)
    sa_p = sa.clone()  # NaN code in every scale byte of the padding rows / columns
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a, b, sa_p, sb, 0.75, dtype, dev)
        assert out.shape == (m, n)
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_mxfp8(a, b, sa_p, sb, 0.75, dtype, dev))


@pytest.mark.parametrize("shape", [(100, 14336, 640), (160, 7168, 2048), (250, 7744, 256), (192, 6144, 128), (48, 28672, 384),
                                   (128, 14336, 4096)])
def test_mxfp8_gemm_streaming_form_with_four_wavefronts(dev, shape):
    """More 64-row x 64-column workgroups than compute units, at most twice as many: the form with 4 wavefronts and a
    one-slot ring, of which two workgroups share a compute unit, so that one round does.  Ragged last slabs (36, 32 and 58 of
    64 rows, one slab of 48), K of one and two chunks (wavefronts without any chunk add zeros); every element compared,
    both output types, NaN codes in all scale padding, run-to-run bit equality."""
    from fuser_amd import capi

    m, n, k = shape
    gen = torch.Generator().manual_seed(m + n + k)
    a, sa = _mxfp8_operand(m, k, gen, 1.0)
    b, sb = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 0.75)
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    sa_p, sb_p = sa.clone(), sb.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    sb_p[O.linear_to_swizzled_128_4(torch.ones(n, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    plan = capi.describe_dispatch("mxfp8_scaled_mm", m, n, k)
    assert plan.startswith("mxfp8_skinny_kernel<RT=4,TT=4,W=4>") and ";" not in plan, plan
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a, b, sa_p, sb_p, 0.75, dtype, dev)
        assert out.shape == (m, n) and torch.isfinite(out.float()).all()
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_mxfp8(a, b, sa_p, sb_p, 0.75, dtype, dev))


@pytest.mark.parametrize("nk", [(1024, 2048), (2048, 4096), (4096, 2048), (6144, 2176), (4096, 7168), (8192, 1152), (14336, 640),
                                (528, 2176), (2080, 1152), (1040, 4096)])
def test_mxfp8_gemm_slab_height_and_weight_tiles_by_cost(dev, nk):
    """33..256 rows (and more, while the estimate prefers it to the persistent kernel): the weight-streaming kernel runs
    as slabs of 128, 64 or 32 rows with 1, 2 or 4 weight tiles per workgroup, picked by a cost estimate.  Row counts on
    both sides of the slab heights (ragged last slabs), shapes that select each form; every element compared, both
    output types, run-to-run bit equality."""
    from fuser_amd import capi

    n, k = nk
    gen = torch.Generator().manual_seed(n + k)
    b, sb = _mxfp8_operand(n, k, gen, 1.0)
    forms = set()
    for m in (33, 48, 64, 65, 96, 100, 128, 129, 192, 200, 256, 384, 520):
        plan = capi.describe_dispatch("mxfp8_scaled_mm", m, n, k)
        forms.add(plan.split(" ")[0])
        a, sa = _mxfp8_operand(m, k, gen, 1.0)
        ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 0.75)
        scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        for dtype in (torch.bfloat16, torch.float16):
            if dtype == torch.float16 and ref.abs().max() > 6e4:
                continue
            out = _run_mxfp8(a, b, sa, sb, 0.75, dtype, dev)
            assert out.shape == (m, n)
            assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (m, n, k, dtype, plan)
            assert torch.equal(out, _run_mxfp8(a, b, sa, sb, 0.75, dtype, dev))
    assert any(f.startswith("mxfp8_skinny_kernel<") for f in forms), forms


@pytest.mark.parametrize("shape", [(300, 2048, 2048), (512, 1536, 2304), (384, 3072, 2048), (640, 528, 2176), (1000, 272, 2560),
                                   (257, 16, 2048), (1024, 768, 2048), (2100, 96, 4096)])
def test_mxfp8_gemm_many_rows_small_n_deep_k(dev, shape):
    """More than 256 rows with K >= 2048 and an N small enough that the workgroups of the kernel for decode-sized
    activations (one per 128 rows x 16 columns) cover the compute units at most three times: all slabs go in one
    launch (3 to 66 slabs of 128, 64 or 32 rows), the last one ragged (44, 104, 1, 52 rows or whole).  Every output
    element is compared with the oracle, with poisoned scale padding, both output types and run-to-run determinism."""
    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 31 + n)
    a, sa = _mxfp8_operand(m, k, gen, 1.0)
    b, sb = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 0.75)
    sa_p = sa.clone()  # NaN code in every scale byte of the padding rows / columns
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a, b, sa_p, sb, 0.75, dtype, dev)
        assert out.shape == (m, n)
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_mxfp8(a, b, sa_p, sb, 0.75, dtype, dev))


@pytest.mark.parametrize("shape", [(4096, 2048, 512), (2560, 3328, 384), (2048, 4096, 256), (8192, 1024, 1152),
                                   (4096, 8192, 256), (8192, 4096, 384), (4352, 4096, 640), (1152, 2048, 384),
                                   (256, 13312, 256), (128, 28672, 384), (256, 10240, 512),
                                   (4096, 1536, 256), (2048, 3840, 256), (4096, 1280, 256)])
def test_mxfp8_gemm_persistent_256_tile_kernel_full_compare(dev, shape):
    """Shapes with N % 256 == K % 128 == 0 and M % 128 == 0 take the persistent LDS-direct kernel with
    256x256 tiles ((2560, 3328): a tile grid that is not a multiple of the 8 x 4 blocking; the two 512-tile
    shapes: two tiles per workgroup, so that the load stream wraps across tiles) or with 128x256 tiles where
    those fill the compute units better (the 128-tile shapes, 272 tiles, and M = 1152, which is no multiple
    of 256); two, three, five and nine K steps per tile; 128 and 256 rows with an N so wide that one round of
    128x256 tiles beats the kernel for decode-sized activations.  Every output element is compared with the
    oracle."""
    m, n, k = shape
    gen = torch.Generator().manual_seed(k)
    a, sa = _mxfp8_operand(m, k, gen, 1.0)
    b, sb = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 1.5)
    out = _run_mxfp8(a, b, sa, sb, 1.5, torch.bfloat16, dev)
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL
    out2 = _run_mxfp8(a, b, sa, sb, 1.5, torch.bfloat16, dev)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("shape", [(300, 14336, 512), (136, 12288, 512), (80, 28672, 256), (520, 14336, 512), (640, 14336, 1024),
                                   (700, 12288, 256), (2049, 4096, 512), (390, 8192, 1280), (200, 65536, 256), (130, 65536, 256),
                                   (300, 14336, 352), (520, 14336, 288), (700, 12288, 320), (1000, 5632, 2880)])
def test_mxfp8_gemm_last_row_tile_with_fewer_rows_on_the_persistent_kernel(dev, shape):
    """M no multiple of the tile height, N % 256 == K % 128 == 0 and enough tiles: the persistent kernel's variant whose
    last row tile clamps the rows of its activation loads and stores only the rows that exist.  128-row tiles with 44,
    8 and 80 rows in the last one (one tile row in all for the 80), 256-row tiles with 8 rows (the tile's second scale
    tile does not exist: the last one is read instead), 128 (M % 256 == 128), 188 and 1 row, and a single 256-row tile row
    with 200 and 130 rows; two to ten K steps; the last four shapes with a short last K step as well (K % 128 = 96, 32,
    64, 64).  NaN
    code in every scale byte of the padding rows, both output types, every element compared, rows are written once
    (a result buffer pre-filled with a pattern keeps it past row M), run-to-run determinism."""
    from fuser_amd import capi

    m, n, k = shape
    plan = capi.describe_dispatch("mxfp8_scaled_mm", m, n, k)
    assert plan.startswith("mxfp8_gemm_256_kernel<") and "ragged_m" in plan and ";" not in plan, plan
    gen = torch.Generator().manual_seed(m * 31 + n)
    a, sa = _mxfp8_operand(m, k, gen, 1.0)
    b, sb = _mxfp8_operand(n, k, gen, 1.0)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 0.75)
    sa_p = sa.clone()
    sa_p[O.linear_to_swizzled_128_4(torch.ones(m, k // 32, dtype=torch.uint8)) == 0] = 0xFF
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    for dtype in (torch.bfloat16, torch.float16):
        if dtype == torch.float16 and ref.abs().max() > 6e4:
            continue
        out = _run_mxfp8(a, b, sa_p, sb, 0.75, dtype, dev)
        assert out.shape == (m, n)
        assert ((out.float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL, (shape, dtype)
        assert torch.equal(out, _run_mxfp8(a, b, sa_p, sb, 0.75, dtype, dev))
    # through the C ABI into the first M rows of a larger buffer: the rows after them keep their contents
    from fuser_amd import capi as C
    buf = torch.full((m + 130, n), 7.0, dtype=torch.bfloat16, device=dev)
    ad, bd = a.to(dev), b.to(dev)
    sad, sbd = sa_p.to(dev), sb.to(dev)
    alpha = torch.tensor(0.75, dtype=torch.float32, device=dev)
    C.check(C.lib().nvf_mxfp8_scaled_mm(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), alpha.data_ptr(), buf.data_ptr(),
                                        m, n, k, C.BF16, None))
    torch.cuda.synchronize()
    assert ((buf[:m].float().cpu() - ref).abs() / scale).max().item() <= GEMM_MAX_REL
    assert bool((buf[m:] == 7.0).all())


def test_mxfp8_gemm_8192_cubed_sampled_against_oracle(dev):
    """BASELINE config 2 at full size.  The CPU oracle is applied to a sample of output rows/columns;
    determinism and the K-split additivity property are checked on the whole output."""
    from fuser_amd import nvf_cutlass, ops

    m = n = k = 8192
    gen = torch.Generator(device=dev).manual_seed(2)
    a = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    b = torch.randn(n, k, device=dev, generator=gen).bfloat16()
    qa, sa = ops.nv_block_quantize(a, None, True, 32, torch.float8_e4m3fn)
    qb, sb = ops.nv_block_quantize(b, None, True, 32, torch.float8_e4m3fn)
    one = torch.tensor(1.0, device=dev)
    out = nvf_cutlass.mxfp8_scaled_mm(qa, qb, sa, sb, one, torch.bfloat16)
    out2 = nvf_cutlass.mxfp8_scaled_mm(qa, qb, sa, sb, one, torch.bfloat16)
    assert torch.equal(out, out2)
    rows = torch.randint(0, m, (48,), generator=torch.Generator().manual_seed(3))
    cols = torch.randint(0, n, (64,), generator=torch.Generator().manual_seed(4))
    rows[:3] = torch.tensor([0, 255, m - 1])
    cols[:3] = torch.tensor([0, 256, n - 1])
    sal = O.swizzled_to_linear_128_4(sa.view(torch.uint8).cpu(), m, k // 32)
    sbl = O.swizzled_to_linear_128_4(sb.view(torch.uint8).cpu(), n, k // 32)
    ra = qa.view(torch.uint8)[rows.to(dev)].cpu()
    rb = qb.view(torch.uint8)[cols.to(dev)].cpu()
    ref = O.ref_mxfp8_scaled_mm(ra, rb, O.linear_to_swizzled_128_4(sal[rows]), O.linear_to_swizzled_128_4(sbl[cols]), 1.0)
    got = out[rows.to(dev)][:, cols.to(dev)]
    assert max_rel(got, ref) <= GEMM_MAX_REL
    # additivity over K halves, fp16 outputs of the halves summed in fp32 vs the full product
    h = k // 2
    def half(lo):
        sl = slice(lo, lo + h)
        sah = O.linear_to_swizzled_128_4(sal[:, lo // 32 : (lo + h) // 32]).to(dev)
        sbh = O.linear_to_swizzled_128_4(sbl[:, lo // 32 : (lo + h) // 32]).to(dev)
        return nvf_cutlass.mxfp8_scaled_mm(qa[:, sl].contiguous(), qb[:, sl].contiguous(), e8m0(sah), e8m0(sbh), one, torch.bfloat16).float()
    total = half(0) + half(h)
    denom = out.float().abs().max()
    assert ((total - out.float()).abs().max() / denom).item() <= GEMM_MAX_REL


def test_nvfp4_gemm_8192_cubed_sampled_against_oracle(dev):
    """The NVFP4 GEMM at the size the metric names (M=N=K=8192: four 256x256 tiles per workgroup of the persistent
    kernel, 64 spans of K per tile).  The CPU oracle is applied to a sample of output rows / columns (row-wise
    tolerance); determinism and additivity over the two halves of K are checked on the whole output."""
    from fuser_amd import nvf_cutlass, ops

    m = n = k = 8192
    gen = torch.Generator(device=dev).manual_seed(5)
    a = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    b = (torch.randn(n, k, device=dev, generator=gen) * 0.02).bfloat16()
    ga, gb = (2688.0 / a.float().abs().max()).float(), (2688.0 / b.float().abs().max()).float()
    qa, sa = ops.nv_block_quantize(a, ga, True, 16)
    qb, sb = ops.nv_block_quantize(b, gb, True, 16)
    del a, b
    alpha = (1.0 / (ga * gb)).float()
    out = nvf_cutlass.nvfp4_scaled_mm(qa, qb, sa, sb, alpha, torch.bfloat16)
    assert torch.equal(out, nvf_cutlass.nvfp4_scaled_mm(qa, qb, sa, sb, alpha, torch.bfloat16))
    rows = torch.randint(0, m, (48,), generator=torch.Generator().manual_seed(3))
    cols = torch.randint(0, n, (64,), generator=torch.Generator().manual_seed(4))
    rows[:4] = torch.tensor([0, 255, 256, m - 1])
    cols[:4] = torch.tensor([0, 255, 256, n - 1])
    sal = O.swizzled_to_linear_128_4(sa.view(torch.uint8).cpu(), m, k // 16)
    sbl = O.swizzled_to_linear_128_4(sb.view(torch.uint8).cpu(), n, k // 16)
    ra, rb = qa.view(torch.uint8)[rows.to(dev)].cpu(), qb.view(torch.uint8)[cols.to(dev)].cpu()
    ref = O.ref_nvfp4_scaled_mm(ra, rb, O.linear_to_swizzled_128_4(sal[rows]), O.linear_to_swizzled_128_4(sbl[cols]), float(alpha))
    got = out[rows.to(dev)][:, cols.to(dev)]
    assert max_rel(got, ref) <= GEMM_MAX_REL and max_rel_rowwise(got, ref) <= GEMM_MAX_REL
    h = k // 2

    def half(lo):  # fp16 results of one half of K
        sah = O.linear_to_swizzled_128_4(sal[:, lo // 16 : (lo + h) // 16]).to(dev)
        sbh = O.linear_to_swizzled_128_4(sbl[:, lo // 16 : (lo + h) // 16]).to(dev)
        qah = qa.view(torch.uint8)[:, lo // 2 : (lo + h) // 2].contiguous()
        qbh = qb.view(torch.uint8)[:, lo // 2 : (lo + h) // 2].contiguous()
        return nvf_cutlass.nvfp4_scaled_mm(fp4(qah), fp4(qbh), e4m3(sah), e4m3(sbh), alpha, torch.bfloat16).float()

    total = half(0) + half(h)
    assert ((total - out.float()).abs().max() / out.float().abs().max()).item() <= GEMM_MAX_REL


def test_gemm_through_raw_c_abi(dev):
    from fuser_amd import capi

    gen = torch.Generator().manual_seed(21)
    m, n, k = 192, 160, 256
    a, sa, ga = _nvfp4_operand(m, k, 1.0, gen)
    b, sb, gb = _nvfp4_operand(n, k, 1.0, gen)
    alpha = torch.tensor(1.0 / (ga * gb), device=dev)
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    capi.check(capi.lib().nvf_nvfp4_scaled_mm(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), alpha.data_ptr(),
                                              out.data_ptr(), m, n, k, capi.BF16, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    assert max_rel(out, O.ref_nvfp4_scaled_mm(a, b, sa, sb, float(alpha))) <= GEMM_MAX_REL
    a8, s8a = _mxfp8_operand(m, k, gen)
    b8, s8b = _mxfp8_operand(n, k, gen)
    a8d, b8d, s8ad, s8bd = a8.to(dev), b8.to(dev), s8a.to(dev), s8b.to(dev)
    one = torch.tensor(1.0, device=dev)
    out16 = torch.empty(m, n, dtype=torch.float16, device=dev)
    capi.check(capi.lib().nvf_mxfp8_scaled_mm(a8d.data_ptr(), b8d.data_ptr(), s8ad.data_ptr(), s8bd.data_ptr(), one.data_ptr(),
                                              out16.data_ptr(), m, n, k, capi.F16, None))
    torch.cuda.synchronize()
    assert max_rel(out16, O.ref_mxfp8_scaled_mm(a8, b8, s8a, s8b, 1.0)) <= GEMM_MAX_REL


def test_dense_ops_reject_bad_inputs_on_device(dev):
    from fuser_amd import nvf_cutlass

    a = fp4(torch.zeros(128, 32, dtype=torch.uint8, device=dev))
    sa = e4m3(torch.zeros(128, 4, dtype=torch.uint8, device=dev))
    alpha = torch.tensor(1.0, device=dev)
    with pytest.raises(RuntimeError, match="Unsupported output data type"):
        nvf_cutlass.nvfp4_scaled_mm(a, a, sa, sa, alpha, torch.float32)
    with pytest.raises(RuntimeError, match="scale_a must be padded and swizzled"):
        nvf_cutlass.nvfp4_scaled_mm(a, a, e4m3(torch.zeros(64, 4, dtype=torch.uint8, device=dev)), sa, alpha, torch.bfloat16)
    with pytest.raises(RuntimeError, match="Expected FP8_E4M3 for Blockscale scale_a"):
        nvf_cutlass.nvfp4_scaled_mm(a, a, sa.view(torch.uint8), sa, alpha, torch.bfloat16)
    with pytest.raises(RuntimeError, match="Expected FP32 for alpha"):
        nvf_cutlass.nvfp4_scaled_mm(a, a, sa, sa, alpha.half(), torch.bfloat16)
    with pytest.raises(RuntimeError, match="is not divisible by"):
        nvf_cutlass.nvfp4_scaled_mm(fp4(torch.zeros(128, 24, dtype=torch.uint8, device=dev)), fp4(torch.zeros(128, 24, dtype=torch.uint8, device=dev)), sa, sa, alpha, torch.bfloat16)
    with pytest.raises(RuntimeError, match="contiguous"):
        nvf_cutlass.nvfp4_scaled_mm(fp4(torch.zeros(128, 64, dtype=torch.uint8, device=dev)[:, ::2]), a, sa, sa, alpha, torch.bfloat16)
    assert nvf_cutlass.get_sm_version() == 950 and nvf_cutlass.get_multiprocessor_count() == 256
