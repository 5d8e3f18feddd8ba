"""Seeded random-shape sweep of every GEMM entry point against the oracle: the shapes are drawn so that
all kernel variants and their dispatch borders are hit (decode-sized / persistent 256-tile / general
tiles of 256, 128 and 64; tile grids that are and are not multiples of the XCD blocking; K with one to
many steps; ragged M and N)."""
import pytest
import torch

from helpers import GEMM_MAX_REL, e4m3, e8m0, fp4, gs_of, start_offsets
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def _rowwise_rel(out, ref):
    scale = ref.abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    return ((out.float().cpu() - ref).abs() / scale).max().item()


def _shapes(seed, count, m_choices, n_choices, k_choices):
    gen = torch.Generator().manual_seed(seed)
    pick = lambda c: c[int(torch.randint(0, len(c), (1,), generator=gen))]
    return [(pick(m_choices), pick(n_choices), pick(k_choices)) for _ in range(count)]


NVFP4_SHAPES = (_shapes(1, 10, [1, 3, 16, 31, 64, 100, 128], [32, 96, 512, 2080, 4096], [128, 256, 640, 1152])  # decode-sized
                + _shapes(2, 6, [2048, 2304, 4096], [2048, 2560, 4096], [256, 384, 512])                        # persistent
                + _shapes(3, 10, [129, 200, 257, 515, 1000], [32, 160, 288, 1056], [32, 96, 160, 416]))         # general


@pytest.mark.parametrize("shape", NVFP4_SHAPES)
def test_nvfp4_scaled_mm_random_shapes(dev, shape):
    from fuser_amd import nvf_cutlass

    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 1000003 + n * 1009 + k)
    a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=gen)
    b = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=gen)
    sa = O.linear_to_swizzled_128_4(torch.randint(0x20, 0x50, (m, k // 16), dtype=torch.uint8, generator=gen))
    sb = O.linear_to_swizzled_128_4(torch.randint(0x20, 0x50, (n, k // 16), dtype=torch.uint8, generator=gen))
    alpha = 0.75
    ref = O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)
    out = nvf_cutlass.nvfp4_scaled_mm(fp4(a.to(dev)), fp4(b.to(dev)), e4m3(sa.to(dev)), e4m3(sb.to(dev)),
                                      torch.tensor(alpha, device=dev), torch.bfloat16)
    torch.cuda.synchronize()
    assert out.shape == (m, n) and _rowwise_rel(out, ref) <= GEMM_MAX_REL


MXFP8_SHAPES = (_shapes(4, 6, [2048, 2304, 4096], [2048, 2560, 4096], [256, 384, 640])      # persistent
                + _shapes(5, 12, [1, 17, 128, 200, 515, 1000], [16, 48, 256, 1040], [32, 96, 128, 416]))  # general


@pytest.mark.parametrize("shape", MXFP8_SHAPES)
def test_mxfp8_scaled_mm_random_shapes(dev, shape):
    from fuser_amd import nvf_cutlass

    m, n, k = shape
    gen = torch.Generator().manual_seed(m * 1000003 + n * 1009 + k + 1)

    def operand(rows):
        q = torch.randint(0, 256, (rows, k), dtype=torch.uint8, generator=gen)
        q[(q & 0x7F) == 0x7F] = 0x3C  # no NaN payload codes
        s = O.linear_to_swizzled_128_4(torch.randint(120, 134, (rows, k // 32), dtype=torch.uint8, generator=gen))
        return q, s

    a, sa = operand(m)
    b, sb = operand(n)
    ref = O.ref_mxfp8_scaled_mm(a, b, sa, sb, 1.25)
    out = nvf_cutlass.mxfp8_scaled_mm(a.to(dev).view(torch.float8_e4m3fn), b.to(dev).view(torch.float8_e4m3fn), e8m0(sa.to(dev)),
                                      e8m0(sb.to(dev)), torch.tensor(1.25, device=dev), torch.bfloat16)
    torch.cuda.synchronize()
    assert out.shape == (m, n) and _rowwise_rel(out, ref) <= GEMM_MAX_REL


def _random_sizes(gen, groups, total):
    cuts = torch.sort(torch.randint(0, total + 1, (groups - 1,), generator=gen)).values.tolist()
    sizes = [b - a for a, b in zip([0] + cuts, cuts + [total])]
    sizes[int(torch.randint(0, groups, (1,), generator=gen))] += 0
    return sizes


@pytest.mark.parametrize("case", [(3, 700, 64, 96, torch.bfloat16), (6, 2000, 264, 136, torch.float16), (5, 4096, 2048, 128, torch.bfloat16),
                                  (9, 4608, 1024, 320, torch.float16), (2, 4100, 2304, 64, torch.bfloat16), (17, 300, 128, 72, torch.bfloat16)])
def test_grouped_mm_random_groups(dev, case):
    from fuser_amd import nvf_cutlass

    groups, m, n, k, dtype = case
    gen = torch.Generator().manual_seed(groups * 7919 + m)
    sizes = _random_sizes(gen, groups, m)
    a = torch.randn(m, k, generator=gen).to(dtype)
    b = (torch.randn(groups, n, k, generator=gen) * 0.1).to(dtype)
    ps = torch.tensor([[t, n, k] for t in sizes], dtype=torch.int32)
    eo = start_offsets(sizes)
    st = torch.full((groups,), k, dtype=torch.int64, device=dev)
    ct = torch.full((groups,), n, dtype=torch.int64, device=dev)
    out = nvf_cutlass.grouped_mm(a.to(dev), b.to(dev), st, ct, ps.to(dev), eo.to(dev))
    torch.cuda.synchronize()
    ref = O.ref_grouped_mm(a, b, ps, eo)
    assert _rowwise_rel(out, ref) <= GEMM_MAX_REL


@pytest.mark.parametrize("case", [(4, 600, 128, 128), (7, 1500, 256, 192), (3, 2048, 512, 320), (12, 900, 384, 64),
                                  # prefill-sized with many small experts and a deep K: every kernel of the grouped op in one call
                                  (40, 2600, 512, 4096), (33, 2200, 1024, 4224), (64, 4200, 512, 4352)])
def test_nvfp4_scaled_grouped_mm_random_groups(dev, case):
    from fuser_amd import nvf_cutlass, ops

    groups, m, n, k = case
    gen = torch.Generator().manual_seed(groups * 104729 + m)
    sizes = _random_sizes(gen, groups, m)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(groups, n, k, generator=gen) * 0.05).bfloat16()
    eo = start_offsets(sizes)
    so = start_offsets([O.round_up(s, 128) for s in sizes])
    gx = gs_of(x)
    qx, sx = O.grouped_block_quantize_nvfp4(x, eo, so, gx)
    qw, sw, alphas = [], [], []
    for g in range(groups):
        gw = gs_of(w[g])
        q, s = O.block_quantize_nvfp4(w[g], gw, True)
        qw.append(q); sw.append(s); alphas.append(1.0 / (gx * gw))
    qw, sw = torch.stack(qw), torch.stack(sw)
    alphas = torch.tensor(alphas, dtype=torch.float32)
    ps = torch.tensor([[t, n, k] for t in sizes], dtype=torch.int32)
    ref = O.ref_nvfp4_scaled_grouped_mm(qx, qw, sx, sw, alphas, ps, eo, so)
    st = torch.full((groups,), k, dtype=torch.int64, device=dev)
    ct = torch.full((groups,), n, dtype=torch.int64, device=dev)
    out = nvf_cutlass.nvfp4_scaled_grouped_mm(fp4(qx.to(dev)), fp4(qw.to(dev)), e4m3(sx.to(dev)), e4m3(sw.to(dev)), alphas.to(dev), st, ct,
                                              ps.to(dev), eo.to(dev), so.to(dev), torch.bfloat16)
    torch.cuda.synchronize()
    assert _rowwise_rel(out, ref) <= GEMM_MAX_REL
