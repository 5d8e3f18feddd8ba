"""GPU parity of the grouped GEMMs (cutlass/group_mm.cu, cutlass/nvfp4_scaled_group_mm.cu) against
per-expert fp32 oracles; configurations of tests/python/direct/test_cutlass_gemm.py:17-70 and
test_cutlass_nvfp4_gemm.py:178-281 verbatim, then BASELINE configs 4 and 5."""
import pytest
import torch

from helpers import GEMM_MAX_REL, e4m3, fp4, gs_of, max_rel, max_rel_rowwise, start_offsets
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def _grouped_args(sizes, n, k, dev):
    g = len(sizes)
    ps = torch.tensor([[t, n, k] for t in sizes], dtype=torch.int32)
    eo = start_offsets(sizes)
    st = torch.full((g,), k, dtype=torch.int64, device=dev)
    ct = torch.full((g,), n, dtype=torch.int64, device=dev)
    return ps, eo, st, ct


@pytest.mark.parametrize("config", [[1024, 128, 256], [267, 128, 256]])
@pytest.mark.parametrize("tokens_per_expert_neg_one", [[115, 144, 8], [5, 7, 9]])
@pytest.mark.parametrize("tensor_dtype", [torch.bfloat16, torch.float16])
def test_grouped_mm_reference_configs(dev, config, tokens_per_expert_neg_one, tensor_dtype):
    from fuser_amd import nvf_cutlass

    m, n, k = config
    sizes = list(tokens_per_expert_neg_one)
    sizes.append(m - sum(sizes))
    g = len(sizes)
    gen = torch.Generator().manual_seed(0)
    mat1 = (torch.rand(m, k, generator=gen) * 18 - 9).to(tensor_dtype)  # make_tensor's default range
    mat2 = (torch.rand(g, n, k, generator=gen) * 18 - 9).to(tensor_dtype)
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    out = nvf_cutlass.grouped_mm(mat1.to(dev), mat2.to(dev), st, ct, ps.to(dev), eo.to(dev))
    torch.cuda.synchronize()
    assert out.dtype == tensor_dtype and out.shape == (m, n)
    ref = O.ref_grouped_mm(mat1, mat2, ps, eo)
    assert not ref.isnan().any()
    assert max_rel(out, ref) <= GEMM_MAX_REL
    assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL
    torch.testing.assert_close(out.float().cpu(), ref.to(tensor_dtype).float(), atol=1e-2 * ref.abs().max().item(), rtol=1e-2)


def test_grouped_mm_empty_groups_and_untouched_rows(dev):
    from fuser_amd import capi

    sizes = [0, 70, 0, 0, 130, 0]
    m, n, k = 300, 264, 136  # 100 trailing rows belong to no group; n, k only multiples of 8
    gen = torch.Generator().manual_seed(5)
    a = torch.randn(m, k, generator=gen).bfloat16()
    b = torch.randn(len(sizes), n, k, generator=gen).bfloat16()
    ps, eo, _, _ = _grouped_args(sizes, n, k, dev)
    ad, bd, psd, eod = a.to(dev), b.to(dev), ps.to(dev), eo.to(dev)
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    capi.check(capi.lib().nvf_grouped_mm(ad.data_ptr(), bd.data_ptr(), out.data_ptr(), psd.data_ptr(), eod.data_ptr(), len(sizes), m, n, k,
                                         capi.BF16, None))
    torch.cuda.synchronize()
    ref = O.ref_grouped_mm(a, b, ps, eo)
    assert ref[200:].isnan().all() and (out[200:] == 7.0).all()
    assert max_rel_rowwise(out[:200], ref[:200]) <= GEMM_MAX_REL


@pytest.mark.parametrize("tensor_dtype,k,n", [(torch.bfloat16, 192, 2048), (torch.float16, 128, 2048), (torch.bfloat16, 1088, 2048),
                                              (torch.bfloat16, 128, 4096), (torch.float16, 192, 4096)])
def test_grouped_mm_persistent_256_tile_kernel_full_compare(dev, tensor_dtype, k, n):
    """Large enough for the persistent LDS-direct kernel (N % 256 == 0, K % 64 == 0, >= 256 rows per
    group on average): groups that end inside a tile, an empty group, a one-row group and a group of
    257 rows; every output element compared, rows past the last group untouched.  N = 4096 gives 288
    tiles, i.e. two tiles for some workgroups, with two and three K steps per tile."""
    from fuser_amd import capi

    sizes = [1000, 0, 1791, 257, 1, 1000]
    m = sum(sizes) + 47
    gen = torch.Generator().manual_seed(k)
    a = torch.randn(m, k, generator=gen).to(tensor_dtype)
    b = (torch.randn(len(sizes), n, k, generator=gen) * 0.05).to(tensor_dtype)
    ps, eo, _, _ = _grouped_args(sizes, n, k, dev)
    ad, bd, psd, eod = a.to(dev), b.to(dev), ps.to(dev), eo.to(dev)
    out = torch.full((m, n), 7.0, dtype=tensor_dtype, device=dev)
    dt = capi.BF16 if tensor_dtype == torch.bfloat16 else capi.F16
    for _ in range(2):
        capi.check(capi.lib().nvf_grouped_mm(ad.data_ptr(), bd.data_ptr(), out.data_ptr(), psd.data_ptr(), eod.data_ptr(), len(sizes),
                                             m, n, k, dt, None))
    torch.cuda.synchronize()
    ref = O.ref_grouped_mm(a, b, ps, eo)
    rows = sum(sizes)
    assert (out[rows:] == 7.0).all()
    scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL


@pytest.mark.parametrize("n,k", [(2048, 192), (2304, 128), (4096, 320), (2304, 1024)])
def test_grouped_mm_group_ends_inside_tiles(dev, n, k):
    """Persistent 256-row-tile kernel: groups that end 128, 129, 1, 100 and 127 rows into a tile, groups smaller than
    half a tile, N with 8 | N/256 (n-tiles dealt to the XCDs) and without, two to 16 K steps.  Every element
    compared, rows after the last group untouched."""
    from fuser_amd import capi

    sizes = [384, 128, 129, 895, 100, 2048 + 127, 256, 0, 257]
    m = sum(sizes) + 5
    gen = torch.Generator().manual_seed(n + k)
    a = torch.randn(m, k, generator=gen).bfloat16()
    b = (torch.randn(len(sizes), n, k, generator=gen) * 0.05).bfloat16()
    ps, eo, _, _ = _grouped_args(sizes, n, k, dev)
    ad, bd, psd, eod = a.to(dev), b.to(dev), ps.to(dev), eo.to(dev)
    assert capi.describe_dispatch("grouped_mm", m, n, k, groups=len(sizes)).startswith("grouped16_gemm_256_kernel")
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    capi.check(capi.lib().nvf_grouped_mm(ad.data_ptr(), bd.data_ptr(), out.data_ptr(), psd.data_ptr(), eod.data_ptr(), len(sizes),
                                         m, n, k, capi.BF16, None))
    torch.cuda.synchronize()
    ref = O.ref_grouped_mm(a, b, ps, eo)
    rows = sum(sizes)
    assert (out[rows:] == 7.0).all()
    scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
    assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL


@pytest.mark.parametrize("n,k", [(14336, 192), (8192, 128)])
def test_grouped_mm_persistent_kernel_from_128_rows_per_group(dev, n, k):
    """128 to 255 rows per group on average and a wide N: the persistent kernel (most of its 256-row tiles are short,
    one group is empty, two have a single tile of 1 and of 255 rows).  Every element compared, rows after the last
    group untouched, both operand types."""
    from fuser_amd import capi

    sizes = [130, 0, 255, 1, 200, 128, 300, 129, 90, 257]
    m = sum(sizes) + 5
    assert 128 * len(sizes) <= m < 256 * len(sizes)
    assert capi.describe_dispatch("grouped_mm", m, n, k, groups=len(sizes)).startswith("grouped16_gemm_256_kernel")
    for tensor_dtype, dt in ((torch.bfloat16, capi.BF16), (torch.float16, capi.F16)):
        gen = torch.Generator().manual_seed(n + k)
        a = torch.randn(m, k, generator=gen).to(tensor_dtype)
        b = (torch.randn(len(sizes), n, k, generator=gen) * 0.05).to(tensor_dtype)
        ps, eo, _, _ = _grouped_args(sizes, n, k, dev)
        ad, bd, psd, eod = a.to(dev), b.to(dev), ps.to(dev), eo.to(dev)
        out = torch.full((m, n), 7.0, dtype=tensor_dtype, device=dev)
        capi.check(capi.lib().nvf_grouped_mm(ad.data_ptr(), bd.data_ptr(), out.data_ptr(), psd.data_ptr(), eod.data_ptr(), len(sizes),
                                             m, n, k, dt, None))
        torch.cuda.synchronize()
        ref = O.ref_grouped_mm(a, b, ps, eo)
        rows = sum(sizes)
        assert (out[rows:] == 7.0).all()
        scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL, tensor_dtype


def _moe_sizes_top2(tokens, experts, seed):
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=gen) + torch.linspace(-1.5, 1.5, experts)
    return torch.bincount(logits.topk(2, dim=1).indices.flatten(), minlength=experts).tolist()


@pytest.mark.parametrize("near_empty", [False, True])
def test_config4_bf16_grouped_moe(dev, near_empty):
    """BASELINE config 4: 8 experts, K=4096, N=14336, 4096 tokens top-2 (8192 rows), uneven groups: exactly the
    group sizes bench.py times ([40, 90, 220, 427, 872, 1413, 2211, 2919]), and the same with one expert
    emptied down to 3 rows."""
    from fuser_amd import nvf_cutlass

    g, k, n = 8, 4096, 14336
    sizes = _moe_sizes_top2(4096, g, seed=0)
    assert sizes == [40, 90, 220, 427, 872, 1413, 2211, 2919]
    if near_empty:
        sizes[3] += sizes[5] - 3
        sizes[5] = 3
    m = sum(sizes)
    assert m == 8192
    gen = torch.Generator(device=dev).manual_seed(1)
    a = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    b = (torch.randn(g, n, k, device=dev, generator=gen) * 0.02).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    out = nvf_cutlass.grouped_mm(a, b, st, ct, ps.to(dev), eo.to(dev))
    torch.cuda.synchronize()
    # oracle on a sample of rows (every expert: first and last row, the rows either side of every 128-row border, random
    # ones) and of columns (first, last, random)
    cols = torch.unique(torch.cat([torch.tensor([0, n - 1]), torch.randint(0, n, (254,), generator=torch.Generator().manual_seed(2))]))
    worst = 0.0
    for e in range(g):
        lo, hi = int(eo[e]), int(eo[e]) + sizes[e]
        borders = torch.tensor([r for b128 in range(128, sizes[e], 128) for r in (lo + b128 - 1, lo + b128)], dtype=torch.long)
        rows = torch.unique(torch.cat([torch.tensor([lo, hi - 1]), borders, torch.randint(lo, hi, (24,), generator=torch.Generator().manual_seed(e))]))
        ref = a[rows.to(dev)].float().cpu() @ b[e][cols.to(dev)].float().cpu().t()
        got = out[rows.to(dev)][:, cols.to(dev)]
        worst = max(worst, max_rel_rowwise(got, ref))
    assert worst <= GEMM_MAX_REL


@pytest.mark.parametrize("config", [[1024, 128, 256]])
@pytest.mark.parametrize("tokens_per_expert_neg_one", [[115, 144, 8]])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_nvfp4_grouped_mm_reference_config(dev, config, tokens_per_expert_neg_one, out_dtype):
    from fuser_amd import nvf_cutlass, ops

    m, n, k = config
    sizes = list(tokens_per_expert_neg_one)
    sizes.append(m - sum(sizes))
    g = len(sizes)
    gen = torch.Generator().manual_seed(0)
    mat1 = (torch.rand(m, k, generator=gen) * 18 - 9)
    mat2 = (torch.rand(g, n, k, generator=gen) * 18 - 9)
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8)
    mat2_gs = torch.empty(g)
    for e in range(g):
        gs = float(2688.0 / mat2[e].max())
        bq[e], bsf[e] = O.block_quantize_nvfp4(mat2[e], gs, True)
        mat2_gs[e] = gs
    # activations quantized per group by the GPU grouped quantizer, no global scale (as in the reference test)
    aq, asf = ops.nv_grouped_block_quantize(mat1.to(dev), eo.to(dev), so.to(dev), None, 16)
    raq, rasf = O.grouped_block_quantize_nvfp4(mat1, eo, so, None)
    assert torch.equal(aq.view(torch.uint8).cpu(), raq)
    alphas = 1.0 / mat2_gs
    out = nvf_cutlass.nvfp4_scaled_grouped_mm(aq, fp4(bq.to(dev)), asf, e4m3(bsf.to(dev)), alphas.to(dev), st, ct, ps.to(dev), eo.to(dev),
                                              so.to(dev), out_dtype)
    torch.cuda.synchronize()
    assert out.dtype == out_dtype and out.shape == (m, n)
    ref = O.ref_nvfp4_scaled_grouped_mm(raq, bq, rasf, bsf, alphas, ps, eo, so)
    assert max_rel(out, ref) <= GEMM_MAX_REL
    assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2 * ref.abs().max().item(), rtol=1e-2)


def test_nvfp4_grouped_mm_empty_and_tiny_groups(dev):
    from fuser_amd import nvf_cutlass

    sizes = [0, 1, 0, 129, 64, 0, 300, 2]
    n, k = 256, 320
    m = sum(sizes)
    gen = torch.Generator().manual_seed(8)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(len(sizes), n, k, generator=gen) * 0.02).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, asf = O.grouped_block_quantize_nvfp4(x, eo, so, None)
    bq = torch.empty(len(sizes), n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(len(sizes), n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(len(sizes))
    for e in range(len(sizes)):
        gs = gs_of(w[e])
        bq[e], bsf[e] = O.block_quantize_nvfp4(w[e], gs, True)
        alphas[e] = 1.0 / gs
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, bq, asf, bsf, alphas, ps, eo, so)
    out = nvf_cutlass.nvfp4_scaled_grouped_mm(fp4(aq.to(dev)), fp4(bq.to(dev)), e4m3(asf.to(dev)), e4m3(bsf.to(dev)), alphas.to(dev), st, ct,
                                              ps.to(dev), eo.to(dev), so.to(dev), torch.bfloat16)
    torch.cuda.synchronize()
    assert max_rel_rowwise(out, ref) <= GEMM_MAX_REL


@pytest.mark.parametrize("m_total,n,k", [(1, 256, 256), (8, 2048, 7168), (32, 7168, 2048), (31, 384, 4096), (20, 512, 1024)])
def test_nvfp4_grouped_mm_fewer_rows_in_all_than_the_smallest_mid_sized_group(dev, m_total, n, k):
    """A decode step of a few tokens: at most 32 rows in the whole call, so the launches that serve groups of 33 rows and
    more have nothing to do (and must not be launched with an empty grid).  Every element compared."""
    from fuser_amd import capi, nvf_cutlass

    g = 8
    gen = torch.Generator().manual_seed(m_total + n)
    cuts = sorted(torch.randint(0, m_total + 1, (g - 1,), generator=gen).tolist())
    sizes = [b - a for a, b in zip([0] + cuts, cuts + [m_total])]
    assert sum(sizes) == m_total
    assert "grid=0" not in capi.describe_dispatch("nvfp4_scaled_grouped_mm", m_total, n, k, groups=g)
    x = torch.randn(m_total, k, generator=gen).bfloat16()
    w = (torch.randn(g, n, k, generator=gen) * 0.05).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, asf = O.grouped_block_quantize_nvfp4(x, eo, so, None)
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(g)
    for e in range(g):
        gs = gs_of(w[e])
        bq[e], bsf[e] = O.block_quantize_nvfp4(w[e], gs, True)
        alphas[e] = (e + 1) / gs
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, bq, asf, bsf, alphas, ps, eo, so)
    out = nvf_cutlass.nvfp4_scaled_grouped_mm(fp4(aq.to(dev)), fp4(bq.to(dev)), e4m3(asf.to(dev)), e4m3(bsf.to(dev)), alphas.to(dev), st, ct,
                                              ps.to(dev), eo.to(dev), so.to(dev), torch.bfloat16)
    torch.cuda.synchronize()
    assert max_rel_rowwise(out[:m_total], ref[:m_total]) <= GEMM_MAX_REL


@pytest.mark.parametrize("sizes,n,k", [([600, 0, 256, 255, 1, 1030, 512, 3600], 512, 384), ([300, 2100, 0, 257, 3585], 256, 256),
                                       ([2560, 700, 3000, 0, 1280, 2900], 2048, 256), ([511] * 13, 512, 640),
                                       ([3700, 2248, 130, 400], 256, 384),
                                       ([40, 64, 2100, 33, 65, 100, 128, 50, 0, 32, 3620], 256, 512),
                                       ([40, 64, 2100, 33, 65, 100, 128, 50, 0, 32, 3620], 384, 256),
                                       ([600, 0, 256, 255, 1, 1030, 512, 3600], 512, 320), ([3700, 2248, 130, 400], 256, 448),
                                       ([219, 130, 300, 0, 1, 257, 129, 500], 12288, 256), ([90, 40, 700, 64, 33, 1400, 128, 160, 8, 500], 22528, 256)])
def test_nvfp4_grouped_mm_whole_tiles_and_group_ends(dev, sizes, n, k):
    """A prefill-sized call (6144 rows or more; the last two cases: fewer rows against weights so wide that the 256-row
    tiles of the large groups fill a round with 128 rows per group, or two rounds), N % 256 == 0 (the last two cases with K % 128 = 64: a short last span): the whole 256-row tiles of every group, and a last tile of
    more than 128 rows, run on the persistent 256x256 kernel (the rows past such a group read as zero payload
    with whatever the scale padding holds - it is poisoned here - and are not stored), the other group ends
    on the 128x128 tile kernel.  Groups with no whole tile, only whole tiles, one row past a tile, 255 of 256
    rows, empty groups; two, three and five spans per tile; the third case has more than 320 tiles, i.e. two
    per workgroup for some; the [3700, 2248, 130, 400] case ends with a 144-row tile whose 256 rows would reach past the
    activation tensor.  The last two cases add groups of every
    weight-streaming class next to a large one (wavefronts owning rows, and wavefronts splitting K).  Every
    output element is compared."""
    from fuser_amd import nvf_cutlass

    g, m = len(sizes), sum(sizes) + 33
    gen = torch.Generator().manual_seed(n + k)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(g, n, k, generator=gen) * 0.05).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, asf = O.grouped_block_quantize_nvfp4(x, eo, so, None)
    asf[asf == 0] = 0x7F  # poison: padding rows of the scale slabs must not reach any output
    valid = O.grouped_block_quantize_nvfp4(x, eo, so, None)[1]
    lin = torch.zeros_like(asf, dtype=torch.bool)
    for e, t in enumerate(sizes):
        if t:
            ones = O.linear_to_swizzled_128_4(torch.ones(t, k // 16, dtype=torch.uint8))
            lin[int(so[e]) : int(so[e]) + ones.shape[0]] |= ones.bool()
    asf = torch.where(lin, valid, torch.full_like(valid, 0x7F))
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(g)
    for e in range(g):
        gs = gs_of(w[e])
        bq[e], bsf[e] = O.block_quantize_nvfp4(w[e], gs, True)
        alphas[e] = (e + 1) / gs  # a different alpha for every group
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, bq, valid, bsf, alphas, ps, eo, so)
    rows = sum(sizes)
    for dtype in (torch.bfloat16, torch.float16):
        out = nvf_cutlass.nvfp4_scaled_grouped_mm(fp4(aq.to(dev)), fp4(bq.to(dev)), e4m3(asf.to(dev)), e4m3(bsf.to(dev)), alphas.to(dev),
                                                  st, ct, ps.to(dev), eo.to(dev), so.to(dev), dtype)
        torch.cuda.synchronize()
        scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL, (sizes, dtype)


@pytest.mark.parametrize("n,k", [(128, 128), (384, 384), (256, 1152), (128, 2048), (256, 4096), (512, 5120), (256, 320), (512, 2880), (128, 192)])
def test_nvfp4_grouped_mm_small_groups_stream_their_weights(dev, n, k):
    """Groups of 1..32 and of 33..128 rows each run on the weight-streaming kernel (one workgroup
    per group and 64 weight rows), larger groups on the tile kernels, which skip the small ones; the last three
    shapes have K % 128 = 64 (a short last chunk).  Sizes on
    both sides of every class border, empty groups, a different alpha per group, poisoned padding of the
    activation scale slabs, one to forty 128-deep chunks (wavefronts without work); N % 256 == 0 with K < 4096
    takes the variant whose wavefronts own different weight rows, the rest the one that splits K; every
    element compared, rows after the last group untouched, run-to-run bit equality."""
    from fuser_amd import nvf_cutlass

    sizes = [0, 1, 16, 17, 32, 33, 64, 65, 128, 129, 300, 0, 2, 100]
    g, m = len(sizes), sum(sizes) + 5
    gen = torch.Generator().manual_seed(n * 7 + k)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(g, n, k, generator=gen) * 0.05).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, valid = O.grouped_block_quantize_nvfp4(x, eo, so, None)
    lin = torch.zeros_like(valid, dtype=torch.bool)
    for e, t in enumerate(sizes):
        if t:
            ones = O.linear_to_swizzled_128_4(torch.ones(t, k // 16, dtype=torch.uint8))
            lin[int(so[e]) : int(so[e]) + ones.shape[0]] |= ones.bool()
    asf = torch.where(lin, valid, torch.full_like(valid, 0x7F))  # NaN code wherever no row owns the byte
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(g)
    for e in range(g):
        gs = gs_of(w[e])
        bq[e], bsf[e] = O.block_quantize_nvfp4(w[e], gs, True)
        alphas[e] = (e + 1) / gs
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, bq, valid, bsf, alphas, ps, eo, so)
    rows = sum(sizes)
    args = (fp4(aq.to(dev)), fp4(bq.to(dev)), e4m3(asf.to(dev)), e4m3(bsf.to(dev)), alphas.to(dev), st, ct, ps.to(dev), eo.to(dev), so.to(dev))
    from fuser_amd import capi
    assert "nvfp4_skinny_ring_kernel<" in capi.describe_dispatch("nvfp4_scaled_grouped_mm", m, n, k, g)
    for dtype in (torch.bfloat16, torch.float16):
        out = nvf_cutlass.nvfp4_scaled_grouped_mm(*args, dtype)
        torch.cuda.synchronize()
        scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL, (n, k, dtype)
        assert torch.equal(out[:rows], nvf_cutlass.nvfp4_scaled_grouped_mm(*args, dtype)[:rows])


@pytest.mark.parametrize("n,k", [(512, 4096), (1024, 4224), (512, 2048), (1024, 1024), (512, 1152)])
def test_nvfp4_grouped_mm_mid_sized_groups_of_a_prefill(dev, n, k):
    """A prefill-sized call (6144 rows or more) with K >= 1024 and N % 512 == 0: groups of 33..80 rows run on the kernel
    that converts a group's activation rows once per 512 weight rows (work items found from the device-resident
    sizes; three, four and five row tiles, sizes on both sides of its borders), their neighbours of 81..128 rows and
    the ends of the larger ones on 128x256 tiles of the persistent kernel, the rest of those on its 256x256 tiles.  8, 9,
    16, 32 and 33 K chunks: the odd and the even LDS slot both end a walk.  A different alpha per group, poisoned
    padding of the activation scale slabs; every element compared, rows after the last group untouched, run-to-run
    bit equality."""
    from fuser_amd import capi, nvf_cutlass

    sizes = [33, 80, 48, 49, 64, 65, 81, 32, 0, 128, 34, 47, 79, 300, 66, 50, 40, 72, 1, 129] + [56, 77, 35, 63] * 6 + [3400]
    g, m = len(sizes), sum(sizes) + 3
    assert sum(sizes) >= 6144
    assert "nvfp4_group_panel_kernel" in capi.describe_dispatch("nvfp4_scaled_grouped_mm", m, n, k, groups=g)
    gen = torch.Generator().manual_seed(n + k)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(g, n, k, generator=gen) * 0.05).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, valid = O.grouped_block_quantize_nvfp4(x, eo, so, None)
    lin = torch.zeros_like(valid, dtype=torch.bool)
    for e, t in enumerate(sizes):
        if t:
            ones = O.linear_to_swizzled_128_4(torch.ones(t, k // 16, dtype=torch.uint8))
            lin[int(so[e]) : int(so[e]) + ones.shape[0]] |= ones.bool()
    asf = torch.where(lin, valid, torch.full_like(valid, 0x7F))  # NaN code wherever no row owns the byte
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(g)
    for e in range(g):
        gs = gs_of(w[e])
        bq[e], bsf[e] = O.block_quantize_nvfp4(w[e], gs, True)
        alphas[e] = (e % 7 + 1) / gs
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, bq, valid, bsf, alphas, ps, eo, so)
    rows = sum(sizes)
    args = (fp4(aq.to(dev)), fp4(bq.to(dev)), e4m3(asf.to(dev)), e4m3(bsf.to(dev)), alphas.to(dev), st, ct, ps.to(dev), eo.to(dev), so.to(dev))
    for dtype in (torch.bfloat16, torch.float16):
        out = nvf_cutlass.nvfp4_scaled_grouped_mm(*args, dtype)
        torch.cuda.synchronize()
        scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL, (n, k, dtype)
        assert torch.equal(out[:rows], nvf_cutlass.nvfp4_scaled_grouped_mm(*args, dtype)[:rows])


@pytest.mark.parametrize("n,k,few_rows", [(256, 4096, False), (128, 4224, False), (256, 512, False), (256, 512, True), (128, 4096, True),
                                          (1024, 4096, False), (2048, 512, True)])
def test_nvfp4_grouped_mm_mid_sized_groups_below_the_prefill_size(dev, n, k, few_rows):
    """300 experts, most of them with 0..3 rows, a few with 33..128 at indices on both sides of the borders at which
    the streaming kernel counts the groups of a size class (63 | 64, 255 | 256, the last one), two large ones.  Up to
    1024 rows in all, or below 6144 with K >= 4096, the mid-sized groups stream their weights from a launch with one
    block of workgroups per group of 33 rows that the call could hold (the block finds its group by rank); otherwise
    they run as 128x256 tiles of the persistent kernel.  The last two shapes give that launch more workgroups than compute
    units: workgroups of 4 wavefronts, two to a compute unit.  A different alpha per group, poisoned padding of the activation
    scale slabs; every element compared, rows after the last group untouched, run-to-run bit equality."""
    from fuser_amd import capi, nvf_cutlass

    g = 300
    if few_rows:
        sizes = [1 if i % 5 == 0 else 0 for i in range(g)]
        for i, t in {63: 33, 64: 128, 256: 40, 299: 100, 130: 129}.items():
            sizes[i] = t
    else:
        sizes = [i % 4 for i in range(g)]
        for i, t in {2: 33, 63: 128, 64: 100, 70: 64, 255: 90, 256: 77, 257: 128, 299: 40, 130: 400, 131: 129}.items():
            sizes[i] = t
    m = sum(sizes) + 3
    assert (m <= 1024) == few_rows and m < 6144
    got = capi.describe_dispatch("nvfp4_scaled_grouped_mm", m, n, k, groups=g)
    mid = [part for part in got.split("; ") if "rows=33..128" in part]
    assert len(mid) == 1 and mid[0].startswith("nvfp4_skinny_ring_kernel<" if few_rows or k >= 4096 else "nvfp4_gemm_256_kernel<grouped=1,TM=2"), got
    assert (",W=4>" in mid[0]) == (n >= 1024), got
    gen = torch.Generator().manual_seed(n + k + few_rows)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(8, n, k, generator=gen) * 0.05).bfloat16()  # eight different experts, repeated
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, valid = O.grouped_block_quantize_nvfp4(x, eo, so, None)
    lin = torch.zeros_like(valid, dtype=torch.bool)
    for e, t in enumerate(sizes):
        if t:
            ones = O.linear_to_swizzled_128_4(torch.ones(t, k // 16, dtype=torch.uint8))
            lin[int(so[e]) : int(so[e]) + ones.shape[0]] |= ones.bool()
    asf = torch.where(lin, valid, torch.full_like(valid, 0x7F))  # NaN code wherever no row owns the byte
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(g)
    quantized = [O.block_quantize_nvfp4(w[e], gs_of(w[e]), True) for e in range(8)]
    for e in range(g):
        bq[e], bsf[e] = quantized[e % 8]
        alphas[e] = (e % 11 + 1) / gs_of(w[e % 8])
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, bq, valid, bsf, alphas, ps, eo, so)
    rows = sum(sizes)
    args = (fp4(aq.to(dev)), fp4(bq.to(dev)), e4m3(asf.to(dev)), e4m3(bsf.to(dev)), alphas.to(dev), st, ct, ps.to(dev), eo.to(dev), so.to(dev))
    for dtype in (torch.bfloat16, torch.float16):
        out = nvf_cutlass.nvfp4_scaled_grouped_mm(*args, dtype)
        torch.cuda.synchronize()
        scale = ref[:rows].abs().amax(dim=1, keepdim=True).clamp(min=1e-30)
        assert ((out[:rows].float().cpu() - ref[:rows]).abs() / scale).max().item() <= GEMM_MAX_REL, (n, k, dtype)
        assert torch.equal(out[:rows], nvf_cutlass.nvfp4_scaled_grouped_mm(*args, dtype)[:rows])


def _zipf_sizes(tokens, topk, experts, s, seed):
    gen = torch.Generator().manual_seed(seed)
    p = 1.0 / torch.arange(1, experts + 1).float() ** s
    p = p[torch.randperm(experts, generator=gen)]
    idx = torch.multinomial(p.expand(tokens, experts), topk, replacement=False, generator=gen).flatten()
    return torch.bincount(idx, minlength=experts).tolist()


@pytest.mark.parametrize("kn", [(7168, 2048), (2048, 7168)])
def test_config5_nvfp4_grouped_large_moe(dev, kn):
    """BASELINE config 5: 256 experts, 8192 tokens top-8 (65536 rows), Zipf(1.1) loads, K/N = 7168/2048
    and the down projection.  Activations quantized per group on the GPU; weights quantized per expert
    on the GPU with a per-expert global scale.  Oracle applied to sampled rows of sampled experts."""
    from fuser_amd import nvf_cutlass, ops

    k, n = kn
    g = 256
    sizes = _zipf_sizes(8192, 8, g, 1.1, seed=0)
    m = sum(sizes)
    assert m == 65536 and min(sizes) < 64
    gen = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    ps, eo, st, ct = _grouped_args(sizes, n, k, dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes])
    aq, asf = ops.nv_grouped_block_quantize(x, eo.to(dev), so.to(dev), None, 16)
    bq = torch.empty(g, n, k // 2, dtype=torch.uint8, device=dev)
    bsf = torch.empty(g, n, k // 16, dtype=torch.uint8, device=dev)
    alphas = torch.empty(g, device=dev)
    for e in range(g):
        w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).bfloat16()
        gs = (2688.0 / w.float().abs().max()).float()
        q, s = ops.nv_block_quantize(w, gs, True, 16)
        bq[e], bsf[e], alphas[e] = q.view(torch.uint8), s.view(torch.uint8), 1.0 / gs
    out = nvf_cutlass.nvfp4_scaled_grouped_mm(aq, fp4(bq), asf, e4m3(bsf), alphas, st, ct, ps.to(dev), eo.to(dev), so.to(dev), torch.bfloat16)
    torch.cuda.synchronize()
    # two experts of every class of the dispatch (they run on different kernels): 1-32 rows, 33-80, 81-128, 129-255, and
    # 256 and more with a last partial tile of at most 128 rows / of more than 128 rows (or none); plus the largest
    classes = {"1-32": lambda t: 1 <= t <= 32, "33-80": lambda t: 33 <= t <= 80, "81-128": lambda t: 81 <= t <= 128,
               "129-255": lambda t: 129 <= t <= 255, "256+, short end": lambda t: t >= 256 and 1 <= t % 256 <= 128,
               "256+, long end": lambda t: t >= 256 and (t % 256 == 0 or t % 256 > 128)}
    picked = [max(range(g), key=lambda e: sizes[e])]
    for name, member in classes.items():
        of_class = [e for e in range(g) if member(sizes[e])]
        assert len(of_class) >= 2, name
        picked += [of_class[0], of_class[-1]]
    cols = torch.unique(torch.cat([torch.tensor([0, n - 1]), torch.randint(0, n, (126,), generator=torch.Generator().manual_seed(6))]))
    worst = 0.0
    aq8, asf8 = aq.view(torch.uint8), asf.view(torch.uint8)
    for e in picked:
        t = sizes[e]
        lo, slo = int(eo[e]), int(so[e])
        # first and last row, the rows either side of the last 256-row and 128-row borders, random ones: 32 at most
        edge = [0, t - 1] + [r for b in ((t - 1) // 256 * 256, (t - 1) // 128 * 128) for r in (b - 1, b) if 0 <= r < t]
        local = torch.unique(torch.cat([torch.tensor(edge), torch.randint(0, t, (26,), generator=torch.Generator().manual_seed(e))]))
        a_rows = aq8[(lo + local).to(dev)].cpu()
        sf_lin = O.swizzled_to_linear_128_4(asf8[slo : slo + O.round_up(t, 128)].cpu(), t, k // 16)[local]
        b_rows = bq[e][cols.to(dev)].cpu()
        sb_lin = O.swizzled_to_linear_128_4(bsf[e].cpu(), n, k // 16)[cols]
        ref = O.ref_nvfp4_scaled_mm(a_rows, b_rows, O.linear_to_swizzled_128_4(sf_lin), O.linear_to_swizzled_128_4(sb_lin), float(alphas[e]))
        got = out[(lo + local).to(dev)][:, cols.to(dev)]
        worst = max(worst, max_rel_rowwise(got, ref))
    assert worst <= GEMM_MAX_REL


def test_grouped_ops_reject_bad_inputs_on_device(dev):
    from fuser_amd import nvf_cutlass

    a = torch.zeros(8, 64, dtype=torch.bfloat16, device=dev)
    b = torch.zeros(2, 16, 64, dtype=torch.bfloat16, device=dev)
    i64 = torch.full((2,), 64, dtype=torch.int64, device=dev)
    ps = torch.zeros(2, 3, dtype=torch.int32, device=dev)
    eo = torch.zeros(2, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="Expected BFloat16 or Half for Operand A"):
        nvf_cutlass.grouped_mm(a.float(), b, i64, i64, ps, eo)
    with pytest.raises(RuntimeError):
        nvf_cutlass.grouped_mm(a, b, i64.int(), i64, ps, eo)  # strides must be int64
    with pytest.raises(RuntimeError):
        nvf_cutlass.grouped_mm(a, b, i64, i64, ps.long(), eo)  # problem_sizes must be int32
    with pytest.raises(RuntimeError, match="not a multiple of"):
        nvf_cutlass.grouped_mm(a[:, :60].contiguous(), b[:, :, :60].contiguous(), i64, i64, ps, eo)
    with pytest.raises(RuntimeError, match="Expected Operand B to be a 3D tensor"):
        nvf_cutlass.grouped_mm(a, b[0], i64, i64, ps, eo)
    out = nvf_cutlass.grouped_mm(a, b, i64, i64, ps, eo)  # all groups empty: nothing computed, still returns [8, 16]
    assert out.shape == (8, 16)
