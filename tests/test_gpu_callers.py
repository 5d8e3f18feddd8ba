"""GPU parity of the caller conventions (csrc/ir/composite_nodes.cpp:1133-1162, 1427-1459, 1663-1712) and of
torch.ops.nvf_cutlass.f16a_nvfp4weight_scaled_grouped_mm against the oracle, fed the graph-level operand
layouts (transposed weight views, END offsets) that the reference's expression nodes receive."""
import pytest
import torch

from helpers import GEMM_MAX_REL, e4m3, fp4, gs_of, max_rel, start_offsets
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def _nvfp4(x, gs):
    q, s = O.block_quantize_nvfp4(x, gs, True)
    return q, s


def test_scaled_mma_runs_the_kernel_on_the_graph_level_layout(dev):
    from fuser_amd import _C

    m, n, k = 200, 160, 192
    gen = torch.Generator().manual_seed(1)
    x, w = torch.randn(m, k, generator=gen).bfloat16(), (torch.randn(n, k, generator=gen) * 0.05).bfloat16()
    gx, gw = gs_of(x), gs_of(w)
    (xq, xs), (wq, ws) = _nvfp4(x, gx), _nvfp4(w, gw)
    alpha = torch.tensor(1.0 / (gx * gw), dtype=torch.float32)
    mat2 = fp4(wq.to(dev)).t()  # [K/2, N] view, as the fusion holds the weight
    out = _C.callers.scaled_mma(fp4(xq.to(dev)), mat2, e4m3(xs.to(dev)), e4m3(ws.to(dev)), alpha.to(dev), out_dtype=torch.float16)
    assert out is not None and out.dtype == torch.float16 and out.shape == (m, n)
    ref = O.ref_nvfp4_scaled_mm(xq, wq, xs, ws, float(alpha))
    assert max_rel(out, ref) <= GEMM_MAX_REL
    # an N the kernel does not take (not a multiple of 32): the caller is told to fall back
    mat2_bad = fp4(wq[:150].contiguous().to(dev)).t()
    assert _C.callers.scaled_mma(fp4(xq.to(dev)), mat2_bad, e4m3(xs.to(dev)), e4m3(ws.to(dev)), alpha.to(dev)) is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_grouped_mma_from_end_offsets(dev, dtype):
    from fuser_amd import _C

    sizes = [70, 0, 130, 1, 55]
    m, n, k = sum(sizes), 136, 72
    gen = torch.Generator().manual_seed(2)
    a = torch.randn(m, k, generator=gen).to(dtype)
    w = (torch.randn(len(sizes), n, k, generator=gen) * 0.1).to(dtype)  # stored [G, N, K]
    ends = torch.cumsum(torch.tensor(sizes), 0).to(torch.int32)
    out = _C.callers.grouped_mma(a.to(dev), w.to(dev).transpose(1, 2), ends.to(dev))
    assert out is not None and out.dtype == dtype and out.shape == (m, n)
    ps = torch.tensor([[t, n, k] for t in sizes], dtype=torch.int32)
    ref = O.ref_grouped_mm(a, w, ps, start_offsets(sizes))
    assert max_rel(out, ref) <= GEMM_MAX_REL


def _moe_case(sizes, k, n, seed, dev):
    g = len(sizes)
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(sum(sizes), k, generator=gen).bfloat16()
    w = (torch.randn(g, n, k, generator=gen) * 0.05).bfloat16()
    wq = torch.empty(g, n, k // 2, dtype=torch.uint8)
    ws = torch.empty(g, n, k // 16, dtype=torch.uint8)
    alphas = torch.empty(g)
    for e in range(g):
        gs = gs_of(w[e])
        wq[e], ws[e] = O.block_quantize_nvfp4(w[e], gs, True)
        alphas[e] = 1.0 / gs
    return x, wq, ws, alphas


def test_custom_op_quantizes_activations_per_group_and_multiplies(dev):
    from fuser_amd import custom_ops

    sizes = [100, 0, 29, 300, 1]
    k, n = 256, 384
    x, wq, ws, alphas = _moe_case(sizes, k, n, 3, dev)
    starts = start_offsets(sizes).to(dev)
    xd = x.to(dev)
    so, ps = custom_ops.compute_auxiliary_tensors(xd, starts, n)
    w_view = fp4(wq.to(dev)).transpose(1, 2)  # [G, K/2, N], as the layer stores it
    out = torch.ops.nvf_cutlass.f16a_nvfp4weight_scaled_grouped_mm(xd, w_view, e4m3(ws.to(dev)), alphas.to(dev), starts, so, ps)
    assert out.dtype == torch.bfloat16 and out.shape == (sum(sizes), n)
    aq, asf = O.grouped_block_quantize_nvfp4(x, starts.cpu(), so.cpu(), None)
    ref = O.ref_nvfp4_scaled_grouped_mm(aq, wq, asf, ws, alphas, ps.cpu(), starts.cpu(), so.cpu())
    assert max_rel(out, ref) <= GEMM_MAX_REL
    # leading dimensions are kept: [2, M/2, K] -> [2, M/2, N]
    out3 = torch.ops.nvf_cutlass.f16a_nvfp4weight_scaled_grouped_mm(xd.view(2, -1, k), w_view, e4m3(ws.to(dev)), alphas.to(dev),
                                                                    starts, so, ps)
    assert out3.shape == (2, sum(sizes) // 2, n) and torch.equal(out3.view(-1, n), out)


def test_grouped_swiglu_layer_end_to_end(dev):
    """gate / up / down projections of an NVFP4 grouped SwiGLU through the registered op, as
    NVFP4InferenceGroupedSwiGLU.forward chains them (layers_for_inference_benchmark.py:495-510); each
    projection is checked against the oracle on the inputs it actually received."""
    from fuser_amd import custom_ops

    op = torch.ops.nvf_cutlass.f16a_nvfp4weight_scaled_grouped_mm
    sizes = [130, 40, 0, 214]
    hidden, inter = 256, 512
    x, gq, gsf, ga = _moe_case(sizes, hidden, inter, 4, dev)
    _, uq, usf, ua = _moe_case(sizes, hidden, inter, 5, dev)
    _, dq, dsf, da = _moe_case(sizes, inter, hidden, 6, dev)
    starts = start_offsets(sizes).to(dev)
    xd = x.to(dev)

    def proj(inp, wq, ws, alphas, out_features):
        so, ps = custom_ops.compute_auxiliary_tensors(inp, starts, out_features)
        out = op(inp, fp4(wq.to(dev)).transpose(1, 2), e4m3(ws.to(dev)), alphas.to(dev), starts, so, ps)
        aq, asf = O.grouped_block_quantize_nvfp4(inp.cpu(), starts.cpu(), so.cpu(), None)
        ref = O.ref_nvfp4_scaled_grouped_mm(aq, wq, asf, ws, alphas, ps.cpu(), starts.cpu(), so.cpu())
        assert max_rel(out, ref) <= GEMM_MAX_REL
        return out

    gate = proj(xd, gq, gsf, ga, inter)
    up = proj(xd, uq, usf, ua, inter)
    mid = torch.nn.functional.silu(gate) * up
    out = proj(mid, dq, dsf, da, hidden)
    assert out.shape == (sum(sizes), hidden) and torch.isfinite(out.float()).all()
