"""The entry points under HIP graph capture: no allocation of their own, no host synchronisation, no
memset nodes.  A chain quantize -> global scale -> GEMMs (dense, decode-sized, split-K with torch-allocated
scratch, grouped, block-scaled result) is captured once and replayed several times with other work on the stream in between;
every replay must reproduce the eager results bit for bit, also after the inputs have been overwritten in
place."""
import pytest
import torch

from helpers import start_offsets
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def test_chain_replays_bit_exactly(dev):
    from fuser_amd import capi, nvf_cutlass, ops

    gen = torch.Generator(device=dev).manual_seed(5)
    m, n, k = 512, 1024, 512
    x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    w = (torch.randn(n, k, device=dev, generator=gen) * 0.05).bfloat16()
    xs = torch.randn(16, k, device=dev, generator=gen).bfloat16()            # decode-sized activations
    xd = torch.randn(72, 8192, device=dev, generator=gen).bfloat16()         # one slab of 65..96 rows, deep K: split K
    wd = (torch.randn(6144, 8192, device=dev, generator=gen) * 0.05).bfloat16()
    sizes = [100, 0, 300, 112]
    eo = start_offsets(sizes).to(dev)
    so = start_offsets([O.round_up(t, 128) for t in sizes]).to(dev)
    ps = torch.tensor([[t, n, k] for t in sizes], dtype=torch.int32, device=dev)
    wg = (torch.randn(len(sizes), n, k, device=dev, generator=gen) * 0.05).bfloat16()
    st = torch.full((len(sizes),), k, dtype=torch.int64, device=dev)
    ct = torch.full((len(sizes),), n, dtype=torch.int64, device=dev)
    one = torch.ones((), device=dev)
    ones_g = torch.ones(len(sizes), device=dev)

    def chain():
        gs = ops.compute_nvfp4_global_scale(x)
        xq, xsf = ops.nv_block_quantize(x, gs, True, 16)
        wq, wsf = ops.nv_block_quantize(w, None, True, 16)
        dense = nvf_cutlass.nvfp4_scaled_mm(xq, wq, xsf, wsf, one, torch.bfloat16)
        sq, ssf = ops.nv_block_quantize(xs, None, True, 16)
        decode = nvf_cutlass.nvfp4_scaled_mm(sq, wq, ssf, wsf, one, torch.bfloat16)
        dq, dsf = ops.nv_block_quantize(xd, None, True, 16)
        wdq, wdsf = ops.nv_block_quantize(wd, None, True, 16)
        split = nvf_cutlass.nvfp4_scaled_mm(dq, wdq, dsf, wdsf, one, torch.float16)
        # the same split with the library's static scratch array (the entry point for callers that cannot allocate;
        # its first call per device, which looks the array's address up, is the eager run below, outside the capture)
        static = torch.empty_like(split)
        capi.check(capi.lib().nvf_nvfp4_scaled_mm_static_ws(dq.data_ptr(), wdq.data_ptr(), dsf.data_ptr(), wdsf.data_ptr(), one.data_ptr(),
                                                            static.data_ptr(), 72, 6144, 8192, capi.F16,
                                                            torch.cuda.current_stream().cuda_stream))
        gq, gsf = ops.nv_grouped_block_quantize(x, eo, so, None, 16)
        wgq = torch.stack([ops.nv_block_quantize(wg[e], None, True, 16)[0].view(torch.uint8) for e in range(len(sizes))])
        wgs = torch.stack([ops.nv_block_quantize(wg[e], None, True, 16)[1].view(torch.uint8) for e in range(len(sizes))])
        grouped = nvf_cutlass.nvfp4_scaled_grouped_mm(gq, wgq.view(torch.float4_e2m1fn_x2), gsf, wgs.view(torch.float8_e4m3fn), ones_g,
                                                      st, ct, ps, eo, so, torch.bfloat16)
        bf = nvf_cutlass.grouped_mm(x, wg, st, ct, ps, eo)
        f8a, e8a = ops.nv_block_quantize(x, None, True, 32, torch.float8_e4m3fn)
        f8b, e8b = ops.nv_block_quantize(w, None, True, 32, torch.float8_e4m3fn)
        mx = nvf_cutlass.mxfp8_scaled_mm(f8a, f8b, e8a, e8b, one, torch.bfloat16)
        # block-scaled result: fused epilogue on the persistent kernel, and a ragged shape whose scale padding is
        # cleared by a fill kernel (no memset node)
        bq, bsf = nvf_cutlass.nvfp4_scaled_mm_blockscale(xq, wq, xsf, wsf, one, one)
        rq, rsf = nvf_cutlass.nvfp4_scaled_mm_blockscale(xq[:200].contiguous(), wq[:160].contiguous(), xsf[:256].contiguous(),
                                                         wsf[:256].contiguous(), one, one)
        return [gs, dense, decode, split, static, grouped[: sum(sizes)], bf[: sum(sizes)], mx, bq.view(torch.uint8), bsf.view(torch.uint8),
                rq.view(torch.uint8), rsf.view(torch.uint8)]

    eager = [t.clone() for t in chain()]  # also the warm-up: function attributes are set outside the capture
    assert capi.lib().nvf_nvfp4_scaled_mm_workspace_bytes(72, 6144, 8192) > 0 and torch.equal(eager[3], eager[4])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = chain()
    torch.cuda.synchronize()
    for replay in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want), replay
        # the program's own eager work between replays
        assert torch.isfinite(nvf_cutlass.grouped_mm(x, wg, st, ct, ps, eo)[: sum(sizes)].float()).all()
    # new data in the captured input buffers: the replay follows it
    x.copy_(torch.randn(m, k, device=dev, generator=gen).bfloat16())
    eager2 = [t.clone() for t in chain()]
    graph.replay()
    torch.cuda.synchronize()
    for got, want in zip(outs, eager2):
        assert torch.equal(got, want)
    assert not torch.equal(eager[1], eager2[1])
