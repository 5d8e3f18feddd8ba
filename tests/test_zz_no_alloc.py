"""nvf_nvfp4_scaled_mm_static_ws: the split-K NVFP4 GEMM with the library's own static scratch array instead of a
caller-provided workspace, for callers that cannot allocate.  Through the raw C ABI its output must be
bit-identical to nvf_nvfp4_scaled_mm_ws (same kernels, same fixed-order reduction), on two calls in a row that
share the array -- the second with a smaller input -- and also after the array has been used by another shape."""
import pytest
import torch

from helpers import GEMM_MAX_REL, gs_of, max_rel
from oracle import nvf_oracle as O

pytestmark = pytest.mark.gpu


def _operand(rows, k, std, gen):
    x = (torch.randn(rows, k, generator=gen) * std).bfloat16()
    gs = gs_of(x)
    q, s = O.block_quantize_nvfp4(x, gs, True)
    return q, s, gs


def test_static_scratch_entry_point_equals_the_workspace_entry_point(dev):
    from fuser_amd import capi

    lib = capi.lib()
    # two split-K shapes of the tile kernel, the second smaller (fewer rows and columns; ragged N / K), one of the
    # weight-streaming kernel; then the first again
    for call, (m, n, k) in enumerate([(640, 4224, 12320), (512, 3104, 12320), (80, 6144, 8192), (640, 4224, 12320)]):
        gen = torch.Generator().manual_seed(100 + call)
        a, sa, ga = _operand(m, k, 1.0, gen)
        b, sb, gb = _operand(n, k, 0.02, gen)
        alpha = 1.0 / (ga * gb)
        need = lib.nvf_nvfp4_scaled_mm_workspace_bytes(m, n, k)
        assert 0 < need <= capi.STATIC_SCRATCH_BYTES
        ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
        al = torch.tensor(alpha, dtype=torch.float32, device=dev)
        ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=dev)
        for dt, code in ((torch.bfloat16, capi.BF16), (torch.float16, capi.F16)):
            want = torch.full((m, n), 7.0, dtype=dt, device=dev)
            got = torch.full((m, n), 9.0, dtype=dt, device=dev)
            capi.check(lib.nvf_nvfp4_scaled_mm_ws(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), al.data_ptr(),
                                                  want.data_ptr(), m, n, k, code, ws.data_ptr(), need, None))
            capi.check(lib.nvf_nvfp4_scaled_mm_static_ws(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), al.data_ptr(),
                                                         got.data_ptr(), m, n, k, code, None))
            torch.cuda.synchronize()
            assert torch.equal(got, want), (call, m, n, k, dt)
            assert max_rel(got, O.ref_nvfp4_scaled_mm(a, b, sa, sb, alpha)) <= GEMM_MAX_REL
    # a shape that needs no scratch runs as nvf_nvfp4_scaled_mm does
    m, n, k = 16, 512, 1024
    gen = torch.Generator().manual_seed(7)
    a, sa, ga = _operand(m, k, 1.0, gen)
    b, sb, gb = _operand(n, k, 0.02, gen)
    al = torch.tensor(1.0 / (ga * gb), dtype=torch.float32, device=dev)
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    want = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    got = torch.empty_like(want)
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(m, n, k) == 0
    capi.check(lib.nvf_nvfp4_scaled_mm(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), al.data_ptr(), want.data_ptr(), m, n, k,
                                       capi.BF16, None))
    capi.check(lib.nvf_nvfp4_scaled_mm_static_ws(ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), al.data_ptr(), got.data_ptr(),
                                                 m, n, k, capi.BF16, None))
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # The largest scratch any split asks for on 256 compute units is the static array (at most 2 x 256 work items of
    # 128 x 128 fp32); the first shape above comes within 4 % of it (3 splits of 5 x 33 tiles).
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(640, 4224, 12320) > 0.96 * capi.STATIC_SCRATCH_BYTES
