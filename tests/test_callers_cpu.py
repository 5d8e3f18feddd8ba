"""Host logic of the caller conventions (csrc/ir/composite_nodes.cpp:1133-1162, 1427-1459, 1663-1712) and of
the torch.library op of the MoE layers (benchmarks/python/layers_for_inference_benchmark.py:217-279,
395-424): argument synthesis against hand-derived values, "return None so the caller falls back", the
fake (shape-only) implementation.  No GPU work."""
import pytest
import torch


def test_grouped_mma_arguments_from_end_offsets():
    from fuser_amd import _C

    # ends [3, 3, 10, 16]: groups of 3, 0, 7 and 6 rows starting at 0, 3, 3, 10
    ps, starts, ab, cs = _C.callers.grouped_mma_arguments(torch.tensor([3, 3, 10, 16], dtype=torch.int32), 64, 32)
    assert ps.dtype == torch.int32 and starts.dtype == torch.int32 and ab.dtype == torch.int64 and cs.dtype == torch.int64
    assert ps.tolist() == [[3, 64, 32], [0, 64, 32], [7, 64, 32], [6, 64, 32]]
    assert starts.tolist() == [0, 3, 3, 10]
    assert ab.tolist() == [32] * 4 and cs.tolist() == [64] * 4
    ps, starts, _, _ = _C.callers.grouped_mma_arguments(torch.tensor([5], dtype=torch.int32), 8, 8)
    assert ps.tolist() == [[5, 8, 8]] and starts.tolist() == [0]
    with pytest.raises(RuntimeError):
        _C.callers.grouped_mma_arguments(torch.zeros(2, 2, dtype=torch.int32), 8, 8)


def test_kernel_branch_declines_operands_it_cannot_take():
    from fuser_amd import _C

    a = torch.zeros(4, 16, dtype=torch.bfloat16)
    w = torch.zeros(2, 8, 16, dtype=torch.bfloat16)  # [G, N, K]
    ends = torch.tensor([2, 4], dtype=torch.int32)
    assert _C.callers.grouped_mma(a, w, ends) is None                  # mat2 must be the [G, K, N] view of it
    assert _C.callers.grouped_mma(a.view(2, 2, 16), w.transpose(1, 2), ends) is None  # mat1 must be 2D
    assert _C.callers.grouped_mma(a.t().contiguous().t(), w.transpose(1, 2), ends) is None  # mat1 not contiguous

    q = torch.zeros(128, 32, dtype=torch.uint8).view(torch.float4_e2m1fn_x2)
    wq = torch.zeros(64, 32, dtype=torch.uint8).view(torch.float4_e2m1fn_x2).t()  # graph-level [K/2, N] view
    s1 = torch.zeros(128, 4, dtype=torch.uint8).view(torch.float8_e4m3fn)
    s2 = torch.zeros(128, 4, dtype=torch.uint8).view(torch.float8_e4m3fn)
    alpha = torch.ones((), dtype=torch.float32)
    # CPU tensors do not validate, a bias / beta is not supported by the kernel, alpha is required
    assert _C.callers.scaled_mma(q, wq, s1, s2, alpha) is None
    assert _C.callers.scaled_mma(q, wq, s1, s2, alpha, bias=torch.zeros(64)) is None
    assert _C.callers.scaled_mma(q, wq, s1, s2, alpha, beta=torch.ones(())) is None
    assert _C.callers.scaled_mma(q, wq, s1, s2, None) is None
    assert _C.callers.scaled_mma(q, wq.reshape(2, 16, 64), s1, s2, alpha) is None


def test_nvfp4_grouped_mma_checks_operand_types_and_problem_sizes():
    from fuser_amd import _C

    q = torch.zeros(8, 32, dtype=torch.uint8)
    w = torch.zeros(2, 16, 32, dtype=torch.uint8)
    sf = torch.zeros(128, 4, dtype=torch.uint8).view(torch.float8_e4m3fn)
    i32 = torch.zeros(2, dtype=torch.int32)
    ps = torch.zeros(2, 3, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="Float4_e2m1fn_x2"):
        _C.callers.cutlass_nvfp4_grouped_mma(q, w.transpose(1, 2), sf, sf, torch.ones(2), ps, i32, i32)
    q4, w4 = q.view(torch.float4_e2m1fn_x2), w.view(torch.float4_e2m1fn_x2)
    with pytest.raises(RuntimeError, match="2D tensor"):
        _C.callers.cutlass_nvfp4_grouped_mma(q4, w4.transpose(1, 2), sf, sf, torch.ones(2), ps.reshape(-1), i32, i32)
    with pytest.raises(RuntimeError, match=r"\(num_experts, 3\)"):
        _C.callers.cutlass_nvfp4_grouped_mma(q4, w4.transpose(1, 2), sf, sf, torch.ones(2), ps[:, :2], i32, i32)


def test_auxiliary_tensors_of_the_grouped_linear():
    from fuser_amd import custom_ops

    hidden = torch.zeros(16, 32)
    starts = torch.tensor([0, 3, 3, 10], dtype=torch.int32)
    so, ps = custom_ops.compute_auxiliary_tensors(hidden, starts, 64)
    assert ps.tolist() == [[3, 64, 32], [0, 64, 32], [7, 64, 32], [6, 64, 32]]
    assert so.dtype == torch.int32 and so.tolist() == [0, 128, 128, 256]   # slabs of 128, 0, 128 rows before
    so, ps = custom_ops.compute_auxiliary_tensors(torch.zeros(400, 32), torch.tensor([0, 129], dtype=torch.int32), 8)
    assert ps[:, 0].tolist() == [129, 271] and so.tolist() == [0, 256]


def test_custom_op_is_registered_with_a_shape_only_implementation():
    from fuser_amd import custom_ops  # noqa: F401  (registers the op)

    op = torch.ops.nvf_cutlass.f16a_nvfp4weight_scaled_grouped_mm
    g, k, n = 2, 64, 48
    act = torch.empty(3, 5, k, dtype=torch.bfloat16, device="meta")
    w = torch.empty(g, n, k // 2, dtype=torch.uint8, device="meta").transpose(1, 2)
    sf = torch.empty(g, n, k // 16, dtype=torch.uint8, device="meta")
    gs = torch.empty(g, device="meta")
    i32 = torch.empty(g, dtype=torch.int32, device="meta")
    ps = torch.empty(g, 3, dtype=torch.int32, device="meta")
    out = op(act, w, sf, gs, i32, i32, ps)
    assert out.shape == (3, 5, n) and out.dtype == torch.bfloat16 and out.device.type == "meta"
    with pytest.raises(ValueError, match="at least 1 dimension"):
        op(torch.empty((), dtype=torch.bfloat16, device="meta"), w, sf, gs, i32, i32, ps)
